// int4 weight-only decode linears for MI355X (gfx950 / CDNA4).
//
// Replaces the bf16 nn.Linear calls of the rollout decode step that the
// reference reaches at vrl/models/families/janus_pro/policy.py:673-678 (Llama
// trunk projections) and policy.py:138-160 (gen_head).  Operand formats and the
// arithmetic contract are stated in include/vrl_int4.h.
//
// Kernels
//   dequant_kernel        packed int4 -> bf16 [N,K], bit-exact, write-bound.
//   gemv_tile_kernel      the hot path.  A workgroup owns TILE_ROWS weight rows;
//                         its waves split K in 128-wide chunks.  Each lane
//                         streams 16-byte pieces of "its" row (lane%16) with
//                         global_load_dwordx4, rebuilds the exactly rounded bf16
//                         weights in registers and feeds them to
//                         v_mfma_f32_16x16x32_bf16 as the B operand; the
//                         activations are staged once per workgroup in LDS (in
//                         the k-order the unpack produces) and read as the A
//                         operand.  Partial sums of the K split meet in LDS.
//   gemv_generic_kernel   any legal shape (K%8, G%8): one wave per row, VALU
//                         dot product, DPP/shuffle reduction.  Correctness
//                         fallback for shapes the tile kernel does not take.
//
// In-register dequant, exact by construction: nibble pairs (i, i+4) of a packed
// word are turned into two bf16 numbers 128+q with one shift and one and-or
// ((v >> 4i) & 0x000F000F | 0x43004300), then
//   v_dot2_f32_bf16(pair, (s,0) or (0,s), c)   with  c = -(128+z)*s  (fp32, exact)
// gives (q-z)*s exactly (16-bit products, 12-bit result), and
// v_cvt_pk_bf16_f32 applies the one round-to-nearest-even the contract asks for.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <type_traits>
#include <vector>

#include "../../include/vrl_int4.h"

namespace {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

// Pointers read out of a plan record lose their address space; loads through these
// typedefs are global_load (vmcnt only) instead of flat_load (vmcnt and lgkmcnt).
typedef const __attribute__((address_space(1))) u32x4_t *gptr_u4;

typedef __attribute__((address_space(1))) uint16_t *gptr_u16;
typedef const __attribute__((address_space(1))) uint16_t *gptr_cu16;
typedef const __attribute__((address_space(1))) uint32_t *gptr_cu32;

__device__ __forceinline__ gptr_u4 as_global(const u32x4_t *p) {
    return (gptr_u4)(uintptr_t)p;
}
__device__ __forceinline__ gptr_u16 as_global(uint16_t *p) { return (gptr_u16)(uintptr_t)p; }
__device__ __forceinline__ gptr_cu16 as_global(const uint16_t *p) { return (gptr_cu16)(uintptr_t)p; }
__device__ __forceinline__ gptr_cu32 as_global(const uint32_t *p) { return (gptr_cu32)(uintptr_t)p; }

constexpr int WAVE = 64;
constexpr int KCHUNK = 128;          // k covered by one wave step (4 lanes x 32 k per row)
constexpr uint32_t PAIR_MASK = 0x000F000Fu;
constexpr uint32_t PAIR_BIAS = 0x43004300u;  // two bf16 128.0

// Device-side problem record (72 bytes).  Also the element type of a grouped plan.
struct DevProblem {
    const uint16_t *x;
    const uint32_t *qweight;
    const uint16_t *scales;
    const uint32_t *qzeros;
    uint16_t *y;
    int32_t M, N, K, G;
    int32_t fused;       // gate||up rows with SiLU epilogue
    int32_t tile_begin;  // first tile index of this problem inside a grouped launch
    int32_t kc;          // k extent of x staged in LDS per pass (multiple of KCHUNK)
    int32_t prepacked;   // bit 0: qweight points at a prepacked blob (scales/qzeros unused);
                         // bit 1: a row of zeros is staged behind the activation rows (PP_ZERO_ROW)
};
static_assert(sizeof(DevProblem) == 72, "plan record layout is part of the plan format");

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits) {
    return __builtin_bit_cast(float, bits << 16);
}

__device__ __forceinline__ uint32_t pack_bf16_rne(float lo, float hi) {
    bf16x2_t r;
    r[0] = (__bf16)lo;  // v_cvt_pk_bf16_f32: round-to-nearest-even
    r[1] = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, r);
}

// Per-(row, group) dequant constants held by a lane.
struct GroupConst {
    uint32_t s_lo;  // bf16 pair (s, 0)
    uint32_t s_hi;  // bf16 pair (0, s)
    float c;        // -(128 + z) * s, exact in fp32
};

__device__ __forceinline__ GroupConst make_group_const(uint32_t scale_bits, uint32_t z) {
    GroupConst g;
    g.s_lo = scale_bits & 0xFFFFu;
    g.s_hi = scale_bits << 16;
    g.c = -(128.0f + (float)z) * bf16_bits_to_f32(scale_bits & 0xFFFFu);
    return g;
}

// One packed word -> 8 exactly rounded bf16 weights in the order
// (w0,w4),(w1,w5),(w2,w6),(w3,w7): four dwords.
//
// One asm block on purpose.  On gfx90a and later the result of a DOT instruction
// may not be read (or overwritten) by a different VALU instruction for three
// wait states and the hardware does not interlock; the compiler cannot see
// inside inline asm, so the order below keeps every v_cvt_pk at least three
// instructions behind the v_dot2 it reads, and the trailing s_nop covers the
// consumer of the last v_cvt_pk.
__device__ __forceinline__ void dequant_word(uint32_t v, const GroupConst &g, uint32_t bias,
                                             uint32_t out[4]) {
    uint32_t p0, p1, p2, p3, d0, d1, d2, d3, d4, d5, d6, d7;
    asm("v_and_or_b32 %[p0], %[v], %[mask], %[bias]\n\t"
        "v_lshrrev_b32 %[p1], 4, %[v]\n\t"
        "v_lshrrev_b32 %[p2], 8, %[v]\n\t"
        "v_lshrrev_b32 %[p3], 12, %[v]\n\t"
        "v_and_or_b32 %[p1], %[p1], %[mask], %[bias]\n\t"
        "v_and_or_b32 %[p2], %[p2], %[mask], %[bias]\n\t"
        "v_and_or_b32 %[p3], %[p3], %[mask], %[bias]\n\t"
        "v_dot2_f32_bf16 %[d0], %[p0], %[slo], %[c]\n\t"
        "v_dot2_f32_bf16 %[d1], %[p0], %[shi], %[c]\n\t"
        "v_dot2_f32_bf16 %[d2], %[p1], %[slo], %[c]\n\t"
        "v_dot2_f32_bf16 %[d3], %[p1], %[shi], %[c]\n\t"
        "v_dot2_f32_bf16 %[d4], %[p2], %[slo], %[c]\n\t"
        "v_dot2_f32_bf16 %[d5], %[p2], %[shi], %[c]\n\t"
        "v_dot2_f32_bf16 %[d6], %[p3], %[slo], %[c]\n\t"
        "v_dot2_f32_bf16 %[d7], %[p3], %[shi], %[c]\n\t"
        "v_cvt_pk_bf16_f32 %[d0], %[d0], %[d1]\n\t"
        "v_cvt_pk_bf16_f32 %[d2], %[d2], %[d3]\n\t"
        "v_cvt_pk_bf16_f32 %[d4], %[d4], %[d5]\n\t"
        "v_cvt_pk_bf16_f32 %[d6], %[d6], %[d7]\n\t"
        "s_nop 1"
        : [p0] "=&v"(p0), [p1] "=&v"(p1), [p2] "=&v"(p2), [p3] "=&v"(p3), [d0] "=&v"(d0),
          [d1] "=&v"(d1), [d2] "=&v"(d2), [d3] "=&v"(d3), [d4] "=&v"(d4), [d5] "=&v"(d5),
          [d6] "=&v"(d6), [d7] "=&v"(d7)
        : [v] "v"(v), [slo] "v"(g.s_lo), [shi] "v"(g.s_hi), [c] "v"(g.c), [mask] "s"(PAIR_MASK),
          [bias] "v"(bias));
    out[0] = d0;
    out[1] = d2;
    out[2] = d4;
    out[3] = d6;
}

// -------------------------------------------------------------------------
// dequant: one thread per packed word, natural k order out
// -------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dequant_kernel(const uint32_t *__restrict__ qweight,
                                                      const uint16_t *__restrict__ scales,
                                                      const uint32_t *__restrict__ qzeros,
                                                      uint16_t *__restrict__ w, int N, int K, int G) {
    const int kwords = K >> 3;
    const int groups = K / G;
    const int zwords = (groups + 7) >> 3;
    const long total = (long)N * kwords;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int n = (int)(idx / kwords);
        const int r = (int)(idx - (long)n * kwords);
        const int g = (r << 3) / G;
        const uint32_t v = qweight[idx];
        const float s = bf16_bits_to_f32(scales[(long)n * groups + g]);
        const int z = (qzeros[(long)n * zwords + (g >> 3)] >> (4 * (g & 7))) & 0xF;
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int q0 = (v >> (8 * i)) & 0xF;
            const int q1 = (v >> (8 * i + 4)) & 0xF;
            o[i] = pack_bf16_rne((float)(q0 - z) * s, (float)(q1 - z) * s);
        }
        u32x4_t ov = {o[0], o[1], o[2], o[3]};
        *reinterpret_cast<u32x4_t *>(w + idx * 8) = ov;
    }
}

// -------------------------------------------------------------------------
// generic GEMV: one wave per output row (pair of rows when fused)
// -------------------------------------------------------------------------
constexpr int GEN_MT = 4;  // activation rows per pass

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
    return v;
}

__device__ __forceinline__ void generic_row_dot(const DevProblem &p, int n, int m0, int mt,
                                                float acc[GEN_MT]) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int kwords = p.K >> 3;
    const int groups = p.K / p.G;
    const int zwords = (groups + 7) >> 3;
#pragma unroll
    for (int j = 0; j < GEN_MT; ++j) acc[j] = 0.0f;
    for (int r = lane; r < kwords; r += WAVE) {
        const int g = (r << 3) / p.G;
        const uint32_t v = p.qweight[(long)n * kwords + r];
        const float s = bf16_bits_to_f32(p.scales[(long)n * groups + g]);
        const int z = (p.qzeros[(long)n * zwords + (g >> 3)] >> (4 * (g & 7))) & 0xF;
        float wv[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int q0 = (v >> (8 * i)) & 0xF;
            const int q1 = (v >> (8 * i + 4)) & 0xF;
            const uint32_t pk = pack_bf16_rne((float)(q0 - z) * s, (float)(q1 - z) * s);
            wv[2 * i] = bf16_bits_to_f32(pk & 0xFFFFu);
            wv[2 * i + 1] = bf16_bits_to_f32(pk >> 16);
        }
#pragma unroll
        for (int j = 0; j < GEN_MT; ++j) {
            if (j < mt) {
                const u32x4_t xv =
                    *reinterpret_cast<const u32x4_t *>(p.x + (long)(m0 + j) * p.K + (r << 3));
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[j] = __builtin_fmaf(bf16_bits_to_f32(xv[i] & 0xFFFFu), wv[2 * i], acc[j]);
                    acc[j] = __builtin_fmaf(bf16_bits_to_f32(xv[i] >> 16), wv[2 * i + 1], acc[j]);
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < GEN_MT; ++j) acc[j] = wave_sum(acc[j]);
}

__global__ __launch_bounds__(256) void gemv_generic_kernel(DevProblem p) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x >> 6;
    const int out_cols = p.fused ? p.N / 2 : p.N;
    const int n = blockIdx.x * (blockDim.x >> 6) + wave;
    if (n >= out_cols) return;  // whole wave leaves together
    for (int m0 = 0; m0 < p.M; m0 += GEN_MT) {
        const int mt = min(GEN_MT, p.M - m0);
        float a[GEN_MT], b[GEN_MT];
        generic_row_dot(p, n, m0, mt, a);
        if (p.fused) generic_row_dot(p, out_cols + n, m0, mt, b);
        if (lane == 0) {
            for (int j = 0; j < mt; ++j) {
                float v = a[j];
                if (p.fused) v = (v / (1.0f + __expf(-v))) * b[j];
                p.y[(long)(m0 + j) * out_cols + n] = (uint16_t)(pack_bf16_rne(v, 0.0f) & 0xFFFFu);
            }
        }
    }
}

// -------------------------------------------------------------------------
// tile GEMV (MFMA dot, VALU dequant)
// -------------------------------------------------------------------------
// R   weight row tiles (16 rows each) per workgroup; fused problems use R/2
//     gate tiles followed by R/2 up tiles and emit 16*R/2 output columns.
// MB  16-row blocks of activations (M <= 16*MB).
// WPB waves per workgroup; wave w owns k-chunks c with c % WPB == w.
template <int R, int MB, int WPB>
struct TileCfg {
    static constexpr int THREADS = WPB * WAVE;
    static constexpr int RED_FLOATS = WPB * R * MB * 256;
};

constexpr int XPAD = 8;  // bf16 elements of padding per staged activation row (16 bytes)

template <int R>
struct Prefetch {
    u32x4_t w[R];
    uint32_t sbits[R];
    uint32_t zword[R];
};

template <int R, int MB, int WPB>
__device__ __forceinline__ void tile_body(const DevProblem &p, int tile, uint8_t *smem) {
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid >> 6;
    const int lc = lane & 15;  // weight row within a tile / activation row within a block
    const int kq = lane >> 4;  // which 32-k quarter of the chunk this lane streams

    const int K = p.K, G = p.G, M = p.M;
    const int kwords = K >> 3;
    const int groups = K / G;
    const int zwords = (groups + 7) >> 3;
    const bool fused = p.fused != 0;
    const int out_cols = fused ? p.N / 2 : p.N;
    const int cols_per_tile = fused ? 16 * (R / 2) : 16 * R;
    const int col0 = tile * cols_per_tile;

    // weight row streamed by this lane for each of the R tiles (clamped: rows past
    // the end are loaded from the last row and their results never stored)
    long row_off[R];
    long sc_off[R];
    long z_off[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        int row;
        if (fused) {
            constexpr int H = R > 1 ? R / 2 : 1;  // fused launches always have R >= 2
            const int half = r / H;
            const int c = col0 + 16 * (r % H) + lc;
            row = half * out_cols + min(c, out_cols - 1);
        } else {
            row = min(col0 + 16 * r + lc, p.N - 1);
        }
        row_off[r] = (long)row * kwords;
        sc_off[r] = (long)row * groups;
        z_off[r] = (long)row * zwords;
    }

    f32x4_t acc[R][MB];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int b = 0; b < MB; ++b) acc[r][b] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    uint16_t *xs = reinterpret_cast<uint16_t *>(smem);
    const int kc = p.kc;                 // staged k extent
    const int xstride = kc + XPAD;       // bf16 elements per staged row
    const uint32_t bias = PAIR_BIAS;

    auto issue = [&](int chunk, Prefetch<R> &pf) {
        const int k0 = chunk * KCHUNK + 32 * kq;
        const int g = k0 / G;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            pf.w[r] = *reinterpret_cast<const u32x4_t *>(p.qweight + row_off[r] + (k0 >> 3));
            pf.sbits[r] = p.scales[sc_off[r] + g];
            pf.zword[r] = p.qzeros[z_off[r] + (g >> 3)];
        }
        return g;
    };

    // the first chunk of weights does not depend on x: request it before staging, so that a
    // small matrix costs one memory round trip instead of two
    Prefetch<R> cur, nxt;
    int g_cur = 0, g_nxt = 0;
    if (wave * KCHUNK < min(kc, K)) g_cur = issue(wave, cur);

    for (int kbase = 0; kbase < K; kbase += kc) {
        const int kext = min(kc, K - kbase);
        // ---- stage x[:, kbase : kbase+kext] into LDS, pair-interleaved per 8 k ----
        if (kbase != 0) __syncthreads();
        {
            const int words_per_row = kext >> 3;  // 16-byte pieces
            const int total = M * words_per_row;
            for (int idx = tid; idx < total; idx += WPB * WAVE) {
                const int m = idx / words_per_row;
                const int j = idx - m * words_per_row;
                const u32x4_t d =
                    *reinterpret_cast<const u32x4_t *>(p.x + (long)m * K + kbase + (j << 3));
                u32x4_t o;
                o[0] = (d[0] & 0xFFFFu) | (d[2] << 16);          // x0, x4
                o[1] = (d[0] >> 16) | (d[2] & 0xFFFF0000u);      // x1, x5
                o[2] = (d[1] & 0xFFFFu) | (d[3] << 16);          // x2, x6
                o[3] = (d[1] >> 16) | (d[3] & 0xFFFF0000u);      // x3, x7
                *reinterpret_cast<u32x4_t *>(xs + m * xstride + (j << 3)) = o;
            }
        }
        __syncthreads();

        const int c_begin = kbase / KCHUNK;
        const int c_end = (kbase + kext) / KCHUNK;
        int chunk = c_begin + wave;
        if (kbase != 0 && chunk < c_end) g_cur = issue(chunk, cur);
        for (; chunk < c_end; chunk += WPB) {
            const bool more = chunk + WPB < c_end;
            if (more) g_nxt = issue(chunk + WPB, nxt);

            // activations for this chunk: A operands, 4 k-steps x MB row blocks
            bf16x8_t xa[4][MB];
            const int kloc = chunk * KCHUNK - kbase + 32 * kq;
#pragma unroll
            for (int b = 0; b < MB; ++b) {
                const int m = min(16 * b + lc, M - 1);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const u32x4_t raw =
                        *reinterpret_cast<const u32x4_t *>(xs + m * xstride + kloc + 8 * t);
                    xa[t][b] = __builtin_bit_cast(bf16x8_t, raw);
                }
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t z = (cur.zword[r] >> (4 * (g_cur & 7))) & 0xFu;
                const GroupConst gc = make_group_const(cur.sbits[r], z);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    uint32_t wb[4];
                    dequant_word(cur.w[r][t], gc, bias, wb);
                    const u32x4_t wv = {wb[0], wb[1], wb[2], wb[3]};
                    const bf16x8_t bop = __builtin_bit_cast(bf16x8_t, wv);
#pragma unroll
                    for (int b = 0; b < MB; ++b)
                        acc[r][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[t][b], bop,
                                                                            acc[r][b], 0, 0, 0);
                }
            }
            if (more) {
                cur = nxt;
                g_cur = g_nxt;
            }
        }
    }

    // ---- meet the K split: partial tiles -> LDS -> sum -> epilogue ----
    __syncthreads();
    float *red = reinterpret_cast<float *>(smem);
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                red[((wave * R + r) * MB + b) * 256 + i * WAVE + lane] = acc[r][b][i];
    __syncthreads();

    // element e of a (tile r, block b) slab: i = e / 64, lane = e % 64 ->
    //   activation row m = 16 b + 4 (lane / 16) + i, column = lane % 16
    const int RO = fused ? R / 2 : R;
    const int count = RO * MB * 256;
    for (int e = tid; e < count; e += WPB * WAVE) {
        const int slab = e >> 8;
        const int r = slab / MB;
        const int b = slab - r * MB;
        const int within = e & 255;
        const int i = within >> 6;
        const int ln = within & 63;
        const int m = 16 * b + 4 * (ln >> 4) + i;
        const int col = col0 + 16 * r + (ln & 15);
        if (m >= M || col >= out_cols) continue;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < WPB; ++w) v += red[((w * R + r) * MB + b) * 256 + within];
        if (fused) {
            float u = 0.f;
#pragma unroll
            for (int w = 0; w < WPB; ++w) u += red[((w * R + r + R / 2) * MB + b) * 256 + within];
            v = (v / (1.0f + __expf(-v))) * u;
        }
        p.y[(long)m * out_cols + col] = (uint16_t)(pack_bf16_rne(v, 0.0f) & 0xFFFFu);
    }
}

template <int R, int MB, int WPB>
__global__ __launch_bounds__(WPB *WAVE) void gemv_tile_kernel(DevProblem p) {
    extern __shared__ __align__(16) uint8_t smem[];
    tile_body<R, MB, WPB>(p, blockIdx.x, smem);
}

// -------------------------------------------------------------------------
// stream GEMV (grouped launches): a wave owns 16 weight rows for all of K
// -------------------------------------------------------------------------
// The tile list of a plan (16 output columns per tile, all problems back to
// back) is cut into one contiguous range per workgroup, balanced by bytes.  A
// workgroup walks its range problem by problem: it stages that problem's
// activations in LDS once, then each wave streams whole tiles - no K split, so
// no partial sums to meet - keeping STREAM_DEPTH 128-k chunks of its 16 rows in
// flight (non-temporal global_load_dwordx4: the weights are read exactly once).
constexpr int STREAM_DEPTH = 4;

template <int RS>
struct Slot {
    u32x4_t w[RS];
    uint32_t sbits[RS];
    uint32_t zword[RS];
};

__device__ __forceinline__ void stage_x(const DevProblem &p, int kbase, int kext, uint16_t *xs,
                                        int xstride, int nthreads) {
    const int words_per_row = kext >> 3;  // 16-byte pieces
    const int total = p.M * words_per_row;
    for (int idx = threadIdx.x; idx < total; idx += nthreads) {
        const int m = idx / words_per_row;
        const int j = idx - m * words_per_row;
        const u32x4_t d = *as_global(reinterpret_cast<const u32x4_t *>(p.x + (long)m * p.K + kbase + (j << 3)));
        u32x4_t o;
        o[0] = (d[0] & 0xFFFFu) | (d[2] << 16);      // x0, x4
        o[1] = (d[0] >> 16) | (d[2] & 0xFFFF0000u);  // x1, x5
        o[2] = (d[1] & 0xFFFFu) | (d[3] << 16);      // x2, x6
        o[3] = (d[1] >> 16) | (d[3] & 0xFFFF0000u);  // x3, x7
        *reinterpret_cast<u32x4_t *>(xs + m * xstride + (j << 3)) = o;
    }
}

// acc += x[:, kbase:kbase+kext] . W[tile rows, kbase:kbase+kext]^T for this wave's tile
template <int MB, bool FUSED>
__device__ __forceinline__ void stream_rows(const DevProblem &p, int tile_local, const uint16_t *xs,
                                            int xstride, int kbase, int kext, int gshift,
                                            f32x4_t (&acc)[FUSED ? 2 : 1][MB]) {
    constexpr int RS = FUSED ? 2 : 1;
    const int lane = threadIdx.x & (WAVE - 1);
    const int lc = lane & 15;
    const int kq = lane >> 4;
    const int kwords = p.K >> 3;
    const int groups = p.K >> gshift;
    const int zwords = (groups + 7) >> 3;
    const int out_cols = FUSED ? p.N / 2 : p.N;

    gptr_cu32 wp[RS];
    gptr_cu16 sp[RS];
    gptr_cu32 zp[RS];
#pragma unroll
    for (int r = 0; r < RS; ++r) {
        const long row = (long)r * out_cols + min(tile_local * 16 + lc, out_cols - 1);
        wp[r] = as_global(p.qweight) + row * kwords + (kbase >> 3) + 4 * kq;
        sp[r] = as_global(p.scales) + row * groups;
        zp[r] = as_global(p.qzeros) + row * zwords;
    }
    const int nch = kext >> 7;
    const uint32_t bias = PAIR_BIAS;
    Slot<RS> ring[STREAM_DEPTH];

    auto issue = [&](Slot<RS> &s, int c) {
        const int g = (kbase + c * KCHUNK + 32 * kq) >> gshift;
#pragma unroll
        for (int r = 0; r < RS; ++r) {
            s.w[r] = __builtin_nontemporal_load((gptr_u4)(wp[r] + c * 16));
            s.sbits[r] = sp[r][g];
            s.zword[r] = zp[r][g >> 3];
        }
    };
    auto compute = [&](const Slot<RS> &s, int c) {
        const int g = (kbase + c * KCHUNK + 32 * kq) >> gshift;
        const int kloc = c * KCHUNK + 32 * kq;
        bf16x8_t xa[4][MB];
#pragma unroll
        for (int b = 0; b < MB; ++b) {
            const int m = min(16 * b + lc, p.M - 1);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const u32x4_t raw = *reinterpret_cast<const u32x4_t *>(xs + m * xstride + kloc + 8 * t);
                xa[t][b] = __builtin_bit_cast(bf16x8_t, raw);
            }
        }
#pragma unroll
        for (int r = 0; r < RS; ++r) {
            const uint32_t z = (s.zword[r] >> (4 * (g & 7))) & 0xFu;
            const GroupConst gc = make_group_const(s.sbits[r], z);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                uint32_t wb[4];
                dequant_word(s.w[r][t], gc, bias, wb);
                const u32x4_t wv = {wb[0], wb[1], wb[2], wb[3]};
                const bf16x8_t bop = __builtin_bit_cast(bf16x8_t, wv);
#pragma unroll
                for (int b = 0; b < MB; ++b)
                    acc[r][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[t][b], bop, acc[r][b], 0, 0, 0);
            }
        }
    };

#pragma unroll
    for (int d = 0; d < STREAM_DEPTH; ++d)
        if (d < nch) issue(ring[d], d);
    for (int c0 = 0; c0 < nch; c0 += STREAM_DEPTH) {
#pragma unroll
        for (int d = 0; d < STREAM_DEPTH; ++d) {
            if (c0 + d < nch) {
                compute(ring[d], c0 + d);
                if (c0 + d + STREAM_DEPTH < nch) issue(ring[d], c0 + d + STREAM_DEPTH);
            }
        }
    }
}

template <int MB, bool FUSED>
__device__ __forceinline__ void store_tile(const DevProblem &p, int tile_local,
                                           const f32x4_t (&acc)[FUSED ? 2 : 1][MB]) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int out_cols = FUSED ? p.N / 2 : p.N;
    const int col = tile_local * 16 + (lane & 15);
    if (col >= out_cols) return;
#pragma unroll
    for (int b = 0; b < MB; ++b)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = 16 * b + 4 * (lane >> 4) + i;
            if (m < p.M) {
                float v = acc[0][b][i];
                if (FUSED) v = (v / (1.0f + __expf(-v))) * acc[FUSED ? 1 : 0][b][i];
                // a global (not flat) store: a pending flat access makes every later wait on
                // the load counter a wait for zero
                as_global(p.y)[(long)m * out_cols + col] = (uint16_t)(pack_bf16_rne(v, 0.0f) & 0xFFFFu);
            }
        }
}

// tiles [t0, t1) of problem p (local tile indices); all waves of the block call this together
template <int MB, bool FUSED, int WPB>
__device__ __forceinline__ void stream_segment(const DevProblem &p, int t0, int t1, uint8_t *smem) {
    constexpr int RS = FUSED ? 2 : 1;
    const int wave = threadIdx.x >> 6;
    const int gshift = __builtin_ctz((unsigned)p.G);
    uint16_t *xs = reinterpret_cast<uint16_t *>(smem);
    const int xstride = p.kc + XPAD;
    if (p.kc >= p.K) {
        __syncthreads();  // readers of whatever was staged before are done
        stage_x(p, 0, p.K, xs, xstride, WPB * WAVE);
        __syncthreads();
        for (int tile = t0 + wave; tile < t1; tile += WPB) {
            f32x4_t acc[RS][MB];
#pragma unroll
            for (int r = 0; r < RS; ++r)
#pragma unroll
                for (int b = 0; b < MB; ++b) acc[r][b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            stream_rows<MB, FUSED>(p, tile, xs, xstride, 0, p.K, gshift, acc);
            store_tile<MB, FUSED>(p, tile, acc);
        }
    } else {
        // activations do not fit: rounds of one tile per wave, K walked in staged passes
        for (int round = t0; round < t1; round += WPB) {
            const int tile = round + wave;
            const bool active = tile < t1;
            f32x4_t acc[RS][MB];
#pragma unroll
            for (int r = 0; r < RS; ++r)
#pragma unroll
                for (int b = 0; b < MB; ++b) acc[r][b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            for (int kbase = 0; kbase < p.K; kbase += p.kc) {
                const int kext = min(p.kc, p.K - kbase);
                __syncthreads();
                stage_x(p, kbase, kext, xs, xstride, WPB * WAVE);
                __syncthreads();
                if (active) stream_rows<MB, FUSED>(p, tile, xs, xstride, kbase, kext, gshift, acc);
            }
            if (active) store_tile<MB, FUSED>(p, tile, acc);
        }
    }
}

// -------------------------------------------------------------------------
// prepacked weights: MFMA-shaped tiles, dequantised by the matrix cores
// -------------------------------------------------------------------------
// A one-time repack (prepack_kernel) turns the canonical operand triple into a
// blob a wave can stream with fully contiguous 1 KB loads and dequantise almost
// without VALU work.  Group sizes 32, 64 and 128.  Per 16-row tile, K padded to 512:
//
//   [meta  : nsc x 64 lanes x gq x 4 B]       word e of super-chunk sc and lane l is
//            (scale bits << 16) | zero  of row (l % 16), group (4*sc + l/16)*gq + e;
//            gq = 128 / G groups lie in the 128 k a lane owns per super-chunk
//   [words : nsc x 4 x 64 lanes x 16 B]       super-chunk sc, load j, lane l, dword d
//
// with l = 16*kq + 4*rq + i.  Nibble nu of a weight dword holds
//   q[row 4*rq + kp][k = 512*sc + 128*kq + 32*j + 8*d + 4*c + i],
//   c = (nu % 4) / 2,  kp = 2*(nu % 2) + (nu >= 4).
// So ((v >> 4s) & 0x000F000F) | 0x43004300 is a bf16 pair (128+q) of two
// neighbouring ROWS at one k, which is the A operand of v_mfma_f32_4x4x4_16b_bf16
// (16 independent 4x4x4 products, one per lane quad): with B = diag(scale of the
// lane's row) and C = -(128+z)*scale it returns the exact fp32 products
// (q-z)*s for the lane's own row at four consecutive k.  v_cvt_pk_bf16_f32
// rounds them (the one RNE of the contract), and two such results are the B
// operand of v_mfma_f32_16x16x32_bf16 against the staged activations.
// Per 8 weights and lane: 7 VALU unpack ops, 4 conversions, 3 MFMA issues.
constexpr int PP_SC = 512;  // k per super-chunk: lane group kq owns one 128-k scale group

__host__ __device__ inline int pp_nsc(int K) { return (K + PP_SC - 1) / PP_SC; }
// groups per lane and super-chunk: a lane owns 128 consecutive k of one row
__host__ __device__ inline int pp_gq(int G) { return 128 / G; }
// 64 lanes x gq words per super-chunk
__host__ __device__ inline long pp_meta_u4(int K, int G) { return (long)pp_nsc(K) * 16 * pp_gq(G); }
__host__ __device__ inline long pp_tile_u4(int K, int G) { return pp_meta_u4(K, G) + (long)pp_nsc(K) * 4 * 64; }

__global__ __launch_bounds__(256) void prepack_kernel(const uint32_t *__restrict__ qweight,
                                                      const uint16_t *__restrict__ scales,
                                                      const uint32_t *__restrict__ qzeros,
                                                      u32x4_t *__restrict__ blob, int N, int K, int G) {
    const int kwords = K >> 3;
    const int groups = K / G;
    const int zwords = (groups + 7) >> 3;
    const int gq = pp_gq(G);
    const long meta_u4 = pp_meta_u4(K, G);
    const long tile_u4 = pp_tile_u4(K, G);
    const long ntiles = (N + 15) / 16;
    const long total = ntiles * tile_u4;
    for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const long tile = idx / tile_u4;
        const long rem = idx - tile * tile_u4;
        u32x4_t out = {0u, 0u, 0u, 0u};
        if (rem < meta_u4) {
            // meta word w of the tile: super-chunk w / (64 gq), lane (w / gq) % 64, sub-group w % gq
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const long w = 4 * rem + e;
                const int sc = (int)(w / (64 * gq));
                const int lane = (int)(w / gq) & 63;
                const long row = tile * 16 + (lane & 15);
                const int g = (4 * sc + (lane >> 4)) * gq + (int)(w % gq);
                if (row < N && g < groups) {
                    const uint32_t sb = scales[row * groups + g];
                    const uint32_t z = (qzeros[row * zwords + (g >> 3)] >> (4 * (g & 7))) & 0xFu;
                    out[e] = (sb << 16) | z;
                }
            }
        } else {
            const long r2 = rem - meta_u4;
            const int sc = (int)(r2 >> 8);
            const int j = (int)((r2 >> 6) & 3);
            const int lane = (int)(r2 & 63);
            const int kq = lane >> 4, rq = (lane >> 2) & 3, i = lane & 3;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                uint32_t word = 0;
#pragma unroll
                for (int nu = 0; nu < 8; ++nu) {
                    const int c = (nu & 3) >> 1;
                    const int kp = 2 * (nu & 1) + (nu >> 2);
                    const long row = tile * 16 + 4 * rq + kp;
                    const int k = sc * PP_SC + kq * 128 + j * 32 + d * 8 + 4 * c + i;
                    if (row < N && k < K) {
                        const uint32_t src = qweight[row * kwords + (k >> 3)];
                        word |= ((src >> (4 * (k & 7))) & 0xFu) << (4 * nu);
                    }
                }
                out[d] = word;
            }
        }
        blob[idx] = out;
    }
}

typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

constexpr int PP_ZERO_ROW = 2;  // DevProblem::prepacked bit

// natural-order staging of x[:, k0:k1) (k beyond K reads as zero), plus a row of zeros at
// row M if the record asks for one
__device__ __forceinline__ void stage_x_natural(const DevProblem &p, int k0, int k1, uint16_t *xs,
                                                int xstride, int nthreads) {
    const int words_per_row = (k1 - k0) >> 3;
    const int total = (p.M + ((p.prepacked & PP_ZERO_ROW) ? 1 : 0)) * words_per_row;
    for (int idx = threadIdx.x; idx < total; idx += nthreads) {
        const int m = idx / words_per_row;
        const int j = idx - m * words_per_row;
        const int k = k0 + (j << 3);
        u32x4_t d = {0u, 0u, 0u, 0u};
        if (k < p.K && m < p.M) d = *as_global(reinterpret_cast<const u32x4_t *>(p.x + (long)m * p.K + k));
        *reinterpret_cast<u32x4_t *>(xs + m * xstride + (j << 3)) = d;
    }
}

struct PPGroup {
    bf16x4_t bdiag;  // B operand of the 4x4x4 product: scale at k' = lane % 4, zero elsewhere
    f32x4_t cq;      // C operand: -(128 + z) * scale in all four rows
};

__device__ __forceinline__ PPGroup pp_group(uint32_t meta_word, int j4) {
    const uint32_t sb = meta_word >> 16;
    const float s = __builtin_bit_cast(float, meta_word & 0xFFFF0000u);
    const float c = -(128.0f + (float)(meta_word & 15u)) * s;
    u32x2_t bd;
    bd[0] = (j4 == 0) ? sb : (j4 == 1 ? (sb << 16) : 0u);
    bd[1] = (j4 == 2) ? sb : (j4 == 3 ? (sb << 16) : 0u);
    PPGroup g;
    g.bdiag = __builtin_bit_cast(bf16x4_t, bd);
    g.cq = f32x4_t{c, c, c, c};
    return g;
}

// Per-wave stream state of the prepacked path: four 16-byte loads per lane in flight (one
// super-chunk) and the meta word that goes with them.
template <int RS, int GQ>
struct PPRing {
    u32x4_t slot[4][RS];
    uint32_t meta[RS][GQ];  // one word per group the lane's 128 k span (GQ = 128 / G)
};

// The prepacked blob is read through a buffer resource: uniform base and size in SGPRs, one
// VGPR (16 * lane) as the per-lane offset for every load, the tile / super-chunk position as
// a scalar offset.  Reads past the blob return zero instead of faulting.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr int BUFFER_NT = 2;  // cache-policy bit: non-temporal (streamed once)
constexpr uint32_t PP_OUT_OF_RANGE = 0x7FFF0000u;  // a per-lane offset no blob reaches (blobs stay below this)

__device__ __forceinline__ rsrc_t pp_blob_rsrc(const DevProblem &p) {
    const uint32_t bytes = (uint32_t)((p.N + 15) / 16) * (uint32_t)(pp_tile_u4(p.K, p.G) * 16);
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t *>(p.qweight), 0, (int)bytes, 0x00020000);
}

template <bool FUSED>
struct PPTilePtr {
    uint32_t words[FUSED ? 2 : 1];  // byte offset of the tile's super-chunk sc0 (16 bytes per lane follow)
    uint32_t meta[FUSED ? 2 : 1];   // byte offset of super-chunk sc0's meta words (4 * GQ bytes per lane follow)
};

// where tile `tile_local` of the blob starts, at super-chunk sc0
template <bool FUSED>
__device__ __forceinline__ PPTilePtr<FUSED> pp_tile_ptr(const DevProblem &p, int tile_local, int sc0) {
    constexpr int RS = FUSED ? 2 : 1;
    const uint32_t meta_bytes = (uint32_t)pp_meta_u4(p.K, p.G) * 16u;
    const uint32_t tile_bytes = (uint32_t)pp_tile_u4(p.K, p.G) * 16u;
    const int out_tiles = (FUSED ? p.N / 2 : p.N + 15) / 16;
    PPTilePtr<FUSED> t;
#pragma unroll
    for (int r = 0; r < RS; ++r) {
        const uint32_t base = (uint32_t)(tile_local + r * out_tiles) * tile_bytes;
        t.words[r] = base + meta_bytes + (uint32_t)sc0 * 4096u;
        t.meta[r] = base + (uint32_t)sc0 * 256u * (uint32_t)pp_gq(p.G);
    }
    return t;
}

// the five loads of one super-chunk: meta words, then four 16-byte slots; slot d alone when
// called with that d, so that a refill can follow each slot's last use
template <bool FUSED, int GQ>
__device__ __forceinline__ void pp_load_slot(rsrc_t rsrc, uint32_t voff, uint32_t mvoff,
                                             const uint32_t (&words)[FUSED ? 2 : 1],
                                             const uint32_t (&meta)[FUSED ? 2 : 1], int d,
                                             PPRing<FUSED ? 2 : 1, GQ> &ring) {
    constexpr int RS = FUSED ? 2 : 1;
#pragma unroll
    for (int r = 0; r < RS; ++r) {
        if (d == 0) {
            if constexpr (GQ == 1) {
                ring.meta[r][0] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, mvoff, meta[r], 0);
            } else if constexpr (GQ == 2) {
                const u32x2_t m = __builtin_amdgcn_raw_buffer_load_b64(rsrc, mvoff, meta[r], 0);
                ring.meta[r][0] = m[0];
                ring.meta[r][1] = m[1];
            } else {
                const u32x4_t m = __builtin_amdgcn_raw_buffer_load_b128(rsrc, mvoff, meta[r], 0);
#pragma unroll
                for (int e = 0; e < 4; ++e) ring.meta[r][e] = m[e];
            }
        }
        ring.slot[d][r] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff + d * 1024, words[r], BUFFER_NT);
    }
}

// per-lane byte offset of the meta words: 4 * GQ bytes per lane
template <int GQ>
__device__ __forceinline__ uint32_t pp_meta_voff(uint32_t voff) { return (voff >> 2) * GQ; }

// issue the loads of a tile's first super-chunk
template <bool FUSED, int GQ>
__device__ __forceinline__ void pp_prime(rsrc_t rsrc, const PPTilePtr<FUSED> &t, PPRing<FUSED ? 2 : 1, GQ> &ring) {
    const uint32_t voff = (threadIdx.x & (WAVE - 1)) * 16u;
#pragma unroll
    for (int d = 0; d < 4; ++d) pp_load_slot<FUSED, GQ>(rsrc, voff, pp_meta_voff<GQ>(voff), t.words, t.meta, d, ring);
}

// acc += x[:, 512*sc0 : 512*sc1) . W[tile rows, same k]^T from a prepacked blob; xs holds x
// for exactly that k range.  On entry the ring holds super-chunk sc0 of this tile (pp_prime);
// if next_tile >= 0 the ring holds that tile's super-chunk sc0 on return, so that the wave
// never runs dry between tiles.
template <int MB, bool FUSED, int GQ>
__device__ __forceinline__ void stream_rows_pp(const DevProblem &p, rsrc_t rsrc, const PPTilePtr<FUSED> &cur,
                                               int next_tile, const uint16_t *xs, int xstride,
                                               int sc0, int sc1, PPRing<FUSED ? 2 : 1, GQ> &ring,
                                               f32x4_t (&acc)[FUSED ? 2 : 1][MB]) {
    constexpr int RS = FUSED ? 2 : 1;
    const int lane = threadIdx.x & (WAVE - 1);
    const int lc = lane & 15;
    const int kq = lane >> 4;
    const int j4 = lane & 3;

    // both must sit in registers for (v & mask) | bias to select v_and_or_b32
    uint32_t mask = PAIR_MASK, bias = PAIR_BIAS;
    asm volatile("" : "+s"(mask));
    asm volatile("" : "+v"(bias));

    static_assert(STREAM_DEPTH == 4, "the ring holds exactly one super-chunk (four loads per lane)");
    PPGroup grp[RS];
    // A-operand rows beyond M are padding: they read the staged row of zeros if there is one
    // (quiet multipliers; the chip runs this kernel at its power limit, so that shows up as
    // clock), else a copy of the last row
    const int pad_row = (p.prepacked & PP_ZERO_ROW) ? p.M : p.M - 1;

    // One super-chunk: 4 loads x 4 words per lane = 16 dequant + dot steps, no branch inside.
    // Each ring slot is reloaded from offset rw (and the meta word from rm, with slot 0) as
    // soon as its last word is consumed.  The scheduling barriers pin the loads there: left alone,
    // the scheduler gathers them at the end of the body and the wave then waits out a whole
    // memory latency per super-chunk.
    auto super_chunk = [&](int sc, uint32_t rv, uint32_t rmv, const uint32_t (&rw)[RS],
                           const uint32_t (&rm)[RS]) {
        // this super-chunk's meta words: the ring's copy is overwritten by the refill that rides
        // with slot 0, the later groups of the lane's span are needed after that
        uint32_t mcur[RS][GQ];
#pragma unroll
        for (int r = 0; r < RS; ++r)
#pragma unroll
            for (int e = 0; e < GQ; ++e) mcur[r][e] = ring.meta[r][e];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            if (d % (4 / GQ) == 0) {  // load d covers 32 k: a new group every 4 / GQ loads
#pragma unroll
                for (int r = 0; r < RS; ++r) grp[r] = pp_group(mcur[r][d * GQ / 4], j4);
            }
            const int kloc = (sc - sc0) * PP_SC + kq * 128 + d * 32;
#pragma unroll
            for (int dd = 0; dd < 4; ++dd) {
                bf16x8_t xa[MB];
#pragma unroll
                for (int b = 0; b < MB; ++b) {
                    const int m = min(16 * b + lc, pad_row);
                    const u32x4_t raw = *reinterpret_cast<const u32x4_t *>(xs + m * xstride + kloc + 8 * dd);
                    xa[b] = __builtin_bit_cast(bf16x8_t, raw);
                }
#pragma unroll
                for (int r = 0; r < RS; ++r) {
                    const uint32_t v = ring.slot[d][r][dd];
                    u32x2_t a0, a1;
                    a0[0] = (v & mask) | bias;
                    a0[1] = ((v >> 4) & mask) | bias;
                    a1[0] = ((v >> 8) & mask) | bias;
                    a1[1] = ((v >> 12) & mask) | bias;
                    const f32x4_t d0 = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(
                        __builtin_bit_cast(bf16x4_t, a0), grp[r].bdiag, grp[r].cq, 0, 0, 0);
                    const f32x4_t d1 = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(
                        __builtin_bit_cast(bf16x4_t, a1), grp[r].bdiag, grp[r].cq, 0, 0, 0);
                    const u32x4_t wv = {pack_bf16_rne(d0[0], d0[1]), pack_bf16_rne(d0[2], d0[3]),
                                        pack_bf16_rne(d1[0], d1[1]), pack_bf16_rne(d1[2], d1[3])};
                    const bf16x8_t bop = __builtin_bit_cast(bf16x8_t, wv);
#pragma unroll
                    for (int b = 0; b < MB; ++b)
                        acc[r][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[b], bop, acc[r][b], 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            pp_load_slot<FUSED, GQ>(rsrc, rv, rmv, rw, rm, d, ring);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // After the last super-chunk the ring is refilled from the next tile's first one.  With no
    // next tile the refill is issued all the same, with a per-lane offset beyond the end of
    // the blob: the buffer range check answers such a load with zeros without touching
    // memory, and the loop body exists once and has no branch.
    const bool has_next = next_tile >= 0;
    const PPTilePtr<FUSED> nxt = pp_tile_ptr<FUSED>(p, has_next ? next_tile : 0, sc0);
    const uint32_t voff = lane * 16u;
    for (int sc = sc0; sc < sc1; ++sc) {
        const bool last = sc + 1 == sc1;
        uint32_t rw[RS], rm[RS];
#pragma unroll
        for (int r = 0; r < RS; ++r) {
            const uint32_t w_same = cur.words[r] + (uint32_t)(sc + 1 - sc0) * 4096u;
            const uint32_t m_same = cur.meta[r] + (uint32_t)(sc + 1 - sc0) * 256u * GQ;
            rw[r] = last ? (has_next ? nxt.words[r] : cur.words[r]) : w_same;
            rm[r] = last ? (has_next ? nxt.meta[r] : cur.meta[r]) : m_same;
        }
        const bool dry = last && !has_next;
        super_chunk(sc, dry ? PP_OUT_OF_RANGE : voff, dry ? PP_OUT_OF_RANGE : pp_meta_voff<GQ>(voff), rw, rm);
    }
}

template <int MB, bool FUSED, int WPB, bool PASSES, int GQ>
__device__ __forceinline__ void stream_segment_pp(const DevProblem &p, int t0, int t1, uint8_t *smem) {
    constexpr int RS = FUSED ? 2 : 1;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: tile offsets stay scalar
    uint16_t *xs = reinterpret_cast<uint16_t *>(smem);
    const int xstride = p.kc + XPAD;
    const int nsc = pp_nsc(p.K);
    const int sc_pass = p.kc / PP_SC;
    if (!PASSES || sc_pass >= nsc) {
        // Tiles of the segment are handed out through a counter in LDS: waves on one SIMD do
        // not progress at equal rates (older waves win the issue arbitration), and with a
        // fixed deal the workgroup would wait at the next barrier for its slowest wave.
        // A wave draws its next tile before it starts the current one, so that the last
        // super-chunk of a tile already pulls in the first of the next.
        __shared__ int next_tile;
        int tile = t0 + wave;
        PPRing<RS, GQ> ring;
        const rsrc_t rsrc = pp_blob_rsrc(p);
        PPTilePtr<FUSED> cur = pp_tile_ptr<FUSED>(p, tile < t1 ? tile : t0, 0);
        if (tile < t1) pp_prime<FUSED, GQ>(rsrc, cur, ring);  // weights are on their way while x is staged
        __syncthreads();
        if (threadIdx.x == 0) next_tile = t0 + WPB;
        stage_x_natural(p, 0, nsc * PP_SC, xs, xstride, WPB * WAVE);
        __syncthreads();
        while (tile < t1) {
            int nt = 0;
            if ((threadIdx.x & (WAVE - 1)) == 0) nt = atomicAdd(&next_tile, 1);
            nt = __builtin_amdgcn_readfirstlane(nt);
            f32x4_t acc[RS][MB];
#pragma unroll
            for (int r = 0; r < RS; ++r)
#pragma unroll
                for (int b = 0; b < MB; ++b) acc[r][b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            stream_rows_pp<MB, FUSED, GQ>(p, rsrc, cur, nt < t1 ? nt : -1, xs, xstride, 0, nsc, ring, acc);
            store_tile<MB, FUSED>(p, tile, acc);
            tile = nt;
            if (tile < t1) cur = pp_tile_ptr<FUSED>(p, tile, 0);
        }
    } else if constexpr (PASSES) {
        // activations do not fit: K is walked in staged passes, and every wave carries T tiles
        // through a pass so that one staging serves T * WPB tiles
        constexpr int T = FUSED ? 1 : (MB == 2 ? 2 : 4);
        const rsrc_t rsrc = pp_blob_rsrc(p);
        for (int round = t0; round < t1; round += WPB * T) {
            f32x4_t acc[T][RS][MB];
#pragma unroll
            for (int i = 0; i < T; ++i)
#pragma unroll
                for (int r = 0; r < RS; ++r)
#pragma unroll
                    for (int b = 0; b < MB; ++b) acc[i][r][b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            for (int sc0 = 0; sc0 < nsc; sc0 += sc_pass) {
                const int sc1 = min(nsc, sc0 + sc_pass);
                __syncthreads();
                stage_x_natural(p, sc0 * PP_SC, sc1 * PP_SC, xs, xstride, WPB * WAVE);
                __syncthreads();
#pragma unroll
                for (int i = 0; i < T; ++i) {
                    const int tile = round + i * WPB + wave;  // neighbouring waves, neighbouring tiles
                    if (tile < t1) {
                        PPRing<RS, GQ> ring;
                        const PPTilePtr<FUSED> cur = pp_tile_ptr<FUSED>(p, tile, sc0);
                        pp_prime<FUSED, GQ>(rsrc, cur, ring);
                        stream_rows_pp<MB, FUSED, GQ>(p, rsrc, cur, -1, xs, xstride, sc0, sc1, ring, acc[i]);
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < T; ++i) {
                const int tile = round + i * WPB + wave;
                if (tile < t1) store_tile<MB, FUSED>(p, tile, acc[i]);
            }
        }
    }
}

// Small plans (fewer tiles than the device has workgroup slots): the waves of a workgroup
// share one tile, each taking a contiguous quarter of its super-chunks, and the partial
// tiles meet in LDS.  A tile is then one or two memory round trips instead of a serial walk
// over K by a single wave; this is the latency mode for launches of a few matrices
// (q|k|v of one layer, one o_proj, ...).  LDS: staged activations, then WPB x RS partial tiles.
template <bool FUSED, int WPB, int GQ>
__device__ __forceinline__ void split_segment_pp(const DevProblem &p, int t0, int t1, uint8_t *smem) {
    constexpr int RS = FUSED ? 2 : 1;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & (WAVE - 1);
    uint16_t *xs = reinterpret_cast<uint16_t *>(smem);
    const int xstride = p.kc + XPAD;
    const int xrows = p.M + ((p.prepacked & PP_ZERO_ROW) ? 1 : 0);
    f32x4_t *red = reinterpret_cast<f32x4_t *>(smem + (size_t)xrows * xstride * 2);
    const int nsc = pp_nsc(p.K);
    const int per = (nsc + WPB - 1) / WPB;
    const int sc0 = min(nsc, wave * per), sc1 = min(nsc, sc0 + per);
    const bool work = sc0 < sc1;  // wave-uniform
    const rsrc_t rsrc = pp_blob_rsrc(p);
    PPRing<RS, GQ> ring;
    PPTilePtr<FUSED> cur = pp_tile_ptr<FUSED>(p, t0, sc0);
    if (work) pp_prime<FUSED, GQ>(rsrc, cur, ring);  // weights are on their way while x is staged
    __syncthreads();
    stage_x_natural(p, 0, nsc * PP_SC, xs, xstride, WPB * WAVE);
    __syncthreads();
    for (int tile = t0; tile < t1; ++tile) {
        const int next = tile + 1 < t1 ? tile + 1 : -1;
        f32x4_t acc[RS][1];
#pragma unroll
        for (int r = 0; r < RS; ++r) acc[r][0] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        if (work) {
            stream_rows_pp<1, FUSED, GQ>(p, rsrc, cur, next, xs + sc0 * PP_SC, xstride, sc0, sc1, ring, acc);
            if (next >= 0) cur = pp_tile_ptr<FUSED>(p, next, sc0);
        }
        if (wave != 0) {
#pragma unroll
            for (int r = 0; r < RS; ++r) red[((wave - 1) * RS + r) * WAVE + lane] = acc[r][0];
        }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int w = 1; w < WPB; ++w)
#pragma unroll
                for (int r = 0; r < RS; ++r) acc[r][0] += red[((w - 1) * RS + r) * WAVE + lane];
            store_tile<1, FUSED>(p, tile, acc);
        }
        if (next >= 0) __syncthreads();  // the partial tiles are read before they are rewritten
    }
}

// the latency kernels take any of the three group sizes in one build (they are not register-critical)
template <bool FUSED, int WPB>
__device__ __forceinline__ void split_by_group(const DevProblem &p, int t0, int t1, uint8_t *smem) {
    if (FUSED && p.fused) {
        if (p.G == 128) split_segment_pp<FUSED, WPB, 1>(p, t0, t1, smem);
        else if (p.G == 64) split_segment_pp<FUSED, WPB, 2>(p, t0, t1, smem);
        else split_segment_pp<FUSED, WPB, 4>(p, t0, t1, smem);
    } else {
        if (p.G == 128) split_segment_pp<false, WPB, 1>(p, t0, t1, smem);
        else if (p.G == 64) split_segment_pp<false, WPB, 2>(p, t0, t1, smem);
        else split_segment_pp<false, WPB, 4>(p, t0, t1, smem);
    }
}

template <bool FUSED, int WPB>
__global__ __launch_bounds__(WPB *WAVE) void gemv_split_kernel(const DevProblem *__restrict__ plan,
                                                               const int2 *__restrict__ block_tab,
                                                               int n_problems) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int2 entry = block_tab[blockIdx.x];
    int t = entry.x;
    const int t_end = block_tab[blockIdx.x + 1].x;
    if (t >= t_end) return;  // block-uniform
    for (int pi = entry.y; t < t_end && pi < n_problems; ++pi) {
        const DevProblem p = plan[pi];
        const int out_cols = p.fused ? p.N / 2 : p.N;
        const int seg_end = min(t_end, p.tile_begin + (out_cols + 15) / 16);
        const int a = t - p.tile_begin, b = seg_end - p.tile_begin;
        split_by_group<FUSED, WPB>(p, a, b, smem);
        t = seg_end;
    }
}

// The same latency mode without a plan in device memory: up to DIRECT_MAX records travel
// as kernel arguments (no dependent loads before the first weight request), one workgroup per
// tile.  This is the single-call path of a prepacked weight (and of q|k|v, gate|up groups).
constexpr int DIRECT_MAX = 4;
struct DirectArgs {
    int32_t n;
    int32_t pad;
    DevProblem recs[DIRECT_MAX];
};

template <bool FUSED, int WPB>
__global__ __launch_bounds__(WPB *WAVE) void gemv_split_direct_kernel(DirectArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int t = blockIdx.x;
    DevProblem p = a.recs[0];
#pragma unroll
    for (int k = 1; k < DIRECT_MAX; ++k)
        if (k < a.n && a.recs[k].tile_begin <= t) p = a.recs[k];  // scalar selects, no indexing
    const int local = t - p.tile_begin;
    split_by_group<FUSED, WPB>(p, local, local + 1, smem);
}

// CANON / PP / FUSED say which kinds of record the plan holds, so that a plan of
// plain prepacked GEMVs runs the variant with the smallest register footprint.
// WPB (waves per workgroup) grows with the LDS the staged activations need, so that
// about 16 waves stay resident per CU; MB = 2 carries up to 32 activation rows per
// record with two A operands per weight tile (weights streamed once); PASSES adds the
// path for prepacked records whose activations do not fit LDS whole (it carries several
// accumulator tiles, so plans that do not need it run a build without it).
template <int WPB, int MB, bool CANON, bool PP, bool FUSED, bool PASSES, int GQ>
__global__ __launch_bounds__(WPB *WAVE) void gemv_stream_kernel(const DevProblem *__restrict__ plan,
                                                                const int2 *__restrict__ block_tab,
                                                                int n_problems) {
    extern __shared__ __align__(16) uint8_t smem[];
    // block_tab[b] = {first tile of workgroup b, record that tile belongs to}
    const int2 entry = block_tab[blockIdx.x];
    int t = entry.x;
    const int t_end = block_tab[blockIdx.x + 1].x;
    if (t >= t_end) return;  // block-uniform
    const int lo = entry.y;
    for (int pi = lo; t < t_end && pi < n_problems; ++pi) {
        const DevProblem p = plan[pi];
        const int out_cols = p.fused ? p.N / 2 : p.N;
        const int seg_end = min(t_end, p.tile_begin + (out_cols + 15) / 16);
        const int a = t - p.tile_begin, b = seg_end - p.tile_begin;
        if (PP && (!CANON || p.prepacked)) {
            if (FUSED && p.fused) stream_segment_pp<MB, FUSED, WPB, PASSES, GQ>(p, a, b, smem);
            else stream_segment_pp<MB, false, WPB, PASSES, GQ>(p, a, b, smem);
        } else if (CANON) {
            if (FUSED && p.fused) stream_segment<MB, FUSED, WPB>(p, a, b, smem);
            else stream_segment<MB, false, WPB>(p, a, b, smem);
        }
        t = seg_end;
    }
}

// -------------------------------------------------------------------------
// host side
// -------------------------------------------------------------------------
constexpr int TILE_WPB = 8;
constexpr int MAX_TILE_M = 16;                  // activation rows one single-launch slab / canonical record takes
constexpr int MAX_PP_M = 32;                    // activation rows a prepacked record of a grouped plan takes
constexpr size_t LDS_X_BUDGET = 40 * 1024;      // split kernel: staged activations per workgroup
constexpr int STAGE_STEP = KCHUNK * TILE_WPB;   // split kernel: shorter staged extents are multiples of this
// stream kernel: workgroup shapes by the LDS the staged activations need
struct StreamShape { int wpb; int per_cu; size_t lds; };
// {waves per workgroup, workgroups per CU to launch when the runtime cannot say how many are
// resident, LDS the shape may use}
constexpr StreamShape STREAM_SHAPES[3] = {{4, 15, 32 * 1024}, {8, 2, 72 * 1024}, {16, 1, 144 * 1024}};
constexpr size_t LDS_PER_CU = 160 * 1024;

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_problem(const void *x, const void *qw, const void *sc, const void *qz, const void *y,
                  long M, long N, long K, long G) {
    if (!x || !qw || !sc || !qz || !y) return VRL_INT4_ENULL;
    if (M < 1 || N < 1 || K < 8 || G < 8) return VRL_INT4_ESHAPE;
    if (K % 8 != 0 || G % 8 != 0 || K % G != 0) return VRL_INT4_ESHAPE;
    if (N * K >= (1L << 40) || M * K >= (1L << 31) || M * N >= (1L << 31)) return VRL_INT4_ESHAPE;
    if (!aligned16(x) || !aligned16(qw) || !aligned16(sc) || !aligned16(qz) || !aligned16(y))
        return VRL_INT4_EALIGN;
    return VRL_INT4_OK;
}

bool pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

// shapes the MFMA kernels take; everything else goes to the generic kernel
bool tile_path_ok(const DevProblem &p) {
    return p.K % KCHUNK == 0 && p.G % 32 == 0 && pow2(p.G) && p.M <= (p.prepacked ? MAX_PP_M : MAX_TILE_M);
}

// split kernel: k extent of x staged per pass, all of K when M rows of it fit the budget,
// else the largest multiple of STAGE_STEP that does (M <= 16 always fits one step)
int staged_k(int M, int K) {
    if ((size_t)M * (K + XPAD) * 2 <= LDS_X_BUDGET) return K;
    long kc = (long)(LDS_X_BUDGET / ((size_t)M * 2)) - XPAD;
    kc -= kc % STAGE_STEP;
    if (kc < STAGE_STEP) kc = STAGE_STEP;
    return (int)(kc < K ? kc : K);
}

// stream kernel, canonical records: all of K if it fits `lds`, else passes that are multiples of KCHUNK
int stream_staged_k(int M, int K, size_t lds) {
    if ((size_t)M * (K + XPAD) * 2 <= lds) return K;
    long kc = (long)(lds / ((size_t)M * 2)) - XPAD;
    kc -= kc % KCHUNK;
    if (kc < KCHUNK) kc = KCHUNK;
    return (int)(kc < K ? kc : K);
}

// prepacked blobs exist for group sizes 32, 64 and 128
// the stream kernel addresses a blob with 32-bit byte offsets, so a blob stays below 2 GiB
bool prepack_ok(long N, long K, long G) {
    if ((G != 128 && G != 64 && G != 32) || K % 128 != 0 || N < 1 || K < 128 || N * K >= (1L << 40)) return false;
    return ((N + 15) / 16) * pp_tile_u4((int)K, (int)G) * 16 < (long)PP_OUT_OF_RANGE;
}

// stream kernel, prepacked records: all of the padded K if it fits, else whole super-chunks per pass
int pp_staged_k(int M, int K, size_t lds) {
    const int kpad = pp_nsc(K) * PP_SC;
    if ((size_t)M * (kpad + XPAD) * 2 <= lds) return kpad;
    long kc = (long)(lds / ((size_t)M * 2)) - XPAD;
    kc -= kc % PP_SC;
    if (kc < PP_SC) kc = PP_SC;
    return (int)kc;
}

template <int R, int MB>
size_t tile_smem_bytes(int M, int kc) {
    const size_t xbytes = (size_t)M * (kc + XPAD) * 2;
    const size_t rbytes = (size_t)TileCfg<R, MB, TILE_WPB>::RED_FLOATS * 4;
    return xbytes > rbytes ? xbytes : rbytes;
}

int device_cu_count() {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
            cus = v;
    }
    return cus;
}

template <int R, int MB>
int launch_tile(const DevProblem &p, hipStream_t stream) {
    const int out_cols = p.fused ? p.N / 2 : p.N;
    const int cols_per_tile = p.fused ? 16 * (R / 2) : 16 * R;
    const int tiles = (out_cols + cols_per_tile - 1) / cols_per_tile;
    const size_t smem = tile_smem_bytes<R, MB>(p.M, p.kc);
    hipLaunchKernelGGL((gemv_tile_kernel<R, MB, TILE_WPB>), dim3(tiles), dim3(TILE_WPB * WAVE), smem,
                       stream, p);
    return (int)hipGetLastError();
}

int launch_problem(DevProblem p, hipStream_t stream) {
    const int out_cols = p.fused ? p.N / 2 : p.N;
    if (!tile_path_ok(p)) {
        // the generic kernel walks activation rows itself, any M
        const int waves = 4;
        hipLaunchKernelGGL(gemv_generic_kernel, dim3((out_cols + waves - 1) / waves),
                           dim3(waves * WAVE), 0, stream, p);
        return (int)hipGetLastError();
    }
    p.kc = staged_k(p.M, p.K);
    // widest tile that still gives every CU two workgroups; narrow tiles otherwise
    const int cus = device_cu_count();
    const int cols_r4 = p.fused ? 32 : 64;
    if ((out_cols + cols_r4 - 1) / cols_r4 >= 2 * cus) return launch_tile<4, 1>(p, stream);
    if (p.fused || (out_cols + 31) / 32 >= 2 * cus) return launch_tile<2, 1>(p, stream);
    return launch_tile<1, 1>(p, stream);
}

int run_rows(const void *x, const void *qw, const void *sc, const void *qz, void *y, int M, int N,
             int K, int G, int fused, void *hip_stream) {
    int rc = check_problem(x, qw, sc, qz, y, M, N, K, G);
    if (rc != VRL_INT4_OK) return rc;
    if (fused && (N % 2 != 0)) return VRL_INT4_ESHAPE;
    const int out_cols = fused ? N / 2 : N;
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
    // activation rows go in slabs of MAX_TILE_M (weights are re-read per slab)
    for (int m0 = 0; m0 < M; m0 += MAX_TILE_M) {
        DevProblem p;
        memset(&p, 0, sizeof p);
        p.x = static_cast<const uint16_t *>(x) + (long)m0 * K;
        p.qweight = static_cast<const uint32_t *>(qw);
        p.scales = static_cast<const uint16_t *>(sc);
        p.qzeros = static_cast<const uint32_t *>(qz);
        p.y = static_cast<uint16_t *>(y) + (long)m0 * out_cols;
        p.M = (M - m0 < MAX_TILE_M) ? (M - m0) : MAX_TILE_M;
        p.N = N;
        p.K = K;
        p.G = G;
        p.fused = fused;
        rc = launch_problem(p, stream);
        if (rc != 0) return rc;
    }
    return VRL_INT4_OK;
}

// Plan blob: [PlanHeader][DevProblem x n_records][int2 {first tile, its record} x (MAX_PLAN_GRID + 1)]
struct PlanHeader {
    uint32_t magic;
    int32_t n_records;
    int32_t total_tiles;
    int32_t grid;
};
static_assert(sizeof(PlanHeader) == 16, "plan header is 16 bytes");
constexpr uint32_t PLAN_MAGIC = 0x34544956u;  // "VIT4"
constexpr int MAX_PLAN_GRID = 4096;
constexpr int VARIANT_CANON = 1, VARIANT_PP = 2, VARIANT_FUSED = 4, VARIANT_MB2 = 8, VARIANT_PASSES = 16,
              VARIANT_SPLIT = 32, VARIANT_G64 = 64, VARIANT_G32 = 128;

// With recs == nullptr nothing is launched: info->grid receives the number of workgroups of
// this build that one CU holds at info->lds_bytes (the plan builder sizes the grid with it).
template <int WPB, int MB, bool CANON, bool PP, bool FUSED, bool PASSES, int GQ = 1>
int launch_stream(vrl_int4_plan_info *info, const DevProblem *recs, const int2 *block_begin,
                  hipStream_t stream) {
    auto kernel = &gemv_stream_kernel<WPB, MB, CANON, PP, FUSED, PASSES, GQ>;
    if (info->lds_bytes > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, info->lds_bytes);
        if (e != hipSuccess) return (int)e;
    }
    if (!recs) {
        int per_cu = 0;
        hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(
            &per_cu, reinterpret_cast<const void *>(kernel), WPB * WAVE, (size_t)info->lds_bytes);
        if (e != hipSuccess) return (int)e;
        info->grid = per_cu;
        return VRL_INT4_OK;
    }
    hipLaunchKernelGGL(kernel, dim3(info->grid), dim3(WPB * WAVE), (size_t)info->lds_bytes,
                       stream, recs, block_begin, info->n_problems);
    return (int)hipGetLastError();
}

// prepacked-only plans: fused or not, staged passes or not (only the widest workgroups ever
// need passes: narrower shapes are chosen because x fits), group size
template <int WPB, int MB, bool FUSED, int GQ>
int launch_stream_pp_g(vrl_int4_plan_info *info, const DevProblem *recs, const int2 *bb, hipStream_t stream,
                       bool passes) {
    if constexpr (WPB == 16) {
        if (passes) return launch_stream<WPB, MB, false, true, FUSED, true, GQ>(info, recs, bb, stream);
    }
    return launch_stream<WPB, MB, false, true, FUSED, false, GQ>(info, recs, bb, stream);
}

template <int WPB, int MB>
int launch_stream_pp(vrl_int4_plan_info *info, const DevProblem *recs, const int2 *bb, hipStream_t stream,
                     bool fused, bool passes, int gq) {
    if (fused) {
        if (gq == 1) return launch_stream_pp_g<WPB, MB, true, 1>(info, recs, bb, stream, passes);
        if (gq == 2) return launch_stream_pp_g<WPB, MB, true, 2>(info, recs, bb, stream, passes);
        return launch_stream_pp_g<WPB, MB, true, 4>(info, recs, bb, stream, passes);
    }
    if (gq == 1) return launch_stream_pp_g<WPB, MB, false, 1>(info, recs, bb, stream, passes);
    if (gq == 2) return launch_stream_pp_g<WPB, MB, false, 2>(info, recs, bb, stream, passes);
    return launch_stream_pp_g<WPB, MB, false, 4>(info, recs, bb, stream, passes);
}

// which record kinds a kernel build must handle, for a given workgroup shape
template <int WPB, int MB>
int launch_stream_variant(vrl_int4_plan_info *info, const DevProblem *recs, const int2 *bb,
                          hipStream_t stream) {
    const int v = info->variant & (VARIANT_CANON | VARIANT_PP | VARIANT_FUSED);
    const bool passes = (info->variant & VARIANT_PASSES) != 0;
    // prepacked-only plans hold one group size (the kernel build is specialised for it)
    const int gq = (info->variant & VARIANT_G32) ? 4 : ((info->variant & VARIANT_G64) ? 2 : 1);
    if (v == VARIANT_PP || v == (VARIANT_PP | VARIANT_FUSED)) {
        return launch_stream_pp<WPB, MB>(info, recs, bb, stream, (v & VARIANT_FUSED) != 0, passes, gq);
    }
    if (gq != 1) return VRL_INT4_EPLAN;
    if constexpr (MB == 1 && WPB != 8) {  // canonical records: narrow and widest workgroups only
        if (v & VARIANT_FUSED) return launch_stream<WPB, 1, true, true, true, WPB == 16>(info, recs, bb, stream);
        return launch_stream<WPB, 1, true, true, false, WPB == 16>(info, recs, bb, stream);
    }
    return VRL_INT4_EPLAN;
}


template <bool FUSED, int WPB>
int launch_split(vrl_int4_plan_info *info, const DevProblem *recs, const int2 *block_tab, hipStream_t stream) {
    auto kernel = &gemv_split_kernel<FUSED, WPB>;
    if (!recs) {
        int per_cu = 0;
        hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(
            &per_cu, reinterpret_cast<const void *>(kernel), WPB * WAVE, (size_t)info->lds_bytes);
        if (e != hipSuccess) return (int)e;
        info->grid = per_cu;
        return VRL_INT4_OK;
    }
    hipLaunchKernelGGL(kernel, dim3(info->grid), dim3(WPB * WAVE), (size_t)info->lds_bytes, stream, recs,
                       block_tab, info->n_problems);
    return (int)hipGetLastError();
}

template <int WPB>
int launch_split_variant(vrl_int4_plan_info *info, const DevProblem *recs, const int2 *block_tab,
                         hipStream_t stream) {
    return (info->variant & VARIANT_FUSED) ? launch_split<true, WPB>(info, recs, block_tab, stream)
                                           : launch_split<false, WPB>(info, recs, block_tab, stream);
}

template <bool FUSED, int WPB>
int launch_direct(const DirectArgs &args, int tiles, size_t lds, hipStream_t stream) {
    hipLaunchKernelGGL((gemv_split_direct_kernel<FUSED, WPB>), dim3(tiles), dim3(WPB * WAVE), lds, stream, args);
    return (int)hipGetLastError();
}

int dispatch_stream(vrl_int4_plan_info *info, const DevProblem *recs, const int2 *block_tab,
                    hipStream_t stream) {
    const bool mb2 = (info->variant & VARIANT_MB2) != 0;
    if (info->variant & VARIANT_SPLIT) {
        if (mb2 || (size_t)info->lds_bytes > 64 * 1024 || (info->variant & (VARIANT_CANON | VARIANT_PASSES)))
            return VRL_INT4_EPLAN;
        switch (info->block_threads) {
            case 4 * WAVE: return launch_split_variant<4>(info, recs, block_tab, stream);
            case 8 * WAVE: return launch_split_variant<8>(info, recs, block_tab, stream);
            case 16 * WAVE: return launch_split_variant<16>(info, recs, block_tab, stream);
            default: return VRL_INT4_EPLAN;
        }
    }
    switch (info->block_threads) {
        case 4 * WAVE: return mb2 ? VRL_INT4_EPLAN : launch_stream_variant<4, 1>(info, recs, block_tab, stream);
        case 8 * WAVE: return mb2 ? VRL_INT4_EPLAN : launch_stream_variant<8, 1>(info, recs, block_tab, stream);
        case 16 * WAVE:
            return mb2 ? launch_stream_variant<16, 2>(info, recs, block_tab, stream)
                       : launch_stream_variant<16, 1>(info, recs, block_tab, stream);
        default: return VRL_INT4_EPLAN;
    }
}

size_t plan_bytes_for(int n_records) {
    return sizeof(PlanHeader) + (size_t)n_records * sizeof(DevProblem) +
           (size_t)(MAX_PLAN_GRID + 1) * sizeof(int2);
}

}  // namespace

extern "C" {

int vrl_int4_abi_version(void) { return VRL_INT4_ABI_VERSION; }

const char *vrl_int4_error_string(int code) {
    switch (code) {
        case VRL_INT4_OK: return "ok";
        case VRL_INT4_ESHAPE: return "shape violates a precondition (M,N>=1; K%8==0; G%8==0; K%G==0)";
        case VRL_INT4_EALIGN: return "pointer is not 16-byte aligned";
        case VRL_INT4_ENULL: return "required pointer is NULL";
        case VRL_INT4_EPLAN: return "malformed or undersized grouped plan";
        default: break;
    }
    if (code > 0 && code < 1000) return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown error code";
}

int vrl_int4_gemv_bf16(const void *x, const void *qweight, const void *scales, const void *qzeros,
                       void *y, int M, int N, int K, int G, void *hip_stream) {
    return run_rows(x, qweight, scales, qzeros, y, M, N, K, G, 0, hip_stream);
}

int vrl_int4_gate_up_silu_bf16(const void *x, const void *qweight_gu, const void *scales_gu,
                               const void *qzeros_gu, void *y, int M, int I, int K, int G,
                               void *hip_stream) {
    if (I < 1 || I > (1 << 29)) return VRL_INT4_ESHAPE;
    return run_rows(x, qweight_gu, scales_gu, qzeros_gu, y, M, 2 * I, K, G, 1, hip_stream);
}

int vrl_int4_dequant_bf16(const void *qweight, const void *scales, const void *qzeros, void *w,
                          int N, int K, int G, void *hip_stream) {
    int rc = check_problem(qweight, qweight, scales, qzeros, w, 1, N, K, G);
    if (rc != VRL_INT4_OK) return rc;
    const long total = (long)N * (K >> 3);
    long blocks = (total + 255) / 256;
    const long cap = (long)device_cu_count() * 32;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(dequant_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       reinterpret_cast<hipStream_t>(hip_stream),
                       static_cast<const uint32_t *>(qweight), static_cast<const uint16_t *>(scales),
                       static_cast<const uint32_t *>(qzeros), static_cast<uint16_t *>(w), N, K, G);
    return (int)hipGetLastError();
}

size_t vrl_int4_prepacked_bytes(int N, int K, int G) {
    if (!prepack_ok(N, K, G)) return 0;
    return (size_t)((N + 15) / 16) * (size_t)pp_tile_u4(K, G) * 16;
}

int vrl_int4_prepack(const void *qweight, const void *scales, const void *qzeros, void *packed,
                     int N, int K, int G, void *hip_stream) {
    int rc = check_problem(qweight, qweight, scales, qzeros, packed, 1, N, K, G);
    if (rc != VRL_INT4_OK) return rc;
    if (!prepack_ok(N, K, G)) return VRL_INT4_ESHAPE;
    const long total = (long)((N + 15) / 16) * pp_tile_u4(K, G);
    long blocks = (total + 255) / 256;
    const long cap = (long)device_cu_count() * 32;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(prepack_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       reinterpret_cast<hipStream_t>(hip_stream),
                       static_cast<const uint32_t *>(qweight), static_cast<const uint16_t *>(scales),
                       static_cast<const uint32_t *>(qzeros), static_cast<u32x4_t *>(packed), N, K, G);
    return (int)hipGetLastError();
}

int vrl_int4_gemv_prepacked_bf16(const vrl_int4_problem *problems, int n_problems, void *hip_stream) {
    if (!problems) return VRL_INT4_ENULL;
    if (n_problems < 1 || n_problems > DIRECT_MAX) return VRL_INT4_ESHAPE;
    DirectArgs args;
    memset(&args, 0, sizeof args);
    args.n = n_problems;
    long tiles = 0;
    bool fused_any = false;
    int max_nsc = 1;
    size_t x_bytes = 0;
    for (int i = 0; i < n_problems; ++i) {
        const vrl_int4_problem &q = problems[i];
        if (!q.prepacked) return VRL_INT4_ESHAPE;
        int rc = check_problem(q.x, q.qweight, q.qweight, q.qweight, q.y, q.M, q.N, q.K, q.G);
        if (rc != VRL_INT4_OK) return rc;
        if (q.M > MAX_TILE_M || !prepack_ok(q.N, q.K, q.G)) return VRL_INT4_ESHAPE;
        if (q.fused_gate_up && (q.N % 2 != 0 || (q.N / 2) % 16 != 0)) return VRL_INT4_ESHAPE;
        DevProblem &p = args.recs[i];
        p.x = static_cast<const uint16_t *>(q.x);
        p.qweight = static_cast<const uint32_t *>(q.qweight);
        p.y = static_cast<uint16_t *>(q.y);
        p.M = q.M; p.N = q.N; p.K = q.K; p.G = q.G;
        p.fused = q.fused_gate_up ? 1 : 0;
        p.prepacked = 1;
        p.kc = pp_nsc(q.K) * PP_SC;
        p.tile_begin = (int)tiles;
        tiles += ((p.fused ? p.N / 2 : p.N) + 15) / 16;
        fused_any |= p.fused != 0;
        max_nsc = std::max(max_nsc, pp_nsc(q.K));
        x_bytes = std::max(x_bytes, (size_t)p.M * (p.kc + XPAD) * 2);
    }
    if (tiles > MAX_PLAN_GRID) return VRL_INT4_ESHAPE;
    const int wpb = max_nsc > 8 ? 16 : (max_nsc > 4 ? 8 : 4);
    const size_t red = (size_t)(wpb - 1) * (fused_any ? 2 : 1) * WAVE * sizeof(f32x4_t);
    // padding rows of the A operand read a staged row of zeros where LDS is plentiful
    size_t xz_bytes = x_bytes;
    for (int i = 0; i < n_problems; ++i) {
        DevProblem &p = args.recs[i];
        const size_t need = (size_t)(p.M + 1) * (p.kc + XPAD) * 2;
        if (p.M < MAX_TILE_M && need + red <= 32 * 1024) {
            p.prepacked |= PP_ZERO_ROW;
            xz_bytes = std::max(xz_bytes, need);
        }
    }
    const size_t lds = xz_bytes + red;
    if (lds > 64 * 1024) return VRL_INT4_ESHAPE;  // activations too large for this path: use a plan
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
    if (fused_any) {
        switch (wpb) {
            case 4: return launch_direct<true, 4>(args, (int)tiles, lds, stream);
            case 8: return launch_direct<true, 8>(args, (int)tiles, lds, stream);
            default: return launch_direct<true, 16>(args, (int)tiles, lds, stream);
        }
    }
    switch (wpb) {
        case 4: return launch_direct<false, 4>(args, (int)tiles, lds, stream);
        case 8: return launch_direct<false, 8>(args, (int)tiles, lds, stream);
        default: return launch_direct<false, 16>(args, (int)tiles, lds, stream);
    }
}

size_t vrl_int4_grouped_plan_size(int n_problems) {
    if (n_problems < 1) return 0;
    return plan_bytes_for(n_problems);
}

int vrl_int4_grouped_plan_build(const vrl_int4_problem *problems, int n_problems, void *plan_host,
                                size_t plan_bytes, vrl_int4_plan_info *info) {
    if (!problems || !plan_host || !info) return VRL_INT4_ENULL;
    if (n_problems < 1 || plan_bytes < vrl_int4_grouped_plan_size(n_problems)) return VRL_INT4_EPLAN;
    uint8_t *base = static_cast<uint8_t *>(plan_host);
    DevProblem *recs = reinterpret_cast<DevProblem *>(base + sizeof(PlanHeader));
    int2 *block_tab = reinterpret_cast<int2 *>(recs + n_problems);
    std::vector<int32_t> block_begin((size_t)MAX_PLAN_GRID + 1, 0);

    long tiles = 0;
    double total_cost = 0.0;
    int variant = 0;
    int pp_group_size = 0;      // group size of the prepacked records, -1 if they differ
    size_t x_need = 0;  // bytes the largest activation matrix needs if staged whole
    for (int i = 0; i < n_problems; ++i) {
        const vrl_int4_problem &q = problems[i];
        variant |= (q.prepacked ? VARIANT_PP : VARIANT_CANON) | (q.fused_gate_up ? VARIANT_FUSED : 0);
        int rc;
        if (q.prepacked)
            rc = check_problem(q.x, q.qweight, q.qweight, q.qweight, q.y, q.M, q.N, q.K, q.G);
        else
            rc = check_problem(q.x, q.qweight, q.scales, q.qzeros, q.y, q.M, q.N, q.K, q.G);
        if (rc != VRL_INT4_OK) return rc;
        if (q.fused_gate_up && q.N % 2 != 0) return VRL_INT4_ESHAPE;
        DevProblem p;
        memset(&p, 0, sizeof p);
        p.x = static_cast<const uint16_t *>(q.x);
        p.qweight = static_cast<const uint32_t *>(q.qweight);
        p.scales = static_cast<const uint16_t *>(q.scales);
        p.qzeros = static_cast<const uint32_t *>(q.qzeros);
        p.y = static_cast<uint16_t *>(q.y);
        p.M = q.M; p.N = q.N; p.K = q.K; p.G = q.G;
        p.fused = q.fused_gate_up ? 1 : 0;
        p.prepacked = q.prepacked ? 1 : 0;
        if (!tile_path_ok(p)) return VRL_INT4_ESHAPE;  // grouped launches take MFMA-path shapes only
        if (p.prepacked && (!prepack_ok(p.N, p.K, p.G) || (p.fused && (p.N / 2) % 16 != 0)))
            return VRL_INT4_ESHAPE;
        if (p.prepacked) pp_group_size = (pp_group_size == 0 || pp_group_size == p.G) ? p.G : -1;
        if (p.M > MAX_TILE_M) variant |= VARIANT_MB2;
        p.tile_begin = (int)tiles;
        const int out_cols = p.fused ? p.N / 2 : p.N;
        const long nt = (out_cols + 15) / 16;
        tiles += nt;
        if (tiles >= (1L << 30)) return VRL_INT4_ESHAPE;
        total_cost += (double)nt * ((double)p.K * (p.fused ? 2 : 1) + 512.0);
        const int kfull = p.prepacked ? pp_nsc(p.K) * PP_SC : p.K;
        const size_t need = (size_t)p.M * (kfull + XPAD) * 2;
        if (need > x_need) x_need = need;
        recs[i] = p;
    }
    // Records go into the blob longest tiles first (the kernel only needs tile_begin to ascend
    // with the record index): the ranges that start last then hold the shortest tiles.
    {
        std::stable_sort(recs, recs + n_problems, [](const DevProblem &a, const DevProblem &b) {
            return (long)a.K * (a.fused ? 2 : 1) > (long)b.K * (b.fused ? 2 : 1);
        });
        long t = 0;
        for (int i = 0; i < n_problems; ++i) {
            recs[i].tile_begin = (int)t;
            t += ((recs[i].fused ? recs[i].N / 2 : recs[i].N) + 15) / 16;
        }
    }
    // more than 16 activation rows per record: prepacked-only plans (two A operands per tile)
    if ((variant & VARIANT_MB2) && (variant & VARIANT_CANON)) return VRL_INT4_ESHAPE;

    // workgroup shape: the narrowest whose LDS holds the largest activation matrix whole
    // (plans with canonical or 32-row records have no 8-wave build); the widest one otherwise,
    // walking K in staged passes
    int shape = 2;
    for (int i = 0; i < 3; ++i) {
        if (x_need > STREAM_SHAPES[i].lds) continue;
        if (i == 1 && (variant & VARIANT_CANON)) continue;
        shape = i;
        break;
    }
    if (variant & VARIANT_MB2) shape = 2;
    const StreamShape sh = STREAM_SHAPES[shape];
    size_t smem = 0;
    for (int i = 0; i < n_problems; ++i) {
        DevProblem &p = recs[i];
        p.kc = p.prepacked ? pp_staged_k(p.M, p.K, sh.lds) : stream_staged_k(p.M, p.K, sh.lds);
        const size_t need = (size_t)p.M * (p.kc + XPAD) * 2;
        if (need > smem) smem = need;
        if (p.prepacked && p.kc < pp_nsc(p.K) * PP_SC) variant |= VARIANT_PASSES;
    }
    int wpb = sh.wpb;  // waves per workgroup of the launch
    // How many workgroups of this build a CU holds at a given LDS size (0: the runtime cannot say).
    auto resident_per_cu = [&](size_t lds_bytes) {
        vrl_int4_plan_info probe;
        memset(&probe, 0, sizeof probe);
        probe.block_threads = wpb * WAVE;
        probe.lds_bytes = (int)lds_bytes;
        probe.variant = variant;
        if (dispatch_stream(&probe, nullptr, nullptr, nullptr) != VRL_INT4_OK) return 0;
        return probe.grid;
    };
    // One contiguous tile range per workgroup, balanced by streamed bytes.  The grid is what the
    // device holds at once (every workgroup runs from start to end, no second round of
    // prologues: measured 1 % faster than a grid twice as deep); if the runtime cannot say how
    // many fit, the table's deeper grid is used and the dispatcher evens out the tail.
    // Plans with fewer tiles than the device has workgroup slots take the latency mode: one
    // workgroup per tile, its waves splitting K (gemv_split_kernel); the partial tiles need LDS
    // behind the staged activations.
    // As many waves share a tile as it has super-chunks (4, 8 or 16), fewer if the plan would
    // not fit the device at that width.
    size_t red_bytes = 0;
    if (shape == 0 && !(variant & (VARIANT_CANON | VARIANT_MB2 | VARIANT_PASSES))) {
        int max_nsc = 1;
        for (int i = 0; i < n_problems; ++i) max_nsc = std::max(max_nsc, pp_nsc(recs[i].K));
        variant |= VARIANT_SPLIT;
        for (int w = max_nsc > 8 ? 16 : (max_nsc > 4 ? 8 : 4); w >= 4; w /= 2) {
            const size_t rb = (size_t)(w - 1) * ((variant & VARIANT_FUSED) ? 2 : 1) * WAVE * sizeof(f32x4_t);
            wpb = w;
            const int slots = resident_per_cu(smem + rb);
            if (slots >= 1 && tiles <= (long)device_cu_count() * slots && tiles <= MAX_PLAN_GRID) {
                red_bytes = rb;
                break;
            }
        }
        if (red_bytes == 0) {
            variant &= ~VARIANT_SPLIT;
            wpb = sh.wpb;
        }
    }
    // The throughput kernel is built per group size: its prepacked records share one, and only
    // 128 goes together with canonical records.  (The latency kernel takes them mixed.)
    if (!(variant & VARIANT_SPLIT) && pp_group_size != 0) {
        if (pp_group_size < 0 || ((variant & VARIANT_CANON) && pp_group_size != 128)) return VRL_INT4_ESHAPE;
        variant |= pp_group_size == 64 ? VARIANT_G64 : (pp_group_size == 32 ? VARIANT_G32 : 0);
    }
    long per_cu = sh.per_cu;
    const int resident = resident_per_cu(smem + red_bytes);
    if (resident >= 1) per_cu = resident;
    // Prepacked records with unused A-operand rows stage one more row, of zeros, for those
    // rows to read, if that costs no residency.
    if (resident >= 1) {
        const int rows_per_record = (variant & VARIANT_MB2) ? 32 : 16;
        size_t smem_z = smem;
        for (int i = 0; i < n_problems; ++i) {
            const DevProblem &p = recs[i];
            const size_t need = (size_t)(p.M + 1) * (p.kc + XPAD) * 2;
            if (p.prepacked && p.M < rows_per_record && need <= sh.lds && need > smem_z) smem_z = need;
        }
        if (smem_z == smem || resident_per_cu(smem_z + red_bytes) == resident) {
            for (int i = 0; i < n_problems; ++i) {
                DevProblem &p = recs[i];
                if (p.prepacked && p.M < rows_per_record && (size_t)(p.M + 1) * (p.kc + XPAD) * 2 <= smem_z)
                    p.prepacked |= PP_ZERO_ROW;
            }
            smem = smem_z;
        }
    }
    smem += red_bytes;
    long grid = (long)device_cu_count() * per_cu;
    if (grid > MAX_PLAN_GRID) grid = MAX_PLAN_GRID;
    const long max_useful = (tiles + sh.wpb - 1) / sh.wpb;
    if (grid > max_useful) grid = max_useful;
    if (variant & VARIANT_SPLIT) {
        grid = tiles;
        for (long k = 0; k <= grid; ++k) block_begin[(size_t)k] = (int)k;
        int rec = 0;
        for (long k = 0; k <= grid; ++k) {
            while (rec + 1 < n_problems && recs[rec + 1].tile_begin <= block_begin[(size_t)k]) ++rec;
            block_tab[k] = make_int2(block_begin[(size_t)k], rec);
        }
    } else
    {
        int b = 0;
        double acc_cost = 0.0;
        block_begin[0] = 0;
        for (int i = 0; i < n_problems; ++i) {
            const DevProblem &p = recs[i];
            const int out_cols = p.fused ? p.N / 2 : p.N;
            const int nt = (out_cols + 15) / 16;
            const double c = (double)p.K * (p.fused ? 2 : 1) + 512.0;
            for (int t = 0; t < nt; ++t) {
                // tile (p.tile_begin + t) starts block b+1 once the blocks so far hold their share
                while (b + 1 < grid && acc_cost >= total_cost * (b + 1) / (double)grid) {
                    ++b;
                    block_begin[b] = p.tile_begin + t;
                }
                acc_cost += c;
            }
        }
        while (b < grid) {
            ++b;
            block_begin[b] = (int)tiles;
        }
        int rec = 0;
        for (long k = 0; k <= grid; ++k) {
            while (rec + 1 < n_problems && recs[rec + 1].tile_begin <= block_begin[(size_t)k]) ++rec;
            block_tab[k] = make_int2(block_begin[(size_t)k], rec);
        }
    }

    PlanHeader hdr;
    hdr.magic = PLAN_MAGIC;
    hdr.n_records = n_problems;
    hdr.total_tiles = (int)tiles;
    hdr.grid = (int)grid;
    memcpy(plan_host, &hdr, sizeof hdr);
    memset(info, 0, sizeof *info);
    info->n_problems = n_problems;
    info->total_tiles = (int)tiles;
    info->grid = (int)grid;
    info->block_threads = wpb * WAVE;
    info->lds_bytes = (int)smem;
    info->variant = variant;
    return VRL_INT4_OK;
}

int vrl_int4_gemv_grouped_bf16(const void *plan_dev, const vrl_int4_plan_info *info,
                               void *hip_stream) {
    if (!plan_dev || !info) return VRL_INT4_ENULL;
    if (info->n_problems < 1 || info->total_tiles < 1 || info->grid < 1 ||
        info->grid > MAX_PLAN_GRID || info->lds_bytes < 0 || (size_t)info->lds_bytes > LDS_PER_CU ||
        !aligned16(plan_dev))
        return VRL_INT4_EPLAN;
    const uint8_t *base = static_cast<const uint8_t *>(plan_dev);
    const DevProblem *recs = reinterpret_cast<const DevProblem *>(base + sizeof(PlanHeader));
    const int2 *block_begin = reinterpret_cast<const int2 *>(recs + info->n_problems);
    vrl_int4_plan_info launch = *info;
    return dispatch_stream(&launch, recs, block_begin, reinterpret_cast<hipStream_t>(hip_stream));
}

}  // extern "C"
