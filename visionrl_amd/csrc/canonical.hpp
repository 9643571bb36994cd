// Kernels over the canonical operand triple (qweight, scales, qzeros): bit-exact dequant, the generic
// fallback, the single-launch split-K tile kernel and the canonical half of the grouped stream kernel.
#pragma once

#include "common.hpp"

namespace {

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

}  // namespace
