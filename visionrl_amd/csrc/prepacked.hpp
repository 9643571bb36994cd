// The prepacked (MFMA-shaped) weight layout: repack kernel, the throughput stream over it and the
// latency kernels whose waves split K.
#pragma once

#include "canonical.hpp"
#include "lora.hpp"

namespace {

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

// Residual add and RMSNorm applied while the activations are staged (plan-free launches only):
// the record's x points into `x0`, a sublayer output; what the tiles multiply is
//   weight * bf16(h * rsqrt(mean(h^2) + eps)),  h = residual ? bf16(x + residual) : x
// with the roundings LlamaDecoderLayer.forward / LlamaRMSNorm.forward apply to bf16 tensors.
// Every workgroup normalises the rows it stages (the row kept in registers: one wave per row, or,
// when there are fewer rows than waves, `split` waves per row whose sums of squares meet in LDS: a
// single wave issues too slowly to hide a row's arithmetic); the first workgroup of a record flagged
// PP_WRITE_H also writes h to `h_out`.
struct NormArgs {
    const uint16_t *x0;        // base of the activation tensor the records' x point into
    const uint16_t *residual;  // same shape as x0, or nullptr
    const uint16_t *weight;    // [K]
    uint16_t *h_out;           // same shape as x0, or nullptr; never the memory of x0 or residual
    float eps;
    int32_t enabled;
};
constexpr int PP_WRITE_H = 4;       // DevProblem::prepacked bit
constexpr int NORM_MAX_K = 4096;    // eight 16-byte words per lane hold a row

// NW: 16-byte words per lane that hold a wave's share of a row (K <= NW * split * 512); `scratch`:
// one float per wave, used when split > 1 (then M * split <= nwaves: one pass)
template <int NW>
__device__ __forceinline__ void stage_x_norm_rows(const DevProblem &p, const NormArgs &n, int kext, uint16_t *xs,
                                                  int xstride, int nwaves, bool write_h, int split,
                                                  float *scratch) {
    typedef __attribute__((address_space(1))) u32x4_t *gptr_w4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & (WAVE - 1);
    const int nthreads = nwaves * WAVE;
    const u32x4_t zero = {0u, 0u, 0u, 0u};
    // k beyond K reads as zero; so does the row behind the activation rows if the record has one
    const int padw = (kext - p.K) >> 3;
    for (int idx = threadIdx.x; idx < p.M * padw; idx += nthreads) {
        const int m = idx / padw;
        *reinterpret_cast<u32x4_t *>(xs + m * xstride + p.K + ((idx - m * padw) << 3)) = zero;
    }
    if (p.prepacked & PP_ZERO_ROW)
        for (int j = threadIdx.x; j < (kext >> 3); j += nthreads)
            *reinterpret_cast<u32x4_t *>(xs + p.M * xstride + (j << 3)) = zero;
    const long base = p.x - n.x0;
    const float inv_k = 1.0f / (float)p.K;
    const int per_pass = nwaves / split, part = wave % split;
    for (int m0 = 0; m0 < p.M; m0 += per_pass) {
        const int m = m0 + wave / split;
        const bool live = m < p.M;  // wave-uniform
        const long row = base + (long)m * p.K;
        u32x4_t h[NW], rv[NW], wv[NW];
        // one memory round trip: the row, its residual and the norm weight are requested together
#pragma unroll
        for (int i = 0; i < NW; ++i) {
            const int k = ((part * NW + i) * WAVE + lane) << 3;
            h[i] = rv[i] = wv[i] = zero;
            if (live && k < p.K) {
                h[i] = *as_global(reinterpret_cast<const u32x4_t *>(n.x0 + row + k));
                if (n.residual) rv[i] = *as_global(reinterpret_cast<const u32x4_t *>(n.residual + row + k));
                wv[i] = *as_global(reinterpret_cast<const u32x4_t *>(n.weight + k));
            }
        }
        float ss = 0.0f;
#pragma unroll
        for (int i = 0; i < NW; ++i) {
            const int k = ((part * NW + i) * WAVE + lane) << 3;
            if (live && k < p.K) {
                if (n.residual) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        h[i][e] = pack_bf16_rne(
                            bf16_bits_to_f32(rv[i][e] & 0xFFFFu) + bf16_bits_to_f32(h[i][e] & 0xFFFFu),
                            bf16_bits_to_f32(rv[i][e] >> 16) + bf16_bits_to_f32(h[i][e] >> 16));
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float lo = bf16_bits_to_f32(h[i][e] & 0xFFFFu), hi = bf16_bits_to_f32(h[i][e] >> 16);
                    ss += lo * lo;
                    ss += hi * hi;
                }
                if (write_h) *(gptr_w4)(uintptr_t)(n.h_out + row + k) = h[i];
            }
        }
        ss = wave_sum(ss);
        if (split > 1) {  // uniform; the row's waves add their shares in one order
            if (lane == 0) scratch[wave] = ss;
            __syncthreads();
            ss = 0.0f;
            for (int q = 0; q < split; ++q) ss += scratch[wave - part + q];
        }
        const float r = rsqrtf(ss * inv_k + n.eps);
#pragma unroll
        for (int i = 0; i < NW; ++i) {
            const int k = ((part * NW + i) * WAVE + lane) << 3;
            if (live && k < p.K) {
                u32x4_t y;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t xn = pack_bf16_rne(bf16_bits_to_f32(h[i][e] & 0xFFFFu) * r,
                                                      bf16_bits_to_f32(h[i][e] >> 16) * r);
                    y[e] = pack_bf16_rne(bf16_bits_to_f32(wv[i][e] & 0xFFFFu) * bf16_bits_to_f32(xn & 0xFFFFu),
                                         bf16_bits_to_f32(wv[i][e] >> 16) * bf16_bits_to_f32(xn >> 16));
                }
                *reinterpret_cast<u32x4_t *>(xs + m * xstride + k) = y;
            }
        }
    }
}

// The same for a wave that holds a whole row of 2049 to 4096 values (eight words per lane, one wave per
// row): the row stays packed in registers, the residual and the norm weight pass through four registers'
// worth of words at a time (the second half of the residual and both halves of the weight are requested when
// their registers are free: round trips into cache beyond the first).  Row, residual and weight held
// together are 96 registers, which made every build of the kernel that contains this path allocate 154 to
// 177 and the 16-wave builds spill.
__device__ __forceinline__ void stage_x_norm_rows_wide(const DevProblem &p, const NormArgs &n, int kext, uint16_t *xs,
                                                       int xstride, int nwaves, bool write_h) {
    typedef __attribute__((address_space(1))) u32x4_t *gptr_w4;
    constexpr int NW = 8, CH = 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & (WAVE - 1);
    const int nthreads = nwaves * WAVE;
    const u32x4_t zero = {0u, 0u, 0u, 0u};
    const int padw = (kext - p.K) >> 3;
    for (int idx = threadIdx.x; idx < p.M * padw; idx += nthreads) {
        const int m = idx / padw;
        *reinterpret_cast<u32x4_t *>(xs + m * xstride + p.K + ((idx - m * padw) << 3)) = zero;
    }
    if (p.prepacked & PP_ZERO_ROW)
        for (int j = threadIdx.x; j < (kext >> 3); j += nthreads)
            *reinterpret_cast<u32x4_t *>(xs + p.M * xstride + (j << 3)) = zero;
    const long base = p.x - n.x0;
    const float inv_k = 1.0f / (float)p.K;
    for (int m0 = 0; m0 < p.M; m0 += nwaves) {
        const int m = m0 + wave;
        const bool live = m < p.M;  // wave-uniform
        const long row = base + (long)m * p.K;
        u32x4_t h[NW], t[CH];
#pragma unroll
        for (int i = 0; i < NW; ++i) {
            const int k = (i * WAVE + lane) << 3;
            h[i] = zero;
            if (live && k < p.K) h[i] = *as_global(reinterpret_cast<const u32x4_t *>(n.x0 + row + k));
        }
        float ss = 0.0f;
#pragma unroll
        for (int c = 0; c < NW; c += CH) {
            if (n.residual) {
#pragma unroll
                for (int i = 0; i < CH; ++i) {
                    const int k = ((c + i) * WAVE + lane) << 3;
                    t[i] = zero;
                    if (live && k < p.K) t[i] = *as_global(reinterpret_cast<const u32x4_t *>(n.residual + row + k));
                }
            }
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                const int k = ((c + i) * WAVE + lane) << 3;
                if (live && k < p.K) {
                    if (n.residual) {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            h[c + i][e] = pack_bf16_rne(
                                bf16_bits_to_f32(t[i][e] & 0xFFFFu) + bf16_bits_to_f32(h[c + i][e] & 0xFFFFu),
                                bf16_bits_to_f32(t[i][e] >> 16) + bf16_bits_to_f32(h[c + i][e] >> 16));
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float lo = bf16_bits_to_f32(h[c + i][e] & 0xFFFFu), hi = bf16_bits_to_f32(h[c + i][e] >> 16);
                        ss += lo * lo;
                        ss += hi * hi;
                    }
                    if (write_h) *(gptr_w4)(uintptr_t)(n.h_out + row + k) = h[c + i];
                }
            }
        }
        ss = wave_sum(ss);
        const float r = rsqrtf(ss * inv_k + n.eps);
#pragma unroll
        for (int c = 0; c < NW; c += CH) {
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                const int k = ((c + i) * WAVE + lane) << 3;
                t[i] = zero;
                if (live && k < p.K) t[i] = *as_global(reinterpret_cast<const u32x4_t *>(n.weight + k));
            }
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                const int k = ((c + i) * WAVE + lane) << 3;
                if (live && k < p.K) {
                    u32x4_t y;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t xn = pack_bf16_rne(bf16_bits_to_f32(h[c + i][e] & 0xFFFFu) * r,
                                                          bf16_bits_to_f32(h[c + i][e] >> 16) * r);
                        y[e] = pack_bf16_rne(bf16_bits_to_f32(t[i][e] & 0xFFFFu) * bf16_bits_to_f32(xn & 0xFFFFu),
                                             bf16_bits_to_f32(t[i][e] >> 16) * bf16_bits_to_f32(xn >> 16));
                    }
                    *reinterpret_cast<u32x4_t *>(xs + m * xstride + k) = y;
                }
            }
        }
    }
}

__device__ __forceinline__ void stage_x_norm(const DevProblem &p, const NormArgs &n, int kext, uint16_t *xs,
                                             int xstride, int nwaves, bool write_h, float *scratch) {
    // rows up to 2048 wide keep half the registers (the 16-wave workgroups have 128 per lane)
    const int words = p.K <= NORM_MAX_K / 2 ? NORM_MAX_K / (16 * WAVE) : NORM_MAX_K / (8 * WAVE);
    int split = 1;
    while (2 * split * p.M <= nwaves && 2 * split <= words) split *= 2;
    switch (words / split) {
        case 8: stage_x_norm_rows_wide(p, n, kext, xs, xstride, nwaves, write_h); break;  // split == 1 here
        case 4: stage_x_norm_rows<4>(p, n, kext, xs, xstride, nwaves, write_h, split, scratch); break;
        case 2: stage_x_norm_rows<2>(p, n, kext, xs, xstride, nwaves, write_h, split, scratch); break;
        default: stage_x_norm_rows<1>(p, n, kext, xs, xstride, nwaves, write_h, split, scratch); break;
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
// if next_tile >= 0 the ring holds that tile's super-chunk sc0 (next_sc0, if given) on return,
// so that the wave never runs dry between tiles.
// prio >= 0: the wave's issue priority rotates with every super-chunk, starting at prio (walks
// in lock-step between barriers, where the hardware's preference for the oldest wave of a SIMD
// would make the whole workgroup wait for the youngest).
// XG: the A operand is not staged in LDS: xpre[b][4 * d + dd] holds it for super-chunk `xpre_sc`
// (fetched by the caller) and is fetched again through `xr`, a range-checked resource over the
// record's x, whenever the walk reaches another super-chunk.
// VDOT (one activation row, kept for the comparison the roofline asks for): the dot product on the
// vector unit instead of the 16x16x32 matrix instruction.  A lane multiplies the eight weights it just
// rebuilt (its row, eight consecutive k) with the matching activations (one LDS read, the same address for
// the 16 lanes of a k quarter) in four v_dot2_f32_bf16 and keeps one running sum, in acc[r][0][0]; the
// four k quarters of a row meet when the tile is stored (store_tile_vdot).
template <int MB, bool FUSED, int GQ, bool XG = false, bool VDOT = false>
__device__ __forceinline__ void stream_rows_pp(const DevProblem &p, rsrc_t rsrc, const PPTilePtr<FUSED> &cur,
                                               int next_tile, const uint16_t *xs, int xstride,
                                               int sc0, int sc1, PPRing<FUSED ? 2 : 1, GQ> &ring,
                                               f32x4_t (&acc)[FUSED ? 2 : 1][MB],
                                               u32x4_t (*xpre)[16] = nullptr, int *xpre_sc = nullptr,
                                               const rsrc_t *xr = nullptr, int next_sc0 = -1,
                                               int prio = -1) {
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
                u32x4_t xrow;   // VDOT: the activation row's eight values
                if constexpr (VDOT) xrow = *reinterpret_cast<const u32x4_t *>(xs + kloc + 8 * dd);
#pragma unroll
                for (int b = 0; b < (VDOT ? 0 : MB); ++b) {
                    if constexpr (XG) {
                        xa[b] = __builtin_bit_cast(bf16x8_t, xpre[b][4 * d + dd]);
                    } else {
                        const int m = min(16 * b + lc, pad_row);
                        const u32x4_t raw = *reinterpret_cast<const u32x4_t *>(xs + m * xstride + kloc + 8 * dd);
                        xa[b] = __builtin_bit_cast(bf16x8_t, raw);
                    }
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
                    if constexpr (VDOT) {
                        // Four running sums, so that no dot instruction accumulates onto the result of one of the
                        // three before it (the hardware does not interlock a DOT result read that early).  Inline
                        // assembly: this toolchain drops all but the first of several independent
                        // __builtin_amdgcn_fdot2_f32_bf16 chains.
                        asm volatile("v_dot2_f32_bf16 %0, %4, %8, %0\n\t"
                                     "v_dot2_f32_bf16 %1, %5, %9, %1\n\t"
                                     "v_dot2_f32_bf16 %2, %6, %10, %2\n\t"
                                     "v_dot2_f32_bf16 %3, %7, %11, %3"
                                     : "+v"(acc[r][0][0]), "+v"(acc[r][0][1]), "+v"(acc[r][0][2]), "+v"(acc[r][0][3])
                                     : "v"(wv[0]), "v"(wv[1]), "v"(wv[2]), "v"(wv[3]), "v"(xrow[0]), "v"(xrow[1]),
                                       "v"(xrow[2]), "v"(xrow[3]));
                    } else {
#pragma unroll
                        for (int b = 0; b < MB; ++b)
                            acc[r][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[b], bop, acc[r][b], 0, 0, 0);
                    }
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
    const PPTilePtr<FUSED> nxt = pp_tile_ptr<FUSED>(p, has_next ? next_tile : 0, next_sc0 < 0 ? sc0 : next_sc0);
    const uint32_t voff = lane * 16u;
    for (int sc = sc0; sc < sc1; ++sc) {
        const bool last = sc + 1 == sc1;
        if (prio >= 0) {  // wave-uniform
            switch ((prio + sc) & 3) {
                case 0: __builtin_amdgcn_s_setprio(0); break;
                case 1: __builtin_amdgcn_s_setprio(1); break;
                case 2: __builtin_amdgcn_s_setprio(2); break;
                default: __builtin_amdgcn_s_setprio(3); break;
            }
        }
        if constexpr (XG) {
            if (*xpre_sc != sc) {  // wave-uniform; never with one super-chunk per wave
                const int kb = sc * PP_SC + kq * 128;
#pragma unroll
                for (int b = 0; b < MB; ++b) {
                    const int row = 16 * b + lc;
                    const uint32_t vo = (row < p.M && kb < p.K) ? (uint32_t)(row * p.K + kb) * 2u : PP_OUT_OF_RANGE;
#pragma unroll
                    for (int i = 0; i < 16; ++i) xpre[b][i] = __builtin_amdgcn_raw_buffer_load_b128(*xr, vo + 16u * i, 0, 0);
                }
                *xpre_sc = sc;
            }
        }
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

// What a workgroup's LDS holds of staged activations, so that a segment over the same x as the one
// before it (q|k|v or gate|up of a layer: records side by side in a plan) does not stage it again.
struct StagedX {
    const uint16_t *x = nullptr;  // nullptr: nothing whole
    int M = 0, K = 0, kc = 0, zero_row = 0;
};

// the four k quarters of each of the tile's 16 rows (lanes l, l + 16, l + 32, l + 48) added up and stored
__device__ __forceinline__ void store_tile_vdot(const DevProblem &p, int tile_local, float part) {
    const int lane = threadIdx.x & (WAVE - 1);
    part = row16_sum_quarters(part);
    const int col = tile_local * 16 + lane;
    if (lane < 16 && col < p.N) as_global(p.y)[col] = (uint16_t)(pack_bf16_rne(part, 0.0f) & 0xFFFFu);
}

template <int MB, bool FUSED, int WPB, bool PASSES, int GQ, bool VDOT = false>
__device__ __forceinline__ void stream_segment_pp(const DevProblem &p, int t0, int t1, uint8_t *smem,
                                                  StagedX &staged) {
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
        const int zero_row = p.prepacked & PP_ZERO_ROW;
        const bool resident = staged.x == p.x && staged.M == p.M && staged.K == p.K && staged.kc == p.kc &&
                              staged.zero_row == zero_row;  // block-uniform
        __syncthreads();
        if (threadIdx.x == 0) next_tile = t0 + WPB;
        if (!resident) stage_x_natural(p, 0, nsc * PP_SC, xs, xstride, WPB * WAVE);
        __syncthreads();
        staged.x = p.x;
        staged.M = p.M;
        staged.K = p.K;
        staged.kc = p.kc;
        staged.zero_row = zero_row;
        while (tile < t1) {
            int nt = 0;
            if ((threadIdx.x & (WAVE - 1)) == 0) nt = atomicAdd(&next_tile, 1);
            nt = __builtin_amdgcn_readfirstlane(nt);
            f32x4_t acc[RS][MB];
#pragma unroll
            for (int r = 0; r < RS; ++r)
#pragma unroll
                for (int b = 0; b < MB; ++b) acc[r][b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            stream_rows_pp<MB, FUSED, GQ, false, VDOT>(p, rsrc, cur, nt < t1 ? nt : -1, xs, xstride, 0, nsc, ring, acc);
            if constexpr (VDOT) {
                asm volatile("s_nop 2" ::: "memory");   // the last dot results are read next
                store_tile_vdot(p, tile, (acc[0][0][0] + acc[0][0][1]) + (acc[0][0][2] + acc[0][0][3]));
            }
            else store_tile<MB, FUSED>(p, tile, acc);
            tile = nt;
            if (tile < t1) cur = pp_tile_ptr<FUSED>(p, tile, 0);
        }
    } else if constexpr (PASSES) {
        // activations do not fit: K is walked in staged passes, and every wave carries T tiles
        // through a pass so that one staging serves T * WPB tiles
        // The ring runs through the whole segment: the last super-chunk of a (tile, pass) step
        // pulls in the first of the wave's next step (its next tile of this pass, else its first
        // tile of the next pass, else of the next round), also across the barriers of a staging.
        constexpr int T = FUSED ? 1 : 4;
        staged.x = nullptr;  // the passes leave a part of K behind
        const rsrc_t rsrc = pp_blob_rsrc(p);
        PPRing<RS, GQ> ring;
        if (t0 + wave < t1) pp_prime<FUSED, GQ>(rsrc, pp_tile_ptr<FUSED>(p, t0 + wave, 0), ring);
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
                        const PPTilePtr<FUSED> cur = pp_tile_ptr<FUSED>(p, tile, sc0);
                        int ntile = -1, nsc0 = sc0;
                        if (i + 1 < T && tile + WPB < t1) {
                            ntile = tile + WPB;
                        } else if (sc1 < nsc) {
                            ntile = round + wave;
                            nsc0 = sc1;
                        } else if (round + WPB * T + wave < t1) {
                            ntile = round + WPB * T + wave;
                            nsc0 = 0;
                        }
                        // waves w, w + 4, w + 8, w + 12 share a SIMD: each starts the pass at
                        // another priority and moves on with every super-chunk
                        const int prio = (wave >> 2) + i * (sc1 - sc0);
                        stream_rows_pp<MB, FUSED, GQ>(p, rsrc, cur, ntile, xs, xstride, sc0, sc1, ring, acc[i],
                                                      nullptr, nullptr, nullptr, nsc0, prio);
                    }
                }
                __builtin_amdgcn_s_setprio(0);
            }
#pragma unroll
            for (int i = 0; i < T; ++i) {
                const int tile = round + i * WPB + wave;
                if (tile < t1) store_tile<MB, FUSED>(p, tile, acc[i]);
            }
        }
    }
}

// Small launches (fewer tiles than the device has workgroup slots): KS waves share one tile,
// each taking a contiguous share of its super-chunks, and the partial tiles meet in LDS.  A
// tile is then one or two memory round trips instead of a serial walk over K by a single
// wave; this is the latency mode for launches of a few matrices (q|k|v of one layer, one
// o_proj, ...).  A workgroup carries TW such tiles at once (KS * TW waves), so that one
// staging of the activations serves TW tiles: that matters once x is tens of KB (8+ rows).
// LDS: staged activations, then TW x (KS - 1) x RS partial tiles.
// XG (plan-free launches of long K): no staging at all.  With K split over the waves and one tile
// per workgroup every activation value is used by exactly one wave, so each wave fetches its own A
// operand (16 rows x 512 k: sixteen 16-byte buffer loads per lane, zeros for rows beyond M and k
// beyond K through the buffer's range check) while its weights arrive, and again for every further
// super-chunk of its share (K > 8192: two per wave); LDS holds only the partial tiles, and 16 rows
// per record fit whatever K is.
// UP instantiations (plan-free launches of one problem) add a LoRA adapter's up-projection to the
// tile before it is stored: y = bf16(bf16(x . W^T) + scaling * t . B^T), the second half of a PEFT
// wrapper's forward (vrl/models/families/janus_pro/policy.py:298-324 attaches the adapters), with t
// the adapter's down-projection of x, handed over in `parts` pieces per row that are summed in order.
struct LoraUpArgs {
    const float *t;      // [M, parts, r] float32
    const void *B;       // [N, r], float32 or bf16
    const uint16_t *x0;  // row 0 of the problem's x: a record's first row is (p.x - x0) / K
    int32_t parts, r, fp32;
    float scaling;
};

// t of the record's rows (pieces summed; rounded to bf16 for a bf16 adapter, whose lora_A output is a
// bf16 tensor) and the rows of B for the workgroup's `cols` columns from `col0`, into LDS with row
// stride r + 4 floats
template <bool FP32>
__device__ __forceinline__ void stage_lora_up(const DevProblem &p, const LoraUpArgs &u, int col0, int cols,
                                              float *ts, float *bs, int nthreads) {
    const int r = u.r, stride = r + 4, r4 = r >> 2, r8 = r >> 3;
    const long m0 = (p.x - u.x0) / p.K;
    for (int idx = threadIdx.x; idx < p.M * r4; idx += nthreads) {
        const int m = idx / r4, j4 = idx - m * r4;
        const float *src = u.t + (m0 + m) * u.parts * r + 4 * j4;
        float4 v = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int q0 = 0; q0 < u.parts; q0 += 16) {   // sixteen pieces requested together, added in order
            float4 w[16];
#pragma unroll
            for (int k = 0; k < 16; ++k)
                w[k] = *reinterpret_cast<const float4 *>(src + (long)(q0 + k < u.parts ? q0 + k : u.parts - 1) * r);
#pragma unroll
            for (int k = 0; k < 16; ++k)
                if (q0 + k < u.parts) v.x += w[k].x, v.y += w[k].y, v.z += w[k].z, v.w += w[k].w;
        }
        if (!FP32) v.x = lora_round_bf16(v.x), v.y = lora_round_bf16(v.y), v.z = lora_round_bf16(v.z), v.w = lora_round_bf16(v.w);
        *reinterpret_cast<float4 *>(ts + m * stride + 4 * j4) = v;
    }
    for (int idx = threadIdx.x; idx < cols * r8; idx += nthreads) {
        const int c = idx / r8, j8 = idx - c * r8;
        const int n = min(col0 + c, p.N - 1);   // columns past the end repeat the last one and are not stored
        float f[8];
        load8<FP32>(u.B, (long)n * r + 8 * j8, f);
        *reinterpret_cast<float4 *>(bs + c * stride + 8 * j8) = float4{f[0], f[1], f[2], f[3]};
        *reinterpret_cast<float4 *>(bs + c * stride + 8 * j8 + 4) = float4{f[4], f[5], f[6], f[7]};
    }
}

// store_tile<1, false> with the adapter added; brow = the B row of the lane's column
template <bool FP32>
__device__ __forceinline__ void store_tile_lora(const DevProblem &p, int tile_local, const f32x4_t &acc,
                                                const LoraUpArgs &u, const float *ts, const float *bs) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int col = tile_local * 16 + (lane & 15);
    if (col >= p.N) return;
    const int stride = u.r + 4;
    const float *brow = bs + (lane & 15) * stride;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = 4 * (lane >> 4) + i;
        if (m < p.M) {
            const float *trow = ts + m * stride;
            float s = 0.0f;
            for (int j = 0; j < u.r; j += 4) {
                const float4 tv = *reinterpret_cast<const float4 *>(trow + j);
                const float4 bv = *reinterpret_cast<const float4 *>(brow + j);
                s += tv.x * bv.x + tv.y * bv.y + tv.z * bv.z + tv.w * bv.w;
            }
            const float delta = FP32 ? s * u.scaling : lora_round_bf16(lora_round_bf16(s) * u.scaling);
            const float base = bf16_bits_to_f32(pack_bf16_rne(acc[i], 0.0f) & 0xFFFFu);  // the base layer's bf16 output
            as_global(p.y)[(long)m * p.N + col] = (uint16_t)(pack_bf16_rne(base + delta, 0.0f) & 0xFFFFu);
        }
    }
}

// Bias and activation of a linear applied to the tile before it is stored (plan-free launches of one plain
// problem): y = act(bf16(bf16(x . W^T) + bias)), the roundings of a bf16 module whose bias is added to its
// output tensor and whose activation is a tensor op of its own (Janus' generation head is Linear, GELU, Linear:
// vrl/models/families/janus_pro/policy.py:138-160 calls it).  Last, a residual stream may be added:
// y = bf16(residual + that), the `hidden_states = residual + hidden_states` that follows o_proj and down_proj in
// LlamaDecoderLayer.forward (reached from policy.py:673-678), so that the launch after it reads one tensor.
struct EpiArgs {
    const uint16_t *bias;      // bf16 [N] or nullptr
    const uint16_t *residual;  // bf16 [M, N] added last (the residual stream a sublayer's output joins), or nullptr
    const uint16_t *y0;        // the problem's y: a record's rows of `residual` lie where its rows of y lie
    int32_t act;               // 0: none; 1: GELU, x / 2 * (1 + erf(x / sqrt 2)) in fp32
    int32_t enabled;
};

__device__ __forceinline__ float epi_round_bf16(float v) {
    return bf16_bits_to_f32(pack_bf16_rne(v, 0.0f) & 0xFFFFu);
}

__device__ __forceinline__ float epi_apply(float acc, float bias, bool has_bias, int act) {
    float v = epi_round_bf16(acc);
    if (has_bias) v = epi_round_bf16(v + bias);
    if (act == 1) v = v * 0.5f * (1.0f + erff(v * 0.70710678118654752440f));
    return v;
}

// What the lane's four outputs of a tile add from the residual stream, requested before the tile's weights are
// streamed so that the values wait in registers when the tile is stored (rows past M repeat the last one).
struct EpiResidual {
    uint16_t v[4];
};
__device__ __forceinline__ EpiResidual epi_residual(const DevProblem &p, int tile_local, const EpiArgs &e) {
    EpiResidual r = {{0, 0, 0, 0}};
    if (e.residual) {   // uniform over the launch
        const int lane = threadIdx.x & (WAVE - 1);
        const int col = min(tile_local * 16 + (lane & 15), p.N - 1);
        const uint16_t *rows = e.residual + (p.y - e.y0);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            r.v[i] = as_global(rows)[(long)min(4 * (lane >> 4) + i, p.M - 1) * p.N + col];
    }
    return r;
}

// store_tile<1, false> with the epilogue
__device__ __forceinline__ void store_tile_epi(const DevProblem &p, int tile_local, const f32x4_t &acc,
                                               const EpiArgs &e, const EpiResidual &res) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int col = tile_local * 16 + (lane & 15);
    if (col >= p.N) return;
    const bool has_bias = e.bias != nullptr;
    const float bias = has_bias ? bf16_bits_to_f32(as_global(e.bias)[col]) : 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = 4 * (lane >> 4) + i;
        if (m < p.M) {
            float v = epi_apply(acc[i], bias, has_bias, e.act);
            if (e.residual) v = epi_round_bf16(epi_round_bf16(v) + bf16_bits_to_f32(res.v[i]));
            as_global(p.y)[(long)m * p.N + col] = (uint16_t)(pack_bf16_rne(v, 0.0f) & 0xFFFFu);
        }
    }
}

template <bool FUSED, int KS, int TW, int GQ, bool NORM, bool XG, bool UP = false, bool EPI = false>
__device__ __forceinline__ void split_segment_pp(const DevProblem &p, int t0, int t1, uint8_t *smem,
                                                 const NormArgs &norm, const LoraUpArgs &up = LoraUpArgs{},
                                                 const EpiArgs &epi = EpiArgs{}) {
    constexpr int RS = FUSED ? 2 : 1;
    static_assert(!EPI || (!FUSED && !UP), "bias, activation and residual join a plain problem");
    static_assert(!XG || (TW == 1 && !NORM), "register-fed activations: one tile per workgroup, no norm");
    static_assert(!UP || (!FUSED && !NORM), "an adapter's up-projection joins a plain problem");
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tw = wave / KS, kw = wave % KS;  // tile of the round, share of K
    const int lane = threadIdx.x & (WAVE - 1);
    uint16_t *xs = reinterpret_cast<uint16_t *>(smem);
    const int xstride = p.kc + XPAD;
    const int xrows = XG ? 0 : p.M + ((p.prepacked & PP_ZERO_ROW) ? 1 : 0);
    f32x4_t *red = reinterpret_cast<f32x4_t *>(smem + (size_t)xrows * xstride * 2) + tw * (KS - 1) * RS * WAVE;
    const int nsc = pp_nsc(p.K);
    const int per = (nsc + KS - 1) / KS;
    const int sc0 = min(nsc, kw * per), sc1 = min(nsc, sc0 + per);
    const rsrc_t rsrc = pp_blob_rsrc(p);
    PPRing<RS, GQ> ring;
    int tile = t0 + tw;
    bool work = sc0 < sc1 && tile < t1;  // wave-uniform
    PPTilePtr<FUSED> cur = pp_tile_ptr<FUSED>(p, work ? tile : t0, sc0);
    if (work) pp_prime<FUSED, GQ>(rsrc, cur, ring);  // weights are on their way while x is staged
    // the adapter's operands sit behind every workgroup's partial tiles; the barrier before the
    // partial tiles are read makes them visible
    float *lora_ts = reinterpret_cast<float *>(smem + (size_t)xrows * xstride * 2) +
                     TW * (KS - 1) * RS * WAVE * 4;
    float *lora_bs = lora_ts + 16 * (UP ? up.r + 4 : 0);   // t of the record's (at most 16) rows, then B
    if constexpr (UP) {
        if (up.fp32) stage_lora_up<true>(p, up, t0 * 16, TW * 16, lora_ts, lora_bs, KS * TW * WAVE);
        else stage_lora_up<false>(p, up, t0 * 16, TW * 16, lora_ts, lora_bs, KS * TW * WAVE);
    }
    u32x4_t xpre[1][16];
    int xpre_sc = sc0;
    rsrc_t xr = rsrc;  // replaced below for XG
    if constexpr (XG) {
        const int lc = lane & 15, kbase = sc0 * PP_SC + (lane >> 4) * 128;  // the lane's row and 128-k span
        xr = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(p.x), 0, p.M * p.K * 2, 0x00020000);
        const uint32_t voff = (work && lc < p.M && kbase < p.K) ? (uint32_t)(lc * p.K + kbase) * 2u : PP_OUT_OF_RANGE;
#pragma unroll
        for (int i = 0; i < 16; ++i) xpre[0][i] = __builtin_amdgcn_raw_buffer_load_b128(xr, voff + 16u * i, 0, 0);
    } else {
        __syncthreads();
        if constexpr (NORM)
            stage_x_norm(p, norm, nsc * PP_SC, xs, xstride, KS * TW,
                         t0 == 0 && (p.prepacked & PP_WRITE_H) && norm.h_out != nullptr,
                         reinterpret_cast<float *>(smem + (size_t)xrows * xstride * 2));  // the partial tiles' space, still free
        else
            stage_x_natural(p, 0, nsc * PP_SC, xs, xstride, KS * TW * WAVE);
        __syncthreads();
    }
    for (int base = t0; base < t1; base += TW) {
        tile = base + tw;
        // a register-fed launch with an epilogue walks one tile per workgroup (the host sees to it): the
        // registers that would hold the next tile's activations are the epilogue's
        const int next = (XG && EPI) ? -1 : (tile + TW < t1 ? tile + TW : -1);
        f32x4_t acc[RS][1];
#pragma unroll
        for (int r = 0; r < RS; ++r) acc[r][0] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        if (work) {
            if constexpr (XG)
                stream_rows_pp<1, FUSED, GQ, true>(p, rsrc, cur, next, nullptr, 0, sc0, sc1, ring, acc, xpre, &xpre_sc, &xr);
            else
                stream_rows_pp<1, FUSED, GQ>(p, rsrc, cur, next, xs + sc0 * PP_SC, xstride, sc0, sc1, ring, acc);
            if (next >= 0) cur = pp_tile_ptr<FUSED>(p, next, sc0);
        }
        if (kw != 0) {
#pragma unroll
            for (int r = 0; r < RS; ++r) red[((kw - 1) * RS + r) * WAVE + lane] = acc[r][0];
        }
        // what the tile adds from the residual stream is requested here, when the wave's operands have left
        // the registers, and arrives while the partial tiles meet
        EpiResidual joins = {{0, 0, 0, 0}};
        if constexpr (EPI) {
            if (kw == 0 && tile < t1) joins = epi_residual(p, tile, epi);
        }
        __syncthreads();
        if (kw == 0 && tile < t1) {
#pragma unroll
            for (int w = 1; w < KS; ++w)
#pragma unroll
                for (int r = 0; r < RS; ++r) acc[r][0] += red[((w - 1) * RS + r) * WAVE + lane];
            if constexpr (UP) {
                const float *brows = lora_bs + (tile - t0) * 16 * (up.r + 4);
                if (up.fp32) store_tile_lora<true>(p, tile, acc[0][0], up, lora_ts, brows);
                else store_tile_lora<false>(p, tile, acc[0][0], up, lora_ts, brows);
            } else {
                if constexpr (EPI) store_tile_epi(p, tile, acc[0][0], epi, joins);
                else store_tile<1, FUSED>(p, tile, acc);
            }
        }
        if constexpr (XG && EPI) break;
        work = work && next >= 0;
        if (base + TW < t1) __syncthreads();  // the partial tiles are read before they are rewritten
    }
}

// the latency kernels take any of the three group sizes in one build (they are not register-critical)
template <bool FUSED, int KS, int TW, bool NORM, bool XG, bool UP = false, bool EPI = false>
__device__ __forceinline__ void split_by_group(const DevProblem &p, int t0, int t1, uint8_t *smem,
                                               const NormArgs &norm, const LoraUpArgs &up = LoraUpArgs{},
                                               const EpiArgs &epi = EpiArgs{}) {
    if constexpr (EPI) {
        if (p.G == 128) split_segment_pp<false, KS, TW, 1, NORM, XG, false, true>(p, t0, t1, smem, norm, up, epi);
        else if (p.G == 64) split_segment_pp<false, KS, TW, 2, NORM, XG, false, true>(p, t0, t1, smem, norm, up, epi);
        else split_segment_pp<false, KS, TW, 4, NORM, XG, false, true>(p, t0, t1, smem, norm, up, epi);
    } else if constexpr (UP) {
        if (p.G == 128) split_segment_pp<false, KS, TW, 1, false, XG, true>(p, t0, t1, smem, norm, up);
        else if (p.G == 64) split_segment_pp<false, KS, TW, 2, false, XG, true>(p, t0, t1, smem, norm, up);
        else split_segment_pp<false, KS, TW, 4, false, XG, true>(p, t0, t1, smem, norm, up);
    } else if (FUSED && p.fused) {
        if (p.G == 128) split_segment_pp<FUSED, KS, TW, 1, NORM, XG>(p, t0, t1, smem, norm);
        else if (p.G == 64) split_segment_pp<FUSED, KS, TW, 2, NORM, XG>(p, t0, t1, smem, norm);
        else split_segment_pp<FUSED, KS, TW, 4, NORM, XG>(p, t0, t1, smem, norm);
    } else {
        if (p.G == 128) split_segment_pp<false, KS, TW, 1, NORM, XG>(p, t0, t1, smem, norm);
        else if (p.G == 64) split_segment_pp<false, KS, TW, 2, NORM, XG>(p, t0, t1, smem, norm);
        else split_segment_pp<false, KS, TW, 4, NORM, XG>(p, t0, t1, smem, norm);
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
        split_by_group<FUSED, WPB, 1, false, false>(p, a, b, smem, NormArgs{});
        t = seg_end;
    }
}

// The same latency mode without a plan in device memory: up to DIRECT_MAX records travel
// as kernel arguments (no dependent loads before the first weight request).  Workgroup g of
// the launch takes the TW * rounds tiles from (g - first workgroup of its record) * TW * rounds of
// that record, TW at a time (rounds > 1 when the launch would otherwise have more workgroups than
// the device holds at once: a second wave of workgroups would stage x and ramp up all over again).
// This is the single-call path of a prepacked weight (and of q|k|v, gate|up groups); the host
// cuts activations of more than 16 rows, or too large for LDS, into row slabs, one record each.
constexpr int DIRECT_MAX = 8;
// LD instantiations carry the down-projection of LoRA adapters over the same input as extra
// workgroups (lora.hpp): the two are independent, so they share the launch.  The extra workgroups
// come first in the grid: they run longer than a tile's and should start first.
struct LoraDownArgs {
    LoraArgs a;
    const uint16_t *x;   // [a.M, a.K]: the input of the launch's problems
    float *t;            // [a.M, r_total]
    int32_t wgs;         // workgroups of the down-projection: the first of the grid
    int32_t fp32;        // the adapters' weight type
};
struct DirectArgs {
    int32_t n;
    int32_t rounds;               // sets of TW tiles a workgroup walks, one after the other
    DevProblem recs[DIRECT_MAX];  // tile_begin holds the record's first workgroup here
    NormArgs norm;                // read by the NORM instantiations only
    LoraDownArgs ld;              // read by the LD instantiations only
    LoraUpArgs up;                // read by the UP instantiations only
    EpiArgs epi;                  // read by the EPI instantiations only: bias, activation, residual before the store
};

template <bool FUSED, int KS, int TW, bool NORM, bool XG, bool LD, bool UP, bool EPI = false>
__global__ __launch_bounds__(KS *TW *WAVE) void gemv_split_direct_kernel(DirectArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    int g = blockIdx.x;
    if constexpr (LD) {
        if (g < a.ld.wgs) {  // uniform over the workgroup
            if constexpr (NORM)   // the adapters read the normalised rows, as the tiles do
                lora_down_workgroup<KS * TW, true>(a.ld.x, a.ld.a, a.ld.t, a.ld.fp32 != 0, g, reinterpret_cast<float *>(smem),
                                                   LoraNorm{a.norm.residual, a.norm.weight, a.norm.eps});
            else
                lora_down_workgroup<KS * TW>(a.ld.x, a.ld.a, a.ld.t, a.ld.fp32 != 0, g, reinterpret_cast<float *>(smem));
            return;
        }
        g -= a.ld.wgs;
    }
    DevProblem p = a.recs[0];
#pragma unroll
    for (int k = 1; k < DIRECT_MAX; ++k)
        if (k < a.n && a.recs[k].tile_begin <= g) p = a.recs[k];  // scalar selects, no indexing
    const int tiles = ((p.fused ? p.N / 2 : p.N) + 15) / 16;
    const int t0 = (g - p.tile_begin) * TW * a.rounds;
    split_by_group<FUSED, KS, TW, NORM, XG, UP, EPI>(p, t0, min(tiles, t0 + TW * a.rounds), smem, a.norm, a.up, a.epi);
}

}  // namespace
