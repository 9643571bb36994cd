// Plan-free launches of 17 to 32 activation rows over long K: activations staged in passes over K, either with one
// record for all the rows (a weight word is read and rebuilt once and multiplied with both blocks of 16 rows) or
// with records of 16 rows.
#pragma once

#include "prepacked.hpp"

namespace {

// The latency mode of split_segment_pp (KS waves share a tile's K, TW tiles per workgroup, partial tiles meet in
// LDS) for records of up to 16 * MB rows.  LDS holds the rows' p.kc values of k at a time: where K is longer, K is walked
// in passes of p.kc (a multiple of 512), x staged again for each, the accumulators kept across them, and the KS
// waves split the super-chunks of every pass; a wave's ring runs on from its share of one pass into its share of
// the next, so the weights of the next pass arrive while x is staged.  One set of TW tiles per workgroup.
// Two row blocks are reduced one after the other through the same LDS space.
template <bool FUSED, int KS, int TW, int GQ, int MB>
__device__ __forceinline__ void rows32_segment(const DevProblem &p, int t0, int t1, uint8_t *smem) {
    constexpr int RS = FUSED ? 2 : 1;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tw = wave / KS, kw = wave % KS;  // tile of the set, share of K
    const int lane = threadIdx.x & (WAVE - 1);
    uint16_t *xs = reinterpret_cast<uint16_t *>(smem);
    const int xstride = p.kc + XPAD;
    const int xrows = p.M + ((p.prepacked & PP_ZERO_ROW) ? 1 : 0);
    f32x4_t *red = reinterpret_cast<f32x4_t *>(smem + (size_t)xrows * xstride * 2) + tw * (KS - 1) * RS * WAVE;
    const int nsc = pp_nsc(p.K);
    const int sc_pass = p.kc / PP_SC;
    const int npass = (nsc + sc_pass - 1) / sc_pass;
    const rsrc_t rsrc = pp_blob_rsrc(p);
    PPRing<RS, GQ> ring;
    const int tile = t0 + tw;
    const bool has_tile = tile < t1;  // wave-uniform
    // the wave's super-chunks of pass q: [a0, a1)
    auto share = [&](int q, int &a0, int &a1) {
        const int b0 = q * sc_pass, b1 = min(nsc, b0 + sc_pass);
        const int per = (b1 - b0 + KS - 1) / KS;
        a0 = min(b1, b0 + kw * per);
        a1 = min(b1, a0 + per);
    };
    // the first pass in which the wave has a share: its weights are on their way while x is staged
    int q_next = -1, n0 = 0, n1 = 0;
    if (has_tile) {
        for (int q = 0; q < npass && q_next < 0; ++q) {
            share(q, n0, n1);
            if (n0 < n1) q_next = q;
        }
    }
    if (q_next >= 0) pp_prime<FUSED, GQ>(rsrc, pp_tile_ptr<FUSED>(p, tile, n0), ring);
    f32x4_t acc[RS][MB];
#pragma unroll
    for (int r = 0; r < RS; ++r)
#pragma unroll
        for (int b = 0; b < MB; ++b) acc[r][b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    for (int q = 0; q < npass; ++q) {
        const int b0 = q * sc_pass, b1 = min(nsc, b0 + sc_pass);
        __syncthreads();  // the pass before is read
        stage_x_natural(p, b0 * PP_SC, b1 * PP_SC, xs, xstride, KS * TW * WAVE);
        __syncthreads();
        if (q == q_next) {  // wave-uniform: the ring holds super-chunk n0 of the tile
            const int a0 = n0, a1 = n1;
            q_next = -1;
            for (int qq = q + 1; qq < npass && q_next < 0; ++qq) {
                share(qq, n0, n1);
                if (n0 < n1) q_next = qq;
            }
            stream_rows_pp<MB, FUSED, GQ>(p, rsrc, pp_tile_ptr<FUSED>(p, tile, a0), q_next >= 0 ? tile : -1,
                                          xs + (a0 - b0) * PP_SC, xstride, a0, a1, ring, acc, nullptr, nullptr,
                                          nullptr, q_next >= 0 ? n0 : -1);
        }
    }
    // the partial tiles meet, one block of 16 rows after the other
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        if (kw != 0) {
#pragma unroll
            for (int r = 0; r < RS; ++r) red[((kw - 1) * RS + r) * WAVE + lane] = acc[r][b];
        }
        __syncthreads();
        if (kw == 0 && has_tile) {
#pragma unroll
            for (int w = 1; w < KS; ++w)
#pragma unroll
                for (int r = 0; r < RS; ++r) acc[r][b] += red[((w - 1) * RS + r) * WAVE + lane];
        }
        if (b + 1 < MB) __syncthreads();  // read before the next block's partial tiles are written
    }
    if (kw == 0 && has_tile) store_tile<MB, FUSED>(p, tile, acc);
}

template <bool FUSED, int KS, int TW, int MB>
__global__ __launch_bounds__(KS *TW *WAVE) void gemv_rows32_direct_kernel(DirectArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int g = blockIdx.x;
    DevProblem p = a.recs[0];
#pragma unroll
    for (int k = 1; k < DIRECT_MAX; ++k)
        if (k < a.n && a.recs[k].tile_begin <= g) p = a.recs[k];  // scalar selects, no indexing
    const int tiles = ((p.fused ? p.N / 2 : p.N) + 15) / 16;
    const int t0 = (g - p.tile_begin) * TW;
    const int t1 = min(tiles, t0 + TW);
    if (FUSED && p.fused) {
        if (p.G == 128) rows32_segment<FUSED, KS, TW, 1, MB>(p, t0, t1, smem);
        else if (p.G == 64) rows32_segment<FUSED, KS, TW, 2, MB>(p, t0, t1, smem);
        else rows32_segment<FUSED, KS, TW, 4, MB>(p, t0, t1, smem);
    } else {
        if (p.G == 128) rows32_segment<false, KS, TW, 1, MB>(p, t0, t1, smem);
        else if (p.G == 64) rows32_segment<false, KS, TW, 2, MB>(p, t0, t1, smem);
        else rows32_segment<false, KS, TW, 4, MB>(p, t0, t1, smem);
    }
}

}  // namespace
