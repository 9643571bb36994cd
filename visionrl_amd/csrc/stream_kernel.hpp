// The throughput kernel of the grouped launches and the flags that name its builds.
#pragma once

#include "prepacked.hpp"

namespace {

// which record kinds a plan holds and which build of the kernel runs it (vrl_int4_plan_info::variant)
constexpr int VARIANT_CANON = 1, VARIANT_PP = 2, VARIANT_FUSED = 4, VARIANT_MB2 = 8, VARIANT_PASSES = 16,
              VARIANT_SPLIT = 32, VARIANT_G64 = 64, VARIANT_G32 = 128;

// CANON / PP / FUSED say which kinds of record the plan holds, so that a plan of
// plain prepacked GEMVs runs the variant with the smallest register footprint.
// WPB (waves per workgroup) grows with the LDS the staged activations need, so that
// about 16 waves stay resident per CU; MB = 2 carries up to 32 activation rows per
// record with two A operands per weight tile (weights streamed once); PASSES adds the
// path for prepacked records whose activations do not fit LDS whole (it carries several
// accumulator tiles, so plans that do not need it run a build without it).
// VDOT: the comparison build whose dot product runs on the vector unit (one activation row, plain prepacked
// records of group size 128 only); the product library holds no such build, the measurement library does.
template <int WPB, int MB, bool CANON, bool PP, bool FUSED, bool PASSES, int GQ, bool VDOT = false>
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
    StagedX staged;
    for (int pi = lo; t < t_end && pi < n_problems; ++pi) {
        const DevProblem p = plan[pi];
        const int out_cols = p.fused ? p.N / 2 : p.N;
        const int seg_end = min(t_end, p.tile_begin + (out_cols + 15) / 16);
        const int a = t - p.tile_begin, b = seg_end - p.tile_begin;
        if (PP && (!CANON || p.prepacked)) {
            if (FUSED && p.fused) stream_segment_pp<MB, FUSED, WPB, PASSES, GQ>(p, a, b, smem, staged);
            else stream_segment_pp<MB, false, WPB, PASSES, GQ, VDOT>(p, a, b, smem, staged);
        } else if (CANON) {
            staged.x = nullptr;  // the canonical walk stages in its own order
            if (FUSED && p.fused) stream_segment<MB, FUSED, WPB>(p, a, b, smem);
            else stream_segment<MB, false, WPB>(p, a, b, smem);
        }
        t = seg_end;
    }
}

}  // namespace
