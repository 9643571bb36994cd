// Cross-lane reductions of a 64-lane wave through DPP and readlane: register to register, without the
// trip through the LDS crossbar that __shfl_xor (ds_bpermute) takes.
#pragma once

#include <hip/hip_runtime.h>

namespace {

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}

// A DPP row is 16 lanes: two quad permutes and two mirrors leave every lane of a row with the row's result.
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_move<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_move<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_move<0x141>(v);  // row_half_mirror
    v += dpp_move<0x140>(v);  // row_mirror
    return v;
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));
    v = fmaxf(v, dpp_move<0x4E>(v));
    v = fmaxf(v, dpp_move<0x141>(v));
    v = fmaxf(v, dpp_move<0x140>(v));
    return v;
}
__device__ __forceinline__ float lane_of(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
// the four rows of the wave meet through readlane; every lane returns the wave's result
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    return (lane_of(v, 0) + lane_of(v, 16)) + (lane_of(v, 32) + lane_of(v, 48));
}
// lanes l, l + 16, l + 32, l + 48 added up in that order; lanes 0..15 hold the results
__device__ __forceinline__ float row16_sum_quarters(float v) {
    const float q1 = __shfl_down(v, 16, 64), q2 = __shfl_down(v, 32, 64), q3 = __shfl_down(v, 48, 64);
    return ((v + q1) + q2) + q3;
}
__device__ __forceinline__ float wave_max(float v) {
    v = row16_max(v);
    return fmaxf(fmaxf(lane_of(v, 0), lane_of(v, 16)), fmaxf(lane_of(v, 32), lane_of(v, 48)));
}

}  // namespace
