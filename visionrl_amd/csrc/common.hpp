// Types, constants and bf16 helpers shared by every kernel of the int4 library; the record a kernel works on.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <type_traits>
#include <vector>

#include "../../include/vrl_int4.h"
#include "launch.hpp"
#include "wave_reduce.hpp"

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

}  // namespace
