// Measurement helpers for bench.py (a library of their own, libvrl_bench.so: nothing in the product
// path loads it).
//
// vrl_bench_stream_read: what a plain streaming read of a buffer achieves on this device, as the
// reference point for the GEMV kernels' GB/s: every wave walks a contiguous share of the buffer with
// non-temporal 16-byte loads per lane (one contiguous KiB per wave load, four in flight per lane: the
// access shape of the prepacked weight stream), folds what it reads into one word and writes that
// word only if it equals a value the data never produces, so nothing is stored.
//
// vrl_bench_gemv_grouped_valu_dot_bf16: the grouped launch of the product library over a plan it built,
// by the comparison build of its throughput kernel whose dot product runs on the vector unit
// (v_dot2_f32_bf16) instead of the matrix cores.  It is slower and exists to be measured.

#include "stream_kernel.hpp"

namespace {

constexpr int NT = BUFFER_NT;  // cache-policy bit: non-temporal

// each wave reads `per_wave` bytes (a multiple of 4 KiB) from its own offset; waves past the end read
// nothing (the buffer range check answers with zeros)
template <int WPB>
__global__ __launch_bounds__(WPB *WAVE) void stream_read_kernel(const void *buf, uint32_t bytes, uint32_t per_wave,
                                                                uint32_t *sink) {
    const rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(buf), 0, (int)bytes, 0x00020000);
    const uint32_t wave = blockIdx.x * WPB + (threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & (WAVE - 1);
    const uint32_t base = __builtin_amdgcn_readfirstlane(wave * per_wave);
    u32x4_t acc = {0u, 0u, 0u, 0u};
    u32x4_t slot[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) slot[d] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane * 16u + d * 1024u, base, NT);
    for (uint32_t off = 4096; off < per_wave; off += 4096) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            acc ^= slot[d];
            slot[d] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane * 16u + d * 1024u, base + off, NT);
        }
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) acc ^= slot[d];
    const uint32_t folded = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (folded == 0x9E3779B9u && sink) sink[0] = folded;  // never for the benchmark's data; keeps the loads alive
}

}  // namespace

extern "C" {

// Enqueues one streaming read of `bytes` (< 4 GiB, 16-byte aligned buffer) on `hip_stream` with
// `waves_per_cu` waves per compute unit in four-wave workgroups.  Returns 0 or a hipError_t value.
int vrl_bench_stream_read(const void *buf, size_t bytes, void *sink, int waves_per_cu, void *hip_stream) {
    if (!buf || bytes == 0 || bytes >= (1ull << 32) || (reinterpret_cast<uintptr_t>(buf) & 15u)) return 1;
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
    }
    if (waves_per_cu < 4) waves_per_cu = 4;
    const uint32_t waves = (uint32_t)cus * (uint32_t)waves_per_cu / 4u * 4u;
    uint64_t per_wave = (bytes + waves - 1) / waves;
    per_wave = (per_wave + 4095) / 4096 * 4096;
    return vrl_launch(&stream_read_kernel<4>, dim3(waves / 4), dim3(4 * WAVE), 0,
                       reinterpret_cast<hipStream_t>(hip_stream), buf, (uint32_t)bytes, (uint32_t)per_wave,
                       static_cast<uint32_t *>(sink));
}

// One grouped launch over `plan_dev` (the device copy of a plan made by vrl_int4_grouped_plan_build of the
// product library) with the vector-unit dot product.  The plan must be the four-wave throughput form over
// plain prepacked records of group size 128 (variant = prepacked only), and every record must carry one
// activation row: the caller knows the records, this function sees only the descriptor.  Returns 0, a
// VRL_INT4_E* code or a hipError_t value.
int vrl_bench_gemv_grouped_valu_dot_bf16(const void *plan_dev, const vrl_int4_plan_info *info, void *hip_stream) {
    if (!plan_dev || !info) return VRL_INT4_ENULL;
    if (info->variant != VARIANT_PP || info->block_threads != 4 * WAVE || info->n_problems < 1 || info->grid < 1 ||
        info->lds_bytes < 0 || info->lds_bytes > 64 * 1024 || (reinterpret_cast<uintptr_t>(plan_dev) & 15u))
        return VRL_INT4_EPLAN;
    const uint8_t *base = static_cast<const uint8_t *>(plan_dev);
    const DevProblem *recs = reinterpret_cast<const DevProblem *>(base + 16);   // behind the plan's 16-byte header
    const int2 *block_tab = reinterpret_cast<const int2 *>(recs + info->n_problems);
    return vrl_launch(&gemv_stream_kernel<4, 1, false, true, false, false, 1, true>, dim3(info->grid),
                       dim3(4 * WAVE), (size_t)info->lds_bytes, reinterpret_cast<hipStream_t>(hip_stream), recs,
                       block_tab, info->n_problems);
}

}  // extern "C"
