// LoRA adapter down-projection t = x . A^T, shared by the launch of its own (decode_layer.hip) and by
// the plan-free int4 launch that carries it as extra workgroups (int4_gemv.hip).
//
// Restates the first half of a PEFT wrapper's forward, result = base_layer(x) + lora_B(lora_A(x)) * scaling
// (vrl/models/families/janus_pro/policy.py:298-324 attaches the adapters): lora_A(x) in float32 for float32
// adapter weights, rounded to bf16 (the module's output tensor) for bf16 ones.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/vrl_decode.h"
#include "../../include/vrl_int4.h"
#include "wave_reduce.hpp"

namespace {

constexpr int LORA_MAX_RANK = 64;
constexpr int LORA_MAX_ADAPTERS = 4;
constexpr int LORA_MAX_ROWS = 32;
constexpr int LORA_MAX_TOTAL = 256;
constexpr int LORA_DOWN_WAVES = 4;   // waves that share one column of t
constexpr int LORA_WAVE = 64;

struct LoraArgs {
    vrl_lora_adapter ad[LORA_MAX_ADAPTERS];
    int32_t off[LORA_MAX_ADAPTERS + 1];  // first column of each adapter in t
    int32_t n, M, K;
};

__device__ __forceinline__ float lora_bf16(uint32_t bits) { return __builtin_bit_cast(float, bits << 16); }
__device__ __forceinline__ float lora_round_bf16(float v) {
    return lora_bf16((uint32_t)__builtin_bit_cast(uint16_t, (__bf16)v));
}

// eight consecutive adapter weights (float32 or bf16) as floats
template <bool FP32>
__device__ __forceinline__ void load8(const void *base, long index, float (&f)[8]) {
    if constexpr (FP32) {
        const float4 a = *reinterpret_cast<const float4 *>(static_cast<const float *>(base) + index);
        const float4 b = *reinterpret_cast<const float4 *>(static_cast<const float *>(base) + index + 4);
        f[0] = a.x, f[1] = a.y, f[2] = a.z, f[3] = a.w, f[4] = b.x, f[5] = b.y, f[6] = b.z, f[7] = b.w;
    } else {
        const uint4 w = *reinterpret_cast<const uint4 *>(static_cast<const uint16_t *>(base) + index);
        const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            f[2 * e] = lora_bf16(u[e] & 0xFFFFu);
            f[2 * e + 1] = lora_bf16(u[e] >> 16);
        }
    }
}

// One column of t (an adapter row) for a block of MB activation rows starting at m_lo, by four waves
// (`gw` = 0..3 within the group): they take interleaved 512-value pieces of K; a lane holds 8 values
// of the A row and requests the matching 8 values of all its activation rows at once, then every row's
// partial sum is reduced over the wave and the four waves meet in `part` (LDS, 4 x MB floats of this
// group).  Written without data-dependent branches: rows past the end repeat the last one (clamped
// index), which costs arithmetic but keeps every load of a lane in flight at once.  Every thread of
// the workgroup must call it (it holds a workgroup barrier); groups with `active` false only wait.
// NORMED (K <= 2048: a lane holds one piece of every row): x is a sublayer output and the adapter reads
//   weight * bf16(h * rsqrt(mean(h^2) + eps)),  h = residual ? bf16(x + residual) : x
// instead, the residual add and RMSNorm that precede q|k|v in LlamaDecoderLayer.forward, with the tensor ops'
// roundings: the rows stay in registers while their sums of squares meet in `part`.
struct LoraNorm {
    const uint16_t *residual;  // same shape as x, or nullptr
    const uint16_t *weight;    // [K]
    float eps;
};

template <bool FP32, int MB>
__device__ __forceinline__ void lora_down_item_normed(const uint16_t *x, const LoraArgs &a, const LoraNorm &nrm,
                                                      float *t, bool active, int col, int m_lo, int gw, int lane,
                                                      float *part) {
    const int total = a.off[a.n];
    const int k = (gw * LORA_WAVE + lane) * 8;
    const bool in = active && k < a.K;
    int rows = 0;
    float af[8];
    uint32_t h[MB][4], wv[4];
#pragma unroll
    for (int e = 0; e < 8; ++e) af[e] = 0.0f;
#pragma unroll
    for (int e = 0; e < 4; ++e) wv[e] = 0u;
#pragma unroll
    for (int u = 0; u < MB; ++u)
#pragma unroll
        for (int e = 0; e < 4; ++e) h[u][e] = 0u;
    if (active) {  // uniform over the group's waves
        int i = 0;
#pragma unroll
        for (int q = 1; q < LORA_MAX_ADAPTERS; ++q)
            if (q < a.n && a.off[q] <= col) i = q;
        const void *A = a.ad[0].A;
        int first = 0;
#pragma unroll
        for (int q = 1; q < LORA_MAX_ADAPTERS; ++q)
            if (q == i) A = a.ad[q].A, first = a.off[q];
        rows = min(MB, a.M - m_lo);
        if (in) {
            load8<FP32>(A, (long)(col - first) * a.K + k, af);
            const uint4 w4 = *reinterpret_cast<const uint4 *>(nrm.weight + k);
            wv[0] = w4.x, wv[1] = w4.y, wv[2] = w4.z, wv[3] = w4.w;
            uint4 xr[MB], rr[MB];
#pragma unroll
            for (int u = 0; u < MB; ++u) {
                const long at = (long)(m_lo + (u < rows ? u : rows - 1)) * a.K + k;
                xr[u] = *reinterpret_cast<const uint4 *>(x + at);
                rr[u] = nrm.residual ? *reinterpret_cast<const uint4 *>(nrm.residual + at) : uint4{0u, 0u, 0u, 0u};
            }
            __builtin_amdgcn_sched_barrier(0);  // all requests before the first use
#pragma unroll
            for (int u = 0; u < MB; ++u) {
                const uint32_t xw[4] = {xr[u].x, xr[u].y, xr[u].z, xr[u].w};
                const uint32_t rw[4] = {rr[u].x, rr[u].y, rr[u].z, rr[u].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (nrm.residual) {   // uniform
                        const float lo = lora_round_bf16(lora_bf16(rw[e] & 0xFFFFu) + lora_bf16(xw[e] & 0xFFFFu));
                        const float hi = lora_round_bf16(lora_bf16(rw[e] >> 16) + lora_bf16(xw[e] >> 16));
                        h[u][e] = (__builtin_bit_cast(uint32_t, lo) >> 16) | (__builtin_bit_cast(uint32_t, hi) & 0xFFFF0000u);
                    } else {
                        h[u][e] = xw[e];
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < MB; ++u) {
            float ss = 0.0f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float lo = lora_bf16(h[u][e] & 0xFFFFu), hi = lora_bf16(h[u][e] >> 16);
                ss += lo * lo;
                ss += hi * hi;
            }
            ss = wave_sum(ss);
            if (lane == 0) part[gw * MB + u] = ss;
        }
    }
    __syncthreads();
    float acc[MB];
    if (active) {
        const float inv_k = 1.0f / (float)a.K;
#pragma unroll
        for (int u = 0; u < MB; ++u) {
            float ss = part[u];
#pragma unroll
            for (int w = 1; w < LORA_DOWN_WAVES; ++w) ss += part[w * MB + u];
            const float r = rsqrtf(ss * inv_k + nrm.eps);
            float sum = 0.0f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float lo = lora_round_bf16(lora_bf16(wv[e] & 0xFFFFu) * lora_round_bf16(lora_bf16(h[u][e] & 0xFFFFu) * r));
                const float hi = lora_round_bf16(lora_bf16(wv[e] >> 16) * lora_round_bf16(lora_bf16(h[u][e] >> 16) * r));
                sum += lo * af[2 * e] + hi * af[2 * e + 1];
            }
            acc[u] = sum;
        }
    }
    __syncthreads();  // the sums of squares are read before the partial products take their place
    if (active) {
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const float v = wave_sum(acc[m]);
            if (lane == 0) part[gw * MB + m] = v;
        }
    }
    __syncthreads();
    if (active && gw == 0 && lane < rows) {
        float v = part[lane];
#pragma unroll
        for (int w = 1; w < LORA_DOWN_WAVES; ++w) v += part[w * MB + lane];
        if (!FP32) v = lora_round_bf16(v);  // lora_A's output tensor is bf16 then
        t[(long)(m_lo + lane) * total + col] = v;
    }
}

template <bool FP32, int MB>
__device__ __forceinline__ void lora_down_item(const uint16_t *x, const LoraArgs &a, float *t, bool active,
                                               int col, int m_lo, int gw, int lane, float *part) {
    const int total = a.off[a.n];
    int rows = 0;
    float acc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[m] = 0.0f;
    if (active) {  // uniform over the group's waves
        int i = 0;
#pragma unroll
        for (int k = 1; k < LORA_MAX_ADAPTERS; ++k)
            if (k < a.n && a.off[k] <= col) i = k;
        const void *A = a.ad[0].A;
        int first = 0;
#pragma unroll
        for (int k = 1; k < LORA_MAX_ADAPTERS; ++k)
            if (k == i) A = a.ad[k].A, first = a.off[k];   // scalar selects, no indexing of the argument block
        const long arow = (long)(col - first) * a.K;
        rows = min(MB, a.M - m_lo);
        x += (long)m_lo * a.K;
        for (int k = (gw * LORA_WAVE + lane) * 8; k < a.K; k += LORA_DOWN_WAVES * LORA_WAVE * 8) {
            float af[8];
            load8<FP32>(A, arow + k, af);
            uint4 xr[MB];
#pragma unroll
            for (int u = 0; u < MB; ++u)
                xr[u] = *reinterpret_cast<const uint4 *>(x + (long)(u < rows ? u : rows - 1) * a.K + k);
            __builtin_amdgcn_sched_barrier(0);  // all requests before the first use
#pragma unroll
            for (int u = 0; u < MB; ++u) {
                const uint32_t w[4] = {xr[u].x, xr[u].y, xr[u].z, xr[u].w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    acc[u] += lora_bf16(w[e] & 0xFFFFu) * af[2 * e] + lora_bf16(w[e] >> 16) * af[2 * e + 1];
            }
        }
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const float v = wave_sum(acc[m]);
            if (lane == 0) part[gw * MB + m] = v;
        }
    }
    __syncthreads();
    if (active && gw == 0 && lane < rows) {
        float v = part[lane];
#pragma unroll
        for (int w = 1; w < LORA_DOWN_WAVES; ++w) v += part[w * MB + lane];
        if (!FP32) v = lora_round_bf16(v);  // lora_A's output tensor is bf16 then
        t[(long)(m_lo + lane) * total + col] = v;
    }
}

// A workgroup of NW waves (a multiple of four) as NW / 4 groups: group `grp` takes item
// wg * (NW / 4) + grp of the r_total x row-block items; `smem` holds NW x 16 floats.
template <int NW, bool NORMED = false>
__device__ __forceinline__ void lora_down_workgroup(const uint16_t *x, const LoraArgs &a, float *t, bool fp32,
                                                    int wg, float *smem, const LoraNorm &nrm = LoraNorm{}) {
    static_assert(NW % LORA_DOWN_WAVES == 0, "whole groups of four waves");
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & (LORA_WAVE - 1);
    const int grp = wave / LORA_DOWN_WAVES, gw = wave % LORA_DOWN_WAVES;
    const int total = a.off[a.n];
    const int mb = a.M <= 8 ? 8 : 16;
    const int items = total * ((a.M + mb - 1) / mb);
    const int item = wg * (NW / LORA_DOWN_WAVES) + grp;
    const bool active = item < items;
    const int col = item % total, m_lo = (item / total) * mb;
    float *part = smem + grp * LORA_DOWN_WAVES * 16;
    if constexpr (NORMED) {
        if (mb == 8) {
            if (fp32) lora_down_item_normed<true, 8>(x, a, nrm, t, active, col, m_lo, gw, lane, part);
            else lora_down_item_normed<false, 8>(x, a, nrm, t, active, col, m_lo, gw, lane, part);
        } else {
            if (fp32) lora_down_item_normed<true, 16>(x, a, nrm, t, active, col, m_lo, gw, lane, part);
            else lora_down_item_normed<false, 16>(x, a, nrm, t, active, col, m_lo, gw, lane, part);
        }
        return;
    }
    if (mb == 8) {
        if (fp32) lora_down_item<true, 8>(x, a, t, active, col, m_lo, gw, lane, part);
        else lora_down_item<false, 8>(x, a, t, active, col, m_lo, gw, lane, part);
    } else {
        if (fp32) lora_down_item<true, 16>(x, a, t, active, col, m_lo, gw, lane, part);
        else lora_down_item<false, 16>(x, a, t, active, col, m_lo, gw, lane, part);
    }
}

// workgroups of NW waves that cover every item
inline int lora_down_workgroups(const LoraArgs &a, int nw) {
    const int mb = a.M <= 8 ? 8 : 16;
    const int items = a.off[a.n] * ((a.M + mb - 1) / mb);
    const int per = nw / LORA_DOWN_WAVES;
    return (items + per - 1) / per;
}

inline bool lora_misaligned(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }

// host side: one argument block for the LoRA launches
inline int lora_args(LoraArgs &a, int M, int K, const vrl_lora_adapter *adapters, int n, bool need_y) {
    if (!adapters) return VRL_INT4_ENULL;
    if (n < 1 || n > LORA_MAX_ADAPTERS || M < 1 || M > LORA_MAX_ROWS || K < 8 || K % 8 != 0) return VRL_INT4_ESHAPE;
    a.n = n;
    a.M = M;
    a.K = K;
    a.off[0] = 0;
    for (int i = 0; i < n; ++i) {
        const vrl_lora_adapter &ad = adapters[i];
        if (!ad.A || !ad.B || (need_y && !ad.y)) return VRL_INT4_ENULL;
        if (ad.r < 8 || ad.r % 8 != 0 || ad.r > LORA_MAX_RANK || ad.N < 1) return VRL_INT4_ESHAPE;
        if (lora_misaligned(ad.A, 16) || lora_misaligned(ad.B, 16) || lora_misaligned(ad.y, 2)) return VRL_INT4_EALIGN;
        if ((ad.weights_fp32 != 0) != (adapters[0].weights_fp32 != 0)) return VRL_INT4_ESHAPE;  // one type per launch
        a.ad[i] = ad;
        a.off[i + 1] = a.off[i] + ad.r;
    }
    for (int i = n; i < LORA_MAX_ADAPTERS; ++i) a.off[i + 1] = a.off[n];
    if (a.off[n] > LORA_MAX_TOTAL) return VRL_INT4_ESHAPE;
    return VRL_INT4_OK;
}

}  // namespace
