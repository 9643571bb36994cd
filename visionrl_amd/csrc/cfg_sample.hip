// Tail of an autoregressive decode step after the image-token head, as one kernel:
// classifier-free-guidance combine, softmax, one multinomial draw, log-probability of the draw.
//
// Restates vrl/models/families/janus_pro/policy.py:686-693 with the arithmetic torch applies to
// bf16 tensors there (every tensor op computes in fp32 and rounds its result to bf16):
//   guided  = uncond + w * (cond - uncond)            three roundings
//   probs   = softmax(guided / T)                     division by a host scalar = product with fl(1/T)
//   sampled = multinomial(probs, 1)                   = argmax(probs / q), q ~ Exp(1) drawn by the caller
//                                                       with the call torch.multinomial makes itself
//   lp      = log_softmax(cond / T)[sampled]
// One workgroup per batch row, three passes over the row (maxima, sums, draw).  The kernel is bound
// by instruction issue on the row's one CU, so a row of up to 16384 entries is read once and its
// scaled logits and exponentials stay in registers between the passes; longer (or unaligned) rows
// are walked three times and stay in cache between the walks (6 bytes per vocabulary entry).

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/vrl_int4.h"
#include "launch.hpp"
#include "wave_reduce.hpp"

namespace {

constexpr int THREADS = 1024;
constexpr int WAVE = 64;
constexpr int WAVES = THREADS / WAVE;

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }

// round to nearest even through the hardware conversion (NaN stays NaN): what a torch bf16 kernel stores
__device__ __forceinline__ float round_bf16(float v) {
    return __builtin_bit_cast(float, (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)v) << 16);
}

struct Row {
    const uint16_t *cond;
    const uint16_t *uncond;
    const uint16_t *noise;
};

template <bool MAX>
__device__ __forceinline__ void block_reduce2(float &a, float &b, float (*lds)[WAVES]) {
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    a = MAX ? wave_max(a) : wave_sum(a);
    b = MAX ? wave_max(b) : wave_sum(b);
    __syncthreads();  // the buffer may still be read from the previous reduction
    if (lane == 0) {
        lds[0][wave] = a;
        lds[1][wave] = b;
    }
    __syncthreads();
    a = lds[0][0];
    b = lds[1][0];
#pragma unroll
    for (int k = 1; k < WAVES; ++k) {  // same order in every thread: every thread holds the same result
        a = MAX ? fmaxf(a, lds[0][k]) : a + lds[0][k];
        b = MAX ? fmaxf(b, lds[1][k]) : b + lds[1][k];
    }
}

// VEC = 8: every thread takes 8 consecutive vocabulary entries per step with 16-byte loads, all
// steps of a walk requested before the first is used (V % 8 == 0, 16-byte aligned rows); VEC = 1
// is the form for any V.
template <int VEC>
__device__ __forceinline__ void load_entries(const uint16_t *p, uint16_t (&v)[VEC]) {
    if constexpr (VEC == 8) {
        const uint4 w = *reinterpret_cast<const uint4 *>(p);
        const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[2 * e] = (uint16_t)(u[e] & 0xFFFFu);
            v[2 * e + 1] = (uint16_t)(u[e] >> 16);
        }
    } else {
        v[0] = *p;
    }
}

// guided / T and cond / T of one vocabulary entry (c, u: its two logits), as bf16 values held in floats
__device__ __forceinline__ void scaled_pair(float c, float u, float w, float inv_t, float &gt, float &ct) {
    const float d = round_bf16(c - u);
    const float g = round_bf16(u + round_bf16(w * d));
    gt = round_bf16(g * inv_t);
    ct = round_bf16(c * inv_t);
}

// the better of two draws: the larger ratio, the lower index among equals, a NaN over any number (torch's argmax)
__device__ __forceinline__ void take_better(float &bv, int &bi, float ov, int oi) {
    const bool other_nan = ov != ov, mine_nan = bv != bv;
    const bool take = mine_nan ? (other_nan && oi < bi) : (other_nan || ov > bv || (ov == bv && oi < bi));
    if (take) {
        bv = ov;
        bi = oi;
    }
}

// the workgroup's best draw, then the row's two outputs
__device__ __forceinline__ void finish_row(const Row &r, float bv, int bi, float mc, float sc, float w, float inv_t,
                                           int V, long long *sampled, float *logprob, float *best_v, int *best_i) {
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) take_better(bv, bi, __shfl_xor(bv, off, WAVE), __shfl_xor(bi, off, WAVE));
    if (lane == 0) {
        best_v[wave] = bv;
        best_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int k = 1; k < WAVES; ++k) take_better(bv, bi, best_v[k], best_i[k]);
        if (bi >= V) bi = 0;  // V >= 1, so only if every ratio compared false: cannot happen for finite input
        float gt, ct;
        scaled_pair(bf16_to_f32(r.cond[bi]), bf16_to_f32(r.uncond[bi]), w, inv_t, gt, ct);
        sampled[blockIdx.x] = bi;
        logprob[blockIdx.x] = round_bf16(ct - mc - logf(sc));
    }
}

template <int VEC>
__global__ __launch_bounds__(THREADS) void cfg_sample_kernel(const uint16_t *__restrict__ logits,
                                                             const uint16_t *__restrict__ noise,
                                                             long long *__restrict__ sampled,
                                                             float *__restrict__ logprob, int B, int V,
                                                             float w, float inv_t) {
    __shared__ float red[2][WAVES];
    __shared__ float best_v[WAVES];
    __shared__ int best_i[WAVES];
    const int b = blockIdx.x;
    Row r;
    r.cond = logits + (long)b * V;
    r.uncond = logits + (long)(B + b) * V;
    r.noise = noise + (long)b * V;

    constexpr int STEP = THREADS * VEC;
    // walk 1: maxima of guided / T and of cond / T
    float mg = -INFINITY, mc = -INFINITY;
#pragma unroll 4
    for (int i = threadIdx.x * VEC; i < V; i += STEP) {
        uint16_t cb[VEC], ub[VEC];
        load_entries<VEC>(r.cond + i, cb);
        load_entries<VEC>(r.uncond + i, ub);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float gt, ct;
            scaled_pair(bf16_to_f32(cb[e]), bf16_to_f32(ub[e]), w, inv_t, gt, ct);
            mg = fmaxf(mg, gt);
            mc = fmaxf(mc, ct);
        }
    }
    block_reduce2<true>(mg, mc, red);

    // walk 2: the two softmax denominators
    float sg = 0.0f, sc = 0.0f;
#pragma unroll 4
    for (int i = threadIdx.x * VEC; i < V; i += STEP) {
        uint16_t cb[VEC], ub[VEC];
        load_entries<VEC>(r.cond + i, cb);
        load_entries<VEC>(r.uncond + i, ub);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float gt, ct;
            scaled_pair(bf16_to_f32(cb[e]), bf16_to_f32(ub[e]), w, inv_t, gt, ct);
            sg += expf(gt - mg);
            sc += expf(ct - mc);
        }
    }
    block_reduce2<false>(sg, sc, red);

    // walk 3: argmax of probs / q, lowest index among equal maxima
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
#pragma unroll 4
    for (int i = threadIdx.x * VEC; i < V; i += STEP) {
        uint16_t cb[VEC], ub[VEC], nb[VEC];
        load_entries<VEC>(r.cond + i, cb);
        load_entries<VEC>(r.uncond + i, ub);
        load_entries<VEC>(r.noise + i, nb);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float gt, ct;
            scaled_pair(bf16_to_f32(cb[e]), bf16_to_f32(ub[e]), w, inv_t, gt, ct);
            const float p = round_bf16(expf(gt - mg) / sg);
            const float ratio = round_bf16(p / bf16_to_f32(nb[e]));
            if (ratio > bv || (ratio == bv && i + e < bi) || (ratio != ratio && bv == bv)) {
                bv = ratio;   // a NaN ratio wins over numbers, as in torch's argmax
                bi = i + e;
            }
        }
    }
    finish_row(r, bv, bi, mc, sc, w, inv_t, V, sampled, logprob, best_v, best_i);
}

// Rows of at most STEPS * 8192 entries (V % 8 == 0, 16-byte aligned): every thread reads its 8 * STEPS
// entries once; same arithmetic and the same order of sums as the walking kernel.
template <int STEPS>
__global__ __launch_bounds__(THREADS) void cfg_sample_resident_kernel(const uint16_t *__restrict__ logits,
                                                                      const uint16_t *__restrict__ noise,
                                                                      long long *__restrict__ sampled,
                                                                      float *__restrict__ logprob, int B, int V,
                                                                      float w, float inv_t) {
    __shared__ float red[2][WAVES];
    __shared__ float best_v[WAVES];
    __shared__ int best_i[WAVES];
    const int b = blockIdx.x;
    Row r;
    r.cond = logits + (long)b * V;
    r.uncond = logits + (long)(B + b) * V;
    r.noise = noise + (long)b * V;
    constexpr int N = 8 * STEPS;
    uint16_t cb[STEPS][8], ub[STEPS][8], nb[STEPS][8];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {   // entries past the end repeat the thread's first in-range ones, uncounted
        const int i = (s * THREADS + threadIdx.x) * 8;
        const int ii = i < V ? i : 0;
        load_entries<8>(r.cond + ii, cb[s]);
        load_entries<8>(r.uncond + ii, ub[s]);
        load_entries<8>(r.noise + ii, nb[s]);
    }
    float gt[N], ct[N];
    float mg = -INFINITY, mc = -INFINITY;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        const bool in = (s * THREADS + threadIdx.x) * 8 < V;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            scaled_pair(bf16_to_f32(cb[s][e]), bf16_to_f32(ub[s][e]), w, inv_t, gt[8 * s + e], ct[8 * s + e]);
            mg = fmaxf(mg, in ? gt[8 * s + e] : -INFINITY);
            mc = fmaxf(mc, in ? ct[8 * s + e] : -INFINITY);
        }
    }
    block_reduce2<true>(mg, mc, red);
    float sg = 0.0f, sc = 0.0f;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        const bool in = (s * THREADS + threadIdx.x) * 8 < V;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            gt[8 * s + e] = expf(gt[8 * s + e] - mg);   // kept for the draw
            const float ec = expf(ct[8 * s + e] - mc);
            if (in) {
                sg += gt[8 * s + e];
                sc += ec;
            }
        }
    }
    block_reduce2<false>(sg, sc, red);
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        const int i = (s * THREADS + threadIdx.x) * 8;
        if (i < V) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float p = round_bf16(gt[8 * s + e] / sg);
                const float ratio = round_bf16(p / bf16_to_f32(nb[s][e]));
                if (ratio > bv || (ratio == bv && i + e < bi) || (ratio != ratio && bv == bv)) {
                    bv = ratio;
                    bi = i + e;
                }
            }
        }
    }
    finish_row(r, bv, bi, mc, sc, w, inv_t, V, sampled, logprob, best_v, best_i);
}

}  // namespace

extern "C" int vrl_cfg_sample_bf16(const void *logits, const void *noise, int64_t *sampled, float *logprob,
                                   int B, int V, float cfg_weight, float temperature, void *hip_stream) {
    if (!logits || !noise || !sampled || !logprob) return VRL_INT4_ENULL;
    if (B < 1 || V < 1 || B > (1 << 20) || (long)B * V >= (1L << 40) || !(temperature > 0.0f)) return VRL_INT4_ESHAPE;
    if ((reinterpret_cast<uintptr_t>(logits) & 1u) || (reinterpret_cast<uintptr_t>(noise) & 1u) ||
        (reinterpret_cast<uintptr_t>(sampled) & 7u) || (reinterpret_cast<uintptr_t>(logprob) & 3u))
        return VRL_INT4_EALIGN;
    const bool wide = V % 8 == 0 && ((reinterpret_cast<uintptr_t>(logits) | reinterpret_cast<uintptr_t>(noise)) & 15u) == 0;
    auto kernel = !wide ? &cfg_sample_kernel<1>
                  : V <= THREADS * 8 ? &cfg_sample_resident_kernel<1>
                  : V <= THREADS * 16 ? &cfg_sample_resident_kernel<2>
                                      : &cfg_sample_kernel<8>;
    return vrl_launch(kernel, dim3(B), dim3(THREADS), 0, reinterpret_cast<hipStream_t>(hip_stream),
                       static_cast<const uint16_t *>(logits), static_cast<const uint16_t *>(noise),
                       reinterpret_cast<long long *>(sampled), logprob, B, V, cfg_weight, 1.0f / temperature);
}
