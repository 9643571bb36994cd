// The parts of a Llama decoder layer between its linears, for one new token per row:
// residual add + RMSNorm, and rotary embedding + cache append + attention over a static cache.
//
// Restates, with the roundings torch applies to bf16 tensors (each tensor op computes in fp32
// and rounds its result to bf16), what the trunk call of a decode step runs between the
// projections (vrl/models/families/janus_pro/policy.py:673-678 -> transformers LlamaDecoderLayer.forward,
// LlamaRMSNorm.forward, apply_rotary_pos_emb, StaticLayer.update, sdpa_attention_forward):
//   h = bf16(residual + x);  normed = bf16(weight * bf16(h * rsqrt(mean(h^2) + eps)))
//   q' = bf16(bf16(q * cos) + bf16(rotate_half(q) * sin)), same for k
//   cache[p] = k', v;  out = bf16(softmax(q' . K^T * scaling, masked slots out) . V)
// The attention keeps scores, probabilities and a running softmax in fp32 (the library kernel it
// stands for rounds the probabilities to bf16 before the second product), so it agrees with it to
// a bf16 rounding of the output, not bit for bit.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include "../../include/vrl_decode.h"
#include "../../include/vrl_int4.h"
#include "launch.hpp"
#include "lora.hpp"
#include "wave_reduce.hpp"

// The split form of the attention hands partial results from workgroup to workgroup through device-scope
// stores, a wait on the store counter and a relaxed counter increment (see the comment at the hand-over):
// an argument about this architecture's caches, not one the language's memory model makes for every target.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "decode_layer.hip: the split attention's hand-over is written for gfx950; revisit it before building for another target"
#endif

namespace {

constexpr int WAVE = 64;
constexpr int THREADS = 256;
constexpr int WAVES = THREADS / WAVE;
constexpr int MAX_NORM_K = 16384;
constexpr int MAX_CACHE_LEN = 8192;

__device__ __forceinline__ float bf16_to_f32(uint32_t bits) { return __builtin_bit_cast(float, bits << 16); }

// round to nearest even through the hardware conversion, value kept in a float
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float v) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)v);
}
__device__ __forceinline__ float round_bf16(float v) { return bf16_to_f32(f32_to_bf16_bits(v)); }

// every thread returns the block's total; `red` holds WAVES floats and is free for reuse afterwards
template <bool MAX>
__device__ __forceinline__ float block_reduce(float v, float *red) {
    v = MAX ? wave_max(v) : wave_sum(v);
    __syncthreads();  // earlier readers of red are done
    if ((threadIdx.x & (WAVE - 1)) == 0) red[threadIdx.x / WAVE] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int k = 1; k < WAVES; ++k) r = MAX ? fmaxf(r, red[k]) : r + red[k];
    return r;
}

// ---------------------------------------------------------------- residual add + RMSNorm
template <bool ADD>
__global__ __launch_bounds__(THREADS) void add_rmsnorm_kernel(const uint16_t *x, const uint16_t *residual,
                                                              const uint16_t *__restrict__ weight,
                                                              uint16_t *h_out, uint16_t *__restrict__ y,
                                                              int K, float eps) {
    extern __shared__ __align__(16) uint16_t hs[];  // the row after the add, K values
    __shared__ float red[WAVES];
    const long row = (long)blockIdx.x * K;
    float ss = 0.0f;
    for (int i = threadIdx.x * 8; i < K; i += THREADS * 8) {
        uint4 xv = *reinterpret_cast<const uint4 *>(x + row + i);
        if (ADD) {
            const uint4 rv = *reinterpret_cast<const uint4 *>(residual + row + i);
            const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w}, rw[4] = {rv.x, rv.y, rv.z, rv.w};
            uint32_t hw[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t lo = f32_to_bf16_bits(bf16_to_f32(rw[e] & 0xFFFFu) + bf16_to_f32(xw[e] & 0xFFFFu));
                const uint32_t hi = f32_to_bf16_bits(bf16_to_f32(rw[e] >> 16) + bf16_to_f32(xw[e] >> 16));
                hw[e] = lo | (hi << 16);
            }
            xv = make_uint4(hw[0], hw[1], hw[2], hw[3]);
        }
        const uint32_t w4[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float lo = bf16_to_f32(w4[e] & 0xFFFFu), hi = bf16_to_f32(w4[e] >> 16);
            ss += lo * lo;
            ss += hi * hi;
        }
        *reinterpret_cast<uint4 *>(hs + i) = xv;
        if (h_out) *reinterpret_cast<uint4 *>(h_out + row + i) = xv;
    }
    const float total = block_reduce<false>(ss, red);
    const float r = rsqrtf(total * (1.0f / (float)K) + eps);  // mean as sum * (1/K), as the tensor op does
    for (int i = threadIdx.x * 8; i < K; i += THREADS * 8) {  // every thread reads back what it wrote
        const uint4 hv = *reinterpret_cast<const uint4 *>(hs + i);
        const uint4 wv = *reinterpret_cast<const uint4 *>(weight + i);
        const uint32_t h4[4] = {hv.x, hv.y, hv.z, hv.w}, w4[4] = {wv.x, wv.y, wv.z, wv.w};
        uint32_t o4[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float lo = round_bf16(bf16_to_f32(h4[e] & 0xFFFFu) * r);
            const float hi = round_bf16(bf16_to_f32(h4[e] >> 16) * r);
            o4[e] = f32_to_bf16_bits(bf16_to_f32(w4[e] & 0xFFFFu) * lo) |
                    (f32_to_bf16_bits(bf16_to_f32(w4[e] >> 16) * hi) << 16);
        }
        *reinterpret_cast<uint4 *>(y + row + i) = make_uint4(o4[0], o4[1], o4[2], o4[3]);
    }
}

// ---------------------------------------------------------------- rotary + cache append + attention
constexpr int ATTN_MAX_SPLITS = 8;   // workgroups that share the cached slots of one (row, head) in the split form
// A row with fewer cached slots than this is left to the first workgroup of each of its pairs by a split launch
// (the exchange of the split form costs more than it saves there: a decode step at 2 rows takes 0.82 against
// 0.85 ms at 450 slots, 0.86 against 0.86 at 530, 0.91 against 0.86 at 610).
constexpr int ATTN_SPLIT_FROM = 512;
// ... and with two workgroups per pair (65 to 128 pairs: half the compute units are busy without it) from 768:
// a decode step at 8 rows takes 1.07 against 1.03 ms at 580 slots and 1.10 against 1.11 ms at 810.
constexpr int ATTN_SPLIT_FROM_TWO = 768;

struct AttnArgs {
    const uint16_t *q, *k, *v;
    uint16_t *k_cache, *v_cache;
    const uint16_t *cos, *sin;
    const uint8_t *mask;
    const long long *position;
    int position_stride;     // 0: one position for every row; 1: position[m] is row m's
    uint16_t *out;
    int q_stride, kv_stride;
    int n_heads, n_kv_heads, L_max;
    float scaling;
    // adapters whose up-projection is added while q, k, v are read (LORA instantiations only)
    const float *t;          // [M, t_stride] down-projections
    int t_stride;
    const void *lb[3];       // B [N, r] of the q, k, v adapter, nullptr for none
    int lr[3], loff[3];      // rank, first column in t
    float lscale[3];
    // adapter on the projection that consumes `out`: this head's share of out . A^T goes to ot
    const void *oa;          // A [orank, n_heads * D], nullptr for none
    float *ot;               // [M, n_heads, orank]
    int orank;
    // SPLIT instantiations: the cached slots of a (row, head) are divided over gridDim.z workgroups
    uint32_t *arrived;       // [M, n_heads] counters, zero between launches
    float *partials;         // [M, n_heads, gridDim.z, D + 2]: unnormalised output, maximum, sum
};

// Raw cache vectors: D / 16 bf16 values of one slot per lane (16 or 8 bytes).
template <int VEC>
struct RawVec {
    uint32_t w[VEC / 2];
};

// NT: a non-temporal load (the line is not kept in the caches).  A cache that is larger than the
// memory-side cache is streamed once per step and layer, and keeping its lines only evicts what
// could stay: measured -6 % on a decode step at 32 rows (86 MB of keys and values per layer).  The
// caches of one image (6 MB per layer at 2 rows, all layers together within the memory-side cache's
// 256 MB) stay there from step to step, and plain loads are 4 % faster.  The host picks by the bytes
// one layer's caches hold.
template <int VEC, bool NT>
__device__ __forceinline__ RawVec<VEC> load_raw(const uint16_t *p) {
    typedef __attribute__((ext_vector_type(4))) uint32_t raw_u32x4;
    typedef __attribute__((ext_vector_type(2))) uint32_t raw_u32x2;
    RawVec<VEC> r;
    if constexpr (VEC == 8) {
        const raw_u32x4 *q = reinterpret_cast<const raw_u32x4 *>(p);
        const raw_u32x4 v = NT ? __builtin_nontemporal_load(q) : *q;
        r.w[0] = v[0], r.w[1] = v[1], r.w[2] = v[2], r.w[3] = v[3];
    } else {
        const raw_u32x2 *q = reinterpret_cast<const raw_u32x2 *>(p);
        const raw_u32x2 v = NT ? __builtin_nontemporal_load(q) : *q;
        r.w[0] = v[0], r.w[1] = v[1];
    }
    return r;
}

// Running softmax state of a set of slots: their maximum score m, sum of exp(score - m), and
// the exp-weighted sum of value rows (the lane's VEC columns of it).
template <int VEC>
struct Partial {
    float m, l, acc[VEC];
};

template <int VEC>
__device__ __forceinline__ void merge(Partial<VEC> &a, float m2, float l2, const float (&acc2)[VEC]) {
    const float m = fmaxf(a.m, m2);
    const float ref = m == -INFINITY ? 0.0f : m;  // both empty: keep zeros, avoid inf - inf
    const float c1 = __expf(a.m - ref), c2 = __expf(m2 - ref);
    a.m = m;
    a.l = a.l * c1 + l2 * c2;
#pragma unroll
    for (int i = 0; i < VEC; ++i) a.acc[i] = a.acc[i] * c1 + acc2[i] * c2;
}


// One workgroup of ATT_WAVES waves per (head, row): 16 when there are few workgroups (each should
// keep many requests in flight), 8 when there are at least two per CU (several then share a CU
// and overlap each other's prologue and epilogue).  Sixteen lanes share a cache slot (D / 16 values
// each), so a wave reads four consecutive slots (4 * D * 2 bytes, contiguous) per load and the
// workgroup 64.  Every 16-lane group keeps its own running softmax over the slots it visits
// (key and value loads of ATT_UNROLL slots are issued together: values do not wait for scores);
// the groups, the waves and the new token's own slot are merged at the end.
// ATT_UNROLL: slots per 16-lane group in flight (keys and values: 2 * ATT_UNROLL vector loads per lane)
// LORA: 0 none, 1 float32 adapter weights, 2 bf16 adapter weights
// SPLIT: with few (row, head) pairs a workgroup's compute unit becomes the limit (its vector memory path
// moves 64 bytes per cycle: 128 KB of keys and values per 256 slots take 2.9 us, and a cache of 830
// slots four such trips), so gridDim.z workgroups share the slots of a pair, a contiguous range each.
// Each leaves its running softmax state (unnormalised output, maximum, sum) in `partials` and counts
// itself in `arrived`; whichever counts last merges the states in index order (the same sums
// whatever the order of arrival), writes the output and clears the counter.  Nobody waits for anybody.
// The states and the counter are exchanged through device-scope atomic stores, loads and adds (they
// bypass the per-XCD caches), and a workgroup counts itself only when its stores have completed, so
// no cache write-back or invalidate is needed.
template <int D, int ATT_WAVES, int ATT_UNROLL, int LORA, bool STREAMED, bool SPLIT = false>
__global__ __launch_bounds__(ATT_WAVES *WAVE) void rope_attn_decode_kernel(AttnArgs a) {
    static_assert(!SPLIT || LORA == 0, "the split form carries no adapters");
    constexpr int VEC = D / 16;
    __shared__ float qs[D];                 // rotated query
    __shared__ float ks[D];                 // rotated key of the new token
    __shared__ float vs[D];                 // value of the new token
    __shared__ float pm[ATT_WAVES], pl[ATT_WAVES];
    __shared__ float pacc[ATT_WAVES][D];
    __shared__ float s_new;                 // score of the new token's own slot
    __shared__ uint32_t s_before;           // SPLIT: workgroups of the pair that had arrived before this one

    const int h = blockIdx.x, m = blockIdx.y;
    const int group = a.n_heads / a.n_kv_heads;
    const int hk = h / group;
    const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE;
    const int sub = lane >> 4, l16 = lane & 15;
    const long cache_base = ((long)m * a.n_kv_heads + hk) * a.L_max * D;
    const uint8_t *mask = a.mask + (long)m * a.L_max;
    const uint16_t *kc = a.k_cache + cache_base + l16 * VEC;
    const uint16_t *vc = a.v_cache + cache_base + l16 * VEC;
    constexpr int STEP = 4 * ATT_WAVES * ATT_UNROLL;  // slots the workgroup visits per batch
    RawVec<VEC> kraw[ATT_UNROLL], vraw[ATT_UNROLL];
    // Whether a slot counts: its flag computed where the slot is requested (the compiler then waits there for the
    // mask byte, and with it for every load issued before: one round trip per slot of a batch), or the mask bytes
    // kept as loaded until the batch is used (MASK_LATE: one round trip per batch).  Per launch, from HIP graphs of
    // 24: 16.9 -> 16.3 us for the 8-wave workgroups of 32 rows and 9.3 -> 8.9 us in the split form, but 7.0 ->
    // 7.5 us for the 16-wave one-workgroup form at 2 rows and 8.5 -> 9.0 us at 8, which keeps the early flags.
    constexpr bool MASK_LATE = SPLIT || ATT_WAVES < 16;
    bool live[ATT_UNROLL];
    uint8_t mraw[ATT_UNROLL];
    // the workgroup's share of the cached slots 0..p-1: all of them, or the z-th of gridDim.z ranges of a
    // multiple of 64 slots (what the workgroup's waves visit together).  A split launch over a cache that is
    // still short (fewer than ATTN_SPLIT_FROM slots filled, ATTN_SPLIT_FROM_TWO with two workgroups per pair: the launch is captured once for a whole
    // generation, which begins short) leaves a pair to its first workgroup: `whole`.
    const int n_split = SPLIT ? (int)gridDim.z : 1, split = SPLIT ? (int)blockIdx.z : 0;
    const long long p64 = a.position[(long)m * a.position_stride];
    int p = 0, j_lo = 0, j_hi = 0;
    bool whole = !SPLIT;
    auto slot_range = [&]() {   // needs p64
        p = (int)p64;
        whole = !SPLIT || p < (n_split > 2 ? ATTN_SPLIT_FROM : ATTN_SPLIT_FROM_TWO);
        const int share = whole ? p : ((p + n_split - 1) / n_split + 4 * ATT_WAVES - 1) / (4 * ATT_WAVES) * (4 * ATT_WAVES);
        j_lo = min(p, split * share);
        j_hi = min(p, j_lo + share);
    };
    auto request = [&](int j0) {  // slot j0 + u * 4 * ATT_WAVES + wave * 4 + sub for u = 0..ATT_UNROLL-1; needs j_hi > j_lo
#pragma unroll
        for (int u = 0; u < ATT_UNROLL; ++u) {
            const int j = j0 + u * 4 * ATT_WAVES + wave * 4 + sub;
            const int jj = j < j_hi ? j : j_hi - 1;  // slots past the end repeat the last one and are not counted
            // SPLIT: a range is often shorter than a batch, and a whole group of slots past its end (uniform) asks
            // for nothing (8.9 -> 8.6 us per launch at 600 slots; the other builds measure slower with the branch)
            if (!SPLIT || j0 + u * 4 * ATT_WAVES < j_hi) {
                kraw[u] = load_raw<VEC, STREAMED>(kc + (long)jj * D);
                vraw[u] = load_raw<VEC, STREAMED>(vc + (long)jj * D);
                if constexpr (MASK_LATE) mraw[u] = mask[jj];
                else live[u] = j < j_hi && mask[jj] != 0;
            } else {
#pragma unroll
                for (int i = 0; i < VEC / 2; ++i) kraw[u].w[i] = vraw[u].w[i] = 0u;
                mraw[u] = 0;
            }
        }
    };
    // The cached slots do not depend on the new token: the first batch of keys and values is
    // requested before anything else and arrives while the query is rotated.  A pair's first (or only)
    // workgroup begins at slot 0 wherever the row stands: which slots its first batch visits does not depend
    // on the position, only how many of them count, and neither do the new token's query, key and value, so
    // all are requested before the position is looked at (it comes from memory, and what waited for it
    // would start a round trip later); the slots at or past the range's end are dropped before the batch
    // is used.
    const bool ahead = split == 0;   // uniform
    if (ahead) {
#pragma unroll
        for (int u = 0; u < ATT_UNROLL; ++u) {
            const int j = u * 4 * ATT_WAVES + wave * 4 + sub;
            const int jj = j < a.L_max ? j : a.L_max - 1;
            kraw[u] = load_raw<VEC, STREAMED>(kc + (long)jj * D);
            vraw[u] = load_raw<VEC, STREAMED>(vc + (long)jj * D);
            if constexpr (MASK_LATE) mraw[u] = mask[jj];
            else live[u] = mask[jj] != 0;
        }
    } else {
        if (p64 < 0 || p64 >= a.L_max) return;  // uniform over the workgroups of the row
        slot_range();
        if (whole) return;                      // the pair's first workgroup has it all
        if (j_hi > j_lo) request(j_lo);
    }

    // The adapter of the projection that follows: thread (j, l16) holds the lane's VEC columns of row j
    // of A (rows j, j + OJ, ... if the rank exceeds OJ; the first is requested here, ahead of its use).
    constexpr int OJ = ATT_WAVES * WAVE / 16;
    const int oj = tid >> 4;
    float oaw[VEC];
    auto request_oa = [&](int j) {
        const long at = (long)j * a.n_heads * D + (long)h * D + l16 * VEC;
        if constexpr (VEC == 8) {
            load8<LORA == 1>(a.oa, at, oaw);
        } else if constexpr (LORA == 1) {
            const float4 w4 = *reinterpret_cast<const float4 *>(static_cast<const float *>(a.oa) + at);
            oaw[0] = w4.x, oaw[1] = w4.y, oaw[2] = w4.z, oaw[3] = w4.w;
        } else {
            const uint2 w2 = *reinterpret_cast<const uint2 *>(static_cast<const uint16_t *>(a.oa) + at);
            oaw[0] = bf16_to_f32(w2.x & 0xFFFFu), oaw[1] = bf16_to_f32(w2.x >> 16);
            oaw[2] = bf16_to_f32(w2.y & 0xFFFFu), oaw[3] = bf16_to_f32(w2.y >> 16);
        }
    };
    if constexpr (LORA != 0) {
        if (a.oa && oj < a.orank) request_oa(oj);
    }

    if constexpr (LORA != 0) {
        // q, k, v of this head with their adapters added: base + scaling * sum_j t[j] * B[n, j] with the
        // roundings of the adapter wrapper's forward (what the projection's output would hold after an
        // up-projection launch).  Consecutive threads take consecutive pieces of eight ranks: the ranks of a
        // column are contiguous in B and so are the columns of a head, so a wave's request covers whole cache
        // lines (one thread per column, each reading its own row of B, asked for 64 lines per instruction:
        // 21.7 against 20.2 us per launch at 32 rows, where several workgroups share a CU's L1).  The requests of the three projections are independent: one memory round
        // trip; the pieces of a column meet in LDS in a fixed order, and the values go on through LDS because
        // the rotation pairs columns.
        constexpr bool FP32 = LORA == 1;
        constexpr int NT = ATT_WAVES * WAVE;
        constexpr int NC = LORA_MAX_RANK / 8;   // pieces of a column at most
        __shared__ float lpart[3][NC][D];
        const float *trow = a.t + (long)m * a.t_stride;
        const long nbase[3] = {(long)h * D, (long)hk * D, (long)hk * D};
        float base3[3] = {0.0f, 0.0f, 0.0f};
        if (tid < D) {
            base3[0] = bf16_to_f32(a.q[(long)m * a.q_stride + nbase[0] + tid]);
            base3[1] = bf16_to_f32(a.k[(long)m * a.kv_stride + nbase[1] + tid]);
            base3[2] = bf16_to_f32(a.v[(long)m * a.kv_stride + nbase[2] + tid]);
        }
        {
            float bw[3][8], tw[3][8];
            int col3[3], jc3[3];
            bool on[3];
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                const int cpr = a.lb[i] ? a.lr[i] >> 3 : 0;   // uniform
                on[i] = tid < D * cpr;
                col3[i] = on[i] ? tid / cpr : 0;
                jc3[i] = on[i] ? tid - col3[i] * cpr : 0;
                if (on[i]) {
                    load8<FP32>(a.lb[i], (nbase[i] + col3[i]) * a.lr[i] + jc3[i] * 8, bw[i]);
                    load8<true>(trow, a.loff[i] + jc3[i] * 8, tw[i]);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) bw[i][e] = tw[i][e] = 0.0f;
                }
            }
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                float u = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) u += tw[i][e] * bw[i][e];
                if (on[i]) lpart[i][jc3[i]][col3[i]] = u;
            }
        }
        for (int i = 0; i < 3; ++i) {   // what one trip of the workgroup did not reach (ranks beyond 32 with eight waves)
            const int cpr = a.lb[i] ? a.lr[i] >> 3 : 0;
            for (int c = tid + NT; c < D * cpr; c += NT) {
                const int col = c / cpr, jc = c - col * cpr;
                float bw[8], tw[8];
                load8<FP32>(a.lb[i], (nbase[i] + col) * a.lr[i] + jc * 8, bw);
                load8<true>(trow, a.loff[i] + jc * 8, tw);
                float u = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) u += tw[e] * bw[e];
                lpart[i][jc][col] = u;
            }
        }
        __syncthreads();
        if (tid < D) {
            float fixed[3];
#pragma unroll
            for (int i = 0; i < 3; ++i) {
                const int cpr = a.lb[i] ? a.lr[i] >> 3 : 0;
                float u = 0.0f;
                for (int jc = 0; jc < cpr; ++jc) u += lpart[i][jc][tid];
                const float delta = FP32 ? u * a.lscale[i] : round_bf16(round_bf16(u) * a.lscale[i]);
                fixed[i] = a.lb[i] ? round_bf16(base3[i] + delta) : base3[i];
            }
            qs[tid] = fixed[0];
            ks[tid] = fixed[1];
            vs[tid] = fixed[2];
        }
        __syncthreads();
    }
    float q_own = 0.0f, q_pair = 0.0f, k_own = 0.0f, k_pair = 0.0f, v_own = 0.0f;
    if (tid < D) {
        const int partner = tid < D / 2 ? tid + D / 2 : tid - D / 2;
        if constexpr (LORA != 0) {
            q_own = qs[tid], q_pair = qs[partner], k_own = ks[tid], k_pair = ks[partner], v_own = vs[tid];
        } else {
            const uint16_t *qrow = a.q + (long)m * a.q_stride + h * D;
            const uint16_t *krow = a.k + (long)m * a.kv_stride + hk * D;
            q_own = bf16_to_f32(qrow[tid]), q_pair = bf16_to_f32(qrow[partner]);
            k_own = bf16_to_f32(krow[tid]), k_pair = bf16_to_f32(krow[partner]);
            v_own = bf16_to_f32(a.v[(long)m * a.kv_stride + hk * D + tid]);
        }
    }
    if constexpr (LORA != 0) __syncthreads();  // everyone has read its pair before the rotated values go in
    if (ahead) {
        if (p64 < 0 || p64 >= a.L_max) return;  // uniform over the workgroups of the row
        slot_range();
    }
    if (tid < D) {
        const float sign = tid < D / 2 ? -1.0f : 1.0f;  // rotate_half: (-x2, x1)
        const float c = bf16_to_f32(a.cos[(long)p * D + tid]), s = bf16_to_f32(a.sin[(long)p * D + tid]);
        const float qe = round_bf16(round_bf16(q_own * c) + round_bf16(sign * q_pair * s));
        const float ke = round_bf16(round_bf16(k_own * c) + round_bf16(sign * k_pair * s));
        qs[tid] = qe;
        ks[tid] = ke;
        vs[tid] = v_own;
        if (h % group == 0 && split == 0) {  // one workgroup per kv head appends; readers of slot p use their own copy
            a.k_cache[cache_base + (long)p * D + tid] = (uint16_t)f32_to_bf16_bits(ke);
            a.v_cache[cache_base + (long)p * D + tid] = (uint16_t)f32_to_bf16_bits(v_own);
        }
    }
    __syncthreads();

    // the lane's VEC values of the rotated query as bf16 pairs (exact: they are bf16 values), so that a
    // key word needs no conversion: v_dot2_f32_bf16 takes two products per instruction
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
    bf16x2_t qpair[VEC / 2];
#pragma unroll
    for (int i = 0; i < VEC / 2; ++i) {
        const uint32_t bits = f32_to_bf16_bits(qs[l16 * VEC + 2 * i]) | (f32_to_bf16_bits(qs[l16 * VEC + 2 * i + 1]) << 16);
        qpair[i] = __builtin_bit_cast(bf16x2_t, bits);
    }
    if (wave == 0) {  // the new token's own slot
        float dot = 0.0f;
        for (int d = lane; d < D; d += WAVE) dot += qs[d] * ks[d];
        dot = wave_sum(dot);
        if (lane == 0) s_new = (mask[p] && split == 0) ? dot * a.scaling : -INFINITY;  // one workgroup of a pair counts it
    }

    if (ahead) {
        // a slot at or past the range's end may hold anything (also what is not a number): it gets weight
        // zero below, and zeros in place of its values keep 0 * value at zero
#pragma unroll
        for (int u = 0; u < ATT_UNROLL; ++u) {
            const bool inside = u * 4 * ATT_WAVES + wave * 4 + sub < j_hi;
            if constexpr (!MASK_LATE) live[u] = live[u] && inside;
#pragma unroll
            for (int i = 0; i < VEC / 2; ++i) {
                kraw[u].w[i] = inside ? kraw[u].w[i] : 0u;
                vraw[u].w[i] = inside ? vraw[u].w[i] : 0u;
            }
        }
    }
    Partial<VEC> st;
    st.m = -INFINITY;
    st.l = 0.0f;
#pragma unroll
    for (int i = 0; i < VEC; ++i) st.acc[i] = 0.0f;

    // cached slots 0..p-1, a batch per trip; the batch of the first trip is already on its way.
    // The running softmax is rescaled once per batch: one maximum over the batch's scores and the
    // state, one exponential per score and one for the state.
    for (int j0 = j_lo; j0 < j_hi; j0 += STEP) {
        if (j0 > j_lo) request(j0);
        float sc[ATT_UNROLL];
        float mx = st.m;
#pragma unroll
        for (int u = 0; u < ATT_UNROLL; ++u) {
            float dot = 0.0f;
#pragma unroll
            for (int i = 0; i < VEC / 2; ++i)
                dot = __builtin_amdgcn_fdot2_f32_bf16(qpair[i], __builtin_bit_cast(bf16x2_t, kraw[u].w[i]), dot, false);
            dot = row16_sum(dot);  // the sixteen lanes that share the slot
            const bool counts = MASK_LATE ? (j0 + u * 4 * ATT_WAVES + wave * 4 + sub < j_hi) & (mraw[u] != 0) : live[u];
            sc[u] = counts ? dot * a.scaling : -INFINITY;
            mx = fmaxf(mx, sc[u]);
        }
        const float ref = mx == -INFINITY ? 0.0f : mx;  // nothing attendable yet: keep zeros, avoid inf - inf
        const float c0 = __expf(st.m - ref);
        st.m = mx;
        st.l *= c0;
#pragma unroll
        for (int i = 0; i < VEC; ++i) st.acc[i] *= c0;
#pragma unroll
        for (int u = 0; u < ATT_UNROLL; ++u) {
            const float w = __expf(sc[u] - ref);
            st.l += w;
#pragma unroll
            for (int i = 0; i < VEC / 2; ++i) {
                st.acc[2 * i] += w * bf16_to_f32(vraw[u].w[i] & 0xFFFFu);
                st.acc[2 * i + 1] += w * bf16_to_f32(vraw[u].w[i] >> 16);
            }
        }
    }
    // the four 16-lane groups of the wave
#pragma unroll
    for (int off = 16; off <= 32; off <<= 1) {
        const float m2 = __shfl_xor(st.m, off, WAVE), l2 = __shfl_xor(st.l, off, WAVE);
        float acc2[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc2[i] = __shfl_xor(st.acc[i], off, WAVE);
        merge<VEC>(st, m2, l2, acc2);
    }
    if (sub == 0) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) pacc[wave][l16 * VEC + i] = st.acc[i];
    }
    if (lane == 0) {
        pm[wave] = st.m;
        pl[wave] = st.l;
    }
    __syncthreads();
    if (tid < D) {
        float mx = s_new;
#pragma unroll
        for (int w = 0; w < ATT_WAVES; ++w) mx = fmaxf(mx, pm[w]);
        float o = 0.0f, sum = 0.0f;
        if (mx != -INFINITY) {  // else every slot is masked: the output is zero
            const float cn = __expf(s_new - mx);
            o = cn * vs[tid];
            sum = cn;
#pragma unroll
            for (int w = 0; w < ATT_WAVES; ++w) {
                const float c = __expf(pm[w] - mx);
                o += c * pacc[w][tid];
                sum += c * pl[w];
            }
            if (whole) o /= sum;
        }
        if (!whole) {
            // this workgroup's state: o and sum relative to mx (zeros and -inf if it saw nothing attendable)
            float *mine = a.partials + (((long)m * a.n_heads + h) * n_split + split) * (D + 2);
            __hip_atomic_store(mine + tid, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (tid == 0) {
                __hip_atomic_store(mine + D, mx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(mine + D + 1, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            // Ordering of the hand-over, stated at the level it rests on (the gfx950 memory system, which the
            // guard at the top of this file pins): the state goes out as device-scope stores, which are written
            // through to the level every compute die shares; s_waitcnt vmcnt(0) returns when they have been
            // acknowledged there, so the counter increment below, issued after it, is performed after the
            // state is in place; the workgroup that reads n_split - 1 from the counter therefore finds every
            // state with device-scope loads, which do not read the per-die caches.  A release on the increment
            // and an acquire in the merging workgroup would express the same in the language's memory model;
            // the release costs a write-back of the die's whole L2 per workgroup, and the acquire (a fence at
            // agent scope for the one merging workgroup of a pair) was measured at 2.8 us per launch, 0.82 ->
            // 0.89 ms per decode step at 520 cached slots, for an invalidate of caches that these loads bypass.
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stores have completed before the workgroup counts itself
        } else {
            const uint32_t bits = f32_to_bf16_bits(o);
            a.out[((long)m * a.n_heads + h) * D + tid] = (uint16_t)bits;
            if constexpr (LORA != 0) qs[tid] = bf16_to_f32(bits);  // what the next projection reads
        }
    }
    if (!whole) {
        uint32_t *count = a.arrived + (long)m * a.n_heads + h;
        __syncthreads();
        if (tid == 0) s_before = __hip_atomic_fetch_add(count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (s_before != (uint32_t)(n_split - 1)) return;  // uniform: somebody else arrives last
        if (tid < D) {
            const float *all = a.partials + ((long)m * a.n_heads + h) * n_split * (D + 2);
            // every state is requested before any is used: one memory round trip
            float pm_[ATTN_MAX_SPLITS], ps_[ATTN_MAX_SPLITS], po_[ATTN_MAX_SPLITS];
#pragma unroll
            for (int z = 0; z < ATTN_MAX_SPLITS; ++z) {
                pm_[z] = -INFINITY, ps_[z] = 0.0f, po_[z] = 0.0f;
                if (z < n_split) {
                    const float *part = all + z * (D + 2);
                    pm_[z] = __hip_atomic_load(part + D, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    ps_[z] = __hip_atomic_load(part + D + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    po_[z] = __hip_atomic_load(part + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            float mx = -INFINITY;
#pragma unroll
            for (int z = 0; z < ATTN_MAX_SPLITS; ++z) mx = fmaxf(mx, pm_[z]);
            float o = 0.0f, sum = 0.0f;
            if (mx != -INFINITY) {
#pragma unroll
                for (int z = 0; z < ATTN_MAX_SPLITS; ++z) {   // index order: the same sums whoever merges
                    const float c = __expf(pm_[z] - mx);
                    o += c * po_[z];
                    sum += c * ps_[z];
                }
                o /= sum;
            }
            a.out[((long)m * a.n_heads + h) * D + tid] = (uint16_t)f32_to_bf16_bits(o);
        }
        if (tid == 0) __hip_atomic_store(count, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    }
    if constexpr (LORA != 0) {
        if (a.oa) {  // uniform
            __syncthreads();
            float ov[VEC];
#pragma unroll
            for (int i = 0; i < VEC; ++i) ov[i] = qs[l16 * VEC + i];
            for (int j = oj; j < a.orank; j += OJ) {
                if (j != oj) request_oa(j);
                float part = 0.0f;
#pragma unroll
                for (int i = 0; i < VEC; ++i) part += ov[i] * oaw[i];
                part = row16_sum(part);  // the sixteen lanes that share row j
                if (l16 == 0) a.ot[((long)m * a.n_heads + h) * a.orank + j] = part;
            }
        }
    }
}

// ---------------------------------------------------------------- LoRA adapters over an int4 projection
// One workgroup per column of t (an adapter row) and block of MB rows (8 or 16; blockIdx.y picks the
// block): lora_down_item.  FP32 is the adapters' weight type.
template <bool FP32, int MB>
__global__ __launch_bounds__(THREADS) void lora_down_kernel(const uint16_t *__restrict__ x, LoraArgs a,
                                                            float *__restrict__ t) {
    __shared__ float part[LORA_DOWN_WAVES * MB];
    lora_down_item<FP32, MB>(x, a, t, true, blockIdx.x, blockIdx.y * MB, threadIdx.x / WAVE, threadIdx.x % WAVE, part);
}

// One thread per output column, 64 columns per workgroup, eight rows per workgroup (blockIdx.z): t of
// the adapter and those rows staged in LDS, the column's row of B (up to RB values, zero beyond the
// rank) in registers, 16-byte LDS reads shared by the wave.  The rows' products are formed while
// their base outputs are on the way (one memory round trip per workgroup).
constexpr int UP_THREADS = 64;
constexpr int UP_ROWS = 8;
template <bool FP32, int RB>
__global__ __launch_bounds__(UP_THREADS) void lora_up_add_kernel(const float *__restrict__ t, int parts, LoraArgs a) {
    extern __shared__ __align__(16) float ts[];  // UP_ROWS x r of this adapter
    const int i = blockIdx.y;
    vrl_lora_adapter ad = a.ad[0];
    int first = 0;
#pragma unroll
    for (int k = 1; k < LORA_MAX_ADAPTERS; ++k)
        if (k == i) ad = a.ad[k], first = a.off[k];
    const int total = a.off[a.n], r = ad.r;
    if (blockIdx.x * UP_THREADS >= ad.N) return;  // uniform: adapters of one launch differ in width
    const int m_lo = blockIdx.z * UP_ROWS, rows = min(UP_ROWS, a.M - m_lo);
    const int n = blockIdx.x * UP_THREADS + threadIdx.x;
    const int nn = n < ad.N ? n : ad.N - 1;  // lanes past the last column repeat it and store nothing
    uint16_t *y = static_cast<uint16_t *>(ad.y);
    uint16_t base[UP_ROWS];
#pragma unroll
    for (int d = 0; d < UP_ROWS; ++d)  // rows past the end repeat the last one and are not stored
        base[d] = y[(long)(m_lo + (d < rows ? d : rows - 1)) * ad.N + nn];
    {   // t of this adapter: rows of r floats (r % 8 == 0), four at a time; a row given as `parts`
        // partial rows is their sum in order (a bf16 adapter's t is rounded once the sum is complete)
        const int r4 = r >> 2, count = rows * r4;
        for (int idx = threadIdx.x; idx < count; idx += UP_THREADS) {
            const int m = idx / r4;
            const float *src = t + (long)(m_lo + m) * parts * total + first + 4 * (idx - m * r4);
            float4 v = {0.0f, 0.0f, 0.0f, 0.0f};
            for (int q0 = 0; q0 < parts; q0 += 16) {   // sixteen pieces requested together, added in order
                float4 w[16];
#pragma unroll
                for (int u = 0; u < 16; ++u)
                    w[u] = *reinterpret_cast<const float4 *>(src + (long)(q0 + u < parts ? q0 + u : parts - 1) * total);
#pragma unroll
                for (int u = 0; u < 16; ++u)
                    if (q0 + u < parts) v.x += w[u].x, v.y += w[u].y, v.z += w[u].z, v.w += w[u].w;
            }
            if (!FP32) v.x = round_bf16(v.x), v.y = round_bf16(v.y), v.z = round_bf16(v.z), v.w = round_bf16(v.w);
            *reinterpret_cast<float4 *>(ts + 4 * idx) = v;
        }
    }
    float bf[RB];
#pragma unroll
    for (int g = 0; g < RB / 8; ++g) {
        float piece[8];
        load8<FP32>(ad.B, (long)nn * r + (8 * g < r ? 8 * g : r - 8), piece);
        const float keep = 8 * g < r ? 1.0f : 0.0f;   // beyond the rank: zeros
#pragma unroll
        for (int e = 0; e < 8; ++e) bf[8 * g + e] = piece[e] * keep;
    }
    __syncthreads();
    if (n >= ad.N) return;
#pragma unroll
    for (int d = 0; d < UP_ROWS; ++d) {
        if (d < rows) {   // uniform
            const float *row = ts + d * r;
            float u = 0.0f;
#pragma unroll
            for (int g = 0; g < RB / 4; ++g) {
                const float4 tv = *reinterpret_cast<const float4 *>(row + (4 * g < r ? 4 * g : r - 4));  // x 0 beyond r
                u += tv.x * bf[4 * g] + tv.y * bf[4 * g + 1] + tv.z * bf[4 * g + 2] + tv.w * bf[4 * g + 3];
            }
            float delta;
            if (!FP32) delta = round_bf16(round_bf16(u) * ad.scaling);  // lora_B's output, then * scaling
            else delta = u * ad.scaling;
            y[(long)(m_lo + d) * ad.N + n] = (uint16_t)f32_to_bf16_bits(bf16_to_f32(base[d]) + delta);
        }
    }
}

template <bool FP32, int MB>
int launch_lora_down(const uint16_t *x, const LoraArgs &a, float *t, hipStream_t stream) {
    return vrl_launch(&lora_down_kernel<FP32, MB>, dim3(a.off[a.n], (a.M + MB - 1) / MB), dim3(THREADS), 0, stream,
                      x, a, t);
}

template <bool FP32, int RB>
int launch_lora_up(const float *t, int parts, const LoraArgs &a, int max_n, int max_r, hipStream_t stream) {
    return vrl_launch(&lora_up_add_kernel<FP32, RB>,
                      dim3((max_n + UP_THREADS - 1) / UP_THREADS, a.n, (a.M + UP_ROWS - 1) / UP_ROWS),
                      dim3(UP_THREADS), (size_t)UP_ROWS * max_r * sizeof(float), stream, t, parts, a);
}

bool misaligned(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }


}  // namespace

extern "C" int vrl_add_rmsnorm_bf16(const void *x, const void *residual, const void *weight, void *h_out,
                                    void *y, int M, int K, float eps, void *hip_stream) {
    if (!x || !weight || !y || (residual && !h_out)) return VRL_INT4_ENULL;
    if (M < 1 || M > (1 << 20) || K < 8 || K % 8 != 0 || K > MAX_NORM_K || !(eps >= 0.0f)) return VRL_INT4_ESHAPE;
    if (misaligned(x, 16) || misaligned(weight, 16) || misaligned(y, 16) || misaligned(residual, 16) ||
        misaligned(h_out, 16))
        return VRL_INT4_EALIGN;
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
    const size_t lds = (size_t)K * sizeof(uint16_t);
    auto xs = static_cast<const uint16_t *>(x);
    auto rs = static_cast<const uint16_t *>(residual);
    auto ws = static_cast<const uint16_t *>(weight);
    auto hs = static_cast<uint16_t *>(h_out);
    auto ys = static_cast<uint16_t *>(y);
    if (residual) return vrl_launch(&add_rmsnorm_kernel<true>, dim3(M), dim3(THREADS), lds, stream, xs, rs, ws, hs, ys, K, eps);
    return vrl_launch(&add_rmsnorm_kernel<false>, dim3(M), dim3(THREADS), lds, stream, xs, rs, ws, hs, ys, K, eps);
}

namespace {
template <int LORA, bool STREAMED>
int launch_attn_build(const AttnArgs &a, int M, int D, hipStream_t stream) {
    const bool many = (long)a.n_heads * M >= 512;
    const dim3 grid(a.n_heads, M);
    // few workgroups: 16 waves each (256 slots per trip); many: 8 waves, several workgroups per CU
    // (a deeper unroll of the 16-wave form, 512 slots per trip, measured slower)
    if (D == 128 && many)
        return vrl_launch(&rope_attn_decode_kernel<128, 8, 4, LORA, STREAMED>, grid, dim3(8 * WAVE), 0, stream, a);
    if (D == 128)
        return vrl_launch(&rope_attn_decode_kernel<128, 16, 4, LORA, STREAMED>, grid, dim3(16 * WAVE), 0, stream, a);
    if (many)
        return vrl_launch(&rope_attn_decode_kernel<64, 8, 4, LORA, STREAMED>, grid, dim3(8 * WAVE), 0, stream, a);
    return vrl_launch(&rope_attn_decode_kernel<64, 16, 4, LORA, STREAMED>, grid, dim3(16 * WAVE), 0, stream, a);
}

// keys and values of one layer beyond this many bytes are read with non-temporal loads: a model's
// layers together then exceed the memory-side cache, and nothing of them survives to the next step
constexpr long STREAMED_CACHE_BYTES = 10L << 20;

// the split form: `splits` workgroups of 16 waves per (row, head)
int attn_splits(long pairs) { return pairs <= 32 ? 8 : (pairs <= 64 ? 4 : (pairs <= 128 ? 2 : 1)); }
size_t attn_counter_bytes(long pairs) { return (size_t)(pairs * sizeof(uint32_t) + 255) / 256 * 256; }

template <bool STREAMED>
int launch_attn_split(const AttnArgs &a, int M, int D, int splits, hipStream_t stream) {
    const dim3 grid(a.n_heads, M, splits);
    if (D == 128)
        return vrl_launch(&rope_attn_decode_kernel<128, 16, 4, 0, STREAMED, true>, grid, dim3(16 * WAVE), 0, stream, a);
    return vrl_launch(&rope_attn_decode_kernel<64, 16, 4, 0, STREAMED, true>, grid, dim3(16 * WAVE), 0, stream, a);
}

template <int LORA>
int launch_attn(const AttnArgs &a, int M, int D, hipStream_t stream) {
    const long cache_bytes = (long)M * a.n_kv_heads * a.L_max * D * 2 * 2;
    if constexpr (LORA == 0) {
        const int splits = a.partials ? attn_splits((long)a.n_heads * M) : 1;
        if (splits > 1) {
            if (cache_bytes > STREAMED_CACHE_BYTES) return launch_attn_split<true>(a, M, D, splits, stream);
            return launch_attn_split<false>(a, M, D, splits, stream);
        }
    }
    if (cache_bytes > STREAMED_CACHE_BYTES) return launch_attn_build<LORA, true>(a, M, D, stream);
    return launch_attn_build<LORA, false>(a, M, D, stream);
}

int attn_decode(const void *q, const void *k, const void *v, int q_stride, int kv_stride, void *k_cache,
                void *v_cache, const void *cos, const void *sin, const void *mask, const int64_t *position,
                void *out, int M, int n_heads, int n_kv_heads, int D, int L_max, float scaling,
                const vrl_attn_lora *lora, void *hip_stream, void *workspace = nullptr, size_t workspace_bytes = 0,
                bool position_per_row = false) {
    if (!q || !k || !v || !k_cache || !v_cache || !cos || !sin || !mask || !position || !out) return VRL_INT4_ENULL;
    if (M < 1 || M > 65535 || n_heads < 1 || n_kv_heads < 1 || n_heads % n_kv_heads != 0 || n_heads > 65535 ||
        (D != 64 && D != 128) || L_max < 1 || L_max > MAX_CACHE_LEN || q_stride < n_heads * D ||
        kv_stride < n_kv_heads * D || q_stride % 8 != 0 || kv_stride % 8 != 0)
        return VRL_INT4_ESHAPE;
    if (misaligned(q, 16) || misaligned(k, 16) || misaligned(v, 16) || misaligned(k_cache, 16) ||
        misaligned(v_cache, 16) || misaligned(cos, 2) || misaligned(sin, 2) || misaligned(position, 8) ||
        misaligned(out, 2))
        return VRL_INT4_EALIGN;
    AttnArgs a;
    memset(&a, 0, sizeof a);
    a.q = static_cast<const uint16_t *>(q);
    a.k = static_cast<const uint16_t *>(k);
    a.v = static_cast<const uint16_t *>(v);
    a.k_cache = static_cast<uint16_t *>(k_cache);
    a.v_cache = static_cast<uint16_t *>(v_cache);
    a.cos = static_cast<const uint16_t *>(cos);
    a.sin = static_cast<const uint16_t *>(sin);
    a.mask = static_cast<const uint8_t *>(mask);
    a.position = reinterpret_cast<const long long *>(position);
    a.position_stride = (position_per_row || (lora && lora->position_per_row)) ? 1 : 0;
    a.out = static_cast<uint16_t *>(out);
    a.q_stride = q_stride;
    a.kv_stride = kv_stride;
    a.n_heads = n_heads;
    a.n_kv_heads = n_kv_heads;
    a.L_max = L_max;
    a.scaling = scaling;
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
    if (workspace) {
        const long pairs = (long)n_heads * M;
        const size_t need = attn_counter_bytes(pairs) + (size_t)pairs * ATTN_MAX_SPLITS * (D + 2) * sizeof(float);
        if (lora) return VRL_INT4_ESHAPE;
        if (workspace_bytes < need) return VRL_INT4_EPLAN;
        if (misaligned(workspace, 256)) return VRL_INT4_EALIGN;
        a.arrived = static_cast<uint32_t *>(workspace);
        a.partials = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + attn_counter_bytes(pairs));
    }
    if (!lora) return launch_attn<0>(a, M, D, stream);
    const void *bs[3] = {lora->q_B, lora->k_B, lora->v_B};
    bool any = false;
    for (int i = 0; i < 3; ++i) {
        a.lb[i] = bs[i];
        a.lr[i] = lora->r[i];
        a.loff[i] = lora->offset[i];
        a.lscale[i] = lora->scaling[i];
        if (!bs[i]) continue;
        any = true;
        if (!lora->t) return VRL_INT4_ENULL;
        if (misaligned(lora->t, 16) || lora->t_stride < 8 || lora->t_stride % 4 != 0) return VRL_INT4_ESHAPE;
        if (lora->r[i] < 8 || lora->r[i] % 8 != 0 || lora->r[i] > LORA_MAX_RANK || lora->offset[i] < 0 ||
            lora->offset[i] % 4 != 0 || lora->offset[i] + lora->r[i] > lora->t_stride)
            return VRL_INT4_ESHAPE;
        if (misaligned(bs[i], 16)) return VRL_INT4_EALIGN;
    }
    if (lora->o_A) {
        if (!lora->o_t) return VRL_INT4_ENULL;
        if (lora->o_r < 8 || lora->o_r % 8 != 0 || lora->o_r > LORA_MAX_RANK) return VRL_INT4_ESHAPE;
        if (misaligned(lora->o_A, 16) || misaligned(lora->o_t, 16)) return VRL_INT4_EALIGN;
        a.oa = lora->o_A;
        a.ot = lora->o_t;
        a.orank = lora->o_r;
        any = true;
    }
    if (!any) return VRL_INT4_ENULL;
    a.t = lora->t;
    a.t_stride = lora->t_stride;
    if (lora->weights_fp32) return launch_attn<1>(a, M, D, stream);
    return launch_attn<2>(a, M, D, stream);
}
}  // namespace

extern "C" int vrl_rope_attn_decode_bf16(const void *q, const void *k, const void *v, int q_stride, int kv_stride,
                                         void *k_cache, void *v_cache, const void *cos, const void *sin,
                                         const void *mask, const int64_t *position, void *out,
                                         int M, int n_heads, int n_kv_heads, int D, int L_max, float scaling,
                                         void *hip_stream) {
    return attn_decode(q, k, v, q_stride, kv_stride, k_cache, v_cache, cos, sin, mask, position, out, M, n_heads,
                       n_kv_heads, D, L_max, scaling, nullptr, hip_stream);
}

extern "C" size_t vrl_rope_attn_decode_split_workspace_bytes(int M, int n_heads, int D) {
    if (M < 1 || n_heads < 1 || (D != 64 && D != 128) || (long)M * n_heads > (1L << 24)) return 0;
    const long pairs = (long)n_heads * M;
    return attn_counter_bytes(pairs) + (size_t)pairs * ATTN_MAX_SPLITS * (D + 2) * sizeof(float);
}

extern "C" int vrl_rope_attn_decode_split_bf16(const void *q, const void *k, const void *v, int q_stride,
                                               int kv_stride, void *k_cache, void *v_cache, const void *cos,
                                               const void *sin, const void *mask, const int64_t *position, void *out,
                                               int M, int n_heads, int n_kv_heads, int D, int L_max, float scaling,
                                               void *workspace, size_t workspace_bytes, void *hip_stream) {
    if (!workspace) return VRL_INT4_ENULL;
    return attn_decode(q, k, v, q_stride, kv_stride, k_cache, v_cache, cos, sin, mask, position, out, M, n_heads,
                       n_kv_heads, D, L_max, scaling, nullptr, hip_stream, workspace, workspace_bytes);
}

extern "C" int vrl_rope_attn_decode_rows_bf16(const void *q, const void *k, const void *v, int q_stride, int kv_stride,
                                              void *k_cache, void *v_cache, const void *cos, const void *sin,
                                              const void *mask, const int64_t *positions, void *out,
                                              int M, int n_heads, int n_kv_heads, int D, int L_max, float scaling,
                                              void *workspace, size_t workspace_bytes, void *hip_stream) {
    return attn_decode(q, k, v, q_stride, kv_stride, k_cache, v_cache, cos, sin, mask, positions, out, M, n_heads,
                       n_kv_heads, D, L_max, scaling, nullptr, hip_stream, workspace, workspace_bytes, true);
}

extern "C" int vrl_rope_attn_decode_lora_bf16(const void *q, const void *k, const void *v, int q_stride,
                                              int kv_stride, void *k_cache, void *v_cache, const void *cos,
                                              const void *sin, const void *mask, const int64_t *position, void *out,
                                              int M, int n_heads, int n_kv_heads, int D, int L_max, float scaling,
                                              const vrl_attn_lora *lora, void *hip_stream) {
    if (!lora) return VRL_INT4_ENULL;
    return attn_decode(q, k, v, q_stride, kv_stride, k_cache, v_cache, cos, sin, mask, position, out, M, n_heads,
                       n_kv_heads, D, L_max, scaling, lora, hip_stream);
}


extern "C" int vrl_lora_down_bf16(const void *x, int M, int K, const vrl_lora_adapter *adapters, int n_adapters,
                                  float *t, void *hip_stream) {
    if (!x || !t) return VRL_INT4_ENULL;
    if (misaligned(x, 16) || misaligned(t, 16)) return VRL_INT4_EALIGN;
    LoraArgs a;
    memset(&a, 0, sizeof a);
    const int rc = lora_args(a, M, K, adapters, n_adapters, false);
    if (rc != VRL_INT4_OK) return rc;
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
    auto xs = static_cast<const uint16_t *>(x);
    const bool fp32 = a.ad[0].weights_fp32 != 0;
    if (M <= 8) return fp32 ? launch_lora_down<true, 8>(xs, a, t, stream) : launch_lora_down<false, 8>(xs, a, t, stream);
    return fp32 ? launch_lora_down<true, 16>(xs, a, t, stream) : launch_lora_down<false, 16>(xs, a, t, stream);
}

extern "C" int vrl_lora_up_add_bf16(const float *t, int t_parts, int M, const vrl_lora_adapter *adapters,
                                    int n_adapters, void *hip_stream) {
    if (!t) return VRL_INT4_ENULL;
    if (t_parts < 1 || t_parts > 256) return VRL_INT4_ESHAPE;
    if (misaligned(t, 16)) return VRL_INT4_EALIGN;
    LoraArgs a;
    memset(&a, 0, sizeof a);
    const int rc = lora_args(a, M, 8, adapters, n_adapters, true);
    if (rc != VRL_INT4_OK) return rc;
    int max_n = 0, max_r = 0;
    for (int i = 0; i < a.n; ++i) {
        max_n = a.ad[i].N > max_n ? a.ad[i].N : max_n;
        max_r = a.ad[i].r > max_r ? a.ad[i].r : max_r;
    }
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
    const bool fp32 = a.ad[0].weights_fp32 != 0;
    if (fp32) return max_r <= 32 ? launch_lora_up<true, 32>(t, t_parts, a, max_n, max_r, stream)
                                 : launch_lora_up<true, 64>(t, t_parts, a, max_n, max_r, stream);
    return max_r <= 32 ? launch_lora_up<false, 32>(t, t_parts, a, max_n, max_r, stream)
                       : launch_lora_up<false, 64>(t, t_parts, a, max_n, max_r, stream);
}

// ---------------------------------------------------------------- a step's launches from one host call
extern "C" int vrl_decode_run_calls(const vrl_step_call *calls, int n_calls, int *failed_at, void *hip_stream) {
    if (!calls) return VRL_INT4_ENULL;
    if (n_calls < 0) return VRL_INT4_ESHAPE;
    for (int n = 0; n < n_calls; ++n) {
        const vrl_step_call &c = calls[n];
        const void *const *p = c.p;
        const int64_t *i = c.i;
        void *s = hip_stream;
        auto w = [&](int k) { return const_cast<void *>(p[k]); };   // a pointer the callee writes through
        int rc;
        switch (c.kind) {
            case VRL_CALL_GEMV:
                rc = vrl_int4_gemv_prepacked_bf16(static_cast<const vrl_int4_problem *>(p[0]), (int)i[0], s);
                break;
            case VRL_CALL_GEMV_NORM:
                rc = vrl_int4_gemv_prepacked_norm_bf16(static_cast<const vrl_int4_problem *>(p[0]), (int)i[0],
                                                       static_cast<const vrl_int4_norm *>(p[1]), s);
                break;
            case VRL_CALL_GEMV_EPILOGUE:
                rc = vrl_int4_gemv_prepacked_epilogue_bf16(static_cast<const vrl_int4_problem *>(p[0]),
                                                           static_cast<const vrl_int4_norm *>(p[1]),
                                                           static_cast<const vrl_int4_epilogue *>(p[2]), s);
                break;
            case VRL_CALL_GEMV_LORA:
                rc = vrl_int4_gemv_prepacked_lora_bf16(static_cast<const vrl_int4_problem *>(p[0]), (int)i[0],
                                                       static_cast<const vrl_lora_adapter *>(p[1]), (int)i[1],
                                                       static_cast<float *>(w(2)), s);
                break;
            case VRL_CALL_GEMV_LORA_UP:
                rc = vrl_int4_gemv_prepacked_lora_up_bf16(static_cast<const vrl_int4_problem *>(p[0]),
                                                          static_cast<const vrl_lora_adapter *>(p[1]),
                                                          static_cast<const float *>(p[2]), (int)i[0], s);
                break;
            case VRL_CALL_ADD_RMSNORM:
                rc = vrl_add_rmsnorm_bf16(p[0], p[1], p[2], w(3), w(4), (int)i[0], (int)i[1], c.f[0], s);
                break;
            case VRL_CALL_ATTN:
                rc = vrl_rope_attn_decode_bf16(p[0], p[1], p[2], (int)i[0], (int)i[1], w(3), w(4), p[5], p[6], p[7],
                                               static_cast<const int64_t *>(p[8]), w(9), (int)i[2], (int)i[3],
                                               (int)i[4], (int)i[5], (int)i[6], c.f[0], s);
                break;
            case VRL_CALL_ATTN_SPLIT:
                rc = vrl_rope_attn_decode_split_bf16(p[0], p[1], p[2], (int)i[0], (int)i[1], w(3), w(4), p[5], p[6],
                                                     p[7], static_cast<const int64_t *>(p[8]), w(9), (int)i[2],
                                                     (int)i[3], (int)i[4], (int)i[5], (int)i[6], c.f[0], w(10),
                                                     (size_t)i[7], s);
                break;
            case VRL_CALL_ATTN_ROWS:
                rc = vrl_rope_attn_decode_rows_bf16(p[0], p[1], p[2], (int)i[0], (int)i[1], w(3), w(4), p[5], p[6],
                                                    p[7], static_cast<const int64_t *>(p[8]), w(9), (int)i[2],
                                                    (int)i[3], (int)i[4], (int)i[5], (int)i[6], c.f[0], w(10),
                                                    (size_t)i[7], s);
                break;
            case VRL_CALL_ATTN_LORA:
                rc = vrl_rope_attn_decode_lora_bf16(p[0], p[1], p[2], (int)i[0], (int)i[1], w(3), w(4), p[5], p[6],
                                                    p[7], static_cast<const int64_t *>(p[8]), w(9), (int)i[2],
                                                    (int)i[3], (int)i[4], (int)i[5], (int)i[6], c.f[0],
                                                    static_cast<const vrl_attn_lora *>(p[10]), s);
                break;
            case VRL_CALL_LORA_DOWN:
                rc = vrl_lora_down_bf16(p[0], (int)i[0], (int)i[1], static_cast<const vrl_lora_adapter *>(p[1]),
                                        (int)i[2], static_cast<float *>(w(2)), s);
                break;
            case VRL_CALL_LORA_UP_ADD:
                rc = vrl_lora_up_add_bf16(static_cast<const float *>(p[0]), (int)i[0], (int)i[1],
                                          static_cast<const vrl_lora_adapter *>(p[1]), (int)i[2], s);
                break;
            case VRL_CALL_GEMV_NORM_LORA:
                rc = vrl_int4_gemv_prepacked_norm_lora_bf16(static_cast<const vrl_int4_problem *>(p[0]), (int)i[0],
                                                            static_cast<const vrl_int4_norm *>(p[1]),
                                                            static_cast<const vrl_lora_adapter *>(p[2]), (int)i[1],
                                                            static_cast<float *>(w(3)), s);
                break;
            default:
                rc = VRL_INT4_ESHAPE;
        }
        if (rc != 0) {
            if (failed_at) *failed_at = n;
            return rc;
        }
    }
    return 0;
}
