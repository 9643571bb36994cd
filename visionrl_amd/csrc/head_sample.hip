// The image-token head and the sampling tail of a decode step in one launch.
//
// Replaces vrl/models/families/janus_pro/policy.py:684-693 for an int4 head: the gen_head linear over
// the [2B, K] hidden rows (conditional rows first), then
//   guided  = uncond + w * (cond - uncond)
//   probs   = softmax(guided / T)
//   sampled = multinomial(probs, 1)                  = argmax(probs / q), q ~ Exp(1) drawn by the caller
//   lp      = log_softmax(cond / T)[sampled]
// with the roundings torch applies to bf16 tensors (every op in fp32, result rounded to bf16), as
// cfg_sample.hip states them.  The [2B, V] logits never make the round trip through memory that a
// head launch followed by a tail launch costs, and the tail is not one workgroup per row any more.
//
// Every workgroup computes 16-column tiles of the head exactly as the plan-free launch of prepacked.hpp
// does (waves split K of a tile, partial tiles meet in LDS).  The wave that holds a finished tile rounds
// the logits to bf16, forms guided / T and cond / T for its B x 16 entries and leaves in a workspace:
//   gt, ct   [B, V] bf16    the two scaled rows (read back only where a draw can win)
//   part     [B, tiles]     {max, sum exp(. - max)} of the tile's 16 entries, for both rows
//   mask     [B, tiles]     which of the 16 entries can still win the draw: those whose
//                           exp(gt - tile max) / q lies within 2^-5 of the tile's largest.  The final
//                           ratio bf16(bf16(exp(gt - max) / sum) / q) is that quantity times one
//                           factor per row, through two monotone roundings of relative size 2^-8 each,
//                           so an entry further below its tile's best than that can neither win nor tie.
// The last workgroup to finish (a counter in the workspace) then takes one wave per batch row: the row's
// maxima and sums from the tile partials in a fixed order, the ratio of every marked entry with exactly
// the arithmetic of cfg_sample.hip, the lowest index among equal maxima, and the log-probability.
// No workgroup waits for another: the last one is whichever increments the counter last.

#include <atomic>

#include "prepacked.hpp"

namespace {

struct HeadArgs {
    DevProblem p;            // x [2B, K] (M = 2B), the head's prepacked blob, y = logits [2B, V] or nullptr
    const uint16_t *noise;   // [B, V] bf16, strictly positive
    long long *sampled;      // [B]
    float *logprob;          // [B]
    uint32_t *counter;       // zero between launches
    f32x4_t *part;           // [B, tiles]: {max gt, sum exp(gt - max), max ct, sum exp(ct - max)}
    uint16_t *mask;          // [B, tiles]
    uint16_t *gt;            // [B, V]
    uint16_t *ct;            // [B, V]
    int32_t B, tiles, rounds, reserved;
    float w, inv_t;
};

__device__ __forceinline__ float hs_round_bf16(float v) {
    return __builtin_bit_cast(float, (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)v) << 16);
}
__device__ __forceinline__ uint16_t hs_bf16_bits(float v) { return __builtin_bit_cast(uint16_t, (__bf16)v); }

// guided / T and cond / T of one vocabulary entry (c, u: its two logits), as bf16 values held in floats
__device__ __forceinline__ void hs_scaled_pair(float c, float u, float w, float inv_t, float &gt, float &ct) {
    const float d = hs_round_bf16(c - u);
    const float g = hs_round_bf16(u + hs_round_bf16(w * d));
    gt = hs_round_bf16(g * inv_t);
    ct = hs_round_bf16(c * inv_t);
}

// the better of two draws: the larger ratio, the lower index among equals, a NaN over any number (torch's argmax)
__device__ __forceinline__ void hs_take_better(float &bv, int &bi, float ov, int oi) {
    const bool other_nan = ov != ov, mine_nan = bv != bv;
    const bool take = mine_nan ? (other_nan && oi < bi) : (other_nan || ov > bv || (ov == bv && oi < bi));
    if (take) {
        bv = ov;
        bi = oi;
    }
}

constexpr float HS_MARGIN = 1.0f - 0.03125f;   // 2^-5 below the tile's best: out of the draw

// The wave that holds tile `tile` ([2B rows] x 16 columns, accumulators in the MFMA layout: lane % 16 =
// column, rows 16 b + 4 (lane / 16) + i): logits to bf16, scaled rows, tile partials and draw mask.
// `tb` is the wave's own [16 * MB][16] floats of LDS.
template <int MB>
__device__ __forceinline__ void head_epilogue(const HeadArgs &a, int tile, const f32x4_t (&acc)[1][MB], float *tb) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int col = lane & 15, rg = lane >> 4;
    const int B = a.B, V = a.p.N;
#pragma unroll
    for (int b = 0; b < MB; ++b)
#pragma unroll
        for (int i = 0; i < 4; ++i) tb[(16 * b + 4 * rg + i) * 16 + col] = hs_round_bf16(acc[0][b][i]);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int n = tile * 16 + col;
    const bool col_ok = n < V;
#pragma unroll
    for (int j = 0; j < 2 * MB; ++j) {
        const int b = rg + 4 * j;                 // uniform over the 16 lanes of a DPP row
        const bool ok = b < B && col_ok;
        const int bb = b < B ? b : 0;
        float gtv, ctv;
        hs_scaled_pair(tb[bb * 16 + col], tb[(B + bb) * 16 + col], a.w, a.inv_t, gtv, ctv);
        const long at = (long)bb * V + (col_ok ? n : 0);
        const float q = bf16_bits_to_f32(as_global(a.noise)[at]);
        if (ok) {
            as_global(a.gt)[at] = hs_bf16_bits(gtv);
            as_global(a.ct)[at] = hs_bf16_bits(ctv);
        }
        const float gm = row16_max(ok ? gtv : -INFINITY), cm = row16_max(ok ? ctv : -INFINITY);
        const float eg = ok ? expf(gtv - gm) : 0.0f, ec = ok ? expf(ctv - cm) : 0.0f;
        const float gs = row16_sum(eg), cs = row16_sum(ec);
        // which entries can still win the draw (a NaN or an infinity compares in their favour)
        const float e = eg / q;
        const float eb = row16_max(e == e ? e : INFINITY);
        const bool cand = ok && !(e < eb * HS_MARGIN);
        const uint64_t votes = __ballot(cand);
        if (col == 0 && b < B) {
            typedef __attribute__((address_space(1))) f32x4_t *gptr_f4;
            *(gptr_f4)(uintptr_t)(a.part + (long)b * a.tiles + tile) = f32x4_t{gm, gs, cm, cs};
            as_global(a.mask)[(long)b * a.tiles + tile] = (uint16_t)((votes >> (16 * rg)) & 0xFFFFu);
        }
    }
}

// One wave finishes batch row b from what every tile left behind.
__device__ __forceinline__ void head_final_row(const HeadArgs &a, int b) {
    typedef const __attribute__((address_space(1))) f32x4_t *gptr_cf4;
    const int lane = threadIdx.x & (WAVE - 1);
    const int tiles = a.tiles, V = a.p.N;
    gptr_cf4 part = (gptr_cf4)(uintptr_t)(a.part + (long)b * tiles);
    float gm = -INFINITY, cm = -INFINITY;
    for (int t = lane; t < tiles; t += WAVE) {
        const f32x4_t pt = part[t];
        gm = fmaxf(gm, pt[0]);
        cm = fmaxf(cm, pt[2]);
    }
    gm = wave_max(gm);
    cm = wave_max(cm);
    float gs = 0.0f, cs = 0.0f;
    for (int t = lane; t < tiles; t += WAVE) {     // a fixed order: the same sums whichever workgroup is last
        const f32x4_t pt = part[t];
        gs += pt[1] * expf(pt[0] - gm);
        cs += pt[3] * expf(pt[2] - cm);
    }
    gs = wave_sum(gs);
    cs = wave_sum(cs);
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
    for (int t = lane; t < tiles; t += WAVE) {
        uint32_t m = as_global(a.mask)[(long)b * tiles + t];
        while (m) {
            const int bit = __builtin_ctz(m);
            m &= m - 1;
            const int idx = 16 * t + bit;
            const float gt = bf16_bits_to_f32(as_global(a.gt)[(long)b * V + idx]);
            const float q = bf16_bits_to_f32(as_global(a.noise)[(long)b * V + idx]);
            const float p = hs_round_bf16(expf(gt - gm) / gs);
            hs_take_better(bv, bi, hs_round_bf16(p / q), idx);
        }
    }
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1)
        hs_take_better(bv, bi, __shfl_xor(bv, off, WAVE), __shfl_xor(bi, off, WAVE));
    if (lane == 0) {
        if (bi >= V) bi = 0;   // only if no entry was marked at all: cannot happen for finite logits
        const float ct = bf16_bits_to_f32(as_global(a.ct)[(long)b * V + bi]);
        a.sampled[b] = bi;
        a.logprob[b] = hs_round_bf16(ct - cm - logf(cs));
    }
}

// KS waves split K of a tile, TW tiles per round, MB blocks of 16 activation rows (M = 2B <= 16 MB).
// LDS: staged activations, then TW x (KS - 1) x MB partial tiles.
template <int KS, int TW, int GQ, int MB>
__global__ __launch_bounds__(KS *TW *WAVE) void head_sample_kernel(HeadArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    __shared__ int is_last;
    const DevProblem &p = a.p;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tw = wave / KS, kw = wave % KS;
    const int lane = threadIdx.x & (WAVE - 1);
    uint16_t *xs = reinterpret_cast<uint16_t *>(smem);
    const int xstride = p.kc + XPAD;
    uint8_t *after_x = smem + (size_t)p.M * xstride * 2;
    f32x4_t *red = reinterpret_cast<f32x4_t *>(after_x) + tw * (KS - 1) * MB * WAVE;
    // the logit tile takes the place of the tile's partial sums once they are added up (2 KiB per row block
    // in at least 3 KiB): between two barriers only the wave that finishes the tile touches that space
    float *tb = reinterpret_cast<float *>(red);
    static_assert((KS - 1) * WAVE * sizeof(f32x4_t) >= 16 * 16 * sizeof(float), "the logit tile fits the partial tiles");
    const int nsc = pp_nsc(p.K);
    const int per = (nsc + KS - 1) / KS;
    const int sc0 = min(nsc, kw * per), sc1 = min(nsc, sc0 + per);
    const rsrc_t rsrc = pp_blob_rsrc(p);
    const int t0 = blockIdx.x * TW * a.rounds, t1 = min(a.tiles, t0 + TW * a.rounds);
    PPRing<1, GQ> ring;
    int tile = t0 + tw;
    bool work = sc0 < sc1 && tile < t1;   // wave-uniform
    PPTilePtr<false> cur = pp_tile_ptr<false>(p, work ? tile : t0, sc0);
    if (work) pp_prime<false, GQ>(rsrc, cur, ring);   // weights are on their way while x is staged
    stage_x_natural(p, 0, nsc * PP_SC, xs, xstride, KS * TW * WAVE);
    __syncthreads();
    for (int base = t0; base < t1; base += TW) {
        tile = base + tw;
        const int next = tile + TW < t1 ? tile + TW : -1;
        f32x4_t acc[1][MB];
#pragma unroll
        for (int b = 0; b < MB; ++b) acc[0][b] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        if (work) {
            stream_rows_pp<MB, false, GQ>(p, rsrc, cur, next, xs + sc0 * PP_SC, xstride, sc0, sc1, ring, acc);
            if (next >= 0) cur = pp_tile_ptr<false>(p, next, sc0);
        }
        if (kw != 0) {
#pragma unroll
            for (int b = 0; b < MB; ++b) red[((kw - 1) * MB + b) * WAVE + lane] = acc[0][b];
        }
        __syncthreads();
        if (kw == 0 && tile < t1) {
#pragma unroll
            for (int w = 1; w < KS; ++w)
#pragma unroll
                for (int b = 0; b < MB; ++b) acc[0][b] += red[((w - 1) * MB + b) * WAVE + lane];
            if (p.y) store_tile<MB, false>(p, tile, acc);
            head_epilogue<MB>(a, tile, acc, tb);
        }
        work = work && next >= 0;
        if (base + TW < t1) __syncthreads();   // the partial tiles are read before they are rewritten
    }
    // whoever arrives last finishes the rows; what the others wrote is visible to it: every workgroup
    // releases its stores before it counts itself, the last one acquires after it saw the count
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t seen = atomicAdd(a.counter, 1u);
        is_last = seen == gridDim.x - 1;
    }
    __syncthreads();
    if (!is_last) return;   // block-uniform
    __threadfence();
    for (int b = wave; b < a.B; b += KS * TW) head_final_row(a, b);
    if (threadIdx.x == 0) *a.counter = 0u;   // the next launch starts from zero again
}

constexpr int HS_MAX_B = 16;
constexpr size_t HS_LDS_CAP = 160 * 1024 - 64;   // what a workgroup can have, less the kernel's static word
constexpr size_t HS_COUNTER_BYTES = 256;

size_t hs_align(size_t v) { return (v + 255) & ~(size_t)255; }

struct HeadLayout {
    size_t part, mask, gt, ct, total;
};

HeadLayout head_layout(int B, int V) {
    const size_t tiles = ((size_t)V + 15) / 16;
    HeadLayout l;
    l.part = HS_COUNTER_BYTES;
    l.mask = l.part + hs_align((size_t)B * tiles * sizeof(f32x4_t));
    l.gt = l.mask + hs_align((size_t)B * tiles * sizeof(uint16_t));
    l.ct = l.gt + hs_align((size_t)B * V * sizeof(uint16_t));
    l.total = l.ct + hs_align((size_t)B * V * sizeof(uint16_t));
    return l;
}

template <int KS, int TW, int GQ, int MB>
int launch_head(const HeadArgs &args, int workgroups, size_t lds, hipStream_t stream) {
    auto kernel = &head_sample_kernel<KS, TW, GQ, MB>;
    if (lds > 64 * 1024) {
        static std::atomic<uint64_t> raised{0};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess) dev = 0;
        const uint64_t bit = 1ull << (dev & 63);
        if (!(raised.load(std::memory_order_relaxed) & bit)) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)HS_LDS_CAP);
            if (e != hipSuccess) return (int)e;
            raised.fetch_or(bit, std::memory_order_relaxed);
        }
    }
    (void)hipGetLastError();  // what an earlier call left behind is not this launch's status
    hipLaunchKernelGGL(kernel, dim3(workgroups), dim3(KS * TW * WAVE), lds, stream, args);
    return (int)hipGetLastError();
}

template <int KS, int TW, int MB>
int launch_head_group(const HeadArgs &args, int workgroups, size_t lds, hipStream_t stream) {
    if (args.p.G == 128) return launch_head<KS, TW, 1, MB>(args, workgroups, lds, stream);
    if (args.p.G == 64) return launch_head<KS, TW, 2, MB>(args, workgroups, lds, stream);
    return launch_head<KS, TW, 4, MB>(args, workgroups, lds, stream);
}

int cu_count() {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
    }
    return cus;
}

int head_sample_launch(const vrl_int4_problem *head, const void *noise, int64_t *sampled, float *logprob, int B,
                       float cfg_weight, float temperature, void *workspace, size_t workspace_bytes,
                       void *hip_stream) {
    if (!head || !noise || !sampled || !logprob || !workspace) return VRL_INT4_ENULL;
    if (!head->x || !head->qweight) return VRL_INT4_ENULL;
    if (!head->prepacked || head->fused_gate_up) return VRL_INT4_ESHAPE;
    const int V = head->N, K = head->K, G = head->G;
    if (B < 1 || B > HS_MAX_B || head->M != 2 * B || V < 16 || V > 65536 || V % 16 != 0 || !(temperature > 0.0f))
        return VRL_INT4_ESHAPE;
    if ((G != 128 && G != 64 && G != 32) || K % 128 != 0 || K < 128) return VRL_INT4_ESHAPE;
    if (vrl_int4_prepacked_bytes(V, K, G) == 0) return VRL_INT4_ESHAPE;
    if ((reinterpret_cast<uintptr_t>(head->x) | reinterpret_cast<uintptr_t>(head->qweight) |
         reinterpret_cast<uintptr_t>(head->y) | reinterpret_cast<uintptr_t>(noise)) & 15u)
        return VRL_INT4_EALIGN;
    if ((reinterpret_cast<uintptr_t>(workspace) & 255u) || (reinterpret_cast<uintptr_t>(sampled) & 7u) ||
        (reinterpret_cast<uintptr_t>(logprob) & 3u))
        return VRL_INT4_EALIGN;
    const HeadLayout lay = head_layout(B, V);
    if (workspace_bytes < lay.total) return VRL_INT4_ESHAPE;

    const int nsc = pp_nsc(K);
    if (nsc > 16) return VRL_INT4_ESHAPE;
    const int M = 2 * B;
    const int mb = M > 16 ? 2 : 1;
    const int ks = nsc > 8 ? 16 : (nsc > 4 ? 8 : 4);
    const int tw = M >= 8 ? 16 / ks : 1;
    const size_t x_bytes = (size_t)M * (nsc * PP_SC + XPAD) * 2;
    const size_t lds = x_bytes + (size_t)tw * (ks - 1) * mb * WAVE * sizeof(f32x4_t);
    if (lds > HS_LDS_CAP) return VRL_INT4_ESHAPE;   // the rows of this K do not fit LDS: head and tail as two launches

    HeadArgs args;
    memset(&args, 0, sizeof args);
    args.p.x = static_cast<const uint16_t *>(head->x);
    args.p.qweight = static_cast<const uint32_t *>(head->qweight);
    args.p.y = static_cast<uint16_t *>(head->y);
    args.p.M = M; args.p.N = V; args.p.K = K; args.p.G = G;
    args.p.prepacked = 1;
    args.p.kc = nsc * PP_SC;
    uint8_t *ws = static_cast<uint8_t *>(workspace);
    args.noise = static_cast<const uint16_t *>(noise);
    args.sampled = reinterpret_cast<long long *>(sampled);
    args.logprob = logprob;
    args.counter = reinterpret_cast<uint32_t *>(ws);
    args.part = reinterpret_cast<f32x4_t *>(ws + lay.part);
    args.mask = reinterpret_cast<uint16_t *>(ws + lay.mask);
    args.gt = reinterpret_cast<uint16_t *>(ws + lay.gt);
    args.ct = reinterpret_cast<uint16_t *>(ws + lay.ct);
    args.B = B;
    args.tiles = V / 16;
    args.w = cfg_weight;
    args.inv_t = 1.0f / temperature;
    // as many workgroups as the device holds at once: a second round of workgroups would stage x again
    const long per_cu = std::max<long>(1, std::min<long>(16 / (ks * tw), (long)(160 * 1024 / std::max<size_t>(lds, 1024))));
    const long capacity = per_cu * cu_count();
    long workgroups = (args.tiles + tw - 1) / tw;
    args.rounds = (int)std::min<long>(16, (workgroups + capacity - 1) / capacity);
    workgroups = (args.tiles + tw * args.rounds - 1) / (tw * args.rounds);
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
    if (mb == 1) {
        if (ks == 4 && tw == 1) return launch_head_group<4, 1, 1>(args, (int)workgroups, lds, stream);
        if (ks == 4 && tw == 4) return launch_head_group<4, 4, 1>(args, (int)workgroups, lds, stream);
        if (ks == 8 && tw == 1) return launch_head_group<8, 1, 1>(args, (int)workgroups, lds, stream);
        if (ks == 8 && tw == 2) return launch_head_group<8, 2, 1>(args, (int)workgroups, lds, stream);
        return launch_head_group<16, 1, 1>(args, (int)workgroups, lds, stream);
    }
    if (ks == 4) return launch_head_group<4, 4, 2>(args, (int)workgroups, lds, stream);
    if (ks == 8) return launch_head_group<8, 2, 2>(args, (int)workgroups, lds, stream);
    return launch_head_group<16, 1, 2>(args, (int)workgroups, lds, stream);
}

}  // namespace

extern "C" {

size_t vrl_int4_head_sample_workspace_bytes(int B, int V) {
    if (B < 1 || B > HS_MAX_B || V < 16 || V > 65536 || V % 16 != 0) return 0;
    return head_layout(B, V).total;
}

int vrl_int4_head_sample_bf16(const vrl_int4_problem *head, const void *noise, int64_t *sampled, float *logprob,
                              int B, float cfg_weight, float temperature, void *workspace, size_t workspace_bytes,
                              void *hip_stream) {
    return head_sample_launch(head, noise, sampled, logprob, B, cfg_weight, temperature, workspace, workspace_bytes,
                              hip_stream);
}

}  // extern "C"
