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
//   gt, ct   [B, V] bf16    the two scaled rows (read back only for the rare second candidates of a tile)
//   rec      [B, tiles]     32 bytes per tile: {max, sum exp(. - max)} of the tile's 16 entries for both
//                           rows; the entry with the tile's largest exp(gt - tile max) / q (its gt, q, ct
//                           and column), which is the tile's first candidate for the draw; and a mask of
//                           the entries within 2^-5 of that largest.  The final ratio
//                           bf16(bf16(exp(gt - max) / sum) / q) is that quantity times one factor per
//                           row, through two monotone roundings of relative size 2^-8 each, so an entry
//                           further below its tile's best than that can neither win nor tie.
// A second, small launch of the same call (one workgroup per batch row, a thread per tile) then finishes
// the rows: the row's maxima and sums from the tile partials in a fixed order, the ratio of the marked
// entries with exactly the arithmetic of cfg_sample.hip, the lowest index among equal maxima, and the
// log-probability.  (Finishing the rows inside the first launch, by whichever workgroup counts itself
// last, was built and measured: the device-wide visibility it needs within one launch - a release
// fence per workgroup, or written-through stores and uncached reads - and the registers the last
// workgroup's part adds to every wave cost more than the second launch's 2 us.)

#include <atomic>

#include "prepacked.hpp"

namespace {

struct HeadArgs {
    DevProblem p;            // x [2B, K] (M = 2B), the head's prepacked blob, y = logits [2B, V] or nullptr
    const uint16_t *noise;   // [B, V] bf16, strictly positive
    long long *sampled;      // [B]
    float *logprob;          // [B]
    u32x4_t *rec;            // [B, tiles][2]: {max gt, sum exp(gt - max), max ct, sum exp(ct - max)} as float bits,
                             // then {gt | q << 16, ct | mask << 16, column, 0} of the tile's first candidate
    uint16_t *gt;            // [B, V]
    uint16_t *ct;            // [B, V]
    int32_t B, tiles, rounds, reserved;
    float w, inv_t;
    // optional parts (vrl_int4_head_extras): each pointer may be null
    const uint16_t *bias;         // [V]: logits = bf16(bf16(x . W^T) + bias)
    const uint16_t *embed_table;  // [V, embed_dim]
    uint16_t *next_embeds;        // [2B, embed_dim]
    long long *tokens;            // [B, token_stride]
    float *logprobs;              // [B, token_stride]
    long long *position;          // device scalar: column of tokens / logprobs, incremented by the call
    long long *slot;              // device scalar incremented by the call
    long long *position_seen;     // in the workspace: the position as the first kernel found it
    const uint8_t *active;        // [B]: rows whose draw counts (null: all)
    int32_t embed_dim, token_stride;
    int32_t per_row, reserved2;   // per_row: position is [B] and slot [2B], one counter per row
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
// The wave that summed up tile `tile` ([2B rows] x 16 columns, accumulators in the MFMA layout: lane % 16 =
// column, rows 16 b + 4 (lane / 16) + i) leaves the logits, rounded to bf16 as the head's output tensor
// holds them, in the tile's [16 * MB][16] floats of LDS.
template <int MB>
__device__ __forceinline__ void head_tile_logits(const f32x4_t (&acc)[1][MB], float *tb) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int col = lane & 15, rg = lane >> 4;
#pragma unroll
    for (int b = 0; b < MB; ++b)
#pragma unroll
        for (int i = 0; i < 4; ++i) tb[(16 * b + 4 * rg + i) * 16 + col] = hs_round_bf16(acc[0][b][i]);
}

// the draw of the lane's entry: batch row lane / 16 + 4 j, column lane % 16 of the tile
__device__ __forceinline__ uint16_t head_noise(const HeadArgs &a, int tile, int j) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int b = (lane >> 4) + 4 * j;
    return as_global(a.noise)[(long)(b < a.B ? b : 0) * a.p.N + min(tile * 16 + (lane & 15), a.p.N - 1)];
}

// Wave j of the tile's waves takes the batch rows lane / 16 + 4 j (one per DPP row of 16 lanes, a lane per
// column): scaled rows, tile partials, first candidate and draw mask.  q16: head_noise(tile, j), requested
// before the tile's weights were streamed.
__device__ __forceinline__ void head_epilogue(const HeadArgs &a, int tile, const float *tb, int j, uint16_t q16) {
    typedef __attribute__((address_space(1))) u32x4_t *gptr_w4;
    const int lane = threadIdx.x & (WAVE - 1);
    const int col = lane & 15, rg = lane >> 4;
    const int B = a.B, V = a.p.N;
    const int n = tile * 16 + col;
    const bool col_ok = n < V;
    const int b = rg + 4 * j;                 // uniform over the 16 lanes of a DPP row
    const bool ok = b < B && col_ok;
    const int bb = b < B ? b : 0;
    float gtv, ctv;
    hs_scaled_pair(tb[bb * 16 + col], tb[(B + bb) * 16 + col], a.w, a.inv_t, gtv, ctv);
    const long at = (long)bb * V + (col_ok ? n : 0);
    const float q = bf16_bits_to_f32(q16);
    if (ok) {
        as_global(a.gt)[at] = hs_bf16_bits(gtv);
        as_global(a.ct)[at] = hs_bf16_bits(ctv);
    }
    const float gm = row16_max(ok ? gtv : -INFINITY), cm = row16_max(ok ? ctv : -INFINITY);
    const float eg = ok ? expf(gtv - gm) : 0.0f, ec = ok ? expf(ctv - cm) : 0.0f;
    const float gs = row16_sum(eg), cs = row16_sum(ec);
    // which entries can still win the draw (a NaN or an infinity compares in their favour), and the first of them
    float e = eg / q;
    e = e == e ? e : INFINITY;
    e = ok ? e : -INFINITY;
    const float eb = row16_max(e);
    const bool cand = ok && !(e < eb * HS_MARGIN);
    const uint32_t votes = (uint32_t)((__ballot(cand) >> (16 * rg)) & 0xFFFFu);
    const uint32_t bests = (uint32_t)((__ballot(ok && e == eb) >> (16 * rg)) & 0xFFFFu);
    const int best_col = bests ? __builtin_ctz(bests) : 0;
    const int from = 16 * rg + best_col;
    const uint32_t g_b = __shfl((int)hs_bf16_bits(gtv), from, WAVE) & 0xFFFFu;
    const uint32_t q_b = __shfl((int)q16, from, WAVE) & 0xFFFFu;
    const uint32_t c_b = __shfl((int)hs_bf16_bits(ctv), from, WAVE) & 0xFFFFu;
    if (col == 0 && b < B) {
        gptr_w4 dst = (gptr_w4)(uintptr_t)(a.rec + 2 * ((long)b * a.tiles + tile));
        dst[0] = __builtin_bit_cast(u32x4_t, f32x4_t{gm, gs, cm, cs});
        dst[1] = u32x4_t{g_b | (q_b << 16), c_b | (votes << 16), (uint32_t)best_col, 0u};
    }
}

// the same with the entry's cond / T riding along (the log-probability needs it for the winner)
__device__ __forceinline__ void hs_take_better(float &bv, int &bi, float &bc, float ov, int oi, float oc) {
    const bool other_nan = ov != ov, mine_nan = bv != bv;
    const bool take = mine_nan ? (other_nan && oi < bi) : (other_nan || ov > bv || (ov == bv && oi < bi));
    if (take) {
        bv = ov;
        bi = oi;
        bc = oc;
    }
}

// One workgroup finishes batch row blockIdx.x from what every tile left behind: TPT tiles per thread,
// their records requested as one batch.  The tile's first candidate is evaluated from the record; the
// other marked entries (rare) only if their tile's first comes within 2^-4 of the best ratio of the row
// (an entry the tile ranks below its first can exceed that first's ratio by rounding only: two
// roundings of 2^-8), and those are read from the scaled rows.
constexpr int MERGE_THREADS = 256;
template <int TPT>
__global__ __launch_bounds__(MERGE_THREADS) void head_merge_kernel(HeadArgs a) {
    typedef const __attribute__((address_space(1))) u32x4_t *gptr_cw4;
    constexpr int WAVES = MERGE_THREADS / WAVE;
    __shared__ float red_f[4][WAVES];
    __shared__ int red_i[WAVES];
    const int b = blockIdx.x, tid = threadIdx.x;
    const int wave = tid / WAVE, lane = tid % WAVE;
    const int tiles = a.tiles, V = a.p.N;
    gptr_cw4 rec = (gptr_cw4)(uintptr_t)(a.rec + 2 * (long)b * tiles);
    gptr_cu16 gtp = as_global(a.gt + (long)b * V), ctp = as_global(a.ct + (long)b * V);
    gptr_cu16 qp = as_global(a.noise + (long)b * V);
    f32x4_t pt[TPT];
    u32x4_t first_of[TPT];
#pragma unroll
    for (int k = 0; k < TPT; ++k) {
        const int tt = min(MERGE_THREADS * k + tid, tiles - 1);
        pt[k] = __builtin_bit_cast(f32x4_t, rec[2 * tt]);
        first_of[k] = rec[2 * tt + 1];
    }
    auto block_all = [&](float &v0, float &v1, bool is_max) {   // every thread ends with the block's two results
        v0 = is_max ? wave_max(v0) : wave_sum(v0);
        v1 = is_max ? wave_max(v1) : wave_sum(v1);
        __syncthreads();   // the buffer may still be read from the previous reduction
        if (lane == 0) {
            red_f[0][wave] = v0;
            red_f[1][wave] = v1;
        }
        __syncthreads();
        v0 = red_f[0][0];
        v1 = red_f[1][0];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) {   // one order in every thread
            v0 = is_max ? fmaxf(v0, red_f[0][w]) : v0 + red_f[0][w];
            v1 = is_max ? fmaxf(v1, red_f[1][w]) : v1 + red_f[1][w];
        }
    };
    float gm = -INFINITY, cm = -INFINITY;
#pragma unroll
    for (int k = 0; k < TPT; ++k) {
        const bool in = MERGE_THREADS * k + tid < tiles;
        gm = fmaxf(gm, in ? pt[k][0] : -INFINITY);
        cm = fmaxf(cm, in ? pt[k][2] : -INFINITY);
    }
    block_all(gm, cm, true);
    float gs = 0.0f, cs = 0.0f;
#pragma unroll
    for (int k = 0; k < TPT; ++k) {   // a fixed order of the sums
        const bool in = MERGE_THREADS * k + tid < tiles;
        gs += in ? pt[k][1] * expf(pt[k][0] - gm) : 0.0f;
        cs += in ? pt[k][3] * expf(pt[k][2] - cm) : 0.0f;
    }
    block_all(gs, cs, false);

    float bv = -INFINITY, bc = 0.0f;
    int bi = 0x7FFFFFFF;
    float first[TPT];
    uint32_t m[TPT];
#pragma unroll
    for (int k = 0; k < TPT; ++k) {
        const int t = MERGE_THREADS * k + tid;
        const uint32_t col = first_of[k][2] & 15u;
        const float p = hs_round_bf16(expf(bf16_bits_to_f32(first_of[k][0] & 0xFFFFu) - gm) / gs);
        first[k] = hs_round_bf16(p / bf16_bits_to_f32(first_of[k][0] >> 16));
        m[k] = t < tiles ? (first_of[k][1] >> 16) & ~(1u << col) : 0u;
        if (t < tiles) hs_take_better(bv, bi, bc, first[k], 16 * t + (int)col, bf16_bits_to_f32(first_of[k][1] & 0xFFFFu));
    }
    // the other marked entries of the tiles that are still in the race
    float seen = bv == bv ? bv : INFINITY, unused = 0.0f;
    block_all(seen, unused, true);
    const float floor_ratio = seen * 0.9375f;
    int more = 0;
#pragma unroll
    for (int k = 0; k < TPT; ++k) {
        if (!(first[k] >= floor_ratio) && first[k] == first[k]) m[k] = 0u;   // a NaN keeps its tile in
        more |= m[k] != 0u;
    }
    while (__syncthreads_or(more)) {   // block-uniform
        uint16_t g16[TPT], q16[TPT], c16[TPT];
#pragma unroll
        for (int k = 0; k < TPT; ++k) {
            const int idx = 16 * min(MERGE_THREADS * k + tid, tiles - 1) + (m[k] ? __builtin_ctz(m[k]) : 0);
            g16[k] = gtp[idx];
            q16[k] = qp[idx];
            c16[k] = ctp[idx];
        }
        more = 0;
#pragma unroll
        for (int k = 0; k < TPT; ++k) {
            const int idx = 16 * min(MERGE_THREADS * k + tid, tiles - 1) + (m[k] ? __builtin_ctz(m[k]) : 0);
            const float p = hs_round_bf16(expf(bf16_bits_to_f32(g16[k]) - gm) / gs);
            if (m[k]) hs_take_better(bv, bi, bc, hs_round_bf16(p / bf16_bits_to_f32(q16[k])), idx, bf16_bits_to_f32(c16[k]));
            m[k] &= m[k] - 1;
            more |= m[k] != 0u;
        }
    }
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1)
        hs_take_better(bv, bi, bc, __shfl_xor(bv, off, WAVE), __shfl_xor(bi, off, WAVE), __shfl_xor(bc, off, WAVE));
    __syncthreads();
    if (lane == 0) {
        red_f[2][wave] = bv;
        red_f[3][wave] = bc;
        red_i[wave] = bi;
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < WAVES; ++w) hs_take_better(bv, bi, bc, red_f[2][w], red_i[w], red_f[3][w]);
        if (bi >= V) {   // no tile at all: cannot happen (V >= 16)
            bi = 0;
            bc = bf16_bits_to_f32(ctp[0]);
        }
        a.sampled[b] = bi;
        const float lp = hs_round_bf16(bc - cm - logf(cs));
        a.logprob[b] = lp;
        const bool counts = !a.active || a.active[b] != 0;   // a row outside the step's batch keeps its state
        if (a.position && counts) {   // the step's bookkeeping (policy.py:695-696): token and log-probability at the position
            const long long pos = a.per_row ? a.position[b] : *a.position_seen;
            if (pos >= 0 && pos < a.token_stride) {
                if (a.tokens) a.tokens[(long)b * a.token_stride + pos] = bi;
                if (a.logprobs) a.logprobs[(long)b * a.token_stride + pos] = lp;
            }
            if (a.per_row) {
                a.position[b] = pos + 1;
                if (a.slot) {   // the conditional and the unconditional row of the pair
                    a.slot[b] += 1;
                    a.slot[a.B + b] += 1;
                }
            } else if (b == 0) {
                *a.position = pos + 1;
                if (a.slot) *a.slot += 1;
            }
        }
        red_i[0] = bi;
    }
    if (a.embed_table && (!a.active || a.active[b] != 0)) {   // uniform: the next input of both rows of the pair (policy.py:698-700)
        __syncthreads();
        const int token = red_i[0];
        const int words = a.embed_dim >> 3;   // 16-byte words per row
        gptr_cw4 src = (gptr_cw4)(uintptr_t)(a.embed_table + (long)token * a.embed_dim);
        typedef __attribute__((address_space(1))) u32x4_t *gptr_w4;
        gptr_w4 dst_c = (gptr_w4)(uintptr_t)(a.next_embeds + (long)b * a.embed_dim);
        gptr_w4 dst_u = (gptr_w4)(uintptr_t)(a.next_embeds + (long)(a.B + b) * a.embed_dim);
        for (int j = tid; j < words; j += MERGE_THREADS) {
            const u32x4_t v = src[j];
            dst_c[j] = v;
            dst_u[j] = v;
        }
    }
}

// KS waves split K of a tile, TW tiles per round, MB blocks of 16 activation rows (M = 2B <= 16 MB).
// LDS: staged activations, then TW x (KS - 1) x MB partial tiles.
template <int KS, int TW, int GQ, int MB>
__global__ __launch_bounds__(KS *TW *WAVE) void head_sample_kernel(HeadArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    const DevProblem &p = a.p;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tw = wave / KS, kw = wave % KS;
    const int lane = threadIdx.x & (WAVE - 1);
    uint16_t *xs = reinterpret_cast<uint16_t *>(smem);
    const int xstride = p.kc + XPAD;
    uint8_t *after_x = smem + (size_t)p.M * xstride * 2;
    f32x4_t *red = reinterpret_cast<f32x4_t *>(after_x) + tw * (KS - 1) * MB * WAVE;
    // the logit tile takes the place of the tile's partial sums once they are added up (1 KiB per row block
    // in at least 3 KiB): written by the wave that adds them up, read by the tile's waves after a barrier
    float *tb = reinterpret_cast<float *>(red);
    static_assert((KS - 1) * WAVE * sizeof(f32x4_t) >= 16 * 16 * sizeof(float), "the logit tile fits the partial tiles");
    static_assert(KS >= 2 * MB, "a wave per group of four batch rows");
    const int nsc = pp_nsc(p.K);
    const int per = (nsc + KS - 1) / KS;
    const int sc0 = min(nsc, kw * per), sc1 = min(nsc, sc0 + per);
    const rsrc_t rsrc = pp_blob_rsrc(p);
    const int t0 = blockIdx.x * TW * a.rounds, t1 = min(a.tiles, t0 + TW * a.rounds);
    // the second kernel's workgroups all need the position this call writes at, and one of them moves it on
    if (a.position && !a.per_row && blockIdx.x == 0 && threadIdx.x == 0) *a.position_seen = *a.position;
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
        uint16_t q16 = 0;
        if (kw < 2 * MB && tile < t1) q16 = head_noise(a, tile, kw);   // the tile's draws arrive while its weights stream
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
            if (a.bias) {   // uniform: the module adds its bias to its bf16 output tensor
                const float bias = bf16_bits_to_f32(as_global(a.bias)[min(tile * 16 + (lane & 15), p.N - 1)]);
#pragma unroll
                for (int b = 0; b < MB; ++b)
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[0][b][i] = hs_round_bf16(hs_round_bf16(acc[0][b][i]) + bias);
            }
            if (p.y) store_tile<MB, false>(p, tile, acc);
            head_tile_logits<MB>(acc, tb);
        }
        __syncthreads();   // the logits of the round's tiles are in LDS: the tile's waves share its batch rows
        if (kw < 2 * MB && tile < t1) head_epilogue(a, tile, tb, kw, q16);
        work = work && next >= 0;
        if (base + TW < t1) __syncthreads();   // the partial tiles are read before they are rewritten
    }
}

constexpr int HS_MAX_B = 16;
constexpr size_t HS_LDS_CAP = 160 * 1024;   // what a workgroup can have

size_t hs_align(size_t v) { return (v + 255) & ~(size_t)255; }

struct HeadLayout {
    size_t rec, gt, ct, pos, total;
};

HeadLayout head_layout(int B, int V) {
    const size_t tiles = ((size_t)V + 15) / 16;
    HeadLayout l;
    l.rec = 0;
    l.gt = l.rec + hs_align((size_t)B * tiles * 32);
    l.ct = l.gt + hs_align((size_t)B * V * sizeof(uint16_t));
    l.pos = l.ct + hs_align((size_t)B * V * sizeof(uint16_t));
    l.total = l.pos + 256;
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
    return vrl_launch(kernel, dim3(workgroups), dim3(KS * TW * WAVE), lds, stream, args);
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
                       void *hip_stream, const vrl_int4_head_extras *extras = nullptr) {
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
    args.rec = reinterpret_cast<u32x4_t *>(ws + lay.rec);
    args.gt = reinterpret_cast<uint16_t *>(ws + lay.gt);
    args.ct = reinterpret_cast<uint16_t *>(ws + lay.ct);
    args.B = B;
    args.tiles = V / 16;
    args.w = cfg_weight;
    args.inv_t = 1.0f / temperature;
    if (extras) {
        const vrl_int4_head_extras &e = *extras;
        if (e.embed_table || e.next_embeds) {
            if (!e.embed_table || !e.next_embeds) return VRL_INT4_ENULL;
            if (e.embed_dim < 8 || e.embed_dim % 8 != 0) return VRL_INT4_ESHAPE;
            if ((reinterpret_cast<uintptr_t>(e.embed_table) | reinterpret_cast<uintptr_t>(e.next_embeds)) & 15u)
                return VRL_INT4_EALIGN;
        }
        if ((e.tokens || e.logprobs || e.slot) && !e.position) return VRL_INT4_ENULL;
        if (e.active && !e.position_per_row) return VRL_INT4_ESHAPE;   // a partial batch needs a counter per row
        if (e.position && e.token_stride < 1) return VRL_INT4_ESHAPE;
        if ((reinterpret_cast<uintptr_t>(e.bias) & 1u) || (reinterpret_cast<uintptr_t>(e.tokens) & 7u) ||
            (reinterpret_cast<uintptr_t>(e.logprobs) & 3u) || (reinterpret_cast<uintptr_t>(e.position) & 7u) ||
            (reinterpret_cast<uintptr_t>(e.slot) & 7u))
            return VRL_INT4_EALIGN;
        args.bias = static_cast<const uint16_t *>(e.bias);
        args.embed_table = static_cast<const uint16_t *>(e.embed_table);
        args.next_embeds = static_cast<uint16_t *>(e.next_embeds);
        args.tokens = reinterpret_cast<long long *>(e.tokens);
        args.logprobs = e.logprobs;
        args.position = reinterpret_cast<long long *>(e.position);
        args.slot = reinterpret_cast<long long *>(e.slot);
        args.position_seen = reinterpret_cast<long long *>(ws + lay.pos);
        args.embed_dim = e.embed_dim;
        args.token_stride = e.token_stride;
        args.active = static_cast<const uint8_t *>(e.active);
        args.per_row = e.position_per_row ? 1 : 0;
    }
    // as many workgroups as the device holds at once: a second round of workgroups would stage x again
    const long per_cu = std::max<long>(1, std::min<long>(16 / (ks * tw), (long)(160 * 1024 / std::max<size_t>(lds, 1024))));
    const long capacity = per_cu * cu_count();
    long workgroups = (args.tiles + tw - 1) / tw;
    args.rounds = (int)std::min<long>(16, (workgroups + capacity - 1) / capacity);
    workgroups = (args.tiles + tw * args.rounds - 1) / (tw * args.rounds);
    hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
    int rc;
    if (mb == 1) {
        if (ks == 4 && tw == 1) rc = launch_head_group<4, 1, 1>(args, (int)workgroups, lds, stream);
        else if (ks == 4 && tw == 4) rc = launch_head_group<4, 4, 1>(args, (int)workgroups, lds, stream);
        else if (ks == 8 && tw == 1) rc = launch_head_group<8, 1, 1>(args, (int)workgroups, lds, stream);
        else if (ks == 8 && tw == 2) rc = launch_head_group<8, 2, 1>(args, (int)workgroups, lds, stream);
        else rc = launch_head_group<16, 1, 1>(args, (int)workgroups, lds, stream);
    } else {
        if (ks == 4) rc = launch_head_group<4, 4, 2>(args, (int)workgroups, lds, stream);
        else if (ks == 8) rc = launch_head_group<8, 2, 2>(args, (int)workgroups, lds, stream);
        else rc = launch_head_group<16, 1, 2>(args, (int)workgroups, lds, stream);
    }
    if (rc != VRL_INT4_OK) return rc;
    // the rows: one workgroup each
    if (args.tiles <= 4 * MERGE_THREADS)
        return vrl_launch(&head_merge_kernel<4>, dim3(B), dim3(MERGE_THREADS), 0, stream, args);
    return vrl_launch(&head_merge_kernel<16>, dim3(B), dim3(MERGE_THREADS), 0, stream, args);
}

// ---------------------------------------------------------------------------------------------
// The same launches for callers that cannot bring a workspace along: the library's own scratch.
// One array per GPU, in that GPU's memory from the moment the code object is loaded there until
// the process ends; its address is asked for once per device (the array's name in host code is a
// handle for that query, not a device address).
constexpr int HS_STATIC_MAX_V = 16384;
constexpr size_t HS_STATIC_BYTES = (size_t)HS_MAX_B * (HS_STATIC_MAX_V / 16) * 32 +
                                   2 * (size_t)HS_MAX_B * HS_STATIC_MAX_V * 2 + 256;   // 1,573,120 bytes
static __device__ __align__(256) unsigned char scratch[HS_STATIC_BYTES];

constexpr int HS_MAX_DEVICES = 64;

// the current device's copy of `scratch`
int scratch_address(void **out) {
    static std::atomic<void *> known[HS_MAX_DEVICES];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= HS_MAX_DEVICES) return VRL_INT4_ESHAPE;
    void *ptr = known[dev].load(std::memory_order_acquire);
    if (!ptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!ptr) return (int)hipErrorInvalidSymbol;
        known[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return VRL_INT4_OK;
}

}  // namespace

extern "C" {

int vrl_int4_head_sample_static_bf16(const vrl_int4_problem *head, const void *noise, int64_t *sampled,
                                     float *logprob, int B, float cfg_weight, float temperature,
                                     void *hip_stream) {
    if (!head) return VRL_INT4_ENULL;
    if (B < 1 || B > HS_MAX_B || head->N > HS_STATIC_MAX_V) return VRL_INT4_ELIMIT;
    void *ptr = nullptr;
    const int rc = scratch_address(&ptr);
    if (rc != VRL_INT4_OK) return rc;
    static_assert(HS_STATIC_BYTES % 256 == 0, "whole 256-byte lines");
    return head_sample_launch(head, noise, sampled, logprob, B, cfg_weight, temperature, ptr, HS_STATIC_BYTES,
                              hip_stream);
}

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

int vrl_int4_head_sample_ex_bf16(const vrl_int4_problem *head, const vrl_int4_head_extras *extras, const void *noise,
                                 int64_t *sampled, float *logprob, int B, float cfg_weight, float temperature,
                                 void *workspace, size_t workspace_bytes, void *hip_stream) {
    if (!extras) return VRL_INT4_ENULL;
    return head_sample_launch(head, noise, sampled, logprob, B, cfg_weight, temperature, workspace, workspace_bytes,
                              hip_stream, extras);
}

}  // extern "C"
