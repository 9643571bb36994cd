/*
 * C ABI of the decode-step kernels that sit between the int4 linears of a Llama decoder layer.
 *
 * One decode step of the reference calls the Hugging Face LlamaModel on a single new token per
 * row (vrl/models/families/janus_pro/policy.py:673-678) after concatenating per-row KV caches
 * (policy.py:664-671, vrl/models/ar.py:42-110).  Between the linears that vrl_int4.h covers, each
 * decoder layer of that model computes, on bf16 tensors (every tensor op in fp32, result rounded
 * to bf16):
 *   h      = residual + sublayer_output                       (LlamaDecoderLayer.forward)
 *   normed = weight * bf16( h * rsqrt(mean(h^2) + eps) )      (LlamaRMSNorm.forward)
 *   q, k   = x * cos + rotate_half(x) * sin                   (apply_rotary_pos_emb)
 *   cache[position] = k, v;  out = softmax(q . K^T * scaling + mask) . V   (Cache.update, sdpa)
 * These entry points compute exactly that for one new token per row over a preallocated cache,
 * with the position held in device memory so that a recorded HIP graph can be replayed.
 *
 * Conventions as in vrl_int4.h: caller-owned device memory, calls only enqueue on `hip_stream`
 * of the current device, no allocation, no synchronisation, no state; return 0, a hipError_t
 * value, or a VRL_INT4_E* code (nothing is enqueued then).
 */
#ifndef VRL_DECODE_H
#define VRL_DECODE_H

#include <stddef.h>
#include <stdint.h>

#include "vrl_int4.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Residual add and RMSNorm of M rows of K bf16 values (K % 8 == 0, K <= 16384):
 *   h = residual ? bf16(x + residual) : x;   y = weight * bf16(h * rsqrt(mean(h^2) + eps))
 * `h_out` receives h when it is not NULL (required when residual is given; may alias x or
 * residual).  Stands for `residual + hidden_states` followed by input_layernorm /
 * post_attention_layernorm / the model's final norm.  All pointers 16-byte aligned.
 */
int vrl_add_rmsnorm_bf16(const void *x, const void *residual, const void *weight, void *h_out,
                         void *y, int M, int K, float eps, void *hip_stream);

/*
 * Rotary embedding, cache append and attention of one new token per row.
 *   q        bf16 [M, n_heads * D]       query projections of the new token, row stride q_stride elements
 *   k, v     bf16 [M, n_kv_heads * D]    key / value projections, row stride kv_stride elements
 *   k_cache, v_cache  bf16 [M, n_kv_heads, L_max, D]   (the layout of transformers' StaticLayer)
 *   cos, sin bf16 [L_max, D]             rotary tables, row p = position p
 *   mask     uint8 [M, L_max]            1 = this cache slot may be attended (0 = prompt padding)
 *   position int64 device scalar p, 0 <= p < L_max: the slot the new token takes
 *   out      bf16 [M, n_heads * D]
 * Row m, head h: q and k are rotated with row p of the tables (each product and the sum rounded
 * to bf16, as the tensor ops do), the rotated k and v are written to slot p of the cache, and
 * out = softmax(q . K[0..p]^T * scaling, masked slots excluded) . V[0..p] with fp32 scores and
 * accumulation.  D is 64 or 128; n_heads % n_kv_heads == 0; L_max <= 8192.  A position outside
 * [0, L_max) makes the call a no-op on the device.  Calls for different layers (different
 * caches) are independent; two calls on the same cache must be ordered by the stream.
 */
int vrl_rope_attn_decode_bf16(const void *q, const void *k, const void *v, int q_stride, int kv_stride,
                              void *k_cache, void *v_cache, const void *cos, const void *sin,
                              const void *mask, const int64_t *position, void *out,
                              int M, int n_heads, int n_kv_heads, int D, int L_max, float scaling,
                              void *hip_stream);

/*
 * The same launch for few (row, head) pairs (M * n_heads <= 128; above that it is the launch above): the
 * cached slots of a pair are divided over 8, 4 or 2 workgroups (for up to 32, 64, 128 pairs), so that
 * a long cache is read by many compute units instead of one per pair; each leaves its running softmax
 * state in `workspace`, and whichever finishes last merges them in index order and writes `out`
 * (deterministic; no workgroup waits for another).  Results equal the launch above up to the order of
 * the fp32 sums.  A row at a position below 512 (768 where a pair has two workgroups) is left to one
 * workgroup per pair, with the launch above's arithmetic (one recorded launch serves a generation from its
 * first slot on); the workgroups that then have nothing to do cost about 1 us per launch, so a caller that
 * knows on the host that every row is below that line does better with the launch above.  `workspace`: vrl_rope_attn_decode_split_workspace_bytes(M, n_heads, D) bytes of device
 * memory, 256-byte aligned, whose first M * n_heads * 4 bytes are zero before the first launch (every
 * launch leaves them zero again); launches that share a workspace must be ordered by the stream.
 * No counterpart in the reference (its attention is the library's, policy.py:673-678).
 */
size_t vrl_rope_attn_decode_split_workspace_bytes(int M, int n_heads, int D);
int vrl_rope_attn_decode_split_bf16(const void *q, const void *k, const void *v, int q_stride, int kv_stride,
                                    void *k_cache, void *v_cache, const void *cos, const void *sin,
                                    const void *mask, const int64_t *position, void *out,
                                    int M, int n_heads, int n_kv_heads, int D, int L_max, float scaling,
                                    void *workspace, size_t workspace_bytes, void *hip_stream);

/*
 * vrl_rope_attn_decode_bf16 with one position per row: `positions` is int64 [M] in device memory and row m
 * takes slot positions[m] (rotary tables, cache append, attended range), for a chunk whose rows advance at
 * different times (the scheduler's partial batches: policy.py:631-645 steps a subset of the rows, which
 * vrl/models/ar.py:42-110 cuts out of the cache and puts back; over a static cache every row keeps its own
 * slot counter instead).  A row whose position lies outside [0, L_max) is left alone.  With `workspace`
 * not NULL it is the split form (vrl_rope_attn_decode_split_bf16, same preconditions), else the plain one.
 */
int vrl_rope_attn_decode_rows_bf16(const void *q, const void *k, const void *v, int q_stride, int kv_stride,
                                   void *k_cache, void *v_cache, const void *cos, const void *sin,
                                   const void *mask, const int64_t *positions, void *out,
                                   int M, int n_heads, int n_kv_heads, int D, int L_max, float scaling,
                                   void *workspace, size_t workspace_bytes, void *hip_stream);

/*
 * LoRA adapters on top of an int4 projection, for the decode step of a policy whose attention
 * projections carry PEFT adapters (vrl/models/families/janus_pro/policy.py:298-324: rank 32 on
 * q/k/v/o by default, policy.py:81-88); the wrapper computes
 *   result = base_layer(x) + lora_B(lora_A(x)) * scaling
 * Two launches per group of projections that share an input x [M, K] (bf16, M <= 32):
 *   vrl_lora_down_bf16:    t[m, off_i + j] = sum_k x[m,k] * A_i[j,k]         for every adapter i
 *   vrl_lora_up_add_bf16:  y_i[m,n] = bf16( y_i[m,n] + scaling_i * sum_j t[m, off_i + j] * B_i[n,j] )
 * with t a float32 [M, r_total] scratch buffer of the caller's, off_i the sum of the ranks before
 * adapter i.  The up-projection also takes t in pieces: float32 [M, t_parts, r_total] whose t_parts
 * rows per m are summed in order first (1 <= t_parts <= 256; 1 for what vrl_lora_down_bf16 wrote):
 * vrl_rope_attn_decode_lora_bf16 leaves the down-projection of its output in that form, one piece
 * per head.  Adapter weights are float32 (what PEFT keeps by default: everything in fp32, one
 * rounding when the result returns to bf16) or bf16 (weights_fp32 = 0: t, the up-projection and its
 * scaled value are rounded to bf16 as the bf16 modules round them); one type per launch.
 * 1 <= n_adapters <= 4, r % 8 == 0, r <= 64, K % 8 == 0, pointers 16-byte aligned.
 */
typedef struct vrl_lora_adapter {
    const void *A;     /* [r, K] row-major */
    const void *B;     /* [N, r] row-major */
    void *y;           /* bf16 [M, N], updated in place by vrl_lora_up_add_bf16 */
    int32_t N, r;
    float scaling;
    int32_t weights_fp32;
} vrl_lora_adapter;

int vrl_lora_down_bf16(const void *x, int M, int K, const vrl_lora_adapter *adapters, int n_adapters,
                       float *t, void *hip_stream);
int vrl_lora_up_add_bf16(const float *t, int t_parts, int M, const vrl_lora_adapter *adapters,
                         int n_adapters, void *hip_stream);

/*
 * vrl_int4_gemv_prepacked_bf16 and vrl_lora_down_bf16 of the same input in one launch: the base
 * projections of a group (q|k|v of one layer: the wrapper computes base_layer(x) and lora_A(x) from the
 * same x) and the down-projections of their adapters do not depend on each other, so the latter run
 * as extra workgroups of the same grid.  Every problem must read the same x [M, K] (M <= 32), none
 * may be a fused gate|up problem; `adapters`, `t` as for vrl_lora_down_bf16 (y and B are not used).
 */
int vrl_int4_gemv_prepacked_lora_bf16(const vrl_int4_problem *problems, int n_problems,
                                      const vrl_lora_adapter *adapters, int n_adapters, float *t,
                                      void *hip_stream);

/*
 * The launch above with the residual add and RMSNorm of vrl_int4_gemv_prepacked_norm_bf16 applied to the shared
 * input first, for both the base projections and the adapters (which read the normalised rows, as the wrapper's
 * lora_A does: input_layernorm precedes q|k|v in LlamaDecoderLayer.forward): a decoder layer under adapters then
 * needs no norm launch of its own in front of q|k|v.  `norm` as for vrl_int4_gemv_prepacked_norm_bf16; K <= 2048,
 * M <= 16 (the adapters' workgroups keep their rows in registers).
 */
int vrl_int4_gemv_prepacked_norm_lora_bf16(const vrl_int4_problem *problems, int n_problems,
                                           const vrl_int4_norm *norm, const vrl_lora_adapter *adapters,
                                           int n_adapters, float *t, void *hip_stream);

/*
 * vrl_int4_gemv_prepacked_bf16 of one problem and vrl_lora_up_add_bf16 of its adapter in one launch:
 *   y[m,n] = bf16( bf16(x . W^T)[m,n] + scaling * sum_j t[m,j] * B[n,j] )
 * with t [M, t_parts, r] as for vrl_lora_up_add_bf16 (the down-projection of the same x, e.g. the
 * pieces vrl_rope_attn_decode_lora_bf16 left) and the adapter's N equal to the problem's; A and y
 * of the adapter record are not used (the sum goes to the problem's y).  Not for a fused gate|up
 * problem.
 */
int vrl_int4_gemv_prepacked_lora_up_bf16(const vrl_int4_problem *problem, const vrl_lora_adapter *adapter,
                                         const float *t, int t_parts, void *hip_stream);

/*
 * vrl_rope_attn_decode_bf16 with the up-projections of the q, k, v adapters added while the new
 * token's projections are read, in place of a vrl_lora_up_add_bf16 launch between the int4 launch
 * and the attention: q, k, v hold the base projections' outputs, `t` the down-projections of the
 * group (vrl_lora_down_bf16), and the kernel attends with (and appends to the cache)
 *   q' = bf16(q + scaling_q * t[:, off_q : off_q + r_q] . B_q^T), likewise k', v'
 * with the roundings described above.  A NULL B means the projection has no adapter.  q, k and v
 * themselves are left as they are.
 * The adapter of the projection that consumes `out` (o_proj) can have its down-projection computed
 * here as well, in place of a vrl_lora_down_bf16 launch after the attention: with o_A given, the
 * workgroup of row m, head h writes
 *   o_t[m, h, j] = sum_d out[m, h * D + d] * o_A[j, h * D + d]        (out as rounded to bf16)
 * and vrl_lora_up_add_bf16(o_t, n_heads, ...) adds the up-projection of the heads' sum.
 * At least one of q_B, k_B, v_B, o_A must be given; t may be NULL when only o_A is.
 */
typedef struct vrl_attn_lora {
    const float *t;          /* [M, t_stride] float32, 16-byte aligned */
    int32_t t_stride;        /* a multiple of 4 */
    int32_t weights_fp32;    /* type of every B: 1 float32, 0 bf16 */
    const void *q_B, *k_B, *v_B;   /* [n_heads * D, r_q], [n_kv_heads * D, r_k], [n_kv_heads * D, r_v] */
    int32_t r[3];            /* ranks (q, k, v): multiples of 8 up to 64 */
    int32_t offset[3];       /* first column of each adapter in t, a multiple of 4 */
    float scaling[3];
    int32_t position_per_row; /* 1: `position` of the call is int64 [M], one slot per row (vrl_rope_attn_decode_rows_bf16) */
    const void *o_A;         /* [o_r, n_heads * D] (type as weights_fp32 says), 16-byte aligned, or NULL */
    float *o_t;              /* [M, n_heads, o_r] float32, 16-byte aligned */
    int32_t o_r;             /* a multiple of 8 up to 64 */
    int32_t reserved2;
} vrl_attn_lora;

int vrl_rope_attn_decode_lora_bf16(const void *q, const void *k, const void *v, int q_stride, int kv_stride,
                                   void *k_cache, void *v_cache, const void *cos, const void *sin,
                                   const void *mask, const int64_t *position, void *out,
                                   int M, int n_heads, int n_kv_heads, int D, int L_max, float scaling,
                                   const vrl_attn_lora *lora, void *hip_stream);

/*
 * The launches of a decode step issued from one host call.  A step of the native decoder layer is a list of
 * some 120 calls of the entry points above and of vrl_int4.h, and a host loop in an interpreted language needs
 * about as long to issue them as the device needs to run them.  A record names the entry point (`kind`) and
 * holds its arguments in the order of its declaration: pointers in p[], integers (int, size_t) in i[], floats
 * in f[]; `hip_stream` is the stream of every call.  The calls are issued in order; the first that fails ends
 * the walk: its return value is returned and, if `failed_at` is not NULL, its index is written there (nothing
 * is written when all succeed).  The records, and whatever they point to, stay the caller's.
 * No counterpart in the reference, whose step is the model's forward (policy.py:673-678).
 */
enum {
    VRL_CALL_GEMV = 1,          /* vrl_int4_gemv_prepacked_bf16 */
    VRL_CALL_GEMV_NORM = 2,     /* vrl_int4_gemv_prepacked_norm_bf16 */
    VRL_CALL_GEMV_EPILOGUE = 3, /* vrl_int4_gemv_prepacked_epilogue_bf16 */
    VRL_CALL_GEMV_LORA = 4,     /* vrl_int4_gemv_prepacked_lora_bf16 */
    VRL_CALL_GEMV_LORA_UP = 5,  /* vrl_int4_gemv_prepacked_lora_up_bf16 */
    VRL_CALL_ADD_RMSNORM = 6,   /* vrl_add_rmsnorm_bf16 */
    VRL_CALL_ATTN = 7,          /* vrl_rope_attn_decode_bf16 */
    VRL_CALL_ATTN_SPLIT = 8,    /* vrl_rope_attn_decode_split_bf16 */
    VRL_CALL_ATTN_ROWS = 9,     /* vrl_rope_attn_decode_rows_bf16 */
    VRL_CALL_ATTN_LORA = 10,    /* vrl_rope_attn_decode_lora_bf16 */
    VRL_CALL_LORA_DOWN = 11,    /* vrl_lora_down_bf16 */
    VRL_CALL_LORA_UP_ADD = 12,  /* vrl_lora_up_add_bf16 */
    VRL_CALL_GEMV_NORM_LORA = 13 /* vrl_int4_gemv_prepacked_norm_lora_bf16 */
};
typedef struct vrl_step_call {
    int32_t kind;
    int32_t reserved;        /* 0 */
    const void *p[12];
    int64_t i[8];
    float f[2];
} vrl_step_call;

int vrl_decode_run_calls(const vrl_step_call *calls, int n_calls, int *failed_at, void *hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* VRL_DECODE_H */
