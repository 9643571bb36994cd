/*
 * C ABI of the MI355X (gfx950) int4 weight-only decode linears.
 *
 * These entry points replace, for autoregressive rollout decode, the bf16
 * nn.Linear calls the reference reaches through
 *   vrl/models/families/janus_pro/policy.py:673-678  (Llama trunk: q/k/v/o_proj,
 *                                                      gate/up/down_proj)
 *   vrl/models/families/janus_pro/policy.py:138-160  (gen_head, image-token logits)
 * The reference has no FFI of its own for this path (it is pure Python on
 * torch); a binding is a ctypes stub over this header.
 *
 * Operand formats (row-major, caller-owned device memory, 16-byte aligned):
 *   x        bf16  [M, K]            activations
 *   qweight  int32 [N, K/8]          nibble i (bits 4i..4i+3) of word r = q[n, 8r+i], q in [0,15]
 *   scales   bf16  [N, K/G]          one scale per group of G consecutive k
 *   qzeros   int32 [N, ceil(K/G/8)]  zero-points, same nibble order along the group axis,
 *                                    unused high nibbles of the last word are 0
 *   y        bf16  [M, N]
 * Arithmetic:
 *   w[n,k] = bf16_rne( (float)(q[n,k] - z[n,k/G]) * (float)s[n,k/G] )   (bit-exact)
 *   y[m,n] = bf16_rne( sum_k (float)x[m,k] * w[n,k] )                   (fp32 accumulate,
 *                                                                        order unspecified)
 * Scales must be finite bf16 numbers; zero, negative and subnormal scales are allowed.
 *
 * Every call only enqueues work on `hip_stream` (a hipStream_t, NULL = the
 * default stream) of the current device; it does not allocate, synchronise or
 * keep state, and is re-entrant.  Return value: 0 on success, a hipError_t
 * value (1..999) if the launch failed, or one of the VRL_INT4_E* codes below if
 * the arguments violate a precondition (nothing is enqueued then).
 * Preconditions: M >= 1, N >= 1, K >= 8, K % 8 == 0, G % 8 == 0, K % G == 0,
 * non-NULL 16-byte aligned pointers, N * K < 2^40.
 */
#ifndef VRL_INT4_H
#define VRL_INT4_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VRL_INT4_ABI_VERSION 1

#define VRL_INT4_OK 0
#define VRL_INT4_ESHAPE 1001  /* M, N, K or G violates a precondition */
#define VRL_INT4_EALIGN 1002  /* a pointer is not 16-byte aligned */
#define VRL_INT4_ENULL 1003   /* a required pointer is NULL */
#define VRL_INT4_EPLAN 1004   /* malformed or undersized grouped plan */
#define VRL_INT4_ELIMIT 1005  /* beyond the fixed size of the library's own scratch memory */

int vrl_int4_abi_version(void);

/* Static text for a return code of this library ("hip error" for 1..999). */
const char *vrl_int4_error_string(int code);

/*
 * y[M,N] = x[M,K] . dequant(qweight, scales, qzeros)^T.
 * Replaces one nn.Linear.forward of the decode step
 * (policy.py:673-678 trunk projections; policy.py:160 gen_head).
 */
int vrl_int4_gemv_bf16(const void *x, const void *qweight, const void *scales,
                       const void *qzeros, void *y, int M, int N, int K, int G,
                       void *hip_stream);

/*
 * w[N,K] (bf16) = dequant(qweight, scales, qzeros): the canonical weight tile,
 * bit-exact.  Used by the loader glue and by the train-time replay path that
 * keeps bf16 weights (policy.py:419-424).
 */
int vrl_int4_dequant_bf16(const void *qweight, const void *scales, const void *qzeros,
                          void *w, int N, int K, int G, void *hip_stream);

/*
 * Fused front half of LlamaMLP (down_proj(act_fn(gate_proj(x)) * up_proj(x)),
 * reached from policy.py:673-678):  y[M,I] = bf16( silu(x.Wg^T) * (x.Wu^T) ),
 * accumulators, SiLU and product in fp32.  The packed operand has 2*I rows:
 * rows 0..I-1 are gate_proj, rows I..2I-1 are up_proj.
 */
int vrl_int4_gate_up_silu_bf16(const void *x, const void *qweight_gu, const void *scales_gu,
                               const void *qzeros_gu, void *y, int M, int I, int K, int G,
                               void *hip_stream);

/*
 * One-time repack of a canonical operand triple (group size 32, 64 or 128) into the
 * MFMA-shaped blob the grouped launch streams fastest: every wave load is one
 * contiguous KiB and the matrix cores do the scale/zero arithmetic.  Loader
 * glue: runs once per weight after the policy is built (the reference builds
 * its policy at vrl/models/families/janus_pro/builder.py:11-33).
 * vrl_int4_prepacked_bytes() is the blob size (0 if the shape has no prepacked
 * form: G not in {32, 64, 128}, K % 128 != 0, or a blob of 2 GiB or more); the
 * blob needs 16-byte alignment.  The
 * arithmetic contract is unchanged: the weights a kernel rebuilds from the blob
 * are bit for bit the canonical dequantised tile.
 */
size_t vrl_int4_prepacked_bytes(int N, int K, int G);
int vrl_int4_prepack(const void *qweight, const void *scales, const void *qzeros, void *packed,
                     int N, int K, int G, void *hip_stream);

/*
 * Grouped launch: several independent GEMVs (for example q/k/v of one layer, or
 * a whole decode step's weight set when the caller streams them back to back)
 * in ONE kernel launch, so small matrices share the machine instead of paying
 * one launch latency each.
 *
 * A plan is a flat byte blob built on the host, copied by the caller into
 * device memory once, and reused for every launch while the pointers stay
 * valid.  vrl_int4_grouped_plan_size() gives its size; vrl_int4_grouped_plan_build()
 * validates every problem against the preconditions above (and, in addition,
 * requires K % 128 == 0, G a power of two >= 32 and M <= 16 per problem; a
 * prepacked problem takes M <= 32, needs G in {32, 64, 128} and, if fused, N/2 a
 * multiple of 16; the prepacked problems of a plan with more tiles than the
 * device has workgroup slots share one group size, which is 128 if the plan
 * also holds canonical problems),
 * fills a host buffer and a small launch descriptor; vrl_int4_gemv_grouped_bf16()
 * takes the DEVICE copy of the blob plus that descriptor.  The plan is built for
 * the current device (its CU count sizes the launch).
 */
typedef struct vrl_int4_problem {
    const void *x;
    const void *qweight;
    const void *scales;
    const void *qzeros;
    void *y;
    int32_t M, N, K, G;
    int32_t fused_gate_up; /* 0: y[M,N]; 1: rows are gate||up, y[M,N/2] with the SiLU epilogue */
    int32_t prepacked;     /* 1: qweight is a blob made by vrl_int4_prepack(); scales/qzeros unused */
    int32_t reserved[2];   /* 0 */
} vrl_int4_problem;

typedef struct vrl_int4_plan_info {
    int32_t n_problems;    /* records in the blob */
    int32_t total_tiles;   /* 16-column output tiles over all problems */
    int32_t grid;          /* workgroups of the launch */
    int32_t block_threads; /* threads per workgroup */
    int32_t lds_bytes;     /* dynamic LDS per workgroup */
    int32_t variant;       /* which record kinds the plan holds (selects the kernel build) */
    int32_t reserved[2];
} vrl_int4_plan_info;

/*
 * Plan-free launch of a few prepacked GEMVs that share a kernel (one nn.Linear.forward over a
 * prepacked weight, or the q|k|v / gate|up linears of one decoder layer, policy.py:673-678):
 * the records travel as kernel arguments, the waves of a workgroup split K of a 16-column
 * tile.  Meant for decode and rollout batches (the launch is one memory round trip).  Every
 * problem must have prepacked = 1; activations are taken in slabs of at most 16 rows (fewer
 * where a slab is staged in LDS and does not fit it: K > 16384, or K > 4096 with adapters'
 * down-projections in the launch), and all slabs of a call together may number at
 * most 8 (for K = 2048: three problems of 32 rows), else VRL_INT4_ESHAPE and the caller uses
 * a grouped plan or vrl_int4_gemv_bf16.  scales and qzeros of the records are ignored.
 */
int vrl_int4_gemv_prepacked_bf16(const vrl_int4_problem *problems, int n_problems, void *hip_stream);

/*
 * The same launch with the residual add and the RMSNorm that precede the linears of a decoder
 * layer applied to the activations on their way in (LlamaDecoderLayer.forward:
 * `hidden_states = residual + hidden_states`, then input_layernorm / post_attention_layernorm,
 * then q|k|v or gate|up; reached from policy.py:673-678):
 *   h = residual ? bf16(x + residual) : x;   x' = weight * bf16(h * rsqrt(mean(h^2) + eps))
 * and every problem multiplies x' (never written to memory) instead of x.  All problems share
 * the input: problems[i].x == norm->x, same M and K, K <= 4096.  `h_out`, when not NULL,
 * receives h ([M, K]); it must not be the memory of x or residual (workgroups read those
 * while another one writes h).  Roundings are those of the tensor ops (see vrl_decode.h).
 */
typedef struct vrl_int4_norm {
    const void *x;        /* bf16 [M, K]: output of the previous sublayer (or the embedding) */
    const void *residual; /* bf16 [M, K] residual stream, NULL for none */
    const void *weight;   /* bf16 [K] norm weight */
    void *h_out;          /* bf16 [M, K] or NULL */
    float eps;
    int32_t reserved;
} vrl_int4_norm;

int vrl_int4_gemv_prepacked_norm_bf16(const vrl_int4_problem *problems, int n_problems,
                                      const vrl_int4_norm *norm, void *hip_stream);

/*
 * The plan-free launch of ONE plain prepacked problem with the linear's bias and a following activation
 * applied to each tile before it is stored:
 *   y = act(bf16(bf16(x . W^T) + bias))
 * i.e. the roundings of a bf16 module that adds its bias to its output tensor and whose activation is a
 * tensor op of its own.  This is the first half of a two-layer image-token head (Linear, GELU, Linear:
 * what `gen_head` is in the Janus-Pro checkpoints, called at policy.py:138-160) and any biased linear.
 * `norm` may be NULL; when given, the residual add and RMSNorm of vrl_int4_gemv_prepacked_norm_bf16 are
 * applied to the activations on their way in (the trunk's final norm in front of the head).
 * bias: bf16 [N] or NULL.  activation: VRL_INT4_ACT_NONE, or VRL_INT4_ACT_GELU for
 * x / 2 * (1 + erf(x / sqrt(2))) evaluated in fp32 on the bf16 value and rounded to bf16 (torch.nn.GELU()).
 * residual: bf16 [M, N] or NULL, added last: y = bf16(residual + that) — the `residual + hidden_states` that
 * follows o_proj and down_proj in LlamaDecoderLayer.forward (reached from policy.py:673-678), so that the
 * residual stream is written by the launch that produces the sublayer's output; it may be the memory of y.
 */
#define VRL_INT4_ACT_NONE 0
#define VRL_INT4_ACT_GELU 1
typedef struct vrl_int4_epilogue {
    const void *bias;
    const void *residual;
    int32_t activation;
    int32_t reserved;   /* 0 */
} vrl_int4_epilogue;

int vrl_int4_gemv_prepacked_epilogue_bf16(const vrl_int4_problem *problem, const vrl_int4_norm *norm,
                                          const vrl_int4_epilogue *epilogue, void *hip_stream);

size_t vrl_int4_grouped_plan_size(int n_problems);

/* Fills plan_host (plan_bytes >= vrl_int4_grouped_plan_size(n_problems)) and *info. */
int vrl_int4_grouped_plan_build(const vrl_int4_problem *problems, int n_problems,
                                void *plan_host, size_t plan_bytes, vrl_int4_plan_info *info);

int vrl_int4_gemv_grouped_bf16(const void *plan_dev, const vrl_int4_plan_info *info,
                               void *hip_stream);

/*
 * Tail of a decode step after the image-token head, one launch (replaces the tensor ops of
 * vrl/models/families/janus_pro/policy.py:686-693):
 *   guided  = uncond + cfg_weight * (cond - uncond)
 *   probs   = softmax(guided / temperature)
 *   sampled = argmax(probs / noise)                  (torch.multinomial(probs, 1) for noise ~ Exp(1))
 *   logprob = log_softmax(cond / temperature)[sampled]
 * logits is bf16 [2B, V] with the conditional rows first (policy.py:685 chunks it that way), noise
 * bf16 [B, V] of strictly positive draws, sampled int64 [B], logprob float [B].  Every step is
 * computed in fp32 and rounded to bf16 where the reference's bf16 tensors are (the division by
 * the temperature is the product with fl(1/temperature), as torch divides by a host scalar);
 * the sums of the two softmaxes are fp32 in a fixed order.  Equal maxima resolve to the lowest index.
 * Preconditions: B >= 1, V >= 1, temperature > 0, non-NULL naturally aligned pointers.
 */
int vrl_cfg_sample_bf16(const void *logits, const void *noise, int64_t *sampled, float *logprob,
                        int B, int V, float cfg_weight, float temperature, void *hip_stream);

/*
 * The image-token head and the tail of the decode step in ONE launch (replaces the head linear of
 * vrl/models/families/janus_pro/policy.py:684 together with the tensor ops of policy.py:685-693):
 *   logits  = x . dequant(head)^T                    bf16 [2B, V], conditional rows first
 *   guided, probs, sampled, logprob                  as vrl_cfg_sample_bf16 states them
 * `head` is one prepacked problem: x bf16 [2B, K] (M = 2B), qweight the blob of the [V, K] head,
 * y NULL (the logits are not wanted: they never reach memory) or bf16 [2B, V]; noise bf16 [B, V];
 * sampled int64 [B]; logprob float [B].  Two kernels are enqueued: the tiles of the head leave
 * per-tile softmax partials, the scaled rows and a mask of the entries that can still win the draw in
 * `workspace`; a small second kernel (one workgroup per batch row) completes the rows from them, with
 * the arithmetic of vrl_cfg_sample_bf16 (the softmax sums are added up in another, fixed order).
 * workspace: device memory of at least vrl_int4_head_sample_workspace_bytes(B, V) bytes, 256-byte
 * aligned, contents irrelevant on entry.  Two calls that overlap in time must not share a workspace.
 * Preconditions beyond the library's: 1 <= B <= 16, 16 <= V <= 65536 with V % 16 == 0, temperature > 0,
 * G in {32, 64, 128}, and the 2B activation rows fit the LDS of a workgroup beside the kernel's partial
 * tiles (for example K = 2048 at up to 32 rows, K = 4096 at up to 16, K = 8192 at up to 8): else
 * VRL_INT4_ESHAPE and the caller launches head and tail separately.
 */
size_t vrl_int4_head_sample_workspace_bytes(int B, int V);
int vrl_int4_head_sample_bf16(const vrl_int4_problem *head, const void *noise, int64_t *sampled,
                              float *logprob, int B, float cfg_weight, float temperature,
                              void *workspace, size_t workspace_bytes, void *hip_stream);

/*
 * vrl_int4_head_sample_bf16 with the parts of the decode step that surround it (each optional):
 *   bias         bf16 [V] of a biased head: logits = bf16(bf16(x . W^T) + bias), the roundings of a bf16 module
 *                that adds its bias to its output tensor (the last linear of Janus' two-layer head has one)
 *   position     device scalar p (0 <= p < token_stride): tokens[b, p] = sampled[b], logprobs[b, p] = logprob[b]
 *                (policy.py:695-696), then p + 1 is stored back; slot, if given, is incremented as well (the
 *                cache slot counter of a static decode loop)
 *   embed_table  bf16 [V, embed_dim], row t the input embedding of image token t (what
 *                prepare_gen_img_embeds returns for it, policy.py:698-700): rows b and B + b of next_embeds
 *                (bf16 [2B, embed_dim]) receive row sampled[b]; embed_dim a multiple of 8, 16-byte aligned rows
 *   position_per_row = 1: position is int64 [B] and slot int64 [2B], one counter per batch row (pair of
 *                rows), for a chunk whose rows advance at different times; `active` (uint8 [B], NULL: all) then
 *                names the rows of this step's batch: only they are written, counted on and given a next input
 *                (sampled / logprob are computed for every row; noise rows of the others are not used)
 * All of it is done by the call's second kernel, one workgroup per batch row.  workspace as for
 * vrl_int4_head_sample_bf16.
 */
typedef struct vrl_int4_head_extras {
    const void *bias;
    const void *embed_table;
    void *next_embeds;
    int64_t *tokens;
    float *logprobs;
    int64_t *position;
    int64_t *slot;
    int32_t embed_dim;
    int32_t token_stride;
    const uint8_t *active;
    int32_t position_per_row;
    int32_t reserved;   /* 0 */
} vrl_int4_head_extras;

int vrl_int4_head_sample_ex_bf16(const vrl_int4_problem *head, const vrl_int4_head_extras *extras, const void *noise,
                                 int64_t *sampled, float *logprob, int B, float cfg_weight, float temperature,
                                 void *workspace, size_t workspace_bytes, void *hip_stream);

/*
 * vrl_int4_head_sample_bf16 without a workspace argument, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): no
 * counterpart in the reference.  The partials, masks and scaled rows go to a fixed array that the
 * library holds in the memory of every GPU it runs on (1,573,120 bytes, kept until the process ends),
 * so the call allocates nothing.  Limits: B <= 16 and V <= 16384, else VRL_INT4_ELIMIT (nothing is
 * enqueued); everything else as vrl_int4_head_sample_bf16.  Every call on a GPU uses that GPU's one
 * array: calls that overlap in time on one GPU (two streams, two threads) race and must be ordered by
 * the caller.  The first call on a device looks the array's address up (no allocation, but make it
 * outside a stream capture).
 */
int vrl_int4_head_sample_static_bf16(const vrl_int4_problem *head, const void *noise, int64_t *sampled,
                                     float *logprob, int B, float cfg_weight, float temperature,
                                     void *hip_stream);

#ifdef __cplusplus
}
#endif

#endif /* VRL_INT4_H */
