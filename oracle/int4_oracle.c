/*
 * CPU oracle for the int4 weight-only decode linears, plain C.
 * TEST INFRASTRUCTURE ONLY: the shipped library never links or calls this.
 *
 * It restates, with scalar loops and its own bf16 rounding, the operator that
 * replaces the bf16 nn.Linear calls the reference makes at
 * vrl/models/families/janus_pro/policy.py:673-678 (Llama trunk: q/k/v/o,
 * gate/up/down projections) and policy.py:138-160 (gen_head):
 *
 *     w[n,k] = bf16_rne( (float)(q[n,k] - z[n,k/G]) * (float)s[n,k/G] )
 *     y[m,n] = bf16_rne( sum_k (float)x[m,k] * w[n,k] )        fp32 accumulate
 *
 * The reference holds no quantised operator and no numeric vector for this
 * path, so parity against it is UNPINNED; tests/test_oracle.py pins this file
 * against exact integer arithmetic, the numpy restatement and torch's bf16
 * rounding instead.
 *
 * Layout: qweight int32 [N, K/8], nibble i of word r = q[n, 8r+i];
 * scales bf16 bits [N, K/G]; qzeros int32 [N, ceil(K/G/8)], same nibble order;
 * x bf16 bits [M, K]; y bf16 bits [M, N].
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bf16_to_f32(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

/* round-to-nearest-even by inspecting the discarded half word */
static uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu) != 0)
        return (uint16_t)((u >> 16) | 0x0040u); /* NaN stays NaN */
    uint32_t keep = u >> 16;
    uint32_t drop = u & 0xFFFFu;
    if (drop > 0x8000u || (drop == 0x8000u && (keep & 1u)))
        keep += 1u;
    return (uint16_t)keep;
}

static int nibble(const int32_t *words, long idx) {
    uint32_t w = (uint32_t)words[idx >> 3];
    return (int)((w >> (4 * (idx & 7))) & 0xFu);
}

static int check(int M, int N, int K, int G) {
    if (M < 0 || N < 0 || K <= 0 || G <= 0) return 1;
    if (K % 8 != 0 || G % 8 != 0 || K % G != 0) return 1;
    return 0;
}

uint16_t vrl_oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }
float vrl_oracle_bf16_to_f32(uint16_t b) { return bf16_to_f32(b); }

/* one dequantised weight, as bf16 bits */
static uint16_t dequant_one(const int32_t *qweight, const uint16_t *scales,
                            const int32_t *qzeros, int n, int k, int K, int G) {
    int groups = K / G;
    int zwords = (groups + 7) / 8;
    int g = k / G;
    int q = nibble(qweight + (long)n * (K / 8), k);
    int z = nibble(qzeros + (long)n * zwords, g);
    float s = bf16_to_f32(scales[(long)n * groups + g]);
    return f32_to_bf16((float)(q - z) * s);
}

int vrl_oracle_dequant_bf16(const int32_t *qweight, const uint16_t *scales,
                            const int32_t *qzeros, uint16_t *w, int N, int K, int G) {
    if (check(0, N, K, G)) return 1;
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k)
            w[(long)n * K + k] = dequant_one(qweight, scales, qzeros, n, k, K, G);
    return 0;
}

/* y in double, no output rounding: the truth the tolerance is measured from;
 * yabs (optional) receives sum_k |x w| */
int vrl_oracle_gemv_f64(const uint16_t *x, const int32_t *qweight, const uint16_t *scales,
                        const int32_t *qzeros, double *y, double *yabs,
                        int M, int N, int K, int G) {
    if (check(M, N, K, G)) return 1;
    for (int n = 0; n < N; ++n) {
        for (int m = 0; m < M; ++m) {
            double acc = 0.0, aacc = 0.0;
            for (int k = 0; k < K; ++k) {
                double w = bf16_to_f32(dequant_one(qweight, scales, qzeros, n, k, K, G));
                double p = (double)bf16_to_f32(x[(long)m * K + k]) * w;
                acc += p;
                aacc += fabs(p);
            }
            y[(long)m * N + n] = acc;
            if (yabs) yabs[(long)m * N + n] = aacc;
        }
    }
    return 0;
}

/* the operator: sequential fp32 accumulation in k order, bf16 output */
int vrl_oracle_gemv_bf16(const uint16_t *x, const int32_t *qweight, const uint16_t *scales,
                         const int32_t *qzeros, uint16_t *y, int M, int N, int K, int G) {
    if (check(M, N, K, G)) return 1;
    for (int n = 0; n < N; ++n) {
        for (int m = 0; m < M; ++m) {
            float acc = 0.0f;
            for (int k = 0; k < K; ++k) {
                float w = bf16_to_f32(dequant_one(qweight, scales, qzeros, n, k, K, G));
                acc += bf16_to_f32(x[(long)m * K + k]) * w;
            }
            y[(long)m * N + n] = f32_to_bf16(acc);
        }
    }
    return 0;
}

/* fused MLP front half over a gate||up operand of 2*I rows:
 * y[m,i] = bf16( silu(acc_gate) * acc_up ), accumulators and epilogue in fp32 */
int vrl_oracle_gate_up_silu_bf16(const uint16_t *x, const int32_t *qweight, const uint16_t *scales,
                                 const int32_t *qzeros, uint16_t *y,
                                 int M, int I, int K, int G) {
    if (check(M, 2 * I, K, G)) return 1;
    for (int i = 0; i < I; ++i) {
        for (int m = 0; m < M; ++m) {
            float g = 0.0f, u = 0.0f;
            for (int k = 0; k < K; ++k) {
                float xv = bf16_to_f32(x[(long)m * K + k]);
                g += xv * bf16_to_f32(dequant_one(qweight, scales, qzeros, i, k, K, G));
                u += xv * bf16_to_f32(dequant_one(qweight, scales, qzeros, I + i, k, K, G));
            }
            float act = g / (1.0f + expf(-g));
            y[(long)m * I + i] = f32_to_bf16(act * u);
        }
    }
    return 0;
}
