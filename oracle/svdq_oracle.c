/*
 * CPU oracle, C restatement (TEST INFRASTRUCTURE -- never linked into the product library).
 *
 * Scalar loops for the byte/integer work of the SVDQuant path, written independently of the
 * tensor-op restatement in svdq_oracle.py so the two can be checked against each other:
 *
 *   - nibble unpack and exact per-group int32 dot products
 *       reference: nunchaku/ops/triton/gemm_w4a4.py:12-14, 400-407, 477-483
 *   - the activation quantizer's fp32 op order (signed and unsigned)
 *       reference: nunchaku/ops/triton/gemm_w4a4.py:1397-1455
 *   - the W4A4 GEMM's scaled accumulation + LoRA-up + bias in fp32
 *       reference: nunchaku/ops/triton/gemm_w4a4.py:156-209, 483
 *   - TinyChat AWQ nibble decode and the per-group GEMV
 *       reference: nunchaku/ops/triton/awq.py:29-47, 137-182
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off: no fused multiply-add may be formed,
 * every fp32 operation below rounds once, exactly as written).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even fp32 -> bf16 (NaN kept quiet) */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static inline int nib(const uint8_t *row, int k, int is_signed) {
    int v = (row[k >> 1] >> ((k & 1) * 4)) & 0xF;
    return (is_signed && v >= 8) ? v - 16 : v;
}

/* p[m*N + n] = sum_{k in group g} a[m,k] * w[n,k]; act (M, K/2), wgt (N, K/2) bytes. */
void oracle_group_acc_i32(const uint8_t *act, const uint8_t *wgt, int32_t *p, int M, int N, int K, int g,
                          int act_unsigned) {
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            int32_t s = 0;
            for (int k = g * 64; k < g * 64 + 64; k++)
                s += nib(act + (size_t)m * (K / 2), k, !act_unsigned) * nib(wgt + (size_t)n * (K / 2), k, 1);
            p[(size_t)m * N + n] = s;
        }
}

/*
 * Quantizer.  x (M, K) bf16 bits; smooth (K) bf16 bits or NULL; out (M, K/2); scales (K/64, ld_s) bf16 bits,
 * element [g, m]; lora_down (K, R) bf16 bits or NULL; lora_act (M, R) fp32.
 */
void oracle_quantize_act(const uint16_t *x, const uint16_t *smooth, const uint16_t *lora_down, uint8_t *out,
                         uint16_t *scales, float *lora_act, int M, int K, int R, int ld_s, int is_unsigned,
                         float shift) {
    const float qmax = is_unsigned ? 15.0f : 7.0f;
    const float lo = is_unsigned ? 0.0f : -8.0f, hi = is_unsigned ? 15.0f : 7.0f;
    for (int m = 0; m < M; m++) {
        if (lora_down)
            for (int r = 0; r < R; r++) lora_act[(size_t)m * R + r] = 0.0f;
        for (int g = 0; g < K / 64; g++) {
            float v[64];
            float gmax = 0.0f; /* max(.., 0) */
            if (lora_down)
                for (int r = 0; r < R; r++) {
                    float s = 0.0f;
                    for (int j = 0; j < 64; j++) {
                        int k = g * 64 + j;
                        s += bf16_to_f32(x[(size_t)m * K + k]) * bf16_to_f32(lora_down[(size_t)k * R + r]);
                    }
                    lora_act[(size_t)m * R + r] += s;
                }
            for (int j = 0; j < 64; j++) {
                int k = g * 64 + j;
                float t = bf16_to_f32(x[(size_t)m * K + k]);
                t = t + shift;
                if (smooth) t = t * (1.0f / bf16_to_f32(smooth[k]));
                v[j] = t;
                float a = is_unsigned ? t : fabsf(t);
                if (a > gmax) gmax = a;
            }
            float scale = gmax / qmax;
            float safe = (scale == 0.0f) ? 1.0f : scale;
            scales[(size_t)g * ld_s + m] = f32_to_bf16(scale);
            float rs = 1.0f / safe;
            for (int j = 0; j < 64; j += 2) {
                int c[2];
                for (int e = 0; e < 2; e++) {
                    volatile float q = v[j + e] * rs;
                    volatile float r = q + 12582912.0f;
                    float rr = r - 12582912.0f;
                    if (rr < lo) rr = lo;
                    if (rr > hi) rr = hi;
                    c[e] = ((int)rr) & 0xF;
                }
                out[(size_t)m * (K / 2) + (g * 64 + j) / 2] = (uint8_t)(c[0] | (c[1] << 4));
            }
        }
    }
}

/*
 * fp32 GEMM result before the final rounding: sequential over groups acc += (f32(p) * as) * ws, then the
 * LoRA-up product on the hidden state rounded to bf16, then bias.  ascales (K/64, lda), wscales (K/64, ldw).
 */
void oracle_gemm_w4a4(const uint8_t *act, const uint8_t *wgt, const uint16_t *ascales, const uint16_t *wscales,
                      const uint16_t *bias, const float *lora_act, const uint16_t *lora_up, float *out, int M,
                      int N, int K, int R, int lda, int ldw, int act_unsigned) {
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            float acc = 0.0f;
            for (int g = 0; g < K / 64; g++) {
                int32_t s = 0;
                for (int k = g * 64; k < g * 64 + 64; k++)
                    s += nib(act + (size_t)m * (K / 2), k, !act_unsigned) * nib(wgt + (size_t)n * (K / 2), k, 1);
                float t = (float)s * bf16_to_f32(ascales[(size_t)g * lda + m]);
                t = t * bf16_to_f32(wscales[(size_t)g * ldw + n]);
                acc = acc + t;
            }
            if (lora_up && R) {
                float l = 0.0f;
                for (int r = 0; r < R; r++)
                    l += bf16_to_f32(f32_to_bf16(lora_act[(size_t)m * R + r])) * bf16_to_f32(lora_up[(size_t)n * R + r]);
                acc = acc + l;
            }
            if (bias) acc = acc + bf16_to_f32(bias[n]);
            out[(size_t)m * N + n] = acc;
        }
}

/* TinyChat decode: logical (n, k) -> uint4, packed int16 [N/4][K]. */
int oracle_awq_nibble(const uint16_t *packed, int K, int n, int k) {
    int a = n / 4, b = n % 4;
    int t = (k / 32) * 8 + (k % 8);
    int e = (t / 16) * 64 + b * 16 + (t % 16);
    return (packed[(size_t)a * K + e] >> (4 * ((k % 32) / 8))) & 0xF;
}

/* out[m*N+n] (fp32) = sum_c s[c,n] * sum_k x q + z[c,n] * sum_k x, group 64. */
void oracle_awq_gemv(const uint16_t *x, const uint16_t *packed, const uint16_t *scales, const uint16_t *zeros,
                     float *out, int M, int N, int K) {
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            float acc = 0.0f;
            for (int c = 0; c < K / 64; c++) {
                float dq = 0.0f, xs = 0.0f;
                for (int k = c * 64; k < c * 64 + 64; k++) {
                    float xv = bf16_to_f32(x[(size_t)m * K + k]);
                    dq += xv * (float)oracle_awq_nibble(packed, K, n, k);
                    xs += xv;
                }
                acc += bf16_to_f32(scales[(size_t)c * N + n]) * dq + bf16_to_f32(zeros[(size_t)c * N + n]) * xs;
            }
            out[(size_t)m * N + n] = acc;
        }
}
