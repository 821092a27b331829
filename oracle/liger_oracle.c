/*
 * liger_oracle.c -- CPU restatement (plain C + OpenMP) of Liger's per-GPU hot path.
 *
 * TEST INFRASTRUCTURE ONLY: the parity checker and the reported CPU baseline.  The shipped GPU
 * path never calls into this file.  See liger_oracle.h for how each function is pinned.
 *
 * Citations are relative to the reference tree (src/...).
 */
#include "liger_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------------------------ */
/* binary16 round trip (software, nearest-even; no dependence on F16C)                         */
/* ------------------------------------------------------------------------------------------ */
uint16_t lo_f32_to_f16_bits(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t mag = x & 0x7fffffffu;
    if (mag >= 0x7f800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((mag > 0x7f800000u) ? 0x200u : 0u));
    }
    if (mag >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (mag < 0x38800000u) { /* subnormal half or zero: |f| < 2^-14 */
        if (mag < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 */
        uint32_t e = mag >> 23;                        /* biased float exponent */
        uint32_t m = (mag & 0x7fffffu) | 0x800000u;    /* 24-bit significand */
        uint32_t shift = 126u - e;                     /* 14..24: bits dropped below half ulp 2^-24 */
        uint32_t half_m = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1u);
        if (rem > halfway || (rem == halfway && (half_m & 1u))) half_m++;
        return (uint16_t)(sign | half_m);
    }
    /* normal */
    uint32_t e = (mag >> 23) - 112u;
    uint32_t m = mag & 0x7fffffu;
    uint32_t h = (e << 10) | (m >> 13);
    uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}

float lo_f16_bits_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    uint32_t x;
    if (e == 0) {
        if (m == 0) {
            x = sign;
        } else {
            float v = (float)m * 5.9604644775390625e-8f; /* 2^-24 */
            memcpy(&x, &v, 4);
            x |= sign;
        }
    } else if (e == 31) {
        x = sign | 0x7f800000u | (m << 13);
    } else {
        x = sign | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

float lo_round_f16(float x) { return lo_f16_bits_to_f32(lo_f32_to_f16_bits(x)); }

void lo_round_f16_array(float* x, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) x[i] = lo_round_f16(x[i]);
}

int lo_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* storage rounding: identity for fp32, binary16 round trip for fp16 */
static inline float st(float x, int dtype) { return dtype == LO_F16 ? lo_round_f16(x) : x; }

/* ------------------------------------------------------------------------------------------ */
/* synthetic data                                                                              */
/* ------------------------------------------------------------------------------------------ */
static inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static inline uint32_t sum16x4(uint64_t r) {
    return (uint32_t)(r & 0xffffu) + (uint32_t)((r >> 16) & 0xffffu) + (uint32_t)((r >> 32) & 0xffffu) +
           (uint32_t)(r >> 48);
}

void lo_fill_normal(float* out, int64_t n, uint64_t seed, uint64_t tensor_id, float mean,
                    float stddev, int dtype) {
    /* 1/sqrt(8*(65536^2-1)/12) as the nearest float */
    const float inv_sigma = 0x1.3988e2p-16f;
    const uint64_t key = splitmix64(seed * 0x100000001B3ull + tensor_id);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        uint64_t a = splitmix64(key + 2ull * (uint64_t)i);
        uint64_t b = splitmix64(key + 2ull * (uint64_t)i + 1ull);
        int32_t s = (int32_t)(sum16x4(a) + sum16x4(b)) - 262140;
        float z = (float)s * inv_sigma;
        float v = stddev * z;
        __asm__ volatile("" : "+x"(v)); /* keeps the compiler from contracting the two roundings into an FMA */
        v = v + mean;
        out[i] = st(v, dtype);
    }
}

/* ------------------------------------------------------------------------------------------ */
/* GEMMs                                                                                       */
/* ------------------------------------------------------------------------------------------ */
void lo_gemm_naive_f64(int M, int N, int K, const float* X, int ldx, const float* W, int ldw,
                       double* Y, int ldy) {
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            double acc = 0.0;
            for (int k = 0; k < K; ++k) acc += (double)X[(int64_t)i * ldx + k] * (double)W[(int64_t)k * ldw + j];
            Y[(int64_t)i * ldy + j] = acc;
        }
}

/* Blocked fp32 GEMM with explicit leading dimensions: Y[M,N] = X[M,K]*W[K,N], row-major.
 * Register tile 4 rows x 16 columns, K blocked so the W panel stays in cache. */
#define KB 256
#define NB 256
static void gemm_rm(int M, int N, int K, const float* X, int64_t ldx, const float* W, int64_t ldw,
                    float* Y, int64_t ldy, int dtype) {
    if (M <= 0 || N <= 0) return;
    const int n_iblk = (M + 3) / 4;
    const int n_jblk = (N + NB - 1) / NB;
#pragma omp parallel for collapse(2) schedule(dynamic, 4)
    for (int jb = 0; jb < n_jblk; ++jb) {
        for (int ib = 0; ib < n_iblk; ++ib) {
            const int i0 = ib * 4, j0 = jb * NB;
            const int mi = (M - i0) < 4 ? (M - i0) : 4;
            const int nj = (N - j0) < NB ? (N - j0) : NB;
            float acc[4][NB];
            for (int r = 0; r < 4; ++r)
                for (int j = 0; j < NB; ++j) acc[r][j] = 0.f;
            for (int k0 = 0; k0 < K; k0 += KB) {
                const int kk = (K - k0) < KB ? (K - k0) : KB;
                if (mi == 4) {
                    const float* x0 = X + (int64_t)(i0 + 0) * ldx + k0;
                    const float* x1 = X + (int64_t)(i0 + 1) * ldx + k0;
                    const float* x2 = X + (int64_t)(i0 + 2) * ldx + k0;
                    const float* x3 = X + (int64_t)(i0 + 3) * ldx + k0;
                    for (int k = 0; k < kk; ++k) {
                        const float* w = W + (int64_t)(k0 + k) * ldw + j0;
                        const float a0 = x0[k], a1 = x1[k], a2 = x2[k], a3 = x3[k];
#pragma omp simd
                        for (int j = 0; j < nj; ++j) {
                            const float wv = w[j];
                            acc[0][j] += a0 * wv;
                            acc[1][j] += a1 * wv;
                            acc[2][j] += a2 * wv;
                            acc[3][j] += a3 * wv;
                        }
                    }
                } else {
                    for (int r = 0; r < mi; ++r) {
                        const float* x = X + (int64_t)(i0 + r) * ldx + k0;
                        for (int k = 0; k < kk; ++k) {
                            const float* w = W + (int64_t)(k0 + k) * ldw + j0;
                            const float a = x[k];
#pragma omp simd
                            for (int j = 0; j < nj; ++j) acc[r][j] += a * w[j];
                        }
                    }
                }
            }
            for (int r = 0; r < mi; ++r) {
                float* y = Y + (int64_t)(i0 + r) * ldy + j0;
                for (int j = 0; j < nj; ++j) y[j] = st(acc[r][j], dtype);
            }
        }
    }
}

void lo_gemm(int M, int N, int K, const float* X, const float* W, float* Y, int dtype) {
    gemm_rm(M, N, K, X, K, W, N, Y, N, dtype);
}

/* generic strided element access: col-major op(A)[i,l] */
static inline float at_cm(const float* A, int lda, int trans, int i, int l) {
    return trans ? A[(int64_t)i * lda + l] : A[(int64_t)l * lda + i];
}

void lo_gemm_ex(int transa, int transb, int m, int n, int k, const float* A, int lda, const float* B,
                int ldb, float* C, int ldc, int dtype) {
    if (!transa && !transb) {
        /* col-major C[m x n] = A[m x k] B[k x n]  ==  row-major C'[n, m] = B'[n, k] A'[k, m] */
        gemm_rm(n, m, k, B, ldb, A, lda, C, ldc, dtype);
        return;
    }
#pragma omp parallel for collapse(2) schedule(static)
    for (int j = 0; j < n; ++j)
        for (int i = 0; i < m; ++i) {
            float acc = 0.f;
            for (int l = 0; l < k; ++l) acc += at_cm(A, lda, transa, i, l) * at_cm(B, ldb, transb, l, j);
            C[(int64_t)j * ldc + i] = st(acc, dtype);
        }
}

void lo_gemm_strided_batched(int transa, int transb, int m, int n, int k, const float* A, int lda,
                             int64_t strideA, const float* B, int ldb, int64_t strideB, float* C,
                             int ldc, int64_t strideC, int batch, int dtype) {
    for (int b = 0; b < batch; ++b)
        lo_gemm_ex(transa, transb, m, n, k, A + b * strideA, lda, B + b * strideB, ldb, C + b * strideC,
                   ldc, dtype);
}

/* ------------------------------------------------------------------------------------------ */
/* bias + GELU   cuda_kernels.cu:9-29 (gelu), :59-84 (add_bias_gelu)                           */
/* ------------------------------------------------------------------------------------------ */
/* gelu(x + b) with the rounding points of the instantiation */
static float bias_gelu_one(float v, float b, int dtype) {
    if (dtype == LO_F32) {
        /* float instantiation, :9-15 */
        float x = v + b;
        float cdf = 0.5f * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
        return x * cdf;
    }
    /* half2 specialisation, :17-29,:72-84: add in half, cube in half (two rounded products), tanh in fp32,
     * cdf rounded to half, product in half */
    float x = lo_round_f16(v + b);
    float x2 = lo_round_f16(x * x);
    float x3 = lo_round_f16(x * x2);
    float cdf = 0.5f * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x3)));
    return lo_round_f16(x * lo_round_f16(cdf));
}

void lo_add_bias_gelu(float* out, const float* bias, int m, int n, int dtype) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < m; ++i) {
        float* row = out + (int64_t)i * n;
        for (int j = 0; j < n; ++j) row[j] = bias_gelu_one(row[j], bias[j], dtype);
    }
}

/* GeGLU (no reference counterpart; the FFN of the GLM family): in [m, 2f] = [gate | up], bias [2f];
 * out[i][j] = gelu(gate + b_gate) * (up + b_up), every operation rounded like the kernels above. */
void lo_add_bias_geglu(float* out, const float* in, const float* bias, int m, int f, int dtype) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < m; ++i) {
        const float* row = in + (int64_t)i * 2 * f;
        for (int j = 0; j < f; ++j) {
            const float g = bias_gelu_one(row[j], bias[j], dtype);
            const float u = st(row[f + j] + bias[f + j], dtype);
            out[(int64_t)i * f + j] = st(g * u, dtype);
        }
    }
}

/* ------------------------------------------------------------------------------------------ */
/* LayerNorm family                                                                            */
/* ------------------------------------------------------------------------------------------ */
/* two-pass statistics exactly as layer_norm_kernel_generalize does them (cuda_kernels.cu:463-508):
 * mean = sum/n; var = sum((x-mean)^2)/n; scale = rsqrt(var + 1e-6).
 * `msrc` holds the values the mean is summed over (x itself for every kernel but add_bias_input_layernorm_2). */
static void ln_row2(const float* x, const float* msrc, const float* gamma, const float* beta, float* y, int n,
                    int dtype) {
    double s = 0.0; /* the GPU tree-reduces in fp32; double here is the mathematically cleaner stand-in */
    for (int j = 0; j < n; ++j) s += msrc[j];
    float mean = (float)(s / n);
    double v = 0.0;
    for (int j = 0; j < n; ++j) {
        float d = x[j] - mean;
        v += (double)d * d;
    }
    float rstd = 1.0f / sqrtf((float)(v / n) + 1e-6f);
    for (int j = 0; j < n; ++j) y[j] = st(((x[j] - mean) * rstd) * gamma[j] + beta[j], dtype);
}

static void ln_row(const float* x, const float* gamma, const float* beta, float* y, int n, int dtype) {
    ln_row2(x, x, gamma, beta, y, n, dtype);
}

void lo_layer_norm(const float* in, const float* gamma, const float* beta, float* out, int m, int n,
                   int dtype) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < m; ++i) ln_row(in + (int64_t)i * n, gamma, beta, out + (int64_t)i * n, n, dtype);
}

/* cuda_kernels.cu:115-185: out = LN(out + input + bias)*gamma + beta, in place, fp32 math on the
 * (half-precision) inputs; the sum is NOT stored before normalising. */
void lo_add_bias_input_layernorm(float* out, const float* input, const float* bias, const float* gamma,
                                 const float* beta, int m, int n, int dtype) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < m; ++i) {
        float* o = out + (int64_t)i * n;
        const float* in = input + (int64_t)i * n;
        float* tmp = (float*)malloc(sizeof(float) * (size_t)n);
        for (int j = 0; j < n; ++j) tmp[j] = o[j] + in[j] + bias[j];
        ln_row(tmp, gamma, beta, o, n, dtype);
        free(tmp);
    }
}

/* cuda_kernels.cu:360-409: output = T(input + output + bias) is stored; the mean is summed over the UNROUNDED fp32
 * sums (:377-384), the variance and the normalised output re-read the stored, rounded values (:392-408).  In half
 * precision the two differ by the mean rounding error of the row, which a row of near-ties makes visible. */
void lo_add_bias_input_layernorm_2(const float* input, const float* gamma, const float* beta,
                                   const float* bias, float* output, float* norm_output, int m, int n,
                                   int dtype) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < m; ++i) {
        float* o = output + (int64_t)i * n;
        const float* in = input + (int64_t)i * n;
        float* raw = (float*)malloc(sizeof(float) * (size_t)n);
        for (int j = 0; j < n; ++j) {
            float t = in[j];
            t += o[j];
            t += bias[j];
            raw[j] = t;
            o[j] = st(t, dtype);
        }
        ln_row2(o, raw, gamma, beta, norm_output + (int64_t)i * n, n, dtype);
        free(raw);
    }
}

/* cuda_kernels.cu:438-452: output = output + input + bias, evaluated left to right in T */
void lo_add_bias_input(float* output, const float* bias, const float* input, int m, int n, int dtype) {
#pragma omp parallel for schedule(static)
    for (int i = 0; i < m; ++i) {
        float* o = output + (int64_t)i * n;
        const float* in = input + (int64_t)i * n;
        for (int j = 0; j < n; ++j) o[j] = st(st(o[j] + in[j], dtype) + bias[j], dtype);
    }
}

/* ------------------------------------------------------------------------------------------ */
/* attention helpers                                                                           */
/* ------------------------------------------------------------------------------------------ */
/* attention_kernels.cu:79-224: buf[b,head,s,:] = X[b,s,head,:] + bias[head,:] */
void lo_add_qkv_bias_transpose(float* q_buf, float* k_buf, float* v_buf, const float* Q,
                               const float* bias_Q, const float* K, const float* bias_K, const float* V,
                               const float* bias_V, int batch, int seq, int head_num, int size_per_head,
                               int dtype) {
    const float* src[3] = {Q, K, V};
    const float* bia[3] = {bias_Q, bias_K, bias_V};
    float* dst[3] = {q_buf, k_buf, v_buf};
    const int n = head_num * size_per_head;
    for (int t = 0; t < 3; ++t) {
#pragma omp parallel for collapse(2) schedule(static)
        for (int b = 0; b < batch; ++b)
            for (int s = 0; s < seq; ++s)
                for (int h = 0; h < head_num; ++h)
                    for (int e = 0; e < size_per_head; ++e) {
                        int64_t si = ((int64_t)(b * seq + s)) * n + h * size_per_head + e;
                        int64_t di = (((int64_t)b * head_num + h) * seq + s) * size_per_head + e;
                        dst[t][di] = st(src[t][si] + bia[t][h * size_per_head + e], dtype);
                    }
    }
}

/* attention_kernels.cu:331-371: QKV packed [M,3,n], bias [3,n] */
void lo_add_fused_qkv_bias_transpose(float* q_buf, float* k_buf, float* v_buf, const float* QKV,
                                     const float* qkv_bias, int batch, int seq, int head_num,
                                     int size_per_head, int dtype) {
    float* dst[3] = {q_buf, k_buf, v_buf};
    const int n = head_num * size_per_head;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < batch; ++b)
        for (int s = 0; s < seq; ++s)
            for (int t = 0; t < 3; ++t)
                for (int h = 0; h < head_num; ++h)
                    for (int e = 0; e < size_per_head; ++e) {
                        int64_t si = (((int64_t)(b * seq + s)) * 3 + t) * n + h * size_per_head + e;
                        int64_t di = (((int64_t)b * head_num + h) * seq + s) * size_per_head + e;
                        dst[t][di] = st(QKV[si] + qkv_bias[(int64_t)t * n + h * size_per_head + e], dtype);
                    }
}

/* attn_softmax_kernelLauncher (attention_kernels.cu:621-680) picks one of three arithmetic variants by seq and T:
 *   t = qk*scalar + (1-mask)*(-10000);  e = exp(t - max t);  s = sum e + 1e-6
 *   odd seq (softmax_kernel / _v2, :397-478)            fp32 math, out = T(e / s)
 *   even seq <= 32, or float (_v3_LE32 / _v3, :482-617) fp32 math, out = T(e * (1/s))
 *   even seq > 32 and half (half2 _v3, :525-576)        t formed in half (scale product, 1-mask, its product with
 *       -10000 and the sum each rounded), max subtracted and exponentiated in half (h2exp), the two columns a thread
 *       holds (2i, 2i+1) added IN HALF before the fp32 block sum, 1/s rounded to half, product in half. */
void lo_attn_softmax(float* buffer, const float* attr_mask, int batch, int seq, int head_num,
                     float scalar, int dtype) {
    const float sc = st(scalar, dtype); /* bert_layer.h:94 stores the scalar as T */
    const int half2_path = dtype != LO_F32 && seq % 2 == 0 && seq > 32;
    const int divide = seq % 2 != 0;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < batch; ++b)
        for (int h = 0; h < head_num; ++h) {
            float* t = (float*)malloc(sizeof(float) * (size_t)(seq > 0 ? seq : 1));
            for (int sq = 0; sq < seq; ++sq) {
                float* row = buffer + (((int64_t)b * head_num + h) * seq + sq) * seq;
                const float* mrow = attr_mask + ((int64_t)b * seq + sq) * seq;
                float mx = -1e20f;
                for (int j = 0; j < seq; ++j) {
                    float v;
                    if (!half2_path) {
                        v = row[j] * sc + (1.0f - mrow[j]) * -10000.0f;
                    } else {
                        float mterm = lo_round_f16(lo_round_f16(1.0f - mrow[j]) * -10000.0f);
                        v = lo_round_f16(lo_round_f16(sc * row[j]) + mterm);
                    }
                    t[j] = v;
                    mx = v > mx ? v : mx;
                }
                float sum = 0.f;
                if (!half2_path) {
                    for (int j = 0; j < seq; ++j) {
                        t[j] = expf(t[j] - mx);
                        sum += t[j];
                    }
                } else {
                    for (int j = 0; j < seq; j += 2) {
                        t[j] = lo_round_f16(expf(lo_round_f16(t[j] - mx)));
                        t[j + 1] = lo_round_f16(expf(lo_round_f16(t[j + 1] - mx)));
                        sum += lo_round_f16(t[j] + t[j + 1]);
                    }
                }
                if (divide) {
                    const float s = sum + 1e-6f;
                    for (int j = 0; j < seq; ++j) row[j] = st(t[j] / s, dtype);
                } else if (!half2_path) {
                    const float inv = 1.0f / (sum + 1e-6f);
                    for (int j = 0; j < seq; ++j) row[j] = st(t[j] * inv, dtype);
                } else {
                    const float inv = lo_round_f16(1.0f / (sum + 1e-6f));
                    for (int j = 0; j < seq; ++j) row[j] = lo_round_f16(t[j] * inv);
                }
            }
            free(t);
        }
}

/* attention_kernels.cu:682-710: dst[b,s,head,:] = src[b,head,s,:] */
void lo_transpose(float* dst, const float* src, int batch, int seq, int head_num, int size_per_head) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < batch; ++b)
        for (int h = 0; h < head_num; ++h)
            for (int s = 0; s < seq; ++s)
                memcpy(dst + (((int64_t)b * seq + s) * head_num + h) * size_per_head,
                       src + (((int64_t)b * head_num + h) * seq + s) * size_per_head,
                       sizeof(float) * (size_t)size_per_head);
}

/* ------------------------------------------------------------------------------------------ */
/* fused prefill attention and decode attention                                                */
/* ------------------------------------------------------------------------------------------ */
void lo_attn_prefill(const float* q_buf, const float* k_buf, const float* v_buf, float* out, int batch,
                     int seq, int head_num, int size_per_head, float scalar, int causal, int dtype) {
    const int S = seq, d = size_per_head;
    const int64_t nbh = (int64_t)batch * head_num;
    float* scores = (float*)malloc(sizeof(float) * (size_t)(nbh * S * S));
    float* mask = (float*)malloc(sizeof(float) * (size_t)((int64_t)batch * S * S));
    for (int b = 0; b < batch; ++b)
        for (int i = 0; i < S; ++i)
            for (int j = 0; j < S; ++j) mask[((int64_t)b * S + i) * S + j] = (!causal || j <= i) ? 1.f : 0.f;
    /* qk_gemm  bert_layer.h:145-150: (T,N, S,S,d, K,d, Q,d, QK,S) */
    lo_gemm_strided_batched(1, 0, S, S, d, k_buf, d, (int64_t)S * d, q_buf, d, (int64_t)S * d, scores, S,
                            (int64_t)S * S, (int)nbh, dtype);
    lo_attn_softmax(scores, mask, batch, S, head_num, scalar, dtype);
    /* qkv_gemm bert_layer.h:158-163: (N,N, d,S,S, V,d, P,S, O,d) */
    lo_gemm_strided_batched(0, 0, d, S, S, v_buf, d, (int64_t)S * d, scores, S, (int64_t)S * S, out, d,
                            (int64_t)S * d, (int)nbh, dtype);
    free(scores);
    free(mask);
}

void lo_attn_decode(const float* q, const float* k_cache, const float* v_cache, float* out, int batch,
                    int head_num, int size_per_head, int len, int max_len, float scalar, int dtype) {
    const int d = size_per_head;
    const float sc = st(scalar, dtype);
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < batch; ++b)
        for (int h = 0; h < head_num; ++h) {
            const float* qv = q + ((int64_t)b * head_num + h) * d;
            const float* kc = k_cache + ((int64_t)b * head_num + h) * max_len * d;
            const float* vc = v_cache + ((int64_t)b * head_num + h) * max_len * d;
            float* o = out + ((int64_t)b * head_num + h) * d;
            float* p = (float*)malloc(sizeof(float) * (size_t)len);
            float mx = -1e20f;
            for (int j = 0; j < len; ++j) {
                float acc = 0.f;
                for (int e = 0; e < d; ++e) acc += qv[e] * kc[(int64_t)j * d + e];
                float sraw = st(acc, dtype); /* the score matrix is stored in T by qk_gemm */
                float v = (dtype == LO_F32) ? sraw * sc : lo_round_f16(lo_round_f16(sc * sraw) + 0.0f);
                p[j] = v;
                mx = v > mx ? v : mx;
            }
            float sum = 0.f;
            for (int j = 0; j < len; ++j) {
                float e = (dtype == LO_F32) ? expf(p[j] - mx)
                                            : lo_round_f16(expf(lo_round_f16(p[j] - lo_round_f16(mx))));
                p[j] = e;
                sum += e;
            }
            float inv = st(1.0f / (sum + 1e-6f), dtype);
            for (int j = 0; j < len; ++j) p[j] = st(p[j] * inv, dtype);
            for (int e = 0; e < d; ++e) {
                float acc = 0.f;
                for (int j = 0; j < len; ++j) acc += p[j] * vc[(int64_t)j * d + e];
                o[e] = st(acc, dtype);
            }
            free(p);
        }
}

/* ------------------------------------------------------------------------------------------ */
/* layer assembly                                                                              */
/* ------------------------------------------------------------------------------------------ */
static float* falloc(int64_t n) { return (float*)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1)); }
static float* zeros(int64_t n) { return (float*)calloc((size_t)(n > 0 ? n : 1), sizeof(float)); }

static int shape_ok(const lo_layer_shape* sh) {
    return sh && sh->batch > 0 && sh->seq > 0 && sh->hidden > 0 && sh->head_num > 0 && sh->size_per_head > 0 &&
           sh->ffn_inner > 0;
}

/* Bert_MHA::forward  bert_layer.h:121-175 */
int lo_mha_forward(const lo_layer_shape* sh, const lo_layer_weights* w, const float* mask, const float* in,
                   float* out) {
    if (!shape_ok(sh)) return -1;
    const int B = sh->batch, S = sh->seq, H = sh->hidden, h = sh->head_num, d = sh->size_per_head;
    const int M = B * S, Hl = h * d, dt = sh->dtype;
    const float scalar = 1.0f / sqrtf((float)d); /* bert_layer.h:94 */
    float *q = falloc((int64_t)M * Hl), *k = falloc((int64_t)M * Hl), *v = falloc((int64_t)M * Hl);
    float *qb = falloc((int64_t)M * Hl), *kb = falloc((int64_t)M * Hl), *vb = falloc((int64_t)M * Hl);
    float *ao = falloc((int64_t)M * Hl), *at = falloc((int64_t)M * Hl);
    lo_gemm(M, Hl, H, in, w->wq, q, dt); /* idx 0..2 */
    lo_gemm(M, Hl, H, in, w->wk, k, dt);
    lo_gemm(M, Hl, H, in, w->wv, v, dt);
    lo_add_qkv_bias_transpose(qb, kb, vb, q, w->bq, k, w->bk, v, w->bv, B, S, h, d, dt); /* idx 3 */
    if (mask && !sh->causal) {
        float* scores = falloc((int64_t)B * h * S * S);
        lo_gemm_strided_batched(1, 0, S, S, d, kb, d, (int64_t)S * d, qb, d, (int64_t)S * d, scores, S,
                                (int64_t)S * S, B * h, dt);                                /* idx 4 */
        lo_attn_softmax(scores, mask, B, S, h, scalar, dt);                                /* idx 5 */
        lo_gemm_strided_batched(0, 0, d, S, S, vb, d, (int64_t)S * d, scores, S, (int64_t)S * S, ao, d,
                                (int64_t)S * d, B * h, dt);                                /* idx 6 */
        free(scores);
    } else {
        lo_attn_prefill(qb, kb, vb, ao, B, S, h, d, scalar, sh->causal, dt);               /* idx 4..6 */
    }
    lo_transpose(at, ao, B, S, h, d);     /* idx 7 */
    lo_gemm(M, H, Hl, at, w->wo, out, dt); /* idx 8 */
    free(q); free(k); free(v); free(qb); free(kb); free(vb); free(ao); free(at);
    return 0;
}

/* Bert_MLP::forward  bert_layer.h:48-62 */
int lo_mlp_forward(const lo_layer_shape* sh, const lo_layer_weights* w, const float* in, float* out) {
    if (!shape_ok(sh)) return -1;
    const int M = sh->batch * sh->seq, H = sh->hidden, F = sh->ffn_inner, dt = sh->dtype;
    float* t = falloc((int64_t)M * F);
    if (sh->ffn_act == LO_FFN_GEGLU) {
        float* t2 = falloc((int64_t)M * 2 * F);
        lo_gemm(M, 2 * F, H, in, w->w1, t2, dt);
        lo_add_bias_geglu(t, t2, w->b1, M, F, dt);
        free(t2);
    } else {
        lo_gemm(M, F, H, in, w->w1, t, dt);   /* idx 11 */
        lo_add_bias_gelu(t, w->b1, M, F, dt); /* idx 12 */
    }
    lo_gemm(M, H, F, t, w->w2, out, dt);  /* idx 13 */
    free(t);
    return 0;
}

/* Bert_Encoder::forward  bert.h:59-79 (LO_POST_NORESID); LO_PRE_LN_RESID chains
 * layer_norm -> MHA -> add_bias_input_layernorm_2 -> MLP -> add_bias_input. */
int lo_encoder_forward(const lo_layer_shape* sh, const lo_layer_weights* w, const float* mask,
                       const float* in, float* out) {
    if (!shape_ok(sh)) return -1;
    const int M = sh->batch * sh->seq, H = sh->hidden, dt = sh->dtype;
    const int64_t n = (int64_t)M * H;
    int rc = 0;
    if (sh->norm_mode == LO_POST_NORESID) {
        float *a = falloc(n), *l = falloc(n), *m = falloc(n);
        rc |= lo_mha_forward(sh, w, mask, in, a);
        lo_layer_norm(a, w->ln1_g, w->ln1_b, l, M, H, dt); /* idx 10 */
        rc |= lo_mlp_forward(sh, w, l, m);
        lo_layer_norm(m, w->ln2_g, w->ln2_b, out, M, H, dt); /* idx 15 */
        free(a); free(l); free(m);
    } else {
        float *n1 = falloc(n), *a = falloc(n), *n2 = falloc(n);
        float* zb = zeros(H);
        lo_layer_norm(in, w->ln1_g, w->ln1_b, n1, M, H, dt);
        rc |= lo_mha_forward(sh, w, mask, n1, a);
        lo_add_bias_input_layernorm_2(in, w->ln2_g, w->ln2_b, w->bo ? w->bo : zb, a, n2, M, H, dt);
        rc |= lo_mlp_forward(sh, w, n2, out);
        lo_add_bias_input(out, w->b2 ? w->b2 : zb, a, M, H, dt);
        free(n1); free(a); free(n2); free(zb);
    }
    return rc;
}

/* One decode step (no reference counterpart; same kernels, M = batch rows, attention over the cache). */
int lo_decoder_step(const lo_layer_shape* sh, const lo_layer_weights* w, const float* x, float* k_cache,
                    float* v_cache, int past, int max_len, float* out) {
    if (!shape_ok(sh) || past < 0 || past + 1 > max_len) return -1;
    const int B = sh->batch, H = sh->hidden, h = sh->head_num, d = sh->size_per_head, F = sh->ffn_inner;
    const int Hl = h * d, dt = sh->dtype;
    const float scalar = 1.0f / sqrtf((float)d);
    float *xin = falloc((int64_t)B * H), *q = falloc((int64_t)B * Hl), *k = falloc((int64_t)B * Hl),
          *v = falloc((int64_t)B * Hl), *ao = falloc((int64_t)B * Hl), *a = falloc((int64_t)B * H),
          *l = falloc((int64_t)B * H), *t = falloc((int64_t)B * F), *m = falloc((int64_t)B * H);
    float* zb = zeros(H);
    if (sh->norm_mode == LO_PRE_LN_RESID)
        lo_layer_norm(x, w->ln1_g, w->ln1_b, xin, B, H, dt);
    else
        memcpy(xin, x, sizeof(float) * (size_t)B * H);
    lo_gemm(B, Hl, H, xin, w->wq, q, dt);
    lo_gemm(B, Hl, H, xin, w->wk, k, dt);
    lo_gemm(B, Hl, H, xin, w->wv, v, dt);
    for (int b = 0; b < B; ++b)
        for (int hh = 0; hh < h; ++hh)
            for (int e = 0; e < d; ++e) {
                int64_t si = (int64_t)b * Hl + hh * d + e;
                int64_t ci = (((int64_t)b * h + hh) * max_len + past) * d + e;
                q[si] = st(q[si] + w->bq[hh * d + e], dt);
                k_cache[ci] = st(k[si] + w->bk[hh * d + e], dt);
                v_cache[ci] = st(v[si] + w->bv[hh * d + e], dt);
            }
    lo_attn_decode(q, k_cache, v_cache, ao, B, h, d, past + 1, max_len, scalar, dt);
    lo_gemm(B, H, Hl, ao, w->wo, a, dt);
    if (sh->norm_mode == LO_POST_NORESID) {
        lo_layer_norm(a, w->ln1_g, w->ln1_b, l, B, H, dt);
    } else {
        lo_add_bias_input_layernorm_2(x, w->ln2_g, w->ln2_b, w->bo ? w->bo : zb, a, l, B, H, dt);
    }
    if (sh->ffn_act == LO_FFN_GEGLU) {
        float* t2 = falloc((int64_t)B * 2 * F);
        lo_gemm(B, 2 * F, H, l, w->w1, t2, dt);
        lo_add_bias_geglu(t, t2, w->b1, B, F, dt);
        free(t2);
    } else {
        lo_gemm(B, F, H, l, w->w1, t, dt);
        lo_add_bias_gelu(t, w->b1, B, F, dt);
    }
    lo_gemm(B, H, F, t, w->w2, m, dt);
    if (sh->norm_mode == LO_POST_NORESID) {
        lo_layer_norm(m, w->ln2_g, w->ln2_b, out, B, H, dt);
    } else {
        lo_add_bias_input(m, w->b2 ? w->b2 : zb, a, B, H, dt);
        memcpy(out, m, sizeof(float) * (size_t)B * H);
    }
    free(xin); free(q); free(k); free(v); free(ao); free(a); free(l); free(t); free(m); free(zb);
    return 0;
}
