/*
 * liger_oracle.h -- CPU restatement of the per-GPU hot path of Liger (PPoPP'24).
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the parity checker and the reported CPU
 * baseline.  Nothing in the shipped GPU path may call, link or import it: only tests/,
 * __graft_entry__.smoke() and the cpu_baseline leg of bench.py do.
 *
 * Every array is plain row-major float32 on the host.  `dtype` selects which template
 * instantiation of the reference is restated:
 *     LO_F32 (0)  the `float` instantiation, fp32 everywhere;
 *     LO_F16 (1)  the `half` instantiation: values are kept in float variables but every
 *                 point where the reference stores or computes in half is rounded to the
 *                 nearest-even binary16 value, so all inputs/outputs are exactly
 *                 representable in fp16.  GEMMs accumulate in fp32 and round once.
 *
 * How each function is pinned (the reference ships no golden vectors and no numeric
 * tests of any kind, and it is CUDA so it cannot be built here):
 *     gemm / gemm_ex / gemm_strided_batched   BLAS definition; fp64 brute force; identity
 *                                             and one-hot operands; numpy matmul
 *     layer_norm family                       closed forms (constant row -> beta, two-point
 *                                             row), shift invariance, torch layer_norm
 *     add_bias_gelu / add_bias_geglu          tabulated tanh-GELU points, torch gelu(tanh) (x up)
 *     attn_softmax                            row-sum identity, uniform rows, mask zeroing,
 *                                             shift invariance, torch softmax
 *     qkv bias+transpose / transpose          exhaustive index check, round trip
 *     attn_decode (no reference counterpart)  equals the last row of causal prefill
 *     encoder / model                         composition + torch fixture (tests/golden)
 *     fill_normal                             integer arithmetic, moments, golden words
 * The one thing that cannot be pinned without running the reference on NVIDIA hardware is
 * cuBLAS's fp16-accumulate rounding (external closed-source library, no version pin in
 * the reference): "parity unpinned" for that rounding; this oracle accumulates in fp32,
 * which the stated tolerance (max rel err <= 1e-2) covers.
 */
#ifndef LIGER_ORACLE_H
#define LIGER_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LO_F32 0
#define LO_F16 1

/* norm_mode of the encoder layer */
#define LO_POST_NORESID 0 /* exactly what src/layer/bert.h:59-79 assembles */
#define LO_PRE_LN_RESID 1 /* pre-LN layer built from the reference's fused residual kernels */

/* ffn_act of the encoder layer */
#define LO_FFN_GELU 0  /* bert_layer.h:43-45: FFN-1 -> bias + GELU -> FFN-2 */
#define LO_FFN_GEGLU 1 /* w1 is [H, 2F] = [gate | up], b1 [2F]: gelu(gate) * up feeds FFN-2 */

/* ---- scalar helpers ---------------------------------------------------------------- */
float lo_round_f16(float x);            /* nearest-even round trip through binary16 */
uint16_t lo_f32_to_f16_bits(float x);
float lo_f16_bits_to_f32(uint16_t h);
void lo_round_f16_array(float* x, int64_t n);
int lo_num_threads(void);

/* ---- deterministic synthetic data ---------------------------------------------------
 * Counter-based: element i of stream (seed, tensor_id) is
 *     s = sum of the eight 16-bit fields of splitmix64(key+2i) and splitmix64(key+2i+1)
 *     z = (float)(s - 262140) * (1 / sqrt(8 * (65536^2 - 1) / 12))        (Irwin-Hall, n = 8)
 *     out = mean + stddev * z          (one fp32 multiply-add, then optional fp16 rounding)
 * Pure integer work plus two exactly-rounded fp32 operations, so the CPU, numpy and the GPU
 * fill kernel agree bit for bit. */
void lo_fill_normal(float* out, int64_t n, uint64_t seed, uint64_t tensor_id, float mean,
                    float stddev, int dtype);

/* ---- GEMMs ---------------------------------------------------------------------------
 * lo_gemm: row-major Y[M,N] = X[M,K] * W[K,N]  (the meaning of Linear_Col / Linear_Row,
 * reference src/layer/linear.h:47-49,99-101 once cuBLAS's column-major view is undone). */
void lo_gemm(int M, int N, int K, const float* X, const float* W, float* Y, int dtype);
/* fp64 triple loop with explicit leading dimensions, for tiny cross-checks */
void lo_gemm_naive_f64(int M, int N, int K, const float* X, int ldx, const float* W, int ldw,
                       double* Y, int ldy);
/* column-major cublasGemmEx subset used by the reference (alpha = 1, beta = 0):
 * C[m x n] = op(A) * op(B); transa/transb: 0 = N, 1 = T.  func_wrapper.h:20-27 */
void lo_gemm_ex(int transa, int transb, int m, int n, int k, const float* A, int lda,
                const float* B, int ldb, float* C, int ldc, int dtype);
/* cublasGemmStridedBatchedEx, same conventions.  func_wrapper.h:30-37 */
void lo_gemm_strided_batched(int transa, int transb, int m, int n, int k, const float* A, int lda,
                             int64_t strideA, const float* B, int ldb, int64_t strideB, float* C,
                             int ldc, int64_t strideC, int batch, int dtype);

/* ---- element-wise / normalisation kernels (src/cuda/cuda_kernels.cu) ------------------ */
void lo_add_bias_gelu(float* out, const float* bias, int m, int n, int dtype);       /* :9-29,59-84 */
/* GeGLU, the FFN activation of the GLM family (no reference counterpart): in [m, 2f] = [gate | up], bias [2f],
 * out [m, f] = gelu(gate + b) * (up + b) */
void lo_add_bias_geglu(float* out, const float* in, const float* bias, int m, int f, int dtype);
void lo_layer_norm(const float* in, const float* gamma, const float* beta, float* out, int m,
                   int n, int dtype);                                                 /* :463-508 */
void lo_add_bias_input_layernorm(float* out, const float* input, const float* bias,
                                 const float* gamma, const float* beta, int m, int n,
                                 int dtype);                                          /* :115-185 */
void lo_add_bias_input_layernorm_2(const float* input, const float* gamma, const float* beta,
                                   const float* bias, float* output, float* norm_output, int m,
                                   int n, int dtype);                                 /* :360-409 */
void lo_add_bias_input(float* output, const float* bias, const float* input, int m, int n,
                       int dtype);                                                    /* :438-452 */

/* ---- attention helper kernels (src/cuda/attention_kernels.cu) ------------------------- */
void lo_add_qkv_bias_transpose(float* q_buf, float* k_buf, float* v_buf, const float* Q,
                               const float* bias_Q, const float* K, const float* bias_K,
                               const float* V, const float* bias_V, int batch, int seq,
                               int head_num, int size_per_head, int dtype);           /* :79-224 */
void lo_add_fused_qkv_bias_transpose(float* q_buf, float* k_buf, float* v_buf, const float* QKV,
                                     const float* qkv_bias, int batch, int seq, int head_num,
                                     int size_per_head, int dtype);                   /* :331-371 */
void lo_attn_softmax(float* buffer, const float* attr_mask, int batch, int seq, int head_num,
                     float scalar, int dtype);                                        /* :395-618 */
void lo_transpose(float* dst, const float* src, int batch, int seq, int head_num,
                  int size_per_head);                                                 /* :682-710 */

/* ---- extensions with no reference counterpart (decode over a KV cache) ----------------
 * q [B,h,d]; k_cache, v_cache [B,h,Lmax,d] with `len` valid positions per sequence (the new
 * token's K/V already appended); out [B,h,d].  Same softmax semantics as lo_attn_softmax with an
 * all-ones mask: p = exp(s - max) / (sum + 1e-6). */
void lo_attn_decode(const float* q, const float* k_cache, const float* v_cache, float* out,
                    int batch, int head_num, int size_per_head, int len, int max_len, float scalar,
                    int dtype);
/* Fused prefill attention = qk_gemm -> attn_softmax -> qkv_gemm (bert_layer.h:145-163) with an
 * implicit mask: causal != 0 -> lower-triangular 0/1 mask, else all ones.
 * q_buf,k_buf,v_buf,out: [B,h,S,d]. */
void lo_attn_prefill(const float* q_buf, const float* k_buf, const float* v_buf, float* out,
                     int batch, int seq, int head_num, int size_per_head, float scalar, int causal,
                     int dtype);

/* ---- layer assembly (src/layer/bert_layer.h, src/layer/bert.h) ------------------------ */
typedef struct lo_layer_weights {
    /* all row-major; Hl = local heads * d, F = local FFN inner */
    const float *wq, *wk, *wv; /* [H, Hl]   Linear_Col  bert_layer.h:98-100 */
    const float *bq, *bk, *bv; /* [Hl]      bert_layer.h:115-117 */
    const float* wo;           /* [Hl, H]   Linear_Row  bert_layer.h:101 */
    const float* bo;           /* [H]  out-proj bias; only used in LO_PRE_LN_RESID (may be NULL = 0) */
    const float *ln1_g, *ln1_b; /* [H]  ln_mha  bert.h:56 */
    const float* w1;           /* [H, F]    bert_layer.h:43 */
    const float* b1;           /* [F]       bert_layer.h:45 */
    const float* w2;           /* [F, H]    bert_layer.h:44 */
    const float* b2;           /* [H]  FFN-2 bias; only used in LO_PRE_LN_RESID (may be NULL = 0) */
    const float *ln2_g, *ln2_b; /* [H]  ln_mlp  bert.h:57 */
} lo_layer_weights;

typedef struct lo_layer_shape {
    int batch, seq, hidden, head_num /* local */, size_per_head, ffn_inner /* local */;
    int causal;    /* 0: use `mask` ([B,S,S] 0/1) if non-NULL else all ones; 1: lower-triangular */
    int norm_mode; /* LO_POST_NORESID / LO_PRE_LN_RESID */
    int dtype;
    int ffn_act;   /* LO_FFN_GELU / LO_FFN_GEGLU */
} lo_layer_shape;

/* One encoder layer.  in/out: [B*S, H].  mask may be NULL.  Returns 0 or -1 on bad shapes. */
int lo_encoder_forward(const lo_layer_shape* sh, const lo_layer_weights* w, const float* mask,
                       const float* in, float* out);
/* attention block only (idx 0..8 of the launch vector): in [M,H] -> out [M,H] */
int lo_mha_forward(const lo_layer_shape* sh, const lo_layer_weights* w, const float* mask,
                   const float* in, float* out);
/* MLP block only (idx 11..13): in [M,H] -> out [M,H] */
int lo_mlp_forward(const lo_layer_shape* sh, const lo_layer_weights* w, const float* in, float* out);

/* One decode step of the same layer for `batch` sequences, one new token each.
 * x [B,H]; caches [B,h,Lmax,d] hold `past` valid positions; the new K/V row is appended at
 * position `past` (caches are modified), attention runs over past+1 positions. out [B,H]. */
int lo_decoder_step(const lo_layer_shape* sh, const lo_layer_weights* w, const float* x,
                    float* k_cache, float* v_cache, int past, int max_len, float* out);

#ifdef __cplusplus
}
#endif
#endif
