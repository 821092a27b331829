// func_wrapper.h -- adaptors from (arguments..., stream context) to the C ABI of the device library.
//
// Counterpart of the reference's src/layer/func_wrapper.h: one adaptor per launcher, same names and argument
// order, `DParams` supplying the stream.  T is float or liger::half; the adaptor picks the _f32 / _f16 entry.
#pragma once
#include "launch_context.h"

namespace liger {

// ---- basic operations  (func_wrapper.h:20-37) ----------------------------------------------------------
inline void GemmEx(const DynamicInitParam& DParams, const GemmDesc& g) {
    if (g.dtype == LG_F16) {
        if (g.epilogue == LG_EPI_NONE)
            note_status(lg_gemm_f16(g.transa, 0, g.m, g.n, g.k, g.A, g.lda, g.B, g.ldb, g.C, g.ldc, DParams.stream), "lg_gemm_f16");
        else
            note_status(lg_gemm_fused_f16(g.transa, g.m, g.n, g.k, g.A, g.lda, g.B, g.ldb, g.C, g.ldc, g.epilogue, g.bias,
                                          g.epi_seq, g.epi_d, g.epi_heads_total, DParams.stream), "lg_gemm_fused_f16");
    } else {
        note_status(lg_gemm_f32(g.transa, 0, g.m, g.n, g.k, (const float*)g.A, g.lda, (const float*)g.B, g.ldb, (float*)g.C,
                                g.ldc, DParams.stream), "lg_gemm_f32");
    }
}

// Q, K and V projections of a decode step as one call (bert_layer.h:127-137 issues them one after the other): the
// descriptors share the activations, the shape and the epilogue arguments and differ in weight, bias and destination.
inline void GemmExGrouped3(const DynamicInitParam& DParams, const GemmDesc& q, const GemmDesc& k, const GemmDesc& v) {
    const void* A[3] = {q.A, k.A, v.A};
    void* C[3] = {q.C, k.C, v.C};
    const int ldc[3] = {q.ldc, k.ldc, v.ldc};
    const void* bias[3] = {q.bias, k.bias, v.bias};
    note_status(lg_gemm_fused_grouped_f16(q.transa, q.m, q.n, q.k, 3, A, q.lda, q.B, q.ldb, C, ldc, q.epilogue, bias, q.epi_seq,
                                          q.epi_d, q.epi_heads_total, DParams.stream), "lg_gemm_fused_grouped_f16");
}

// The same for sequences in arbitrary cache slots at different positions: q goes to row r of its buffer, the K and V rows of
// token r to position pos[r] of cache slot slot[r].  `n` sequences; slot / pos are copied into the launch.
inline void GemmExGrouped3Rows(const DynamicInitParam& DParams, const GemmDesc& q, const GemmDesc& k, const GemmDesc& v, const int* slot,
                               const int* pos) {
    const void* A[3] = {q.A, k.A, v.A};
    void* C[3] = {q.C, k.C, v.C};
    const int ldc[3] = {q.ldc, k.ldc, v.ldc};
    const void* bias[3] = {q.bias, k.bias, v.bias};
    const int use_rows[3] = {0, 1, 1};
    note_status(lg_gemm_fused_grouped_rows_f16(q.transa, q.m, q.n, q.k, 3, A, q.lda, q.B, q.ldb, C, ldc, bias, q.epi_d, q.epi_heads_total,
                                               use_rows, slot, pos, DParams.stream), "lg_gemm_fused_grouped_rows_f16");
}

inline void GemmStridedBatchedEx(const DynamicInitParam& DParams, int dtype, int transa, int transb, int m, int n, int k,
                                 const void* A, int lda, long long strideA, const void* B, int ldb, long long strideB,
                                 void* C, int ldc, long long strideC, int batchCount) {
    if (dtype == LG_F16)
        note_status(lg_gemm_strided_batched_f16(transa, transb, m, n, k, A, lda, strideA, B, ldb, strideB, C, ldc, strideC,
                                                batchCount, DParams.stream), "lg_gemm_strided_batched_f16");
    else
        note_status(lg_gemm_strided_batched_f32(transa, transb, m, n, k, (const float*)A, lda, strideA, (const float*)B, ldb,
                                                strideB, (float*)C, ldc, strideC, batchCount, DParams.stream),
                    "lg_gemm_strided_batched_f32");
}

// ---- attention kernels  (func_wrapper.h:57-81) ---------------------------------------------------------
template <typename T>
void Add_QKV_bias_transpose(T* q_buf, T* k_buf, T* v_buf, T* Q, const T* bias_Q, T* K, const T* bias_K, T* V,
                            const T* bias_V, int batch_size, int seq_len, int head_num, int size_per_head,
                            const DynamicInitParam& DParams) {
    if (dtype_of<T>::value == LG_F16)
        note_status(lg_add_qkv_bias_transpose_f16(q_buf, k_buf, v_buf, Q, bias_Q, K, bias_K, V, bias_V, batch_size, seq_len,
                                                  head_num, size_per_head, DParams.stream), "lg_add_qkv_bias_transpose_f16");
    else
        note_status(lg_add_qkv_bias_transpose_f32((float*)q_buf, (float*)k_buf, (float*)v_buf, (const float*)Q,
                                                  (const float*)bias_Q, (const float*)K, (const float*)bias_K,
                                                  (const float*)V, (const float*)bias_V, batch_size, seq_len, head_num,
                                                  size_per_head, DParams.stream), "lg_add_qkv_bias_transpose_f32");
}

template <typename T>
void Add_fusedQKV_bias_transpose_kernelLauncher(T* q_buf, T* k_buf, T* v_buf, T* QKV, const T* qkv_bias, int batch_size,
                                                int seq_len, int head_num, int size_per_head,
                                                const DynamicInitParam& DParams) {
    if (dtype_of<T>::value == LG_F16)
        note_status(lg_add_fused_qkv_bias_transpose_f16(q_buf, k_buf, v_buf, QKV, qkv_bias, batch_size, seq_len, head_num,
                                                        size_per_head, DParams.stream), "lg_add_fused_qkv_bias_transpose_f16");
    else
        note_status(lg_add_fused_qkv_bias_transpose_f32((float*)q_buf, (float*)k_buf, (float*)v_buf, (const float*)QKV,
                                                        (const float*)qkv_bias, batch_size, seq_len, head_num, size_per_head,
                                                        DParams.stream), "lg_add_fused_qkv_bias_transpose_f32");
}

template <typename T>
void Attn_softmax_kernel(T* buffer, const T* attr_mask, int batch_size, int seq_len, int head_num, float scalar,
                         const DynamicInitParam& DParams) {
    if (dtype_of<T>::value == LG_F16)
        note_status(lg_attn_softmax_f16(buffer, attr_mask, batch_size, seq_len, head_num, scalar, DParams.stream), "lg_attn_softmax_f16");
    else
        note_status(lg_attn_softmax_f32((float*)buffer, (const float*)attr_mask, batch_size, seq_len, head_num, scalar,
                                        DParams.stream), "lg_attn_softmax_f32");
}

template <typename T>
void Transpose_kernel(T* dst, T* src, int batch_size, int seq_len, int head_num, int size_per_head,
                      const DynamicInitParam& DParams) {
    if (dtype_of<T>::value == LG_F16)
        note_status(lg_transpose_f16(dst, src, batch_size, seq_len, head_num, size_per_head, DParams.stream), "lg_transpose_f16");
    else
        note_status(lg_transpose_f32((float*)dst, (const float*)src, batch_size, seq_len, head_num, size_per_head,
                                     DParams.stream), "lg_transpose_f32");
}

// ---- element-wise / normalisation kernels  (func_wrapper.h:85-114) -------------------------------------
template <typename T>
void Add_bias_act_kernelLauncher(T* out, const T* bias, int m, int n, const DynamicInitParam& DParams) {
    if (dtype_of<T>::value == LG_F16) note_status(lg_add_bias_act_f16(out, bias, m, n, DParams.stream), "lg_add_bias_act_f16");
    else note_status(lg_add_bias_act_f32((float*)out, (const float*)bias, m, n, DParams.stream), "lg_add_bias_act_f32");
}

// GeGLU (no reference counterpart): in [m, 2f] = [gate | up] -> out [m, f]
template <typename T>
void Add_bias_geglu_kernelLauncher(T* out, const T* in, const T* bias, const int m, const int f, const DynamicInitParam& DParams) {
    if (dtype_of<T>::value == LG_F16) note_status(lg_add_bias_geglu_f16(out, in, bias, m, f, DParams.stream), "lg_add_bias_geglu_f16");
    else note_status(lg_add_bias_geglu_f32((float*)out, (const float*)in, (const float*)bias, m, f, DParams.stream), "lg_add_bias_geglu_f32");
}

template <typename T>
void Add_bias_input_layernorm_kernelLauncher(T* out, const T* input_tensor, const T* bias, const T* gamma, const T* beta,
                                             int m, int n, const DynamicInitParam& DParams) {
    if (dtype_of<T>::value == LG_F16)
        note_status(lg_add_bias_input_layernorm_f16(out, input_tensor, bias, gamma, beta, m, n, DParams.stream),
                    "lg_add_bias_input_layernorm_f16");
    else
        note_status(lg_add_bias_input_layernorm_f32((float*)out, (const float*)input_tensor, (const float*)bias,
                                                    (const float*)gamma, (const float*)beta, m, n, DParams.stream),
                    "lg_add_bias_input_layernorm_f32");
}

template <typename T>
void Add_bias_input_layernorm_2_kernelLauncher(const T* from_tensor, const T* gamma, const T* beta, const T* bias, T* output,
                                               T* norm_output_buf_, int m, int n, const DynamicInitParam& DParams) {
    if (dtype_of<T>::value == LG_F16)
        note_status(lg_add_bias_input_layernorm_2_f16(from_tensor, gamma, beta, bias, output, norm_output_buf_, m, n,
                                                      DParams.stream), "lg_add_bias_input_layernorm_2_f16");
    else
        note_status(lg_add_bias_input_layernorm_2_f32((const float*)from_tensor, (const float*)gamma, (const float*)beta,
                                                      (const float*)bias, (float*)output, (float*)norm_output_buf_, m, n,
                                                      DParams.stream), "lg_add_bias_input_layernorm_2_f32");
}

template <typename T>
void Add_bias_input_kernelLauncher(T* output, const T* bias, const T* input, int m, int n, const DynamicInitParam& DParams) {
    if (dtype_of<T>::value == LG_F16)
        note_status(lg_add_bias_input_f16(output, bias, input, m, n, DParams.stream), "lg_add_bias_input_f16");
    else
        note_status(lg_add_bias_input_f32((float*)output, (const float*)bias, (const float*)input, m, n, DParams.stream),
                    "lg_add_bias_input_f32");
}

template <typename T>
void Layer_Norm(const T* from_tensor, const T* gamma, const T* beta, T* norm_from_tensor_buf_, int m, int n,
                const DynamicInitParam& DParams) {
    if (dtype_of<T>::value == LG_F16)
        note_status(lg_layer_norm_f16(from_tensor, gamma, beta, norm_from_tensor_buf_, m, n, DParams.stream), "lg_layer_norm_f16");
    else
        note_status(lg_layer_norm_f32((const float*)from_tensor, (const float*)gamma, (const float*)beta,
                                      (float*)norm_from_tensor_buf_, m, n, DParams.stream), "lg_layer_norm_f32");
}

}  // namespace liger
