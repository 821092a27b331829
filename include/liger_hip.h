/*
 * liger_hip.h -- C ABI of the MI355X (gfx950) device library behind Liger's launch vector.
 *
 * Every entry point replaces one host launcher (or cuBLAS call) that the reference's adaptors in
 * src/layer/func_wrapper.h bind into a FuncWrap.  Conventions, identical to the reference's:
 *   - asynchronous: work is enqueued on `stream` (a hipStream_t passed as void*; NULL = default
 *     stream) and the call returns without waiting;
 *   - device pointers are owned by the caller; no kernel entry point allocates, frees or blocks (lg_malloc & co. below
 *     are thin runtime wrappers for host code that does not include HIP headers).  The one piece of device memory the
 *     library owns is a 64 MiB split-K workspace per stream, allocated by lg_stream_create* / lg_stream_attach and freed
 *     by lg_stream_destroy / lg_stream_detach -- the counterpart of the workspace a cuBLAS handle owns (context.h:20-29
 *     binds one handle per stream).  A GEMM on a stream the library was never told about still runs, on kernels that
 *     need no workspace (slower for fewer than 257 token rows);
 *   - several kernels work in place, exactly where the reference's do.
 * Differences: every function returns an int status instead of asserting --
 *   LG_OK, LG_ERR_INVALID (bad / unsupported shape or pointer), LG_ERR_LAUNCH (HIP error; text via
 *   lg_last_error()).  A C++ wrapper that wants the reference's `void` signatures may ignore it.
 * Suffix _f32 / _f16 = the reference's explicit float / half template instantiations; fp16 data is
 * IEEE binary16 (`uint16_t` storage, passed as void*).  fp16 kernels compute in fp32 and round once.
 */
#ifndef LIGER_HIP_H
#define LIGER_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LG_OK 0
#define LG_ERR_INVALID 1
#define LG_ERR_LAUNCH 2

#define LG_F32 0
#define LG_F16 1

/* values of transa in the GEMM entry points: the two cuBLAS operations the reference uses, and a third with no cuBLAS
 * counterpart for weights the caller has re-laid with lg_weight_tile_f16 (fp16 only; see there) */
#define LG_OP_N 0
#define LG_OP_T 1
#define LG_OP_TILED 2

/* most sequences one launch of the per-sequence (varlen / rows) decode entry points can carry */
#define LG_ATTN_DECODE_MAX_SEQS 64

/* ---- library / device ------------------------------------------------------------------------ */
const char* lg_last_error(void);
const char* lg_version(void);
/* Fills name (gcnArchName), CU count, engine clock (kHz), memory clock (kHz), bus width (bits),
 * total device memory (bytes).  Used by the bench to print the roofline denominators. */
int lg_device_info(char* name, int name_len, int* cu_count, int* clock_khz, int* mem_clock_khz,
                   int* bus_width_bits, size_t* total_mem);

/* ---- thin runtime wrappers (context.h:20-29, schedule.h:62-63,226-241, init.h:58-59,269-275) ---- */
int lg_malloc(void** ptr, size_t bytes);
int lg_free(void* ptr);
int lg_memcpy_h2d(void* dst, const void* src, size_t bytes);
int lg_memcpy_d2h(void* dst, const void* src, size_t bytes);
int lg_memcpy_d2d_async(void* dst, const void* src, size_t bytes, void* stream);
int lg_memset_async(void* dst, int value, size_t bytes, void* stream);
int lg_device_synchronize(void);
int lg_stream_create(void** stream);          /* non-blocking stream, default priority */
/* Tells the library about a stream it did not create (the null stream, another runtime's stream): allocates its split-K
 * workspace and records how many compute units its kernels run on (cu_count 0 = all of the device), which is what the
 * launchers size their grids for.  On a stream that is already known only a non-zero cu_count changes anything.  lg_stream_detach frees the workspace (after
 * synchronising the stream); lg_stream_cu_count returns the recorded count (the device's for an unknown stream). */
int lg_stream_attach(void* stream, int cu_count);
int lg_stream_detach(void* stream);
int lg_stream_cu_count(void* stream);
/* Non-blocking stream whose kernels run only on the compute units whose bit is set in cu_mask (mask_words 32-bit
 * words, bit i of word w = mask bit 32*w + i; on this GPU bit i selects a unit of accelerator die i mod 8, and every die must
 * keep at least one unit).  The launchers size their grids for the number of selected units.  Takes the place of the two stream priorities
 * the reference gives its streams (context.h:28-29, schedule.h:54-55): on this platform the two streams of the scheduler
 * are separated in space, not by priority.  The call runs one empty kernel on the new stream and waits for it (a stream of
 * this kind that is destroyed before anything ran on it has blocked in the runtime's destroy call): it may block, like every
 * stream creation here; launches never do. */
int lg_stream_create_cu_mask(void** stream, const unsigned* cu_mask, int mask_words);
/* Non-blocking stream that is verified, by measurement, to run kernels at the same time as `other` (the scheduler's
 * second stream, schedule.h:54-55).  HIP multiplexes a process's streams onto a few hardware queues and two streams
 * that share one execute strictly in turn; candidates are created and probed (a 0.4 ms one-wave spin on `other` next
 * to a one-wave kernel on the candidate) until one overlaps.  *verified = 1 if such a stream was found, 0 if the
 * returned stream is an unverified fallback.  `other` must be a created stream (not the null stream). */
int lg_stream_create_concurrent(void** stream, void* other, int* verified);
/* The same probe for two streams that exist already (both created, not the null stream; CU-masked ones included):
 * *concurrent = 1 when a one-wave kernel on `b` finishes while a 0.4 ms one-wave spin on `a` still runs.  Blocks until
 * both have run (set-up time only).  No reference counterpart: schedule.h:54-55 trusts its two streams to overlap. */
int lg_streams_run_concurrently(void* a, void* b, int* concurrent);
int lg_stream_destroy(void* stream);
int lg_stream_synchronize(void* stream);
int lg_stream_wait_event(void* stream, void* event);
int lg_event_create(void** event);            /* timing-enabled */
int lg_event_destroy(void* event);
int lg_event_record(void* event, void* stream);
int lg_event_synchronize(void* event);
int lg_event_query(void* event);              /* LG_OK when complete, LG_ERR_LAUNCH + 1 (=3) when not ready */
int lg_event_elapsed_ms(float* ms, void* start, void* stop);

/* Deterministic synthetic data on the device: out[i] = mean + stddev * z_i with z from the
 * counter-based Irwin-Hall(8) generator keyed by (seed, tensor_id).  Bit-identical to the CPU
 * oracle's generator.  No reference counterpart (the reference never initialises a buffer). */
int lg_fill_normal_f32(float* out, int64_t n, uint64_t seed, uint64_t tensor_id, float mean, float stddev,
                       void* stream);
int lg_fill_normal_f16(void* out, int64_t n, uint64_t seed, uint64_t tensor_id, float mean, float stddev,
                       void* stream);
int lg_fill_const_f32(float* out, int64_t n, float value, void* stream);
int lg_fill_const_f16(void* out, int64_t n, float value, void* stream);
/* mask[b,i,j] = (j <= i) as 0/1 in T: the lower-triangular attr_mask for causal prefill */
int lg_fill_causal_mask_f32(float* mask, int batch, int seq, void* stream);
int lg_fill_causal_mask_f16(void* mask, int batch, int seq, void* stream);

/* ---- element-wise / normalisation  (src/cuda/cuda_kernels.cuh:23-43) ---------------------------- */
/* layer_norm<T>                        cuda_kernels.cuh:41-43, cuda_kernels.cu:510-532 */
int lg_layer_norm_f32(const float* in, const float* gamma, const float* beta, float* out, int m, int n,
                      void* stream);
int lg_layer_norm_f16(const void* in, const void* gamma, const void* beta, void* out, int m, int n,
                      void* stream);
/* add_bias_act_kernelLauncher<T> (GELU-tanh, in place)   cuda_kernels.cuh:23-24, cuda_kernels.cu:302-319 */
int lg_add_bias_act_f32(float* out, const float* bias, int m, int n, void* stream);
int lg_add_bias_act_f16(void* out, const void* bias, int m, int n, void* stream);
/* GeGLU, the FFN activation of the GLM family; no reference counterpart (the reference's MLP is bias + GELU only,
 * bert_layer.h:43-62).  in [m, 2f] = [gate | up], bias [2f]; out [m, f] = gelu_tanh(gate + b) * (up + b).  out must not
 * overlap in. */
int lg_add_bias_geglu_f32(float* out, const float* in, const float* bias, int m, int f, void* stream);
int lg_add_bias_geglu_f16(void* out, const void* in, const void* bias, int m, int f, void* stream);
/* add_bias_input_layernorm_kernelLauncher<T> (in place on out)   cuda_kernels.cuh:26-30.
 * Unlike the reference (n <= 1024 / 2048) any n is accepted. */
int lg_add_bias_input_layernorm_f32(float* out, const float* input, const float* bias, const float* gamma,
                                    const float* beta, int m, int n, void* stream);
int lg_add_bias_input_layernorm_f16(void* out, const void* input, const void* bias, const void* gamma,
                                    const void* beta, int m, int n, void* stream);
/* add_bias_input_layernorm_2_kernelLauncher<T>   cuda_kernels.cuh:32-36 */
int lg_add_bias_input_layernorm_2_f32(const float* input, const float* gamma, const float* beta,
                                      const float* bias, float* output, float* norm_output, int m, int n,
                                      void* stream);
int lg_add_bias_input_layernorm_2_f16(const void* input, const void* gamma, const void* beta, const void* bias,
                                      void* output, void* norm_output, int m, int n, void* stream);
/* add_bias_input_kernelLauncher<T>   cuda_kernels.cuh:38-39 */
int lg_add_bias_input_f32(float* output, const float* bias, const float* input, int m, int n, void* stream);
int lg_add_bias_input_f16(void* output, const void* bias, const void* input, int m, int n, void* stream);

/* ---- attention helpers  (src/cuda/attention_kernels.cuh:6-54) ------------------------------------ */
/* add_QKV_bias_transpose_kernelLauncher<T>   attention_kernels.cuh:6-21.  Any head_num*size_per_head. */
int lg_add_qkv_bias_transpose_f32(float* q_buf, float* k_buf, float* v_buf, const float* Q, const float* bias_Q,
                                  const float* K, const float* bias_K, const float* V, const float* bias_V,
                                  int batch, int seq, int head_num, int size_per_head, void* stream);
int lg_add_qkv_bias_transpose_f16(void* q_buf, void* k_buf, void* v_buf, const void* Q, const void* bias_Q,
                                  const void* K, const void* bias_K, const void* V, const void* bias_V,
                                  int batch, int seq, int head_num, int size_per_head, void* stream);
/* add_fusedQKV_bias_transpose_kernelLauncher<T>   attention_kernels.cuh:23-34 */
int lg_add_fused_qkv_bias_transpose_f32(float* q_buf, float* k_buf, float* v_buf, const float* QKV,
                                        const float* qkv_bias, int batch, int seq, int head_num,
                                        int size_per_head, void* stream);
int lg_add_fused_qkv_bias_transpose_f16(void* q_buf, void* k_buf, void* v_buf, const void* QKV,
                                        const void* qkv_bias, int batch, int seq, int head_num,
                                        int size_per_head, void* stream);
/* attn_softmax_kernelLauncher<T> (in place)   attention_kernels.cuh:36-44.  Any seq (the reference needs
 * seq <= 1024 fp32 / 2048 fp16).  `scalar` is passed as float and rounded to T as the reference stores it. */
int lg_attn_softmax_f32(float* buffer, const float* attr_mask, int batch, int seq, int head_num, float scalar,
                        void* stream);
int lg_attn_softmax_f16(void* buffer, const void* attr_mask, int batch, int seq, int head_num, float scalar,
                        void* stream);
/* transpose_kernelLauncher<T>   attention_kernels.cuh:46-54.  No batch*head*seq % 4 restriction. */
int lg_transpose_f32(float* dst, const float* src, int batch, int seq, int head_num, int size_per_head,
                     void* stream);
int lg_transpose_f16(void* dst, const void* src, int batch, int seq, int head_num, int size_per_head,
                     void* stream);

/* ---- GEMM  (cuBLAS as called through func_wrapper.h:20-37) --------------------------------------- */
/* cublasGemmEx subset the reference uses: column-major, alpha = 1, beta = 0, C = op(A) * B.
 * transa: 0 = N (linear.h:47-49,99-101), 1 = T (bert_layer.h:145-149); transb must be 0.
 * In row-major words: C'[n, m] = B'[n, k] * W where W is A seen row-major: [k, m] (transa = 0) or
 * [m, k] (transa = 1).  fp16: fp32 accumulate (the reference accumulates in fp16).
 * transa = LG_OP_TILED (fp16, single problems and groups): A is the [m, k] matrix in the tiled layout written by
 * lg_weight_tile_f16, lda must equal k, m % 16 == 0, k % 32 == 0.  A sub-range of features that starts at a multiple of
 * 16 starts (first feature) * k elements into A, as in the [m, k] layout. */
int lg_gemm_f32(int transa, int transb, int m, int n, int k, const float* A, int lda, const float* B, int ldb,
                float* C, int ldc, void* stream);
int lg_gemm_f16(int transa, int transb, int m, int n, int k, const void* A, int lda, const void* B, int ldb,
                void* C, int ldc, void* stream);
/* cublasGemmStridedBatchedEx, same subset.  func_wrapper.h:30-37 */
int lg_gemm_strided_batched_f32(int transa, int transb, int m, int n, int k, const float* A, int lda,
                                int64_t strideA, const float* B, int ldb, int64_t strideB, float* C, int ldc,
                                int64_t strideC, int batch, void* stream);
int lg_gemm_strided_batched_f16(int transa, int transb, int m, int n, int k, const void* A, int lda,
                                int64_t strideA, const void* B, int ldb, int64_t strideB, void* C, int ldc,
                                int64_t strideC, int batch, void* stream);

/* Epilogues for lg_gemm_fused_f16 */
#define LG_EPI_NONE 0
#define LG_EPI_BIAS 1      /* C = acc + bias[m-index]                    */
#define LG_EPI_BIAS_GELU 2 /* C = gelu_tanh(acc + bias[m-index])   == lg_gemm + lg_add_bias_act        */
#define LG_EPI_BIAS_HEADS 3 /* C is written as [batch, head, row, d] == lg_gemm + lg_add_qkv_bias_transpose
                               for one of Q/K/V.  epi_arg0 = seq (tokens per sequence), epi_arg1 =
                               size_per_head, epi_arg2 = heads per batch entry in C (0 -> m / size_per_head;
                               larger when C is a slice of a wider buffer), and ldc = rows reserved per
                               (batch, head) in C (>= seq; > seq when C is a KV cache)                     */
#define LG_EPI_BIAS_GEGLU 5 /* the m output features are the gate and up halves of a GeGLU FFN-1, interleaved in groups
                               of 16: features [32g, 32g+16) are gate columns [16g, 16g+16), features [32g+16, 32g+32)
                               the up columns of the same indices (A and bias are stored in that order); C is
                               [n tokens, m/2] (ldc >= m/2) with C[t, c] = gelu_tanh(gate_c + bias) * (up_c + bias)
                               == lg_gemm + lg_add_bias_geglu on the de-interleaved operands.  m % 32 == 0.   */
/* lg_gemm_f16 with a fused epilogue (the bias / GELU / head-transpose kernels that follow the GEMMs in
 * the launch vector, bert_layer.h:54-56,139-142, folded into the GEMM's store).  No reference
 * counterpart; results equal the two-kernel sequence up to one fp16 rounding. */
int lg_gemm_fused_f16(int transa, int m, int n, int k, const void* A, int lda, const void* B, int ldb, void* C,
                      int ldc, int epilogue, const void* bias, int epi_arg0, int epi_arg1, int epi_arg2,
                      void* stream);

/* `count` (1..3) lg_gemm_fused_f16 calls that share B (the token rows), the shape, lda and the epilogue arguments
 * and differ in A[i], C[i], ldc[i] and bias[i]: the Q, K and V projections of a decode step (linear.h:99-101 issued
 * three times by bert_layer.h:127-137; also the column blocks of one packed [H, 3 Hl] weight: A[i] = the block's first
 * column or row, lda = the packed matrix's).  Few-token problems with weights [out, in] run as ONE launch of the
 * weight-streaming kernels, problems of more than 256 token rows as ONE launch of the pipelined kernel (either weight
 * layout); anything else is executed as `count` plain calls.  Results are those of the plain calls up to the order of the
 * fp32 sum over k (the one launch may use another block width).  No reference counterpart. */
int lg_gemm_fused_grouped_f16(int transa, int m, int n, int k, int count, const void* const* A, int lda, const void* B,
                              int ldb, void* const* C, const int* ldc, int epilogue, const void* const* bias,
                              int epi_arg0, int epi_arg1, int epi_arg2, void* stream);

/* The Q, K and V projections of a decode step over sequences that sit in arbitrary cache slots at different positions (decode
 * steps of different requests batched into one launch): lg_gemm_fused_grouped_f16 with the heads epilogue and one token per
 * sequence, except that a member i with use_rows[i] != 0 writes token row r to position pos[r] of batch entry slot[r] of its
 * destination C[i] = [slots, heads_total, ldc[i], size_per_head] (a KV cache) instead of to position 0 of entry r.  slot and
 * pos are HOST arrays of n ints, copied into the launch (n <= LG_ATTN_DECODE_MAX_SEQS).  pos[r] is checked against ldc[i];
 * how many entries C[i] has is not known here: slot[r] must be a valid entry (the host runtime checks it against the model's
 * cache before it builds a launch).  No reference counterpart. */
int lg_gemm_fused_grouped_rows_f16(int transa, int m, int n, int k, int count, const void* const* A, int lda, const void* B,
                                   int ldb, void* const* C, const int* ldc, const void* const* bias, int size_per_head,
                                   int heads_total, const int* use_rows, const int* slot, const int* pos, void* stream);

/* ---- attention kernels with no reference counterpart --------------------------------------------- */
/* Fused prefill attention: out = softmax(q k^T * scalar + maskterm) v with the reference's softmax
 * semantics (-10000 additive mask, +1e-6 in the denominator); replaces launch-vector entries 4,5,6 (and 7
 * when out_layout = 1).  q_buf [B,h,S,d]; k_buf, v_buf [B,h,kv_rows,d] with the S valid rows first
 * (kv_rows = S for plain buffers, = max_len when they are a KV cache).  causal != 0: implicit
 * lower-triangular mask (attr_mask ignored, may be NULL); causal == 0: attr_mask [B,S,S] of 0/1 or NULL
 * for all ones.  out_layout 0: [B,h,S,d]; 1: [B,S,h,d] (= transpose-back fused).  size_per_head: 64, 96 or 128. */
int lg_attn_prefill_f16(const void* q_buf, const void* k_buf, const void* v_buf, const void* attr_mask,
                        void* out, int batch, int seq, int head_num, int size_per_head, int kv_rows,
                        float scalar, int causal, int out_layout, void* stream);
/* The same for a prefill that continues a sequence (a long prompt processed in chunks over a KV cache): the `seq` queries of
 * q_buf [B,h,seq,d] are positions past .. past + seq - 1, k_buf / v_buf [B,h,kv_rows,d] hold the past + seq keys and values
 * (the chunk's own rows included, past + seq <= kv_rows).  causal != 0: query i sees keys 0 .. past + i; causal == 0: all
 * past + seq keys.  No explicit mask. */
int lg_attn_prefill_past_f16(const void* q_buf, const void* k_buf, const void* v_buf, void* out, int batch, int seq, int past,
                             int head_num, int size_per_head, int kv_rows, float scalar, int causal, int out_layout,
                             void* stream);
/* Decode attention: q [B,h,d]; k_cache, v_cache [B,h,max_len,d] with `len` valid positions; out [B,h,d].
 * size_per_head: 64, 96 or 128.  workspace: float buffer of lg_attn_decode_workspace_bytes(...) bytes (split-KV partials),
 * caller-owned; that size is an upper bound for every batch and every len <= max_len, so a buffer sized once for the
 * largest batch serves all smaller ones. */
size_t lg_attn_decode_workspace_bytes(int batch, int head_num, int size_per_head, int max_len);
int lg_attn_decode_f16(const void* q, const void* k_cache, const void* v_cache, void* out, void* workspace,
                       int batch, int head_num, int size_per_head, int len, int max_len, float scalar,
                       void* stream);
/* The same over sequences that differ in length and sit in arbitrary cache slots (decode steps of different requests
 * batched into one launch): sequence b reads slot[b] of the caches [slots,h,max_len,d] and attends to its first len[b]
 * positions.  slot and len are HOST arrays of `batch` ints, copied into the launch (batch <= LG_ATTN_DECODE_MAX_SEQS). */
int lg_attn_decode_varlen_f16(const void* q, const void* k_cache, const void* v_cache, void* out, void* workspace,
                              int batch, int head_num, int size_per_head, const int* slot, const int* len, int max_len,
                              float scalar, void* stream);
/* lg_attn_decode_f16 for callers that cannot allocate device memory or pass a workspace (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc); no counterpart in the reference.  The split-KV partials live in
 * a fixed array inside the library's device image (2048 partial slots x (2 + 128) floats = 1.02 MiB per GPU, held until
 * the process ends); this call allocates nothing.  Same results as lg_attn_decode_f16, bit for bit.  size_per_head > 128
 * is rejected.  Every call on a GPU uses that GPU's one array: calls that overlap in time on one GPU (two streams)
 * race; calls on one stream are ordered and safe. */
int lg_attn_decode_static_f16(const void* q, const void* k_cache, const void* v_cache, void* out, int batch, int head_num,
                              int size_per_head, int len, int max_len, float scalar, void* stream);
/* Adds the Q/K/V biases to one new token per sequence ([B, h*d] rows straight from the QKV GEMMs), writes
 * q -> q_out [B,h,d] and appends k, v at position `pos` of the caches [B,h,max_len,d]. */
int lg_kv_append_f16(void* q_out, void* k_cache, void* v_cache, const void* Q, const void* bias_Q, const void* K,
                     const void* bias_K, const void* V, const void* bias_V, int batch, int head_num,
                     int size_per_head, int pos, int max_len, void* stream);
/* The same with a cache slot and a position per sequence (HOST arrays of `batch` ints, batch <= LG_ATTN_DECODE_MAX_SEQS):
 * sequence b's k, v go to position pos[b] of slot[b] of the caches [slots,h,max_len,d]. */
int lg_kv_append_varlen_f16(void* q_out, void* k_cache, void* v_cache, const void* Q, const void* bias_Q, const void* K,
                            const void* bias_K, const void* V, const void* bias_V, int batch, int head_num,
                            int size_per_head, const int* slot, const int* pos, int max_len, void* stream);

/* ---- weights in the tiled layout (no reference counterpart: linear.h:40,92 allocate the weights and never say how they
 * are laid out, so a layer that owns its weights may store them as its kernels read them fastest) -------------------- */
/* tiled = the [features, k] matrix cut into blocks of 16 features x 32 k, block (t, c) at element ((t * k / 32) + c) * 512;
 * inside a block, element (feature f, position j) sits at ((j / 8) * 16 + f) * 8 + j % 8 -- the order in which the lanes of a
 * wave hold the B operand of v_mfma_f32_16x16x32_f16.  Every wave-wide load of a block is one contiguous KiB and the blocks
 * of a feature tile follow each other along k: decode GEMMs stream such weights 15-20 % faster than row-major ones (whole
 * 128-byte lines per load, marked non-temporal), prefill GEMMs copy blocks to LDS without a swizzle.
 * plain_transa says how the plain matrix is stored: 0 = [k, features] (ld_plain >= features), 1 = [features, k]
 * (ld_plain >= k, a multiple of 8).  features % 16 == 0, k % 32 == 0, both pointers 16-byte aligned and distinct. */
int lg_weight_tile_f16(void* tiled, const void* plain, int features, int k, int plain_transa, int ld_plain, void* stream);
int lg_weight_untile_f16(void* plain, const void* tiled, int features, int k, int plain_transa, int ld_plain, void* stream);

/* ---- what the device sustains (no reference counterpart; measurement calls for a bench: they time their own kernel with
 * two events on `stream` and BLOCK until it has finished; nothing on the launch path calls them) ------------------------- */
/* A register-only loop of v_mfma_f32_16x16x32_f16 on a 128 x 64 wave tile (no loads, no LDS), 1024 blocks of 8 waves x iters
 * rounds of 32 matrix instructions.  Operands are read once from `operands` (fp16, >= 106504 elements, 16-byte aligned): with
 * the data distribution of a GEMM's inputs the pipes draw more power than with zeros and the clock settles lower, so the
 * figure is the matrix throughput a GEMM on such data cannot exceed on this device.  scratch: >= 64 bytes of device memory.
 * Returns the kernel's milliseconds, TFLOP/s and the shader clock (GHz) seen by the kernel (either may be NULL). */
int lg_probe_mfma_f16(const void* operands, int64_t operand_elems, void* scratch, size_t scratch_bytes, int iters, float* ms,
                      float* tflops, float* shader_ghz, void* stream);
/* The same wave tile and instruction with the operand traffic of the pipelined GEMM's k-loop and nothing else of it: per 64
 * matrix instructions a wave copies 8 KiB from `operands` (a region that stays in L2) to LDS with direct-to-LDS loads and
 * reads 24 fragments of 1 KiB from LDS (two LDS slots of 64 KiB, fragments double-buffered in registers); no barrier and no
 * wait for a particular tile, no epilogue, no stores, no traffic beyond L2.  1024 blocks x 8 waves x iters rounds of 64 matrix
 * instructions.  loads_per_round = 8 and reads_per_step = 12 are the GEMM's traffic; 4 / 0 and 6 / 0 show what half or none of
 * either would leave.  Other arguments and results as lg_probe_mfma_f16: an upper bound for a k-loop whose operands travel
 * L2 -> LDS -> registers at that rate, whatever its synchronisation costs on top. */
int lg_probe_mfma_stream_f16(const void* operands, int64_t operand_elems, void* scratch, size_t scratch_bytes, int iters, int loads_per_round,
                             int reads_per_step, float* ms, float* tflops, float* shader_ghz, void* stream);
/* Reads every byte of src[0, bytes) once per pass (16-byte loads, 8 in flight per lane, 1 KiB per wave instruction;
 * nontemporal != 0 marks them as streaming), `passes` passes after one untimed pass.  On a buffer much larger than the
 * caches (256 MB memory-side cache) the figure is the device's memory read ceiling.  scratch: >= 4 bytes of device memory.
 * Returns milliseconds per pass and GB/s (may be NULL). */
int lg_probe_read(const void* src, size_t bytes, void* scratch, int passes, int nontemporal, float* ms, float* gbps, void* stream);

#ifdef __cplusplus
}
#endif
#endif
