// launch_context.h -- the launch descriptor types of the Liger host runtime on HIP.
//
// Counterpart of the reference's src/context.h: DynamicNvInitParam (:14-31), StaticNvInitParam (:33-57),
// BertInitParam (:59-85), layer_type (:87), GEMM_ARGS (:89-92), FuncWrap (:96-153), kernel_info / KeyHash
// (:155-169).  Same names and meaning; what changed and why:
//   * a stream context holds a HIP stream (void*, from lg_stream_create) instead of stream + cuBLAS handle;
//     stream priorities are not used (both streams run at the default priority);
//   * the GEMM argument tuple is a named struct (GemmDesc) that also carries the split axis and epilogue, so a
//     decomposed piece can offset its operands (the reference's pieces all recompute the first columns);
//   * every FuncWrap carries a resource class (MFMA-bound / HBM-bound / link-bound).  On one GPU there is no
//     COMMUNICATION entry, so the scheduler interleaves MFMA-bound with HBM-bound work instead of compute with
//     communication; with the classic classifier the original behaviour is reproduced.
//   * launch errors are recorded (first_error()) instead of being dropped.
#pragma once
#include <cstdint>
#include <cstdio>
#include <functional>
#include <mutex>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "liger_hip.h"

namespace liger {

// IEEE binary16 storage type for the host side (no arithmetic; device code does the math)
struct half {
    uint16_t bits;
};

template <typename T> struct dtype_of;
template <> struct dtype_of<float> { static constexpr int value = LG_F32; };
template <> struct dtype_of<half> { static constexpr int value = LG_F16; };

// ---- error capture ---------------------------------------------------------------------------------
// The first failing status of the process, written by whichever thread sees it first (the request thread builds vectors, the
// scheduler thread launches them), hence the lock.
struct ErrorState {
    int code = 0;
    std::string text;
};
inline std::mutex& error_mutex() {
    static std::mutex m;
    return m;
}
inline ErrorState& error_state_unlocked() {
    static ErrorState s;
    return s;
}
inline void set_error_state(int code, const std::string& text) {
    std::lock_guard<std::mutex> lk(error_mutex());
    ErrorState& e = error_state_unlocked();
    if (e.code == 0) { e.code = code; e.text = text; }
}
inline void note_status(int rc, const char* what) {
    if (rc != LG_OK) set_error_state(rc, std::string(what) + ": " + lg_last_error());
}
inline int error_code() {
    std::lock_guard<std::mutex> lk(error_mutex());
    return error_state_unlocked().code;
}
inline std::string error_text() {
    std::lock_guard<std::mutex> lk(error_mutex());
    return error_state_unlocked().text;
}
inline int first_error() { return error_code(); }
inline void clear_error() {
    std::lock_guard<std::mutex> lk(error_mutex());
    error_state_unlocked() = ErrorState();
}

// ---- per-stream context  (context.h:14-31) ------------------------------------------------------------
class DynamicInitParam {
  public:
    void* stream = nullptr;
    int stream_id = 0;  // 0 = primary, 1 = secondary; used by traces
    // Copies are handed to every launch callback (as in the reference), so the object does not own its stream: whoever created
    // the context calls destroy() on ONE copy when the stream is idle and no longer needed (a stream that was adopted from
    // elsewhere belongs to whoever made it and is left alone).
    bool adopted = false;
    void destroy() {
        if (!stream) return;
        if (!adopted) {
            note_status(lg_stream_synchronize(stream), "lg_stream_synchronize");
            note_status(lg_stream_destroy(stream), "lg_stream_destroy");
        }
        stream = nullptr;
    }
    DynamicInitParam() { note_status(lg_stream_create(&stream), "lg_stream_create"); }
    // the reference passes a CUDA stream priority here; priorities are deliberately not used on this platform
    explicit DynamicInitParam(int /*priority*/) { note_status(lg_stream_create(&stream), "lg_stream_create"); }
    // A stream created elsewhere.  Wrapping it costs nothing and touches nothing, so it may be done per call on the launch
    // path.  Whether K-sliced GEMMs are available on it is the owner's decision: lg_stream_attach (once, at set-up, where
    // allocating and blocking are allowed) gives it a split-K workspace; without it the launchers simply do not slice K.
    DynamicInitParam(void* existing_stream, int id) : stream(existing_stream), stream_id(id), adopted(true) {}
    // a stream whose kernels run on the compute units selected by the mask only (see lg_stream_create_cu_mask)
    DynamicInitParam(const unsigned* cu_mask, int mask_words, int id) : stream_id(id) {
        note_status(lg_stream_create_cu_mask(&stream, cu_mask, mask_words), "lg_stream_create_cu_mask");
    }
    // a stream that is verified to execute kernels at the same time as `first`'s (two streams of one process may share a
    // hardware queue, on which they would run strictly in turn); `concurrent` tells whether the verification succeeded
    bool concurrent = false;
    DynamicInitParam(int /*priority*/, const DynamicInitParam& first) {
        int verified = 0;
        note_status(lg_stream_create_concurrent(&stream, first.stream, &verified), "lg_stream_create_concurrent");
        concurrent = verified != 0;
    }
};
using DynamicNvInitParam = DynamicInitParam;

// ---- per-rank static context  (context.h:33-57) -------------------------------------------------------
class StaticInitParam {
  public:
    int world_size = 1;
    int world_rank = 0;
    int datatype = LG_F16;  // 0 = fp32, 1 = fp16 (the reference's CUDA_R_32F / CUDA_R_16F)
    StaticInitParam() {}
    StaticInitParam(int world_rank_, int world_size_, int datatype_)
        : world_size(world_size_), world_rank(world_rank_), datatype(datatype_) {}
};
using StaticNvInitParam = StaticInitParam;

enum norm_mode_t { POST_NORESID = 0, PRE_LN_RESID = 1 };
enum ffn_act_t { FFN_GELU = 0, FFN_GEGLU = 1 };

// ---- model / scheduler parameters  (context.h:59-85) --------------------------------------------------
class BertInitParam {
  public:
    int max_batch_size = 0;
    int max_seq_len = 0;
    int head_num = 0;       // GLOBAL head count; layers use head_num / world_size
    int size_per_head = 0;
    int layer_num = 0;
    int kernel_num = 0;     // launch-vector entries per layer
    int factor = 0;         // decomposition factor
    int rq_interval = 0;    // request spacing in microseconds
    // extensions (defaults reproduce the reference)
    int ffn_inner = 0;      // GLOBAL FFN inner size; 0 -> 4 * hidden (bert_layer.h:23,39)
    int norm_mode = POST_NORESID;
    int causal = 0;         // 1 -> lower-triangular attr_mask
    int fused = 0;          // 1 -> bias/GELU/transposes folded into GEMM epilogues, one fused attention kernel
    int max_cache_len = 0;  // > 0 -> layers own a KV cache [max_batch, heads, max_cache_len, d] for decode steps
    int weight_layout = 0;  // 0: weights stored [in, out] (what the reference's (N,N) cuBLAS call implies);
                            // 1: stored [out, in] and multiplied with transa = T (both operands K-contiguous);
                            // 2: the [out, in] matrix in the tiled layout of lg_weight_tile_f16 (transa = LG_OP_TILED; fp16)
    int ffn_act = 0;        // 0: FFN-1 -> bias + GELU -> FFN-2 (bert_layer.h:43-62); 1: GeGLU, FFN-1 is [H, 2F] = [gate | up]
    int packed_qkv = 0;     // 1 (reference-shaped assembly only): one [H, 3 Hl] GEMM + add_fusedQKV_bias_transpose
                            // (attention_kernels.cuh:23-34) instead of three GEMMs + add_QKV_bias_transpose
    BertInitParam() {}
    BertInitParam(int max_batch_size_, int max_seq_len_, int head_num_, int size_per_head_, int layer_num_,
                  int kernel_num_, int factor_, int rq_interval_)
        : max_batch_size(max_batch_size_), max_seq_len(max_seq_len_), head_num(head_num_),
          size_per_head(size_per_head_), layer_num(layer_num_), kernel_num(kernel_num_), factor(factor_),
          rq_interval(rq_interval_) {}
};

enum layer_type { COMMUNICATION, COMPUTATION, GEMM };   // context.h:87
enum resource_class { MFMA_BOUND, HBM_BOUND, LINK_BOUND };
enum split_axis { SPLIT_OUT_COLS = 0, SPLIT_TOKEN_ROWS = 1 };

// Named replacement of GEMM_ARGS (context.h:89-92): cuBLAS column-major convention, alpha = 1, beta = 0.
struct GemmDesc {
    bool valid = false;
    int dtype = LG_F16;
    int transa = 0;
    int m = 0, n = 0, k = 0;        // m = output features, n = tokens (column-major view)
    const void* A = nullptr; int lda = 0;   // weights
    const void* B = nullptr; int ldb = 0;   // activations
    void* C = nullptr; int ldc = 0;
    int epilogue = LG_EPI_NONE;
    const void* bias = nullptr;
    int epi_seq = 0, epi_d = 0, epi_heads_total = 0;
};

class FuncWrap {
  public:
    float duration = 0.f;  // profiled milliseconds
    layer_type type = COMPUTATION;
    resource_class rclass = HBM_BOUND;
    std::function<void(const DynamicInitParam&)> callback;
    GemmDesc args_gemm;
    int name = -1;  // kernel index inside the layer (profile key)
    // a small kernel between the big ones of its layer (normalisation, residual, cache append, row gather): a scheduler that
    // is told to merge minor entries lets it take the scheduling class of the entry before it
    bool minor = false;
    // the primary's round ends behind this entry even though the next one has the same class: the end of a chunk of a long
    // prefill, where the scheduler may give the turn to the decode steps of other requests (no reference counterpart)
    bool yield_after = false;
    const char* label = "";

    FuncWrap() {}
    FuncWrap(float duration_, layer_type type_, std::function<void(const DynamicInitParam&)> cb, const char* label_ = "",
             resource_class rc = HBM_BOUND)
        : duration(duration_), type(type_), rclass(rc), callback(std::move(cb)), label(label_) {}
    FuncWrap(float duration_, layer_type type_, std::function<void(const DynamicInitParam&)> cb, const GemmDesc& g,
             const char* label_ = "", resource_class rc = MFMA_BOUND)
        : duration(duration_), type(type_), rclass(rc), callback(std::move(cb)), args_gemm(g), label(label_) {}
    FuncWrap(int name_, float duration_, layer_type type_, std::function<void(const DynamicInitParam&)> cb,
             const GemmDesc& g, const char* label_ = "", resource_class rc = MFMA_BOUND)
        : duration(duration_), type(type_), rclass(rc), callback(std::move(cb)), args_gemm(g), name(name_), label(label_) {}
    bool not_comm() const { return type != COMMUNICATION; }
};

// profile-dictionary key  (context.h:155-169)
struct kernel_info {
    int kernel_name;
    int batch_size;
    int seq_len;
    bool operator==(const kernel_info& o) const {
        return std::tie(kernel_name, batch_size, seq_len) == std::tie(o.kernel_name, o.batch_size, o.seq_len);
    }
};
struct KeyHash {
    std::size_t operator()(const kernel_info& k) const {
        // the reference XORs the three std::hash values, which collides for permuted keys; mix them instead
        std::size_t h = std::hash<int>{}(k.kernel_name);
        h = h * 1000003u ^ std::hash<int>{}(k.batch_size);
        h = h * 1000003u ^ std::hash<int>{}(k.seq_len);
        return h;
    }
};
using MainDict = std::unordered_map<kernel_info, float, KeyHash>;
using SubDict = std::unordered_map<kernel_info, std::vector<float>, KeyHash>;

}  // namespace liger
