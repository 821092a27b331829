// layers.h -- layer assembly: classes that own device weights and emit the launch vector.
//
// Counterpart of the reference's src/layer/linear.h (Linear_Row :16-64, Linear_Col :68-109), operator.h
// (LayerNorm :16-41), bert_layer.h (Bert_MLP :19-63, Bert_MHA :65-176) and bert.h (Bert_Encoder :18-80,
// Bert_Model :83-118).  Same class names, constructor arguments and `forward(...) -> vector<FuncWrap>` contract;
// no GPU work happens in forward().  Deliberate differences:
//   * weights, biases, gamma/beta and masks are initialised (seeded generator) -- the reference leaves every
//     buffer uninitialised because it only measures time;
//   * workspace slices are computed per request from (batch, seq) and are sized correctly (the reference sizes
//     the score buffer as B*S*n and multiplies element offsets by sizeof(T));
//   * tensor parallelism appears only as `/ world_size` on the shard dimensions, exactly as in the reference,
//     but the all-reduce entry after a row-parallel GEMM is not emitted (single-GPU build: one shard at its real
//     shape, exchange out of scope);
//   * optional assemblies: pre-LN with residuals built from the reference's fused residual kernels, a fused
//     assembly (epilogue-fused GEMMs + one attention kernel) and a decode step over a KV cache.
#pragma once
#include <cmath>
#include <map>
#include <memory>

#include "func_wrapper.h"

namespace liger {

template <typename T>
inline T* dev_alloc(size_t elems) {
    void* p = nullptr;
    note_status(lg_malloc(&p, (elems ? elems : 1) * sizeof(T)), "lg_malloc");
    return (T*)p;
}
inline void dev_free(void* p) {
    if (p) note_status(lg_free(p), "lg_free");
}
template <typename T>
inline void dev_fill_normal(T* p, int64_t n, uint64_t seed, uint64_t tensor_id, float mean, float stddev) {
    if (dtype_of<T>::value == LG_F16) note_status(lg_fill_normal_f16(p, n, seed, tensor_id, mean, stddev, nullptr), "lg_fill_normal_f16");
    else note_status(lg_fill_normal_f32((float*)p, n, seed, tensor_id, mean, stddev, nullptr), "lg_fill_normal_f32");
}
template <typename T>
inline void dev_fill_const(T* p, int64_t n, float v) {
    if (dtype_of<T>::value == LG_F16) note_status(lg_fill_const_f16(p, n, v, nullptr), "lg_fill_const_f16");
    else note_status(lg_fill_const_f32((float*)p, n, v, nullptr), "lg_fill_const_f32");
}

inline int64_t align_up(int64_t x, int64_t a = 128) { return (x + a - 1) / a * a; }

// Named parameters of a layer, for tests that download / upload them.
struct ParamRef {
    std::string name;
    void* ptr;
    int64_t elems;
    int rows = 1, cols = 0;   // logical shape [in, out] of a weight matrix (vectors: rows = 1)
    int transposed = 0;       // bit 0: stored as [out, in]; bit 1: the out dimension (or the vector) is stored with its two
                              // halves interleaved in groups of 16 (stored group 2g = logical [16g, 16g+16) of the first
                              // half, stored group 2g+1 = the same range of the second half); bit 2: the [out, in] matrix is
                              // stored in the tiled layout of lg_weight_tile_f16 (16 x 32 fragment blocks)
};

// ParamRef::transposed bits of a weight layout, and the shapes the tiled layout can hold
inline int layout_bits(int weight_layout) { return weight_layout == 2 ? (1 | 4) : (weight_layout ? 1 : 0); }
inline void check_tiled_shape(int weight_layout, int dtype, int features, int k, const char* who) {
    if (weight_layout != 2) return;
    if (dtype != LG_F16 || features % 16 != 0 || k % 32 != 0)
        set_error_state(LG_ERR_INVALID, std::string(who) + ": the tiled weight layout is fp16 only and needs features % 16 == 0 and k % 32 == 0 (features " +
                        std::to_string(features) + ", k " + std::to_string(k) + ")");
}

// ---------------------------------------------------------------------------------------------------
// Linear layers.  Y[M, N'] = X[M, K'] * W with W stored row-major [K', N'] (the layout cuBLAS's (N,N) call in
// the reference implies: column-major N' x K' with lda = N').
// ---------------------------------------------------------------------------------------------------
template <typename T>
class Linear_Col {  // linear.h:68-109: output features split across ranks
  public:
    int k, n;  // GLOBAL in/out features
    T* weights;
    StaticInitParam SParams;
    std::vector<FuncWrap> FuncWrapVec;

    int weight_layout = 0;  // 0: [k, n_local] row-major; 1: [n_local, k] row-major (multiplied with transa = T); 2: [n_local, k] in
                            // the tiled layout (transa = LG_OP_TILED; fp16, n_local % 16 == 0, k % 32 == 0)
    int interleave16 = 0;   // 1: output features stored as (gate, up) groups of 16 (the GeGLU epilogue's order)

    int lda_view = 0;       // > 0: `weights` points into a wider matrix with this leading dimension (one of q / k / v inside the
                            // packed [H, 3 Hl] projection); the object then owns and initialises nothing

    Linear_Col(const StaticInitParam& SParams_, const int& k_, const int& n_, int weight_layout_ = 0)
        : k(k_), n(n_), SParams(SParams_), weight_layout(weight_layout_) {
        weights = dev_alloc<T>((size_t)k * n / SParams.world_size);
        check_tiled_shape(weight_layout, dtype_of<T>::value, n_local(), k, "Linear_Col");
    }
    Linear_Col(const StaticInitParam& SParams_, const int& k_, const int& n_, int weight_layout_, T* view, int lda)
        : k(k_), n(n_), weights(view), SParams(SParams_), weight_layout(weight_layout_), lda_view(lda) {}
    Linear_Col(const Linear_Col&) = delete;
    Linear_Col& operator=(const Linear_Col&) = delete;
    ~Linear_Col() { if (!lda_view) dev_free(weights); }
    ParamRef param(const std::string& name) { return ParamRef{name, weights, (int64_t)k * n_local(), k, n_local(), layout_bits(weight_layout) | (interleave16 << 1)}; }
    int n_local() const { return n / SParams.world_size; }
    void init_weights(uint64_t seed, uint64_t tensor_id, float stddev = 0.02f) {
        if (!lda_view) dev_fill_normal(weights, (int64_t)k * n_local(), seed, tensor_id, 0.f, stddev);
    }
    GemmDesc desc(T* input, T* output, int m) const {
        GemmDesc g;
        g.valid = true; g.dtype = dtype_of<T>::value; g.transa = weight_layout;
        g.m = n_local(); g.n = m; g.k = k;
        g.A = weights; g.lda = lda_view ? lda_view : (weight_layout ? k : n_local()); g.B = input; g.ldb = k; g.C = output; g.ldc = n_local();
        return g;
    }
    std::vector<FuncWrap> forward(T* input, T* output, int m) {
        FuncWrapVec.clear();
        GemmDesc g = desc(input, output, m);
        FuncWrapVec.push_back(FuncWrap(1.0f, GEMM, [g](const DynamicInitParam& D) { GemmEx(D, g); }, g, "linear_col"));
        return FuncWrapVec;
    }
};

template <typename T>
class Linear_Row {  // linear.h:16-64: input features split across ranks; partial sums
  public:
    int k, n;
    T* weights;
    StaticInitParam SParams;
    std::vector<FuncWrap> FuncWrapVec;

    int weight_layout = 0;  // 0: [k_local, n] row-major; 1: [n, k_local] row-major (multiplied with transa = T); 2: [n, k_local] tiled

    Linear_Row(const StaticInitParam& SParams_, const int& k_, const int& n_, int weight_layout_ = 0)
        : k(k_), n(n_), SParams(SParams_), weight_layout(weight_layout_) {
        weights = dev_alloc<T>((size_t)k * n / SParams.world_size);
        check_tiled_shape(weight_layout, dtype_of<T>::value, n, k_local(), "Linear_Row");
    }
    Linear_Row(const Linear_Row&) = delete;
    Linear_Row& operator=(const Linear_Row&) = delete;
    ~Linear_Row() { dev_free(weights); }
    ParamRef param(const std::string& name) { return ParamRef{name, weights, (int64_t)k_local() * n, k_local(), n, layout_bits(weight_layout)}; }
    int k_local() const { return k / SParams.world_size; }
    void init_weights(uint64_t seed, uint64_t tensor_id, float stddev = 0.02f) {
        dev_fill_normal(weights, (int64_t)k_local() * n, seed, tensor_id, 0.f, stddev);
    }
    GemmDesc desc(T* input, T* output, int m) const {
        GemmDesc g;
        g.valid = true; g.dtype = dtype_of<T>::value; g.transa = weight_layout;
        g.m = n; g.n = m; g.k = k_local();
        g.A = weights; g.lda = weight_layout ? k_local() : n; g.B = input; g.ldb = k_local(); g.C = output; g.ldc = n;
        return g;
    }
    std::vector<FuncWrap> forward(T* input, T* output, int m) {
        FuncWrapVec.clear();
        GemmDesc g = desc(input, output, m);
        FuncWrapVec.push_back(FuncWrap(2.0f, GEMM, [g](const DynamicInitParam& D) { GemmEx(D, g); }, g, "linear_row"));
        // linear.h:55-60 appends the all-reduce of m*n elements here when world_size != 1.  The exchange between
        // GPUs is outside this single-GPU build, so the vector holds this rank's partial product only.
        return FuncWrapVec;
    }
};

template <typename T>
class LayerNorm {  // operator.h:16-41
  public:
    int k;
    T* gamma;
    T* beta;
    StaticInitParam SParams;
    std::vector<FuncWrap> FuncWrapVec;

    LayerNorm(const StaticInitParam& SParams_, const int& k_) : k(k_), SParams(SParams_) {
        gamma = dev_alloc<T>(k);
        beta = dev_alloc<T>(k);
        dev_fill_const(gamma, k, 1.0f);
        dev_fill_const(beta, k, 0.0f);
    }
    LayerNorm(const LayerNorm&) = delete;
    LayerNorm& operator=(const LayerNorm&) = delete;
    ~LayerNorm() { dev_free(gamma); dev_free(beta); }
    void init_weights(uint64_t seed, uint64_t tensor_id) {
        dev_fill_normal(gamma, k, seed, tensor_id, 1.0f, 0.1f);
        dev_fill_normal(beta, k, seed, tensor_id + 1, 0.0f, 0.1f);
    }
    std::vector<FuncWrap> forward(T* input, T* output, int m) {
        FuncWrapVec.clear();
        T *g = gamma, *b = beta;
        int kk = k;
        FuncWrapVec.push_back(FuncWrap(0.1f, COMPUTATION,
                                       [=](const DynamicInitParam& D) { Layer_Norm<T>(input, g, b, output, m, kk, D); },
                                       "layer_norm"));
        FuncWrapVec.back().minor = true;
        return FuncWrapVec;
    }
};

// ---------------------------------------------------------------------------------------------------
// MLP  (bert_layer.h:19-63)
// ---------------------------------------------------------------------------------------------------
template <typename T>
class Bert_MLP {
  public:
    int k, n, intermediate_size;  // GLOBAL sizes
    int mlp_ratio = 4;
    StaticInitParam SParam;
    BertInitParam BertParams;
    T* linear_row_output;  // default inner buffer
    T* bias;               // [F local]   (bert_layer.h:45)
    T* bias2;              // [k] FFN-2 bias: only used by the pre-LN assembly
    Linear_Col<T>* linear_col;
    Linear_Row<T>* linear_row;
    std::vector<FuncWrap> FuncWrapVec;

    Bert_MLP(const BertInitParam& BertParams_, const StaticInitParam& SParam_, const int& k_, const int& n_, T* workspace)
        : k(k_), n(n_), SParam(SParam_), BertParams(BertParams_), linear_row_output(workspace) {
        intermediate_size = BertParams.ffn_inner > 0 ? BertParams.ffn_inner : n * mlp_ratio;
        // GeGLU: FFN-1 produces [gate | up], 2 F local columns
        linear_col = new Linear_Col<T>(SParam, k, intermediate_size * gate_mult(), BertParams.weight_layout);
        linear_row = new Linear_Row<T>(SParam, intermediate_size, k, BertParams.weight_layout);
        linear_col->interleave16 = geglu_fused() ? 1 : 0;
        bias = dev_alloc<T>(f_local() * gate_mult());
        bias2 = dev_alloc<T>(k);
        dev_fill_const(bias, f_local() * gate_mult(), 0.f);
        dev_fill_const(bias2, k, 0.f);
    }
    Bert_MLP(const Bert_MLP&) = delete;
    Bert_MLP& operator=(const Bert_MLP&) = delete;
    ~Bert_MLP() { delete linear_col; delete linear_row; dev_free(bias); dev_free(bias2); }
    int f_local() const { return intermediate_size / SParam.world_size; }
    int gate_mult() const { return BertParams.ffn_act == FFN_GEGLU ? 2 : 1; }
    // GeGLU in the fused fp16 assembly: FFN-1's weight and bias are stored with gate and up interleaved in groups of 16 features,
    // and the product is formed in the GEMM's epilogue (no [gate | up] buffer, no separate pass over it)
    static bool geglu_fused(const BertInitParam& P, const StaticInitParam& S, int hidden) {
        const int64_t F = (P.ffn_inner > 0 ? P.ffn_inner : 4 * hidden) / S.world_size;
        return P.ffn_act == FFN_GEGLU && P.fused && dtype_of<T>::value == LG_F16 && F % 16 == 0;
    }
    bool geglu_fused() const { return geglu_fused(BertParams, SParam, n); }
    // elements of the FFN-1 output buffer per token (unfused GeGLU keeps [gate | up] and the product)
    static int64_t inner_per_token(const BertInitParam& P, const StaticInitParam& S, int hidden) {
        const int64_t F = (P.ffn_inner > 0 ? P.ffn_inner : 4 * hidden) / S.world_size;
        return (P.ffn_act == FFN_GEGLU && !geglu_fused(P, S, hidden)) ? 3 * F : F;
    }
    void init_weights(uint64_t seed, uint64_t base) {
        linear_col->init_weights(seed, base + 0);
        linear_row->init_weights(seed, base + 1);
        dev_fill_normal(bias, f_local() * gate_mult(), seed, base + 2, 0.f, 0.02f);
        dev_fill_normal(bias2, k, seed, base + 3, 0.f, 0.02f);
    }
    void params(const std::string& prefix, std::vector<ParamRef>& out) {
        out.push_back(linear_col->param(prefix + "w1"));
        out.push_back({prefix + "b1", bias, f_local() * gate_mult(), 1, f_local() * gate_mult(), geglu_fused() ? 2 : 0});
        out.push_back(linear_row->param(prefix + "w2"));
        out.push_back({prefix + "b2", bias2, k, 1, k, 0});
    }
    // inner: [m, F local] scratch.  idx 11, 12, 13 of the launch vector (fused: 2 entries).
    std::vector<FuncWrap> forward(T* input, T* output, int m, T* inner = nullptr) {
        FuncWrapVec.clear();
        if (!inner) inner = linear_row_output;
        const int F = f_local();
        if (geglu_fused()) {
            GemmDesc g = linear_col->desc(input, inner, m);
            g.epilogue = LG_EPI_BIAS_GEGLU;
            g.bias = bias;
            g.ldc = F;
            FuncWrapVec.push_back(FuncWrap(1.0f, GEMM, [g](const DynamicInitParam& D) { GemmEx(D, g); }, g, "ffn1+bias+geglu"));
        } else if (BertParams.ffn_act == FFN_GEGLU) {
            // inner holds [m, F] (the product) followed by [m, 2F] (gate | up)
            T* gu = inner + (int64_t)m * F;
            std::vector<FuncWrap> v = linear_col->forward(input, gu, m);
            v[0].label = "ffn1(gate+up)";
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
            T* b = bias;
            FuncWrapVec.push_back(FuncWrap(0.2f, COMPUTATION,
                                           [=](const DynamicInitParam& D) { Add_bias_geglu_kernelLauncher<T>(inner, gu, b, m, F, D); },
                                           "bias+geglu"));
        } else if (BertParams.fused && dtype_of<T>::value == LG_F16) {
            GemmDesc g = linear_col->desc(input, inner, m);
            g.epilogue = LG_EPI_BIAS_GELU;
            g.bias = bias;
            FuncWrapVec.push_back(FuncWrap(1.0f, GEMM, [g](const DynamicInitParam& D) { GemmEx(D, g); }, g, "ffn1+bias+gelu"));
        } else {
            std::vector<FuncWrap> v = linear_col->forward(input, inner, m);
            v[0].label = "ffn1";
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
            T* b = bias;
            FuncWrapVec.push_back(FuncWrap(0.2f, COMPUTATION,
                                           [=](const DynamicInitParam& D) { Add_bias_act_kernelLauncher<T>(inner, b, m, F, D); },
                                           "bias+gelu"));
        }
        std::vector<FuncWrap> v = linear_row->forward(inner, output, m);
        v[0].label = "ffn2";
        FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
        return FuncWrapVec;
    }
};

// ---------------------------------------------------------------------------------------------------
// Multi-head attention  (bert_layer.h:65-176)
// ---------------------------------------------------------------------------------------------------
template <typename T>
struct MhaBuffers {  // per-request slices, all in elements of T
    T *q, *k, *v, *q_buf, *k_buf, *v_buf, *qk_buf, *attn_trans_out, *attn_out;
    T* mask;          // attr_mask [batch, seq, seq] of the reference-shaped assembly
    void* decode_ws;  // split-KV partials of the decode attention
};

// Which (batch, seq, causal) the attr_mask slice of a workspace was last written for.  The slices of a workspace are a function of
// its base and the request's shape, so as long as the same shape keeps using the workspace nothing else overlaps the mask.
// Launch callbacks run on the scheduler's thread, the profiler's on the caller's: hence the lock.
struct MaskState {
    std::mutex mu;
    std::map<const void*, std::tuple<int, int, int>> last;
    bool in_place(const void* ws_base, int batch, int seq, int causal) {
        std::lock_guard<std::mutex> lk(mu);
        const auto want = std::make_tuple(batch, seq, causal);
        auto it = last.find(ws_base);
        if (it != last.end() && it->second == want) return true;
        last[ws_base] = want;
        return false;
    }
};

template <typename T>
class Bert_MHA {
  public:
    int k, n;
    float scalar;
    Linear_Col<T>* linear_q_col;
    Linear_Col<T>* linear_k_col;
    Linear_Col<T>* linear_v_col;
    Linear_Col<T>* linear_qkv_col = nullptr;  // packed_qkv: one [H, 3 Hl] projection, columns [q | k | v]
    T* qkv_bias = nullptr;                    // packed_qkv: [3 Hl]
    Linear_Row<T>* linear_w_row;
    StaticInitParam SParam;
    BertInitParam BertParams;
    T *q_bias, *k_bias, *v_bias, *w_bias;
    T* workspace;
    T *k_cache = nullptr, *v_cache = nullptr;  // [max_batch, heads, max_cache_len, d] when max_cache_len > 0
    std::shared_ptr<MaskState> mask_state = std::make_shared<MaskState>();
    std::vector<FuncWrap> FuncWrapVec;

    Bert_MHA(const BertInitParam& BertParams_, const StaticInitParam& SParam_, const int& k_, const int& n_, T* workspace_)
        : k(k_), n(n_), SParam(SParam_), BertParams(BertParams_), workspace(workspace_) {
        scalar = 1.0f / sqrtf((float)BertParams.size_per_head);  // bert_layer.h:94
        linear_w_row = new Linear_Row<T>(SParam, k, n, BertParams.weight_layout);
        w_bias = dev_alloc<T>(n);
        dev_fill_const(w_bias, n, 0.f);
        if (BertParams.packed_qkv) {
            // one [H, 3 Hl] projection, columns [q | k | v]; the three per-projection objects are views of its column blocks
            // (weights stored [out, in]: row blocks), so every assembly that issues q, k and v separately, or as one grouped
            // launch, reads the packed parameters
            const int wl = BertParams.weight_layout;
            linear_qkv_col = new Linear_Col<T>(SParam, k, 3 * n, wl);
            qkv_bias = dev_alloc<T>(3 * hl());
            dev_fill_const(qkv_bias, 3 * hl(), 0.f);
            T* w = linear_qkv_col->weights;
            const int64_t step = wl ? (int64_t)hl() * k : hl();
            const int lda = wl ? k : 3 * hl();
            linear_q_col = new Linear_Col<T>(SParam, k, n, wl, w, lda);
            linear_k_col = new Linear_Col<T>(SParam, k, n, wl, w + step, lda);
            linear_v_col = new Linear_Col<T>(SParam, k, n, wl, w + 2 * step, lda);
            q_bias = qkv_bias; k_bias = qkv_bias + hl(); v_bias = qkv_bias + 2 * hl();
        } else {
            linear_q_col = new Linear_Col<T>(SParam, k, n, BertParams.weight_layout);
            linear_k_col = new Linear_Col<T>(SParam, k, n, BertParams.weight_layout);
            linear_v_col = new Linear_Col<T>(SParam, k, n, BertParams.weight_layout);
            q_bias = dev_alloc<T>(hl()); k_bias = dev_alloc<T>(hl()); v_bias = dev_alloc<T>(hl());
            dev_fill_const(q_bias, hl(), 0.f); dev_fill_const(k_bias, hl(), 0.f); dev_fill_const(v_bias, hl(), 0.f);
        }
        if (BertParams.max_cache_len > 0) {
            const size_t ce = (size_t)BertParams.max_batch_size * heads() * BertParams.max_cache_len * BertParams.size_per_head;
            k_cache = dev_alloc<T>(ce);
            v_cache = dev_alloc<T>(ce);
            note_status(lg_memset_async(k_cache, 0, ce * sizeof(T), nullptr), "lg_memset_async");
            note_status(lg_memset_async(v_cache, 0, ce * sizeof(T), nullptr), "lg_memset_async");
        }
    }
    Bert_MHA(const Bert_MHA&) = delete;
    Bert_MHA& operator=(const Bert_MHA&) = delete;
    ~Bert_MHA() {
        delete linear_q_col; delete linear_k_col; delete linear_v_col; delete linear_w_row;
        if (linear_qkv_col) { delete linear_qkv_col; dev_free(qkv_bias); }   // q / k / v biases are parts of qkv_bias
        else { dev_free(q_bias); dev_free(k_bias); dev_free(v_bias); }
        dev_free(w_bias); dev_free(k_cache); dev_free(v_cache);
    }
    int heads() const { return BertParams.head_num / SParam.world_size; }
    int hl() const { return heads() * BertParams.size_per_head; }
    void init_weights(uint64_t seed, uint64_t base) {
        linear_q_col->init_weights(seed, base + 0);  // views of the packed projection fill nothing
        linear_k_col->init_weights(seed, base + 1);
        linear_v_col->init_weights(seed, base + 2);
        linear_w_row->init_weights(seed, base + 3);
        if (!linear_qkv_col) {
            dev_fill_normal(q_bias, hl(), seed, base + 4, 0.f, 0.02f);
            dev_fill_normal(k_bias, hl(), seed, base + 5, 0.f, 0.02f);
            dev_fill_normal(v_bias, hl(), seed, base + 6, 0.f, 0.02f);
        }
        dev_fill_normal(w_bias, n, seed, base + 7, 0.f, 0.02f);
        if (linear_qkv_col) {
            linear_qkv_col->init_weights(seed, base + 20);
            dev_fill_normal(qkv_bias, 3 * hl(), seed, base + 21, 0.f, 0.02f);
        }
    }
    void params(const std::string& prefix, std::vector<ParamRef>& out) {
        if (linear_qkv_col) {
            // the packed projection replaces wq / wk / wv and their biases
            out.push_back(linear_qkv_col->param(prefix + "wqkv"));
            out.push_back({prefix + "bqkv", qkv_bias, 3 * hl(), 1, 3 * hl(), 0});
            out.push_back(linear_w_row->param(prefix + "wo"));
            out.push_back({prefix + "bo", w_bias, n, 1, n, 0});
            return;
        }
        out.push_back(linear_q_col->param(prefix + "wq"));
        out.push_back(linear_k_col->param(prefix + "wk"));
        out.push_back(linear_v_col->param(prefix + "wv"));
        out.push_back({prefix + "bq", q_bias, hl(), 1, hl(), 0});
        out.push_back({prefix + "bk", k_bias, hl(), 1, hl(), 0});
        out.push_back({prefix + "bv", v_bias, hl(), 1, hl(), 0});
        out.push_back(linear_w_row->param(prefix + "wo"));
        out.push_back({prefix + "bo", w_bias, n, 1, n, 0});
    }
    static int64_t score_elems(const BertInitParam& P, const StaticInitParam& S, int batch, int seq) {
        const bool fused = P.fused && dtype_of<T>::value == LG_F16;
        return fused ? 0 : align_up((int64_t)batch * (P.head_num / S.world_size) * seq * seq);
    }
    static int64_t decode_ws_elems(const BertInitParam& P, const StaticInitParam& S, int batch) {
        if (P.max_cache_len <= 0) return 0;
        const size_t bytes = lg_attn_decode_workspace_bytes(batch, P.head_num / S.world_size, P.size_per_head, P.max_cache_len);
        return align_up((int64_t)((bytes + sizeof(T) - 1) / sizeof(T)));
    }
    // attr_mask [batch, seq, seq] lives in the request's workspace (reference-shaped assembly only; bert_layer.h:118 keeps one
    // buffer in the layer, which requests of different lengths in flight at the same time could not share)
    static int64_t mask_elems(const BertInitParam& P, int batch, int seq) {
        const bool fused = P.fused && dtype_of<T>::value == LG_F16;
        return fused ? 0 : align_up((int64_t)batch * seq * seq);
    }
    static int64_t workspace_elems(const BertInitParam& P, const StaticInitParam& S, int batch, int seq) {
        const int64_t M = (int64_t)batch * seq, hl_ = (int64_t)(P.head_num / S.world_size) * P.size_per_head;
        return 8 * align_up(M * hl_) + score_elems(P, S, batch, seq) + mask_elems(P, batch, seq) + decode_ws_elems(P, S, batch);
    }
    MhaBuffers<T> slice(T* ws, int batch, int seq) const {
        const int64_t M = (int64_t)batch * seq, a = align_up(M * hl());
        MhaBuffers<T> b;
        b.q = ws; b.k = b.q + a; b.v = b.k + a;
        b.q_buf = b.v + a; b.k_buf = b.q_buf + a; b.v_buf = b.k_buf + a;
        b.attn_trans_out = b.v_buf + a; b.attn_out = b.attn_trans_out + a;
        b.qk_buf = b.attn_out + a;
        b.mask = b.qk_buf + score_elems(BertParams, SParam, batch, seq);
        b.decode_ws = b.mask + mask_elems(BertParams, batch, seq);
        return b;
    }
    // idx 0..8 of the launch vector (9 entries); fused assembly: 5 entries.
    // cache_slot >= 0 (fused only): K/V are written straight into the KV cache rows [cache_slot, cache_slot+batch).
    // past > 0 (fused assembly with a cache slot only): the seq_len tokens continue sequences whose first `past` positions are
    // in the KV cache already (a long prompt prefilled in chunks): K / V go to cache rows past .., the attention sees the past
    // and the chunk's own keys.  No reference counterpart.
    std::vector<FuncWrap> forward(T* input, T* output, int batch_size, int seq_len, T* ws = nullptr, int cache_slot = -1, int past = 0) {
        FuncWrapVec.clear();
        if (!ws) ws = workspace;
        const MhaBuffers<T> b = slice(ws, batch_size, seq_len);
        const int M = batch_size * seq_len, h = heads(), d = BertParams.size_per_head;
        const int dt = dtype_of<T>::value;
        const float sc = scalar;
        if (cache_slot >= 0 && k_cache && (past + seq_len > BertParams.max_cache_len || cache_slot + batch_size > BertParams.max_batch_size)) {
            set_error_state(LG_ERR_INVALID, "Bert_MHA::forward: sequence or cache slot outside the KV cache");
            return FuncWrapVec;
        }
        if (past < 0 || (past > 0 && !(BertParams.fused && dt == LG_F16 && cache_slot >= 0 && k_cache))) {
            set_error_state(LG_ERR_INVALID, "Bert_MHA::forward: a prefill that continues a sequence needs the fused assembly and a KV-cache slot");
            return FuncWrapVec;
        }
        if (BertParams.fused && dt == LG_F16) {
            T* kdst = b.k_buf;
            T* vdst = b.v_buf;
            int kv_rows = seq_len;
            if (cache_slot >= 0 && k_cache) {
                kv_rows = BertParams.max_cache_len;
                kdst = k_cache + (int64_t)cache_slot * h * kv_rows * d;
                vdst = v_cache + (int64_t)cache_slot * h * kv_rows * d;
            }
            Linear_Col<T>* lin[3] = {linear_q_col, linear_k_col, linear_v_col};
            T* dst[3] = {b.q_buf, kdst + (int64_t)past * d, vdst + (int64_t)past * d};  // row `past` of every (sequence, head) slot
            const T* bias[3] = {q_bias, k_bias, v_bias};
            const char* lab[3] = {"q_gemm+bias+heads", "k_gemm+bias+heads", "v_gemm+bias+heads"};
            GemmDesc gd[3];
            for (int t = 0; t < 3; ++t) {
                GemmDesc g = lin[t]->desc(input, dst[t], M);
                g.epilogue = LG_EPI_BIAS_HEADS;
                g.bias = bias[t];
                g.epi_seq = seq_len; g.epi_d = d; g.epi_heads_total = h;
                g.ldc = (t == 0) ? seq_len : kv_rows;  // rows per (batch, head) slot of the destination
                gd[t] = g;
                if (!linear_qkv_col) FuncWrapVec.push_back(FuncWrap(1.0f, GEMM, [g](const DynamicInitParam& D) { GemmEx(D, g); }, g, lab[t]));
            }
            if (linear_qkv_col) {
                // packed projection: ONE launch over the [H, 3 Hl] weight whose epilogue routes the q columns to q_buf and the k
                // and v columns to their buffers or straight into the KV cache (attention_kernels.cu:331-393 does the routing in
                // a separate kernel after the GEMM)
                const GemmDesc gq = gd[0], gk = gd[1], gv = gd[2];
                FuncWrapVec.push_back(FuncWrap(1.0f, COMPUTATION, [gq, gk, gv](const DynamicInitParam& D) { GemmExGrouped3(D, gq, gk, gv); },
                                               "qkv_gemm+bias+heads", MFMA_BOUND));
            }
            T* qb = b.q_buf; T* ao = b.attn_out;
            const int causal = BertParams.causal;
            FuncWrapVec.push_back(FuncWrap(0.8f, COMPUTATION, [=](const DynamicInitParam& D) {
                if (past > 0)
                    note_status(lg_attn_prefill_past_f16(qb, kdst, vdst, ao, batch_size, seq_len, past, h, d, kv_rows, sc, causal, 1, D.stream),
                                "lg_attn_prefill_past_f16");
                else
                    note_status(lg_attn_prefill_f16(qb, kdst, vdst, nullptr, ao, batch_size, seq_len, h, d, kv_rows, sc, causal, 1,
                                                    D.stream), "lg_attn_prefill_f16");
            }, "attn_prefill_fused", MFMA_BOUND));
            std::vector<FuncWrap> v = linear_w_row->forward(b.attn_out, output, M);
            v[0].label = "out_proj";
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
            return FuncWrapVec;
        }

        std::vector<FuncWrap> v;
        if (linear_qkv_col) {
            // packed projection: QKV [M, 3, Hl] in the (contiguous) q, k, v slices, then the reference's fused
            // bias + transpose kernel (attention_kernels.cuh:23-34)
            v = linear_qkv_col->forward(input, b.q, M); v[0].label = "qkv_gemm";
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
            T* qkvb = qkv_bias;
            FuncWrapVec.push_back(FuncWrap(0.2f, COMPUTATION, [=](const DynamicInitParam& D) {
                Add_fusedQKV_bias_transpose_kernelLauncher<T>(b.q_buf, b.k_buf, b.v_buf, b.q, qkvb, batch_size, seq_len, h, d, D);
            }, "fused_qkv_bias_transpose"));
        } else {
            // qkv linear  (bert_layer.h:128-135)
            v = linear_q_col->forward(input, b.q, M); v[0].label = "q_gemm";
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
            v = linear_k_col->forward(input, b.k, M); v[0].label = "k_gemm";
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
            v = linear_v_col->forward(input, b.v, M); v[0].label = "v_gemm";
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
            // bias + transpose  (:139-142)
            T *qbias = q_bias, *kbias = k_bias, *vbias = v_bias;
            FuncWrapVec.push_back(FuncWrap(0.2f, COMPUTATION, [=](const DynamicInitParam& D) {
                Add_QKV_bias_transpose<T>(b.q_buf, b.k_buf, b.v_buf, b.q, qbias, b.k, kbias, b.v, vbias, batch_size, seq_len, h, d, D);
            }, "qkv_bias_transpose"));
        }
        // qk  (:145-150)
        FuncWrapVec.push_back(FuncWrap(0.3f, COMPUTATION, [=](const DynamicInitParam& D) {
            GemmStridedBatchedEx(D, dt, 1, 0, seq_len, seq_len, d, b.k_buf, d, (long long)seq_len * d, b.q_buf, d,
                                 (long long)seq_len * d, b.qk_buf, seq_len, (long long)seq_len * seq_len, batch_size * h);
        }, "qk_gemm", MFMA_BOUND));
        // softmax  (:153-155).  The mask (all ones, or lower-triangular) is written into the request's workspace by the same
        // entry, on the launch stream: building the vector neither allocates nor synchronises.  It is written when the
        // workspace last held another shape's slices (or nothing): the layers of one request, the requests of one shape that
        // follow each other on a context and the repeated launches of the profiler find it in place, so a profiled softmax is
        // the softmax alone.
        const int causal_mask = BertParams.causal;
        std::shared_ptr<MaskState> ms = mask_state;
        FuncWrapVec.push_back(FuncWrap(0.2f, COMPUTATION, [=](const DynamicInitParam& D) {
            if (ms->in_place(b.q, batch_size, seq_len, causal_mask)) {
                // nothing to write
            } else if (dt == LG_F16) {
                if (causal_mask) note_status(lg_fill_causal_mask_f16(b.mask, batch_size, seq_len, D.stream), "lg_fill_causal_mask_f16");
                else note_status(lg_fill_const_f16(b.mask, (int64_t)batch_size * seq_len * seq_len, 1.0f, D.stream), "lg_fill_const_f16");
            } else {
                if (causal_mask) note_status(lg_fill_causal_mask_f32((float*)b.mask, batch_size, seq_len, D.stream), "lg_fill_causal_mask_f32");
                else note_status(lg_fill_const_f32((float*)b.mask, (int64_t)batch_size * seq_len * seq_len, 1.0f, D.stream), "lg_fill_const_f32");
            }
            Attn_softmax_kernel<T>(b.qk_buf, b.mask, batch_size, seq_len, h, sc, D);
        }, "softmax"));
        // qkv  (:158-163)
        FuncWrapVec.push_back(FuncWrap(0.3f, COMPUTATION, [=](const DynamicInitParam& D) {
            GemmStridedBatchedEx(D, dt, 0, 0, d, seq_len, seq_len, b.v_buf, d, (long long)seq_len * d, b.qk_buf, seq_len,
                                 (long long)seq_len * seq_len, b.attn_trans_out, d, (long long)seq_len * d, batch_size * h);
        }, "pv_gemm", MFMA_BOUND));
        // transpose back  (:166-168)
        FuncWrapVec.push_back(FuncWrap(0.1f, COMPUTATION, [=](const DynamicInitParam& D) {
            Transpose_kernel<T>(b.attn_out, b.attn_trans_out, batch_size, seq_len, h, d, D);
        }, "transpose_back"));
        // linear row  (:171)
        v = linear_w_row->forward(b.attn_out, output, M); v[0].label = "out_proj";
        FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
        return FuncWrapVec;
    }

    // One decode step for `batch` sequences whose cache rows start at cache_slot: Q/K/V GEMMs on one token each,
    // bias + append to the cache at position `past`, attention over past+1 positions, output projection.
    // No reference counterpart (the reference has no KV cache).  fp16 only.
    std::vector<FuncWrap> forward_decode(T* input, T* output, int batch, int past, int cache_slot, T* ws = nullptr) {
        FuncWrapVec.clear();
        if (!ws) ws = workspace;
        const MhaBuffers<T> b = slice(ws, batch, 1);
        const int h = heads(), d = BertParams.size_per_head, Lmax = BertParams.max_cache_len;
        // the K/V epilogues write cache row `past` of slots [cache_slot, cache_slot + batch): outside the cache nothing is built
        if (!k_cache || past < 0 || past >= Lmax || cache_slot < 0 || cache_slot + batch > BertParams.max_batch_size) {
            set_error_state(LG_ERR_INVALID, "Bert_MHA::forward_decode: position or cache slot outside the KV cache");
            return FuncWrapVec;
        }
        const float sc = scalar;
        T* kc = k_cache + (int64_t)cache_slot * h * Lmax * d;
        T* vc = v_cache + (int64_t)cache_slot * h * Lmax * d;
        void* dws = b.decode_ws;
        std::vector<FuncWrap> v;
        if (BertParams.fused) {
            // the GEMM epilogues add the bias and write q as [B, h, d] and the new K/V rows straight into the cache at
            // position `past` (one token per sequence: batch index = token index, row 0 of a slot shifted by `past` rows)
            Linear_Col<T>* lin[3] = {linear_q_col, linear_k_col, linear_v_col};
            T* dst[3] = {b.q_buf, kc + (int64_t)past * d, vc + (int64_t)past * d};
            const T* bias[3] = {q_bias, k_bias, v_bias};
            GemmDesc g[3];
            for (int t = 0; t < 3; ++t) {
                g[t] = lin[t]->desc(input, dst[t], batch);
                g[t].epilogue = LG_EPI_BIAS_HEADS;
                g[t].bias = bias[t];
                g[t].epi_seq = 1; g[t].epi_d = d; g[t].epi_heads_total = h;
                g[t].ldc = (t == 0) ? 1 : Lmax;  // rows per (batch, head) slot of the destination
            }
            // one launch for the three projections: they read the same token rows and nothing orders them among themselves
            const GemmDesc gq = g[0], gk = g[1], gv = g[2];
            FuncWrapVec.push_back(FuncWrap(1.0f, COMPUTATION, [gq, gk, gv](const DynamicInitParam& D) { GemmExGrouped3(D, gq, gk, gv); },
                                           "qkv_gemm(decode)", HBM_BOUND));
        } else {
            v = linear_q_col->forward(input, b.q, batch); v[0].label = "q_gemm(decode)"; v[0].rclass = HBM_BOUND;
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
            v = linear_k_col->forward(input, b.k, batch); v[0].label = "k_gemm(decode)"; v[0].rclass = HBM_BOUND;
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
            v = linear_v_col->forward(input, b.v, batch); v[0].label = "v_gemm(decode)"; v[0].rclass = HBM_BOUND;
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
            T *qbias = q_bias, *kbias = k_bias, *vbias = v_bias;
            FuncWrapVec.push_back(FuncWrap(0.05f, COMPUTATION, [=](const DynamicInitParam& D) {
                note_status(lg_kv_append_f16(b.q_buf, kc, vc, b.q, qbias, b.k, kbias, b.v, vbias, batch, h, d, past, Lmax, D.stream), "lg_kv_append_f16");
            }, "kv_append"));
            FuncWrapVec.back().minor = true;
        }
        FuncWrapVec.push_back(FuncWrap(0.15f, COMPUTATION, [=](const DynamicInitParam& D) {
            note_status(lg_attn_decode_f16(b.q_buf, kc, vc, b.attn_out, dws, batch, h, d, past + 1, Lmax, sc, D.stream), "lg_attn_decode_f16");
        }, "attn_decode"));
        v = linear_w_row->forward(b.attn_out, output, batch); v[0].label = "out_proj(decode)"; v[0].rclass = HBM_BOUND;
        FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
        return FuncWrapVec;
    }

    // One decode step for sequences that sit in arbitrary cache slots at different positions (decode steps of different
    // requests as one launch vector): sequence i reads and extends cache slot slots[i], which holds pasts[i] positions.
    // Same entries as forward_decode, with the per-sequence variants of the kernels that touch the cache.
    std::vector<FuncWrap> forward_decode_seqs(T* input, T* output, const std::vector<int>& slots, const std::vector<int>& pasts,
                                              T* ws = nullptr) {
        FuncWrapVec.clear();
        if (!ws) ws = workspace;
        const int batch = (int)slots.size();
        const MhaBuffers<T> b = slice(ws, batch, 1);
        const int h = heads(), d = BertParams.size_per_head, Lmax = BertParams.max_cache_len;
        bool ok = k_cache && batch > 0 && batch <= LG_ATTN_DECODE_MAX_SEQS && pasts.size() == slots.size();
        for (int i = 0; i < batch && ok; ++i) ok = slots[i] >= 0 && slots[i] < BertParams.max_batch_size && pasts[i] >= 0 && pasts[i] < Lmax;
        if (!ok) {
            set_error_state(LG_ERR_INVALID, "Bert_MHA::forward_decode_seqs: a position or cache slot lies outside the KV cache");
            return FuncWrapVec;
        }
        const float sc = scalar;
        T *kc = k_cache, *vc = v_cache;
        void* dws = b.decode_ws;
        std::vector<int> lens(pasts);
        for (int& l : lens) l += 1;
        std::vector<FuncWrap> v;
        if (BertParams.fused) {
            Linear_Col<T>* lin[3] = {linear_q_col, linear_k_col, linear_v_col};
            T* dst[3] = {b.q_buf, kc, vc};
            const T* bias[3] = {q_bias, k_bias, v_bias};
            GemmDesc g[3];
            for (int t = 0; t < 3; ++t) {
                g[t] = lin[t]->desc(input, dst[t], batch);
                g[t].bias = bias[t];
                g[t].epi_seq = 1; g[t].epi_d = d; g[t].epi_heads_total = h;
                g[t].ldc = (t == 0) ? 1 : Lmax;
            }
            const GemmDesc gq = g[0], gk = g[1], gv = g[2];
            FuncWrapVec.push_back(FuncWrap(1.0f, COMPUTATION, [gq, gk, gv, slots, pasts](const DynamicInitParam& D) {
                GemmExGrouped3Rows(D, gq, gk, gv, slots.data(), pasts.data());
            }, "qkv_gemm(decode)", HBM_BOUND));
        } else {
            v = linear_q_col->forward(input, b.q, batch); v[0].label = "q_gemm(decode)"; v[0].rclass = HBM_BOUND;
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
            v = linear_k_col->forward(input, b.k, batch); v[0].label = "k_gemm(decode)"; v[0].rclass = HBM_BOUND;
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
            v = linear_v_col->forward(input, b.v, batch); v[0].label = "v_gemm(decode)"; v[0].rclass = HBM_BOUND;
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
            T *qbias = q_bias, *kbias = k_bias, *vbias = v_bias;
            FuncWrapVec.push_back(FuncWrap(0.05f, COMPUTATION, [=](const DynamicInitParam& D) {
                note_status(lg_kv_append_varlen_f16(b.q_buf, kc, vc, b.q, qbias, b.k, kbias, b.v, vbias, batch, h, d, slots.data(), pasts.data(),
                                                    Lmax, D.stream), "lg_kv_append_varlen_f16");
            }, "kv_append"));
            FuncWrapVec.back().minor = true;
        }
        FuncWrapVec.push_back(FuncWrap(0.15f, COMPUTATION, [=](const DynamicInitParam& D) {
            note_status(lg_attn_decode_varlen_f16(b.q_buf, kc, vc, b.attn_out, dws, batch, h, d, slots.data(), lens.data(), Lmax, sc, D.stream),
                        "lg_attn_decode_varlen_f16");
        }, "attn_decode"));
        v = linear_w_row->forward(b.attn_out, output, batch); v[0].label = "out_proj(decode)"; v[0].rclass = HBM_BOUND;
        FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
        return FuncWrapVec;
    }
};

// ---------------------------------------------------------------------------------------------------
// Encoder layer and model  (bert.h:18-118)
// ---------------------------------------------------------------------------------------------------
template <typename T>
class Bert_Encoder {
    int k, n;
    StaticInitParam SParam;
    BertInitParam BertParam;
    T* workspace;
    std::vector<FuncWrap> FuncWrapVec;

  public:
    Bert_MHA<T>* MHA;
    Bert_MLP<T>* MLP;
    LayerNorm<T>* ln_mha;
    LayerNorm<T>* ln_mlp;

    Bert_Encoder(const BertInitParam& BertParams, const StaticInitParam& SParam_, const int& k_, const int& n_, T* workspace_)
        : k(k_), n(n_), SParam(SParam_), BertParam(BertParams), workspace(workspace_) {
        MHA = new Bert_MHA<T>(BertParams, SParam, k, n, workspace);
        MLP = new Bert_MLP<T>(BertParams, SParam, k, n, workspace);
        ln_mha = new LayerNorm<T>(SParam, k);
        ln_mlp = new LayerNorm<T>(SParam, k);
    }
    Bert_Encoder(const Bert_Encoder&) = delete;
    Bert_Encoder& operator=(const Bert_Encoder&) = delete;
    ~Bert_Encoder() { delete MHA; delete MLP; delete ln_mha; delete ln_mlp; }
    void init_weights(uint64_t seed, uint64_t base) {
        MHA->init_weights(seed, base + 0);
        MLP->init_weights(seed, base + 8);
        ln_mha->init_weights(seed, base + 12);
        ln_mlp->init_weights(seed, base + 14);
    }
    void params(const std::string& prefix, std::vector<ParamRef>& out) {
        MHA->params(prefix, out);
        out.push_back({prefix + "ln1_g", ln_mha->gamma, k, 1, k, 0});
        out.push_back({prefix + "ln1_b", ln_mha->beta, k, 1, k, 0});
        MLP->params(prefix, out);
        out.push_back({prefix + "ln2_g", ln_mlp->gamma, k, 1, k, 0});
        out.push_back({prefix + "ln2_b", ln_mlp->beta, k, 1, k, 0});
    }
    static int64_t workspace_elems(const BertInitParam& P, const StaticInitParam& S, int batch, int seq) {
        const int hidden = P.head_num * P.size_per_head;
        const int64_t M = (int64_t)batch * seq;
        return Bert_MHA<T>::workspace_elems(P, S, batch, seq) + align_up(M * Bert_MLP<T>::inner_per_token(P, S, hidden)) +
               4 * align_up(M * hidden);
    }

    // bert.h:59-79: MHA -> LN -> MLP -> LN (POST_NORESID).  PRE_LN_RESID chains layer_norm -> MHA ->
    // add_bias_input_layernorm_2 -> MLP -> add_bias_input.
    // slots / pasts (both or neither): a decode step over sequences in arbitrary cache slots at different positions
    // prefill_past > 0: the seq_len tokens continue sequences with that many positions in the KV cache (see Bert_MHA::forward)
    std::vector<FuncWrap> forward(T* input, T* output, int batch_size, int seq_len, T* ws = nullptr, int cache_slot = -1,
                                  int decode_past = -1, const std::vector<int>* slots = nullptr, const std::vector<int>* pasts = nullptr,
                                  int prefill_past = 0) {
        FuncWrapVec.clear();
        if (!ws) ws = workspace;
        const bool decode = decode_past >= 0 || slots;
        const int seq = decode ? 1 : seq_len;
        const int M = batch_size * seq;
        T* attn_ws = ws;
        T* mlp_inner = attn_ws + Bert_MHA<T>::workspace_elems(BertParam, SParam, batch_size, seq);
        T* mha_out = mlp_inner + align_up((int64_t)M * Bert_MLP<T>::inner_per_token(BertParam, SParam, k));
        T* ln_mha_out = mha_out + align_up((int64_t)M * n);
        T* mlp_out = ln_mha_out + align_up((int64_t)M * n);
        T* pre_ln_out = mlp_out + align_up((int64_t)M * n);
        auto append = [&](std::vector<FuncWrap> v) { FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end()); };
        auto mha = [&](T* in, T* out) {
            if (slots) return MHA->forward_decode_seqs(in, out, *slots, *pasts, attn_ws);
            return decode ? MHA->forward_decode(in, out, batch_size, decode_past, cache_slot, attn_ws)
                          : MHA->forward(in, out, batch_size, seq_len, attn_ws, cache_slot, prefill_past);
        };
        auto mlp = [&](T* in, T* out) {
            std::vector<FuncWrap> v = MLP->forward(in, out, M, mlp_inner);
            if (decode) for (auto& f : v) f.rclass = HBM_BOUND;
            return v;
        };
        if (BertParam.norm_mode == POST_NORESID) {
            append(mha(input, mha_out));
            append(ln_mha->forward(mha_out, ln_mha_out, M));
            append(mlp(ln_mha_out, mlp_out));
            append(ln_mlp->forward(mlp_out, output, M));
        } else {
            append(ln_mha->forward(input, pre_ln_out, M));
            append(mha(pre_ln_out, mha_out));
            T *g = ln_mlp->gamma, *bt = ln_mlp->beta, *wb = MHA->w_bias;
            const int nn = n;
            FuncWrapVec.push_back(FuncWrap(0.1f, COMPUTATION, [=](const DynamicInitParam& D) {
                Add_bias_input_layernorm_2_kernelLauncher<T>(input, g, bt, wb, mha_out, ln_mha_out, M, nn, D);
            }, "residual+bias+layer_norm"));
            FuncWrapVec.back().minor = true;
            append(mlp(ln_mha_out, output));
            T* b2 = MLP->bias2;
            FuncWrapVec.push_back(FuncWrap(0.1f, COMPUTATION, [=](const DynamicInitParam& D) {
                Add_bias_input_kernelLauncher<T>(output, b2, mha_out, M, nn, D);
            }, "residual+bias"));
            FuncWrapVec.back().minor = true;
        }
        return FuncWrapVec;
    }
};

template <typename T>
class Bert_Model {
  public:
    int k, n;
    StaticInitParam SParam;
    BertInitParam BertParams;
    std::vector<Bert_Encoder<T>*> encoders;
    std::vector<FuncWrap> FuncWrapVec;
    T* workspace;

    Bert_Model(const BertInitParam& BertParams_, const StaticInitParam& SParam_, const int& k_, const int& n_, T* workspace_)
        : k(k_), n(n_), SParam(SParam_), BertParams(BertParams_), workspace(workspace_) {
        for (int i = 0; i < BertParams.layer_num; i++) encoders.push_back(new Bert_Encoder<T>(BertParams, SParam, k, n, workspace));
        // the layers share their workspaces, so they share what is known about the mask slices in them
        for (auto* e : encoders) e->MHA->mask_state = encoders[0]->MHA->mask_state;
    }
    Bert_Model(const Bert_Model&) = delete;
    Bert_Model& operator=(const Bert_Model&) = delete;
    ~Bert_Model() { for (auto* e : encoders) delete e; }   // the workspace belongs to the caller
    void init_weights(uint64_t seed) {
        for (size_t i = 0; i < encoders.size(); ++i) encoders[i]->init_weights(seed, 1000 * (i + 1));
        note_status(lg_device_synchronize(), "lg_device_synchronize");
    }
    std::vector<ParamRef> params() {
        std::vector<ParamRef> out;
        for (size_t i = 0; i < encoders.size(); ++i) encoders[i]->params("layer" + std::to_string(i) + ".", out);
        return out;
    }
    int64_t workspace_elems(int batch, int seq) const { return Bert_Encoder<T>::workspace_elems(BertParams, SParam, batch, seq); }
    // entries per layer of the vector forward() returns for this configuration
    int kernels_per_layer(bool decode = false) const {
        const bool fused = BertParams.fused && dtype_of<T>::value == LG_F16;
        int mha = decode ? (BertParams.fused ? 3 : 6) : (fused ? (BertParams.packed_qkv ? 3 : 5) : (BertParams.packed_qkv ? 7 : 9));
        const int hidden = BertParams.head_num * BertParams.size_per_head;
        int mlp = (fused && (BertParams.ffn_act != FFN_GEGLU || Bert_MLP<T>::geglu_fused(BertParams, SParam, hidden))) ? 2 : 3;
        return mha + mlp + 2 + (BertParams.norm_mode == PRE_LN_RESID ? 1 : 0);
    }

    // bert.h:104-115: layer 0 input -> output, later layers output -> output (in place through the workspace)
    std::vector<FuncWrap> forward(T* input, T* output, int batch_size, int seq_len, T* ws = nullptr, int cache_slot = -1) {
        FuncWrapVec.clear();
        if (!ws) ws = workspace;
        for (int i = 0; i < BertParams.layer_num; i++) {
            std::vector<FuncWrap> v = encoders[i]->forward(i == 0 ? input : output, output, batch_size, seq_len, ws, cache_slot);
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
        }
        return FuncWrapVec;
    }
    // A prefill that continues sequences whose first `past` positions are already in the KV cache of `cache_slot` (a long prompt
    // taken in chunks, each chunk through all layers): input / output are the chunk's own rows [batch, seq_len, hidden].
    std::vector<FuncWrap> forward_prefill_past(T* input, T* output, int batch_size, int seq_len, int past, T* ws, int cache_slot) {
        FuncWrapVec.clear();
        if (!ws) ws = workspace;
        for (int i = 0; i < BertParams.layer_num; i++) {
            std::vector<FuncWrap> v = encoders[i]->forward(i == 0 ? input : output, output, batch_size, seq_len, ws, cache_slot, -1, nullptr, nullptr, past);
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
        }
        return FuncWrapVec;
    }
    // one decode step through all layers for sequences in arbitrary cache slots at different positions
    std::vector<FuncWrap> forward_decode_seqs(T* input, T* output, const std::vector<int>& slots, const std::vector<int>& pasts, T* ws = nullptr) {
        FuncWrapVec.clear();
        if (!ws) ws = workspace;
        if (slots.empty() || slots.size() != pasts.size()) return FuncWrapVec;
        for (int i = 0; i < BertParams.layer_num; i++) {
            std::vector<FuncWrap> v = encoders[i]->forward(i == 0 ? input : output, output, (int)slots.size(), 1, ws, -1, -1, &slots, &pasts);
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
        }
        return FuncWrapVec;
    }
    // one decode step through all layers (KV caches must have been filled by a fused prefill with the same slot)
    std::vector<FuncWrap> forward_decode(T* input, T* output, int batch_size, int past, int cache_slot, T* ws = nullptr) {
        FuncWrapVec.clear();
        if (!ws) ws = workspace;
        for (int i = 0; i < BertParams.layer_num; i++) {
            std::vector<FuncWrap> v = encoders[i]->forward(i == 0 ? input : output, output, batch_size, 1, ws, cache_slot, past);
            FuncWrapVec.insert(FuncWrapVec.end(), v.begin(), v.end());
        }
        return FuncWrapVec;
    }
};

}  // namespace liger
