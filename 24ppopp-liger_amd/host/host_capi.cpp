// host_capi.cpp -- C API over the C++ launch-vector runtime, for drivers that are not C++ (tests, bench).
//
// A model handle owns a Bert_Model<T> (T = float or liger::half), its default workspace and two stream contexts.
// Nothing here computes: vectors are built by the layer classes and launched entry by entry through FuncWrap.
#include <cstdlib>
#include <cstring>
#include <memory>
#include <string>

#include "layers.h"
#include "scheduler.h"

using namespace liger;

namespace {

struct SchedBase {
    virtual ~SchedBase() {}
    virtual void configure(int deep, float contention, int policy, int axis, int seq_bucket, int ignore_num) = 0;
    virtual void make_pool(int count, int ctx_batch) = 0;
    virtual void profile(int bs, int seq_lo, int seq_hi, int seq_step, int itr) = 0;
    virtual void profile_decode(int bs, int past, int itr) = 0;
    virtual bool save(const char* main_file, const char* sub_file) = 0;
    virtual bool load(const char* main_file, const char* sub_file) = 0;
    virtual Report run(int mode, const std::vector<TraceRequest>& trace, int* counters) = 0;
    virtual float lookup(int name, int bs, int seq) = 0;
    virtual int sub_lookup(int name, int bs, int seq, float* out, int cap) = 0;
    virtual void set_profile(int name, int bs, int seq, float ms, const float* sub, int nsub) = 0;
    virtual bool serve(int bs, int seq, int n_decode) = 0;
    virtual bool serve_decode(int bs, int past, int n_steps) = 0;
    virtual bool enable_partition(int hbm_cus) = 0;
    virtual bool profile_partition(int bs, int seq, int dec_bs, int past, float* out7) = 0;
    virtual bool set_partition_factor(int main_class, int sub_class, float v) = 0;
    virtual float get_partition_factor(int main_class, int sub_class) = 0;
    virtual void extra_counters(int* out2) = 0;
    virtual bool enable_batch_decode(bool on, int steps_ahead) = 0;
    virtual void batch_counters(int* out2) = 0;
    virtual void set_recycle(bool on) = 0;
    virtual bool ctx_decode_ptrs(int i, void** a, void** b) = 0;
    virtual void set_factor(int factor) = 0;
    virtual bool ctx_ptrs(int i, void** in, void** out) = 0;
    virtual Report run_queued(int mode, int* counters) = 0;
    virtual bool profile_contention(int bs, int seq, int dec_bs, int past, float* out5) = 0;
    virtual bool set_contention(int main_class, int sub_class, float v) = 0;
    virtual float get_contention(int main_class, int sub_class) = 0;
    virtual bool streams_concurrent() = 0;
    virtual int partition_streams_concurrent() = 0;
    virtual void set_verify_partition_streams(bool on) = 0;
    virtual void set_merge_minor(bool on) = 0;
    virtual void set_prefill_chunk(int rows) = 0;
    virtual void chunk_counters(int* out2) = 0;
    virtual void set_partition_feedback(bool on, int min_samples, int probe, float margin) = 0;
    virtual void feedback_state(double* out5) = 0;
    virtual void set_decode_step_hook(void (*fn)(void*, int, int, const int*, const int*, void*, void*), void* user) = 0;
};

struct ModelBase {
    virtual SchedBase* make_scheduler() = 0;
    virtual ~ModelBase() {
        if (stream0) { stream0->destroy(); delete stream0; }
        dev_free(default_ws); dev_free(io_in); dev_free(io_out);
    }
    virtual std::vector<FuncWrap> build(void* in, void* out, int batch, int seq, void* ws, int slot) = 0;
    virtual std::vector<FuncWrap> build_decode(void* in, void* out, int batch, int past, int slot, void* ws) = 0;
    virtual std::vector<FuncWrap> build_prefill_past(void* in, void* out, int batch, int seq, int past, void* ws, int slot) = 0;
    virtual std::vector<FuncWrap> build_decode_seqs(void* in, void* out, const std::vector<int>& slots, const std::vector<int>& pasts, void* ws) = 0;
    virtual int64_t workspace_elems(int batch, int seq) = 0;
    virtual int kernels_per_layer(bool decode) = 0;
    virtual std::vector<ParamRef> params() = 0;
    virtual size_t elem_size() = 0;
    virtual bool kv_cache(int layer, void** k, void** v) = 0;
    BertInitParam P;
    StaticInitParam S;
    void* default_ws = nullptr;
    int64_t default_ws_elems = 0;
    DynamicInitParam* stream0 = nullptr;
    void *io_in = nullptr, *io_out = nullptr;  // default request buffers [max_batch * max_seq, hidden]
};

template <typename T>
struct SchedT : SchedBase {
    std::unique_ptr<Scheduler<T, Bert_Model<T>>> s;
    void configure(int deep, float contention, int policy, int axis, int seq_bucket, int ignore_num) override {
        s->schedule_deep = deep; s->contention_factor = contention; s->policy = (class_policy)policy;
        s->axis = (split_axis)axis; s->seq_bucket = seq_bucket; s->ignore_num = ignore_num;
    }
    void make_pool(int count, int ctx_batch) override { s->make_pool(count, ctx_batch); }
    void profile(int bs, int seq_lo, int seq_hi, int seq_step, int itr) override {
        s->profile(bs, bs + 1, seq_lo, seq_hi + 1, "", "", seq_step, itr);
    }
    void profile_decode(int bs, int past, int itr) override { s->profile_decode(bs, past, itr); }
    // The measured contention table travels in the main profile file inside the reference's record schema (utils.h:106-127):
    // {"kernel_name": -1, "batch_size": primary class, "seq_len": secondary class, "duration": fraction}.
    bool save(const char* a, const char* b) override {
        auto dict = s->profiling_res_dict;
        for (int m = 0; m < 3; ++m)
            for (int c = 0; c < 3; ++c)
                if (s->contention_table[m][c] >= 0.f) dict[{-1, m, c}] = s->contention_table[m][c];
        return MainDictToFile(dict, a) && SubDictToFile(s->profiling_decompse_res_dict, b);
    }
    bool load(const char* a, const char* b) override {
        if (!MainFileToDict(a, s->profiling_res_dict) || !SubFileToDict(b, s->profiling_decompse_res_dict)) return false;
        for (auto it = s->profiling_res_dict.begin(); it != s->profiling_res_dict.end();) {
            if (it->first.kernel_name == -1) {
                const int m = it->first.batch_size, c = it->first.seq_len;
                if (m >= 0 && m < 3 && c >= 0 && c < 3) s->contention_table[m][c] = it->second;
                it = s->profiling_res_dict.erase(it);
            } else {
                ++it;
            }
        }
        return true;
    }
    Report run(int mode, const std::vector<TraceRequest>& trace, int* counters) override {
        s->reset_run();
        s->serving(trace);
        if (mode == 0) s->run_sequential(); else s->run_stream_sync();
        Report r = s->output_recording(getenv("LGH_PRINT_RECORDS") != nullptr);  // per-request lines as schedule.h:325-348 prints them
        if (counters) { counters[0] = s->rounds; counters[1] = s->secondary_launches; counters[2] = s->splits; counters[3] = s->profile_misses; }
        return r;
    }
    float lookup(int name, int bs, int seq) override { return s->lookup(name, bs, seq); }
    void set_profile(int name, int bs, int seq, float ms, const float* sub, int nsub) override {
        s->profiling_res_dict[{name, bs, seq}] = ms;
        if (sub && nsub > 0) s->profiling_decompse_res_dict[{name, bs, seq}] = std::vector<float>(sub, sub + nsub);
    }
    bool serve(int bs, int seq, int n_decode) override { return s->serve(bs, seq, n_decode); }
    bool serve_decode(int bs, int past, int n_steps) override { return s->serve_decode(bs, past, n_steps); }
    bool enable_partition(int hbm_cus) override {
        if (hbm_cus == 0) { s->disable_partition(); return true; }
        return s->enable_partition(hbm_cus, lg_stream_cu_count(s->DParams0.stream));
    }
    bool profile_partition(int bs, int seq, int dec_bs, int past, float* out7) override {
        auto r = s->profile_partition(bs, seq, dec_bs, past);
        if (r.factor < 0.f) return false;
        out7[0] = r.main_ms; out7[1] = r.sub_ms; out7[2] = r.main_part_ms; out7[3] = r.sub_part_ms; out7[4] = r.factor; out7[5] = r.gain;
        out7[6] = (float)r.sub_repeats;
        return true;
    }
    bool set_partition_factor(int main_class, int sub_class, float v) override {
        if (main_class < 0 || main_class > 2 || sub_class < 0 || sub_class > 2) return false;
        s->partition_table[main_class][sub_class] = v;
        return true;
    }
    float get_partition_factor(int main_class, int sub_class) override {
        return (main_class < 0 || main_class > 2 || sub_class < 0 || sub_class > 2) ? -1.f : s->partition_table[main_class][sub_class];
    }
    void extra_counters(int* out2) override { out2[0] = s->partition_rounds; out2[1] = s->sub_profile_misses; }
    bool enable_batch_decode(bool on, int steps_ahead) override {
        if (steps_ahead > 0) s->decode_steps_ahead = steps_ahead;
        return s->enable_batch_decode(on);
    }
    void batch_counters(int* out2) override { out2[0] = s->batched_steps; out2[1] = s->batched_rows; }
    void set_recycle(bool on) override { s->recycle_contexts = on; }
    bool ctx_decode_ptrs(int i, void** a, void** b) override {
        auto* c = s->context(i);
        if (!c) return false;
        *a = c->dec_a; *b = c->dec_b;
        return true;
    }
    void set_factor(int factor) override { s->BertParams.factor = factor; }
    bool ctx_ptrs(int i, void** in, void** out) override {
        auto* c = s->context(i);
        if (!c) return false;
        *in = c->input; *out = c->output;
        return true;
    }
    Report run_queued(int mode, int* counters) override {
        s->reset_run();
        s->run_stop();  // everything is already queued: the loop ends once it has drained
        if (mode == 0) s->run_sequential(); else s->run_stream_sync();
        Report r = s->output_recording(false);
        if (counters) { counters[0] = s->rounds; counters[1] = s->secondary_launches; counters[2] = s->splits; counters[3] = s->profile_misses; }
        return r;
    }
    bool profile_contention(int bs, int seq, int dec_bs, int past, float* out5) override {
        auto r = s->profile_contention(bs, seq, dec_bs, past);
        if (r.hidden < 0.f) return false;
        out5[0] = r.main_ms; out5[1] = r.sub_ms; out5[2] = r.both_ms; out5[3] = r.hidden; out5[4] = (float)r.sub_repeats;
        return true;
    }
    bool set_contention(int main_class, int sub_class, float v) override {
        if (main_class < 0 || main_class > 2 || sub_class < 0 || sub_class > 2) return false;
        s->contention_table[main_class][sub_class] = v;
        return true;
    }
    float get_contention(int main_class, int sub_class) override { return s->contention(main_class, sub_class); }
    int sub_lookup(int name, int bs, int seq, float* out, int cap) override {
        auto it = s->profiling_decompse_res_dict.find({name, bs, seq});
        if (it == s->profiling_decompse_res_dict.end()) return -1;
        int n = (int)it->second.size();
        for (int i = 0; i < n && i < cap; ++i) out[i] = it->second[i];
        return n;
    }
    bool streams_concurrent() override { return s->DParams1.concurrent; }
    int partition_streams_concurrent() override { return s->partition_hbm_cus > 0 ? s->partition_streams_concurrent : -1; }
    void set_verify_partition_streams(bool on) override { s->verify_partition_streams = on; }
    void set_merge_minor(bool on) override { s->merge_minor = on; }
    void set_prefill_chunk(int rows) override { s->prefill_chunk = rows; }
    void chunk_counters(int* out2) override { out2[0] = s->chunked_prefills; out2[1] = s->yield_turns; }
    void set_partition_feedback(bool on, int min_samples, int probe, float margin) override {
        s->partition_feedback = on;
        if (min_samples > 0) s->partition_feedback_min = min_samples;
        if (probe >= 0) s->partition_feedback_probe = probe;
        if (margin > 0.f) s->partition_feedback_margin = margin;
    }
    void feedback_state(double* out5) override {
        out5[0] = s->feedback_rate(1); out5[1] = s->feedback_rate(2); out5[2] = s->feedback_samples(1); out5[3] = s->feedback_samples(2);
        out5[4] = s->partition_declined;
    }
    void set_decode_step_hook(void (*fn)(void*, int, int, const int*, const int*, void*, void*), void* user) override {
        if (!fn) { s->decode_step_hook = nullptr; return; }
        s->decode_step_hook = [fn, user](int step, const std::vector<int>& slots, const std::vector<int>& pasts, T* rows, const DynamicInitParam& D) {
            fn(user, step, (int)slots.size(), slots.data(), pasts.data(), (void*)rows, D.stream);
        };
    }
};

template <typename T>
struct ModelT : ModelBase {
    std::unique_ptr<Bert_Model<T>> m;
    SchedBase* make_scheduler() override {
        auto* st = new SchedT<T>();
        BertInitParam P2 = P;
        st->s.reset(new Scheduler<T, Bert_Model<T>>(m.get(), P2, S, (T*)io_in, (T*)io_out));
        return st;
    }
    std::vector<FuncWrap> build(void* in, void* out, int batch, int seq, void* ws, int slot) override {
        return m->forward((T*)in, (T*)out, batch, seq, (T*)(ws ? ws : default_ws), slot);
    }
    std::vector<FuncWrap> build_decode(void* in, void* out, int batch, int past, int slot, void* ws) override {
        return m->forward_decode((T*)in, (T*)out, batch, past, slot, (T*)(ws ? ws : default_ws));
    }
    std::vector<FuncWrap> build_prefill_past(void* in, void* out, int batch, int seq, int past, void* ws, int slot) override {
        return m->forward_prefill_past((T*)in, (T*)out, batch, seq, past, (T*)(ws ? ws : default_ws), slot);
    }
    std::vector<FuncWrap> build_decode_seqs(void* in, void* out, const std::vector<int>& slots, const std::vector<int>& pasts, void* ws) override {
        return m->forward_decode_seqs((T*)in, (T*)out, slots, pasts, (T*)(ws ? ws : default_ws));
    }
    int64_t workspace_elems(int batch, int seq) override { return m->workspace_elems(batch, seq); }
    int kernels_per_layer(bool decode) override { return m->kernels_per_layer(decode); }
    std::vector<ParamRef> params() override { return m->params(); }
    size_t elem_size() override { return sizeof(T); }
    bool kv_cache(int layer, void** k, void** v) override {
        if (layer < 0 || layer >= (int)m->encoders.size() || !m->encoders[layer]->MHA->k_cache) return false;
        *k = m->encoders[layer]->MHA->k_cache;
        *v = m->encoders[layer]->MHA->v_cache;
        return true;
    }
};

int fail(const char* msg) {
    set_error_state(LG_ERR_INVALID, msg);
    return LG_ERR_INVALID;
}

bool shape_ok(ModelBase* mb, int batch, int seq) {
    return mb && batch > 0 && seq > 0 && batch <= mb->P.max_batch_size && seq <= mb->P.max_seq_len;
}

// what a prefill (decode_past < 0) or decode-step launch vector may touch: the model's default buffers are sized for
// (max_batch, max_seq), the KV cache for max_batch slots of max_cache_len rows
bool launch_shape_ok(ModelBase* mb, int batch, int seq, int decode_past, int cache_slot) {
    if (!mb || batch <= 0 || batch > mb->P.max_batch_size) return false;
    if (decode_past >= 0)
        return mb->P.max_cache_len > 0 && decode_past < mb->P.max_cache_len && cache_slot >= 0 && cache_slot + batch <= mb->P.max_batch_size;
    if (seq <= 0 || seq > mb->P.max_seq_len) return false;
    return cache_slot < 0 || (mb->P.max_cache_len > 0 && seq <= mb->P.max_cache_len && cache_slot + batch <= mb->P.max_batch_size);
}

}  // namespace

extern "C" {

int lgh_first_error(char* buf, int len) {
    if (buf && len > 0) {
        strncpy(buf, error_text().c_str(), (size_t)len - 1);
        buf[len - 1] = 0;
    }
    return first_error();
}
void lgh_clear_error(void) { clear_error(); }

// dtype 0 = fp32, 1 = fp16.  head_num and ffn_inner are GLOBAL sizes; the model holds the 1/world_size shard.
void* lgh_model_create_ex(int dtype, int max_batch, int max_seq, int head_num, int size_per_head, int layer_num, int world_size,
                          int ffn_inner, int norm_mode, int causal, int fused, int max_cache_len, int factor, int weight_layout,
                          int ffn_act, int packed_qkv, uint64_t seed);
void* lgh_model_create(int dtype, int max_batch, int max_seq, int head_num, int size_per_head, int layer_num, int world_size,
                       int ffn_inner, int norm_mode, int causal, int fused, int max_cache_len, int factor, int weight_layout,
                       uint64_t seed) {
    return lgh_model_create_ex(dtype, max_batch, max_seq, head_num, size_per_head, layer_num, world_size, ffn_inner, norm_mode, causal,
                               fused, max_cache_len, factor, weight_layout, 0, 0, seed);
}
// ffn_act: 0 GELU, 1 GeGLU (FFN-1 is [H, 2F] = [gate | up]); packed_qkv: 1 = one [H, 3 Hl] projection, columns [q | k | v] (the
// reference-shaped assembly follows it with the fused bias/transpose kernel, the fused assembly routes the columns in the GEMM's
// epilogue; decode steps read the same packed parameters)
void* lgh_model_create_ex(int dtype, int max_batch, int max_seq, int head_num, int size_per_head, int layer_num, int world_size,
                          int ffn_inner, int norm_mode, int causal, int fused, int max_cache_len, int factor, int weight_layout,
                          int ffn_act, int packed_qkv, uint64_t seed) {
    if (max_batch <= 0 || max_seq <= 0 || head_num <= 0 || size_per_head <= 0 || layer_num <= 0 || world_size <= 0 ||
        head_num % world_size != 0 || (ffn_inner > 0 && ffn_inner % world_size != 0) || (dtype != 0 && dtype != 1)) {
        fail("lgh_model_create: bad configuration");
        return nullptr;
    }
    if (fused && dtype != 1) { fail("lgh_model_create: the fused assembly is fp16 only"); return nullptr; }
    if (max_cache_len > 0 && !fused) { fail("lgh_model_create: the KV cache needs the fused assembly"); return nullptr; }
    if ((ffn_act != 0 && ffn_act != 1) || (packed_qkv != 0 && packed_qkv != 1)) { fail("lgh_model_create: bad ffn_act / packed_qkv"); return nullptr; }
    BertInitParam P(max_batch, max_seq, head_num, size_per_head, layer_num, 0, factor, 0);
    P.ffn_act = ffn_act; P.packed_qkv = packed_qkv;
    P.ffn_inner = ffn_inner; P.norm_mode = norm_mode; P.causal = causal; P.fused = fused; P.max_cache_len = max_cache_len;
    if (weight_layout < 0 || weight_layout > 2 || (weight_layout == 2 && dtype != 1)) { fail("lgh_model_create: weight_layout is 0 ([in, out]), 1 ([out, in]) or 2 (tiled, fp16 only)"); return nullptr; }
    P.weight_layout = weight_layout;
    StaticInitParam S(0, world_size, dtype);
    const int hidden = head_num * size_per_head;
    ModelBase* mb = nullptr;
    if (dtype == 1) {
        auto* m = new ModelT<half>();
        m->P = P; m->S = S;
        m->default_ws_elems = Bert_Encoder<half>::workspace_elems(P, S, max_batch, max_seq);
        m->default_ws = dev_alloc<half>(m->default_ws_elems);
        m->m.reset(new Bert_Model<half>(P, S, hidden, hidden, (half*)m->default_ws));
        m->m->init_weights(seed);
        mb = m;
    } else {
        auto* m = new ModelT<float>();
        m->P = P; m->S = S;
        m->default_ws_elems = Bert_Encoder<float>::workspace_elems(P, S, max_batch, max_seq);
        m->default_ws = dev_alloc<float>(m->default_ws_elems);
        m->m.reset(new Bert_Model<float>(P, S, hidden, hidden, (float*)m->default_ws));
        m->m->init_weights(seed);
        mb = m;
    }
    mb->P.kernel_num = mb->kernels_per_layer(false);
    mb->stream0 = new DynamicInitParam();
    {
        const size_t io_bytes = (size_t)max_batch * max_seq * hidden * mb->elem_size();
        mb->io_in = dev_alloc<char>(io_bytes);
        mb->io_out = dev_alloc<char>(io_bytes);
        if (dtype == 1) dev_fill_normal((half*)mb->io_in, (int64_t)(io_bytes / 2), seed, 7, 0.f, 1.f);
        else dev_fill_normal((float*)mb->io_in, (int64_t)(io_bytes / 4), seed, 7, 0.f, 1.f);
        note_status(lg_device_synchronize(), "lg_device_synchronize");
    }
    if (first_error()) return nullptr;
    return mb;
}

// Frees a model: its parameters, KV caches, default workspace and buffers, and its stream.  Schedulers built on the model must be
// destroyed first.
int lgh_model_destroy(void* model) {
    ModelBase* mb = (ModelBase*)model;
    if (!mb) return LG_OK;
    lg_device_synchronize();
    delete mb;
    return LG_OK;
}

int lgh_model_kernels_per_layer(void* model, int decode) { return model ? ((ModelBase*)model)->kernels_per_layer(decode != 0) : -1; }
int64_t lgh_model_workspace_elems(void* model, int batch, int seq) { return model ? ((ModelBase*)model)->workspace_elems(batch, seq) : -1; }
void* lgh_model_stream(void* model) { return model ? ((ModelBase*)model)->stream0->stream : nullptr; }

int lgh_model_param_count(void* model) { return model ? (int)((ModelBase*)model)->params().size() : -1; }
int lgh_model_param_info(void* model, int idx, char* name, int name_len, void** ptr, int64_t* elems, int* rows, int* cols,
                         int* transposed) {
    if (!model) return fail("lgh_model_param_info: null model");
    auto ps = ((ModelBase*)model)->params();
    if (idx < 0 || idx >= (int)ps.size()) return fail("lgh_model_param_info: index out of range");
    if (name && name_len > 0) { strncpy(name, ps[idx].name.c_str(), (size_t)name_len - 1); name[name_len - 1] = 0; }
    if (ptr) *ptr = ps[idx].ptr;
    if (elems) *elems = ps[idx].elems;
    if (rows) *rows = ps[idx].rows;
    if (cols) *cols = ps[idx].cols;
    if (transposed) *transposed = ps[idx].transposed;
    return LG_OK;
}

// Takes a parameter over from device memory the caller owns: `src` holds parameter `idx` as a plain row-major array, weight
// matrices either [in, out] (src_layout 0: what the reference's (N,N) cuBLAS call implies, linear.h:47-49,99-101) or [out, in]
// (src_layout 1), vectors flat.  The layer re-lays it into its own storage layout on the device (one kernel on `stream`, null =
// the model's stream; nothing is allocated, the caller synchronises): a copy when the layouts agree, a transpose between the
// two plain layouts, lg_weight_tile_f16 for a layer that stores fragment blocks.  So a model whose weights arrive [in, out]
// runs at the speed of the layout its kernels read fastest.  Parameters stored with interleaved halves (fused GeGLU FFN-1)
// are refused: their order is private to the layer and they are written through the host (upload in logical order).
int lgh_model_load_param(void* model, int idx, const void* src, int src_layout, void* stream) {
    ModelBase* mb = (ModelBase*)model;
    if (!mb || !src) return fail("lgh_model_load_param: null model or source");
    if (src_layout != 0 && src_layout != 1) return fail("lgh_model_load_param: src_layout must be 0 ([in, out]) or 1 ([out, in])");
    auto ps = mb->params();
    if (idx < 0 || idx >= (int)ps.size()) return fail("lgh_model_load_param: index out of range");
    const ParamRef& p = ps[idx];
    if (p.transposed & 2) return fail(("lgh_model_load_param: " + p.name + " is stored with interleaved halves; upload it in logical order through the host").c_str());
    if (src == p.ptr) return fail("lgh_model_load_param: the source is the parameter itself");
    void* st = stream ? stream : mb->stream0->stream;
    const size_t es = mb->elem_size();
    int rc;
    if (p.rows <= 1) {
        rc = lg_memcpy_d2d_async(p.ptr, src, (size_t)p.elems * es, st);
    } else if (p.transposed & 4) {   // fragment blocks of the [out, in] matrix (fp16 by construction)
        rc = lg_weight_tile_f16(p.ptr, src, p.cols, p.rows, src_layout, src_layout ? p.rows : p.cols, st);
    } else if ((p.transposed & 1) == src_layout) {
        rc = lg_memcpy_d2d_async(p.ptr, src, (size_t)p.elems * es, st);
    } else {
        // [a, b] -> [b, a]: the head transpose [1, a, b, 1] -> [1, b, a, 1]
        const int a = src_layout ? p.cols : p.rows, b = src_layout ? p.rows : p.cols;
        rc = es == 2 ? lg_transpose_f16(p.ptr, src, 1, b, a, 1, st) : lg_transpose_f32((float*)p.ptr, (const float*)src, 1, b, a, 1, st);
    }
    if (rc != LG_OK) { note_status(rc, "lgh_model_load_param"); return rc; }
    return LG_OK;
}

// Device pointers of layer `layer`'s KV cache [max_batch, local heads, max_cache_len, size_per_head] (K and V), for callers that
// manage cache contents themselves (loading a saved cache, tests).
int lgh_model_kv_cache(void* model, int layer, void** k_cache, void** v_cache) {
    if (!model || !k_cache || !v_cache || !((ModelBase*)model)->kv_cache(layer, k_cache, v_cache)) return fail("lgh_model_kv_cache: no such layer or no KV cache");
    return LG_OK;
}

// Writes "idx|label|type|class\n" per entry of the vector forward() (or forward_decode()) would return.
int lgh_model_describe(void* model, int batch, int seq, int decode_past, char* buf, int len) {
    ModelBase* mb = (ModelBase*)model;
    if (!shape_ok(mb, batch, decode_past >= 0 ? 1 : seq)) return fail("lgh_model_describe: bad shape");
    std::vector<FuncWrap> v = decode_past >= 0 ? mb->build_decode(mb->default_ws, mb->default_ws, batch, decode_past, 0, nullptr)
                                               : mb->build(mb->default_ws, mb->default_ws, batch, seq, nullptr, -1);
    std::string s;
    const char* tn[3] = {"COMMUNICATION", "COMPUTATION", "GEMM"};
    const char* cn[3] = {"MFMA_BOUND", "HBM_BOUND", "LINK_BOUND"};
    for (size_t i = 0; i < v.size(); ++i)
        s += std::to_string(i) + "|" + v[i].label + "|" + tn[v[i].type] + "|" + cn[v[i].rclass] + "\n";
    if (buf && len > 0) { strncpy(buf, s.c_str(), (size_t)len - 1); buf[len - 1] = 0; }
    return (int)v.size();
}

// Builds the launch vector and launches every entry in order on `stream` (NULL -> the model's own stream).
// Does not synchronise.  cache_slot >= 0 routes K/V into the KV cache (fused assembly).
int lgh_model_run(void* model, void* input, void* output, int batch, int seq, void* workspace, void* stream, int cache_slot) {
    ModelBase* mb = (ModelBase*)model;
    if (!shape_ok(mb, batch, seq) || !input || !output) return fail("lgh_model_run: bad arguments");
    if (cache_slot >= 0 && (mb->P.max_cache_len <= 0 || seq > mb->P.max_cache_len || cache_slot + batch > mb->P.max_batch_size))
        return fail("lgh_model_run: sequence or cache slot outside the KV cache");
    DynamicInitParam D(stream ? stream : mb->stream0->stream, 0);
    for (auto& f : mb->build(input, output, batch, seq, workspace, cache_slot)) f.callback(D);
    return first_error();
}

// The prefill of ONE sequence of `seq` tokens taken in chunks of `chunk` tokens (the last one shorter), every chunk through all
// layers before the next: chunk c attends to the keys and values chunks 0 .. c left in the KV cache of `cache_slot`.  input /
// output are [seq, hidden].  The result equals lgh_model_run(batch 1) up to the rounding of another summation order.
int lgh_model_run_chunked(void* model, void* input, void* output, int seq, int chunk, void* workspace, void* stream, int cache_slot) {
    ModelBase* mb = (ModelBase*)model;
    if (!shape_ok(mb, 1, seq) || !input || !output || chunk <= 0) return fail("lgh_model_run_chunked: bad arguments");
    if (!mb->P.fused || cache_slot < 0 || mb->P.max_cache_len <= 0 || seq > mb->P.max_cache_len || cache_slot >= mb->P.max_batch_size)
        return fail("lgh_model_run_chunked: needs the fused assembly and a KV-cache slot that holds the sequence");
    DynamicInitParam D(stream ? stream : mb->stream0->stream, 0);
    const size_t row_bytes = (size_t)mb->P.head_num * mb->P.size_per_head * mb->elem_size();
    for (int p0 = 0; p0 < seq; p0 += chunk) {
        const int c = std::min(chunk, seq - p0);
        for (auto& f : mb->build_prefill_past((char*)input + (size_t)p0 * row_bytes, (char*)output + (size_t)p0 * row_bytes, 1, c, p0, workspace, cache_slot))
            f.callback(D);
    }
    return first_error();
}

int lgh_model_run_decode(void* model, void* input, void* output, int batch, int past, int cache_slot, void* workspace, void* stream) {
    ModelBase* mb = (ModelBase*)model;
    if (!mb || batch <= 0 || batch > mb->P.max_batch_size || past < 0 || past >= mb->P.max_cache_len || cache_slot < 0 ||
        cache_slot + batch > mb->P.max_batch_size || !input || !output)
        return fail("lgh_model_run_decode: bad arguments");
    DynamicInitParam D(stream ? stream : mb->stream0->stream, 0);
    for (auto& f : mb->build_decode(input, output, batch, past, cache_slot, workspace)) f.callback(D);
    return first_error();
}

// One decode step for `batch` sequences that sit in cache slots slot[i] with past[i] cached positions each (decode steps of
// different requests as one launch vector); input / output are [batch, hidden].
int lgh_model_run_decode_seqs(void* model, void* input, void* output, int batch, const int* slot, const int* past, void* workspace,
                              void* stream) {
    ModelBase* mb = (ModelBase*)model;
    if (!mb || batch <= 0 || batch > mb->P.max_batch_size || batch > LG_ATTN_DECODE_MAX_SEQS || !slot || !past || !input || !output ||
        mb->P.max_cache_len <= 0)
        return fail("lgh_model_run_decode_seqs: bad arguments");
    std::vector<int> slots(slot, slot + batch), pasts(past, past + batch);
    for (int i = 0; i < batch; ++i)
        if (slots[i] < 0 || slots[i] >= mb->P.max_batch_size || pasts[i] < 0 || pasts[i] >= mb->P.max_cache_len)
            return fail("lgh_model_run_decode_seqs: a position or cache slot lies outside the KV cache");
    DynamicInitParam D(stream ? stream : mb->stream0->stream, 0);
    for (auto& f : mb->build_decode_seqs(input, output, slots, pasts, workspace)) f.callback(D);
    return first_error();
}

// Times every entry of the launch vector the way the reference's profiler does (schedule.h:93-112): 2 warm-up
// launches, then `iters` launches between two events on the launch stream, minimum over `trials`.  ms_out gets one
// value per entry; returns the number of entries.
int lgh_model_time_kernels(void* model, void* input, void* output, int batch, int seq, int decode_past, int cache_slot,
                           int iters, int trials, float* ms_out, int ms_cap) {
    ModelBase* mb = (ModelBase*)model;
    if (!mb || !input || !output || iters <= 0 || trials <= 0) { fail("lgh_model_time_kernels: bad arguments"); return -1; }
    if (!launch_shape_ok(mb, batch, seq, decode_past, cache_slot)) { fail("lgh_model_time_kernels: shape, position or cache slot outside the model's buffers"); return -1; }
    std::vector<FuncWrap> v = decode_past >= 0 ? mb->build_decode(input, output, batch, decode_past, cache_slot, nullptr)
                                               : mb->build(input, output, batch, seq, nullptr, cache_slot);
    if ((int)v.size() > ms_cap) { fail("lgh_model_time_kernels: output array too small"); return -1; }
    DynamicInitParam& D = *mb->stream0;
    void *e0 = nullptr, *e1 = nullptr;
    note_status(lg_event_create(&e0), "lg_event_create");
    note_status(lg_event_create(&e1), "lg_event_create");
    // run the whole vector once so that every entry sees valid inputs
    for (auto& f : v) f.callback(D);
    note_status(lg_stream_synchronize(D.stream), "lg_stream_synchronize");
    for (size_t i = 0; i < v.size(); ++i) ms_out[i] = profile_callback(v[i], D, e0, e1, iters, trials);
    lg_event_destroy(e0);
    lg_event_destroy(e1);
    return first_error() ? -1 : (int)v.size();
}

// Times the entries where they run: the whole launch vector is launched `reps` times with an event between every two entries,
// and ms_out[i] gets the mean distance between the events around entry i (its run time plus the gap to the entry before it).
// Unlike lgh_model_time_kernels no launch repeats the one before it, so nothing is re-read from a cache that the previous
// launch of the same kernel filled, and the values add up to the step.  Returns the number of entries.
int lgh_model_time_step(void* model, void* input, void* output, int batch, int seq, int decode_past, int cache_slot, int reps,
                        float* ms_out, int ms_cap) {
    ModelBase* mb = (ModelBase*)model;
    if (!mb || !input || !output || reps <= 0) { fail("lgh_model_time_step: bad arguments"); return -1; }
    if (!launch_shape_ok(mb, batch, seq, decode_past, cache_slot)) { fail("lgh_model_time_step: shape, position or cache slot outside the model's buffers"); return -1; }
    std::vector<FuncWrap> v = decode_past >= 0 ? mb->build_decode(input, output, batch, decode_past, cache_slot, nullptr)
                                               : mb->build(input, output, batch, seq, nullptr, cache_slot);
    if ((int)v.size() > ms_cap) { fail("lgh_model_time_step: output array too small"); return -1; }
    DynamicInitParam& D = *mb->stream0;
    std::vector<void*> ev(v.size() + 1, nullptr);
    for (auto& e : ev) note_status(lg_event_create(&e), "lg_event_create");
    std::vector<double> sum(v.size(), 0.0);
    for (int r = -2; r < reps; ++r) {   // two untimed passes first
        note_status(lg_event_record(ev[0], D.stream), "lg_event_record");
        for (size_t i = 0; i < v.size(); ++i) {
            v[i].callback(D);
            note_status(lg_event_record(ev[i + 1], D.stream), "lg_event_record");
        }
        note_status(lg_stream_synchronize(D.stream), "lg_stream_synchronize");
        for (size_t i = 0; i < v.size() && r >= 0; ++i) {
            float ms = 0.f;
            note_status(lg_event_elapsed_ms(&ms, ev[i], ev[i + 1]), "lg_event_elapsed_ms");
            sum[i] += ms;
        }
    }
    for (size_t i = 0; i < v.size(); ++i) ms_out[i] = (float)(sum[i] / reps);
    for (void* e : ev) if (e) lg_event_destroy(e);
    return first_error() ? -1 : (int)v.size();
}


// ---- scheduler ---------------------------------------------------------------------------------------------------
struct LghReport {
    int records;
    double avg_latency_ms, p99_latency_ms, avg_gpu_ms, avg_queue_ms, total_duration_ms, throughput;
    int rounds, secondary_launches, splits, profile_misses;
    double avg_e2e_ms, p99_e2e_ms;  // arrival -> completion on one clock
    int partition_rounds, sub_profile_misses;
    int batched_steps, batched_rows;
};

// policy: 0 = classic (communication vs rest), 1 = resource classes (MFMA-bound vs HBM-bound)
// axis: 0 = split output features (the reference's axis), 1 = split token rows
void* lgh_sched_create(void* model, int schedule_deep, float contention_factor, int policy, int axis, int seq_bucket,
                       int ignore_num, int pool_count, int ctx_batch) {
    ModelBase* mb = (ModelBase*)model;
    if (!mb || schedule_deep < 1 || contention_factor < 0 || pool_count < 0 || ctx_batch < 0 ||
        (int64_t)pool_count * ctx_batch > mb->P.max_batch_size) {
        fail("lgh_sched_create: bad arguments (pool_count * ctx_batch must not exceed the model's max_batch)");
        return nullptr;
    }
    SchedBase* s = mb->make_scheduler();
    s->configure(schedule_deep, contention_factor, policy, axis, seq_bucket < 1 ? 1 : seq_bucket, ignore_num);
    if (pool_count > 0) s->make_pool(pool_count, ctx_batch);
    return first_error() ? nullptr : s;
}
// Frees a scheduler: its streams (every one holds a hardware queue), events, request contexts and decode-batch buffers.
int lgh_sched_destroy(void* sched) {
    if (!sched) return LG_OK;
    delete (SchedBase*)sched;
    return first_error();
}
int lgh_sched_profile(void* sched, int bs, int seq_lo, int seq_hi, int seq_step, int itr) {
    if (!sched || bs <= 0 || seq_lo <= 0 || seq_hi < seq_lo || seq_step <= 0 || itr <= 0) return fail("lgh_sched_profile: bad arguments");
    ((SchedBase*)sched)->profile(bs, seq_lo, seq_hi, seq_step, itr);
    return first_error();
}
int lgh_sched_profile_decode(void* sched, int bs, int past, int itr) {
    if (!sched || bs <= 0 || past < 0 || itr <= 0) return fail("lgh_sched_profile_decode: bad arguments");
    ((SchedBase*)sched)->profile_decode(bs, past, itr);
    return first_error();
}
// Measures the contention table entry for prefill MFMA-bound kernels || decode-step kernels (see Scheduler::profile_contention);
// out5 = {primary ms, secondary ms, concurrent ms, hidden fraction, secondary repeats}.
int lgh_sched_profile_contention(void* sched, int bs, int seq, int dec_bs, int past, float* out5) {
    if (!sched || bs <= 0 || seq <= 0 || dec_bs <= 0 || past < 0 || !out5) return fail("lgh_sched_profile_contention: bad arguments");
    if (!((SchedBase*)sched)->profile_contention(bs, seq, dec_bs, past, out5))
        return fail("lgh_sched_profile_contention: needs a pool context and a KV cache");
    return LG_OK;
}
// Spatial partition of co-running rounds: hbm_cus compute units (a multiple of 8; 0 switches partitioning off) for the HBM-bound
// side, the rest for the MFMA-bound side (Scheduler::enable_partition).
int lgh_sched_enable_partition(void* sched, int hbm_cus) {
    if (!sched || hbm_cus < 0 || !((SchedBase*)sched)->enable_partition(hbm_cus)) return fail("lgh_sched_enable_partition: bad CU count (a multiple of 8 below the device's) or stream creation failed");
    return LG_OK;
}
// out7 = {prefill kernels alone ms, one decode step alone ms (both on the whole chip), prefill side ms and decode side ms of the
// partitioned co-run, factor, gain, decode steps co-run}; see Scheduler::profile_partition.
int lgh_sched_profile_partition(void* sched, int bs, int seq, int dec_bs, int past, float* out7) {
    if (!sched || bs <= 0 || seq <= 0 || dec_bs <= 0 || past < 0 || !out7) return fail("lgh_sched_profile_partition: bad arguments");
    if (!((SchedBase*)sched)->profile_partition(bs, seq, dec_bs, past, out7))
        return fail("lgh_sched_profile_partition: needs lgh_sched_enable_partition, a pool context, a KV cache and shapes inside them");
    return LG_OK;
}
int lgh_sched_set_partition_factor(void* sched, int main_class, int sub_class, float value) {
    if (!sched || !((SchedBase*)sched)->set_partition_factor(main_class, sub_class, value)) return fail("lgh_sched_set_partition_factor: bad arguments");
    return LG_OK;
}
float lgh_sched_get_partition_factor(void* sched, int main_class, int sub_class) {
    return sched ? ((SchedBase*)sched)->get_partition_factor(main_class, sub_class) : -1.f;
}
// Requests that are in their decode steps at the same time share one launch vector per step (Scheduler::enable_batch_decode);
// needs a pool, a KV cache and one cache slot more than the pool uses.  steps_ahead > 0 sets how many steps one vector holds
// while nothing waits to join.
int lgh_sched_enable_batch_decode(void* sched, int on, int steps_ahead) {
    if (!sched || !((SchedBase*)sched)->enable_batch_decode(on != 0, steps_ahead))
        return fail("lgh_sched_enable_batch_decode: needs per-request contexts, a KV cache and max_batch >= pool_count * ctx_batch + 1");
    return LG_OK;
}
// on = 0: a finished request's context stays out of the pool until the next run, so that a run of no more requests than
// contexts leaves every request's results in a context of its own (requests take the free context with the lowest index)
int lgh_sched_set_recycle_contexts(void* sched, int on) {
    if (!sched) return fail("lgh_sched_set_recycle_contexts: null");
    ((SchedBase*)sched)->set_recycle(on != 0);
    return LG_OK;
}
// the decode ping-pong buffers [ctx_batch, hidden] of the i-th context: after n decode steps a request's last hidden state is in
// the second one when n is odd, in the first when n is even
int lgh_sched_ctx_decode_ptrs(void* sched, int i, void** dec_a, void** dec_b) {
    if (!sched || !dec_a || !dec_b || !((SchedBase*)sched)->ctx_decode_ptrs(i, dec_a, dec_b)) return fail("lgh_sched_ctx_decode_ptrs: no such context");
    return LG_OK;
}
// main_class / sub_class: 0 = MFMA-bound, 1 = HBM-bound, 2 = link-bound; a negative value restores the constant factor
int lgh_sched_set_contention(void* sched, int main_class, int sub_class, float value) {
    if (!sched || !((SchedBase*)sched)->set_contention(main_class, sub_class, value)) return fail("lgh_sched_set_contention: bad arguments");
    return LG_OK;
}
// Resource-class policy: minor entries (LayerNorm, residual, cache append, row gather) take the scheduling class of the entry
// before them: a prefill's LayerNorms no longer cut it into runs and no longer stop it when it is interleaved.  Off by default.
int lgh_sched_set_merge_minor(void* sched, int on) {
    if (!sched) return fail("lgh_sched_set_merge_minor: null");
    ((SchedBase*)sched)->set_merge_minor(on != 0);
    return LG_OK;
}
// With batched decode steps: single-sequence prompts longer than `rows` tokens are prefilled in chunks of `rows`, and the batched
// decode step runs between two chunks (Scheduler::prefill_chunk).  0 switches it off.
int lgh_sched_set_prefill_chunk(void* sched, int rows) {
    if (!sched || rows < 0) return fail("lgh_sched_set_prefill_chunk: bad arguments");
    ((SchedBase*)sched)->set_prefill_chunk(rows);
    return LG_OK;
}
// out2 = {requests of the last run whose prefill was cut into chunks, turns given to the batched decode step between chunks}
int lgh_sched_chunk_counters(void* sched, int* out2) {
    if (!sched || !out2) return fail("lgh_sched_chunk_counters: bad arguments");
    ((SchedBase*)sched)->chunk_counters(out2);
    return LG_OK;
}
// Whether partitioned rounds are checked against whole-chip rounds while a run goes on (Scheduler::partition_feedback; on by
// default).  min_samples <= 0, probe < 0, margin <= 0 keep the current value.
int lgh_sched_set_partition_feedback(void* sched, int on, int min_samples, int probe, float margin) {
    if (!sched) return fail("lgh_sched_set_partition_feedback: null");
    ((SchedBase*)sched)->set_partition_feedback(on != 0, min_samples, probe, margin);
    return LG_OK;
}
// out5 = {progress rate of whole-chip rounds, of partitioned rounds (stand-alone ms of work per ms), samples of each, rounds that
// could have been partitioned and were not} of the last run
int lgh_sched_partition_feedback_state(void* sched, double* out5) {
    if (!sched || !out5) return fail("lgh_sched_partition_feedback_state: bad arguments");
    ((SchedBase*)sched)->feedback_state(out5);
    return LG_OK;
}
// fn(user, step, rows, slots[rows], pasts[rows], batch_rows, stream) is called on the scheduler's thread after the kernels of
// every batched decode step have been launched on `stream` (Scheduler::decode_step_hook); batch_rows is the device buffer
// [rows, hidden] the steps work on in place.  fn = NULL removes the hook.
int lgh_sched_set_decode_step_hook(void* sched, void (*fn)(void*, int, int, const int*, const int*, void*, void*), void* user) {
    if (!sched) return fail("lgh_sched_set_decode_step_hook: null");
    ((SchedBase*)sched)->set_decode_step_hook(fn, user);
    return LG_OK;
}
// 1 when the scheduler's second stream was verified to execute at the same time as the first
int lgh_sched_streams_concurrent(void* sched) { return (sched && ((SchedBase*)sched)->streams_concurrent()) ? 1 : 0; }
// 1 when both (primary, secondary) pairs of CU-masked streams of the share in use were measured to overlap, 0 when a pair could
// not be made to, -1 when they were not probed (no share in use, or verification off when the share's streams were created)
int lgh_sched_partition_streams_concurrent(void* sched) { return sched ? ((SchedBase*)sched)->partition_streams_concurrent() : -1; }
// Whether enable_partition probes the stream pairs of a share it creates (and replaces secondaries that take turns)
int lgh_sched_set_verify_partition_streams(void* sched, int on) {
    if (!sched) return fail("lgh_sched_set_verify_partition_streams: null scheduler");
    ((SchedBase*)sched)->set_verify_partition_streams(on != 0);
    return LG_OK;
}
float lgh_sched_get_contention(void* sched, int main_class, int sub_class) {
    return sched ? ((SchedBase*)sched)->get_contention(main_class, sub_class) : -1.f;
}
int lgh_sched_save(void* sched, const char* main_file, const char* sub_file) {
    return (sched && ((SchedBase*)sched)->save(main_file, sub_file)) ? LG_OK : fail("lgh_sched_save: cannot write");
}
int lgh_sched_load(void* sched, const char* main_file, const char* sub_file) {
    return (sched && ((SchedBase*)sched)->load(main_file, sub_file)) ? LG_OK : fail("lgh_sched_load: cannot read or parse");
}
float lgh_sched_lookup(void* sched, int name, int bs, int seq) { return sched ? ((SchedBase*)sched)->lookup(name, bs, seq) : -1.f; }
int lgh_sched_sub_lookup(void* sched, int name, int bs, int seq, float* out, int cap) {
    return sched ? ((SchedBase*)sched)->sub_lookup(name, bs, seq, out, cap) : -1;
}
// mode 0 = sequential baseline (run_sequential), 1 = interleaved (run_stream_sync).  Replays the trace in real time.
int lgh_sched_run_trace(void* sched, int mode, const double* arrival_s, const int* batch, const int* seq, const int* n_decode,
                        int n, LghReport* out) {
    if (!sched || n < 0 || !out) return fail("lgh_sched_run_trace: bad arguments");
    std::vector<TraceRequest> tr;
    for (int i = 0; i < n; ++i) tr.push_back({arrival_s[i], batch[i], seq[i], n_decode ? n_decode[i] : 0});
    int c[4] = {0, 0, 0, 0};
    Report r = ((SchedBase*)sched)->run(mode, tr, c);
    out->records = r.records; out->avg_latency_ms = r.avg_latency_ms; out->p99_latency_ms = r.p99_latency_ms;
    out->avg_gpu_ms = r.avg_gpu_ms; out->avg_queue_ms = r.avg_queue_ms; out->total_duration_ms = r.total_duration_ms;
    out->throughput = r.throughput; out->rounds = c[0]; out->secondary_launches = c[1]; out->splits = c[2]; out->profile_misses = c[3];
    out->avg_e2e_ms = r.avg_e2e_ms; out->p99_e2e_ms = r.p99_e2e_ms;
    { int x[2] = {0, 0}; ((SchedBase*)sched)->extra_counters(x); out->partition_rounds = x[0]; out->sub_profile_misses = x[1]; }
    { int x[2] = {0, 0}; ((SchedBase*)sched)->batch_counters(x); out->batched_steps = x[0]; out->batched_rows = x[1]; }
    return first_error();
}
// Deterministic variant for tests: requests are queued up front with lgh_sched_serve (no request thread, no real-time
// arrivals), then lgh_sched_run_queued drains them.
int lgh_sched_set_profile(void* sched, int name, int bs, int seq, float ms, const float* sub, int nsub) {
    if (!sched) return fail("lgh_sched_set_profile: null");
    ((SchedBase*)sched)->set_profile(name, bs, seq, ms, sub, nsub);
    return LG_OK;
}
int lgh_sched_serve(void* sched, int bs, int seq, int n_decode) {
    if (!sched || bs <= 0 || seq <= 0 || n_decode < 0) return fail("lgh_sched_serve: bad arguments");
    if (!((SchedBase*)sched)->serve(bs, seq, n_decode)) return fail("lgh_sched_serve: request refused");
    return first_error();
}
int lgh_sched_serve_decode(void* sched, int bs, int past, int n_steps) {
    if (!sched || bs <= 0 || past < 0 || n_steps <= 0) return fail("lgh_sched_serve_decode: bad arguments");
    if (!((SchedBase*)sched)->serve_decode(bs, past, n_steps)) return fail("lgh_sched_serve_decode: request refused");
    return first_error();
}
// decomposition factor used by profile() and by the samples queued afterwards
int lgh_sched_set_factor(void* sched, int factor) {
    if (!sched || factor < 1) return fail("lgh_sched_set_factor: bad arguments");
    ((SchedBase*)sched)->set_factor(factor);
    return LG_OK;
}
// input / output buffers of the i-th per-request context (creation order; requests take contexts in that order)
int lgh_sched_ctx_ptrs(void* sched, int i, void** input, void** output) {
    if (!sched || !input || !output || !((SchedBase*)sched)->ctx_ptrs(i, input, output)) return fail("lgh_sched_ctx_ptrs: no such context");
    return LG_OK;
}
int lgh_sched_run_queued(void* sched, int mode, LghReport* out) {
    if (!sched || !out) return fail("lgh_sched_run_queued: bad arguments");
    int c[4] = {0, 0, 0, 0};
    Report r = ((SchedBase*)sched)->run_queued(mode, c);
    out->records = r.records; out->avg_latency_ms = r.avg_latency_ms; out->p99_latency_ms = r.p99_latency_ms;
    out->avg_gpu_ms = r.avg_gpu_ms; out->avg_queue_ms = r.avg_queue_ms; out->total_duration_ms = r.total_duration_ms;
    out->throughput = r.throughput; out->rounds = c[0]; out->secondary_launches = c[1]; out->splits = c[2]; out->profile_misses = c[3];
    out->avg_e2e_ms = r.avg_e2e_ms; out->p99_e2e_ms = r.p99_e2e_ms;
    { int x[2] = {0, 0}; ((SchedBase*)sched)->extra_counters(x); out->partition_rounds = x[0]; out->sub_profile_misses = x[1]; }
    { int x[2] = {0, 0}; ((SchedBase*)sched)->batch_counters(x); out->batched_steps = x[0]; out->batched_rows = x[1]; }
    return first_error();
}
// the report arithmetic alone (known-answer tests against the reference's published logs)
int lgh_summarize(const double* cpu_ms, const double* gpu_ms, int n, double total_duration_ms, LghReport* out) {
    if (n < 0 || !out) return fail("lgh_summarize: bad arguments");
    Report r = summarize_records(std::vector<double>(cpu_ms, cpu_ms + n), std::vector<double>(gpu_ms, gpu_ms + n), total_duration_ms);
    out->records = r.records; out->avg_latency_ms = r.avg_latency_ms; out->p99_latency_ms = r.p99_latency_ms;
    out->avg_gpu_ms = r.avg_gpu_ms; out->avg_queue_ms = r.avg_queue_ms; out->total_duration_ms = r.total_duration_ms;
    out->throughput = r.throughput; out->rounds = out->secondary_launches = out->splits = out->profile_misses = 0;
    out->avg_e2e_ms = out->p99_e2e_ms = 0; out->partition_rounds = out->sub_profile_misses = 0; out->batched_steps = out->batched_rows = 0;
    return LG_OK;
}
int lgh_make_poisson_trace(double lambda, int n, int batch, int seq_lo, int seq_hi, int seq_round, int n_decode, uint64_t seed,
                           double* arrival_s, int* seq_out) {
    if (lambda <= 0 || n < 0 || seq_lo <= 0 || seq_hi < seq_lo) return fail("lgh_make_poisson_trace: bad arguments");
    auto tr = make_poisson_trace(lambda, n, batch, seq_lo, seq_hi, seq_round, n_decode, seed);
    for (int i = 0; i < n; ++i) { arrival_s[i] = tr[i].arrival_s; seq_out[i] = tr[i].seq; }
    return LG_OK;
}


// Launches entry `index` of the vector `iters` times back to back between two events on the model's stream (after one
// full pass of the vector so that its inputs are valid); returns the average milliseconds per launch, or -1.
float lgh_model_time_one(void* model, void* input, void* output, int batch, int seq, int decode_past, int cache_slot, int index,
                         int iters) {
    ModelBase* mb = (ModelBase*)model;
    if (!mb || !input || !output || iters <= 0) { fail("lgh_model_time_one: bad arguments"); return -1.f; }
    if (!launch_shape_ok(mb, batch, seq, decode_past, cache_slot)) { fail("lgh_model_time_one: shape, position or cache slot outside the model's buffers"); return -1.f; }
    std::vector<FuncWrap> v = decode_past >= 0 ? mb->build_decode(input, output, batch, decode_past, cache_slot, nullptr)
                                               : mb->build(input, output, batch, seq, nullptr, cache_slot);
    if (index < 0 || index >= (int)v.size()) { fail("lgh_model_time_one: index out of range"); return -1.f; }
    DynamicInitParam& D = *mb->stream0;
    for (auto& f : v) f.callback(D);
    note_status(lg_stream_synchronize(D.stream), "lg_stream_synchronize");
    void *e0 = nullptr, *e1 = nullptr;
    note_status(lg_event_create(&e0), "lg_event_create");
    note_status(lg_event_create(&e1), "lg_event_create");
    note_status(lg_event_record(e0, D.stream), "lg_event_record");
    for (int i = 0; i < iters; ++i) v[index].callback(D);
    note_status(lg_event_record(e1, D.stream), "lg_event_record");
    note_status(lg_event_synchronize(e1), "lg_event_synchronize");
    float ms = 0.f;
    note_status(lg_event_elapsed_ms(&ms, e0, e1), "lg_event_elapsed_ms");
    lg_event_destroy(e0);
    lg_event_destroy(e1);
    return first_error() ? -1.f : ms / (float)iters;
}

}  // extern "C"
