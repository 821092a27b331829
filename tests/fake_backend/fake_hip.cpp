// fake_hip.cpp -- a host-only stand-in for the device library, for unit tests of the launch-vector runtime.
//
// TEST INFRASTRUCTURE.  It exports every symbol of include/liger_hip.h but computes nothing: each "kernel launch"
// appends a record (stream, kernel name, problem size, pointers, virtual start/end time) to a trace and advances a
// virtual clock by a deterministic cost; streams are timelines, events are timestamps.  With it the Sample / Scheduler
// policy (src/schedule.h:221-278, src/init.h:121-259 of the reference) can be asserted launch by launch on a machine
// without a GPU.  Memory "on the device" is ordinary host memory that is never dereferenced by the fake kernels.
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "liger_hip.h"

namespace {

struct Stream {
    double ready = 0;
    int id = 0;
    int cus = 256;                  // compute units of the stream (a CU-masked stream has fewer)
    unsigned mask[8] = {~0u, ~0u, ~0u, ~0u, ~0u, ~0u, ~0u, ~0u};
};
bool share_cus(const Stream* a, const Stream* b) {
    for (int w = 0; w < 8; ++w)
        if (a->mask[w] & b->mask[w]) return true;
    return false;
}
struct Event { double time = 0; bool recorded = false; };
struct Launch {
    int stream; char name[48]; long long a, b, c;  // problem size (m, n, k) or (rows, cols, 0)
    const void* p0; const void* p1; void* p2; double start, end;
};

std::mutex g_mu;
double g_host_now = 0;          // virtual milliseconds
double g_launch_cost = 0.002;   // host time per launch call
double g_mfma_rate = 1.0e9;     // flop per virtual ms
double g_hbm_rate = 1.0e6;      // bytes per virtual ms
double g_corun_speed = 1.0;     // a kernel launched while another stream is busy runs at this fraction of its speed
double g_share_exp[2] = {1.0, 1.0};  // a kernel on a stream with `cus` of 256 compute units costs (256 / cus)^exp times more:
                                     // [0] matrix kernels, [1] memory kernels (1 = proportional, < 1 = the share hurts less)
thread_local int g_cost_kind = 1;    // kind of the cost computed last on this thread (0 matrix, 1 memory)
std::vector<Stream*> g_streams;
int g_fail_cu_mask_after = -1;  // >= 0: that many CU-masked streams are still created, the ones after them fail
int g_serial_probes = 0;        // that many of the next concurrency probes report streams that run in turn
int g_cu_mask_created = 0;     // CU-masked streams created since the last reset of this counter
int g_live_streams = 0, g_live_allocs = 0;   // created and not yet destroyed / allocated and not yet freed
std::vector<Launch> g_trace;
Stream g_default;

Stream* S(void* s) { return s ? (Stream*)s : &g_default; }

int launch(void* stream, const char* name, long long a, long long b, long long c, const void* p0, const void* p1, void* p2, double cost) {
    std::lock_guard<std::mutex> lk(g_mu);
    Stream* s = S(stream);
    g_host_now += g_launch_cost;
    Launch l;
    l.stream = s->id;
    strncpy(l.name, name, sizeof(l.name) - 1);
    l.name[sizeof(l.name) - 1] = 0;
    l.a = a; l.b = b; l.c = c; l.p0 = p0; l.p1 = p1; l.p2 = p2;
    l.start = std::max(s->ready, g_host_now);
    // a kernel on a CU-masked stream runs on its share of the chip: cost x 256 / cus; a kernel launched while another stream
    // that shares compute units with this one is busy runs at g_corun_speed of its speed
    bool other_busy = (s != &g_default && g_default.ready > l.start && share_cus(s, &g_default));
    for (auto* o : g_streams) other_busy = other_busy || (o != s && o->ready > l.start && share_cus(s, o));
    cost *= std::pow(256.0 / (double)s->cus, g_share_exp[g_cost_kind]);
    l.end = l.start + (other_busy ? cost / g_corun_speed : cost);
    s->ready = l.end;
    g_trace.push_back(l);
    return LG_OK;
}
double gemm_cost(long long m, long long n, long long k) { g_cost_kind = 0; return 0.003 + 2.0 * m * n * k / g_mfma_rate; }
double mem_cost(double bytes) { g_cost_kind = 1; return 0.003 + bytes / g_hbm_rate; }

}  // namespace

extern "C" {

// ---- test controls -------------------------------------------------------------------------------------------------
void fake_reset(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    g_trace.clear();
    g_corun_speed = 1.0;
    g_share_exp[0] = g_share_exp[1] = 1.0;
    g_host_now = 0;
    g_default.ready = 0;
    for (auto* s : g_streams) s->ready = 0;
}
void fake_set_rates(double mfma_flop_per_ms, double hbm_bytes_per_ms, double launch_cost_ms) {
    g_mfma_rate = mfma_flop_per_ms; g_hbm_rate = hbm_bytes_per_ms; g_launch_cost = launch_cost_ms;
}
void fake_set_corun_speed(double speed) { g_corun_speed = speed > 0 ? speed : 1.0; }
void fake_set_share_model(double matrix_exp, double memory_exp) { g_share_exp[0] = matrix_exp; g_share_exp[1] = memory_exp; }
int fake_trace_count(void) { std::lock_guard<std::mutex> lk(g_mu); return (int)g_trace.size(); }
int fake_trace_get(int i, int* stream, char* name, int name_len, long long* abc, unsigned long long* ptrs, double* start_end) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (i < 0 || i >= (int)g_trace.size()) return 1;
    const Launch& l = g_trace[i];
    *stream = l.stream;
    strncpy(name, l.name, (size_t)name_len - 1); name[name_len - 1] = 0;
    abc[0] = l.a; abc[1] = l.b; abc[2] = l.c;
    ptrs[0] = (unsigned long long)(uintptr_t)l.p0; ptrs[1] = (unsigned long long)(uintptr_t)l.p1; ptrs[2] = (unsigned long long)(uintptr_t)l.p2;
    start_end[0] = l.start; start_end[1] = l.end;
    return 0;
}
double fake_host_now(void) { return g_host_now; }
int fake_live_streams(void) { return g_live_streams; }
void fake_fail_cu_mask_streams_after(int n) { g_fail_cu_mask_after = n; }
void fake_serialise_probes(int n) { g_serial_probes = n; }
int fake_cu_mask_streams_created(int reset) { const int n = g_cu_mask_created; if (reset) g_cu_mask_created = 0; return n; }
int fake_live_allocs(void) { return g_live_allocs; }

// ---- library / runtime ------------------------------------------------------------------------------------------------
const char* lg_last_error(void) { return "fake backend: no error text"; }
const char* lg_version(void) { return "liger-fake 0.1 (virtual time)"; }
int lg_device_info(char* name, int name_len, int* cu, int* clk, int* mclk, int* bus, size_t* mem) {
    if (name && name_len > 0) { strncpy(name, "fake", (size_t)name_len - 1); name[name_len - 1] = 0; }
    if (cu) *cu = 256; if (clk) *clk = 2400000; if (mclk) *mclk = 2000000; if (bus) *bus = 8192; if (mem) *mem = (size_t)1 << 38;
    return LG_OK;
}
int lg_malloc(void** ptr, size_t bytes) {
    // address space only: the fake kernels never touch the memory, so reserve small real blocks and hand out
    // distinct, correctly spaced addresses from a bump counter
    static uintptr_t next = 0x100000000ull;
    std::lock_guard<std::mutex> lk(g_mu);
    *ptr = (void*)next;
    next += (bytes + 255) / 256 * 256 + 256;
    ++g_live_allocs;
    return LG_OK;
}
int lg_free(void* p) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (p) --g_live_allocs;
    return LG_OK;
}
int lg_memcpy_h2d(void*, const void*, size_t) { return LG_OK; }
int lg_memcpy_d2h(void*, const void*, size_t) { return LG_OK; }
int lg_memcpy_d2d_async(void* dst, const void* src, size_t bytes, void* stream) { return launch(stream, "memcpy_d2d", (long long)bytes, 0, 0, src, nullptr, dst, mem_cost(2.0 * bytes)); }
int lg_memset_async(void*, int, size_t, void*) { return LG_OK; }
int lg_device_synchronize(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    g_host_now = std::max(g_host_now, g_default.ready);
    for (auto* s : g_streams) g_host_now = std::max(g_host_now, s->ready);
    return LG_OK;
}
int lg_stream_create(void** stream) {
    std::lock_guard<std::mutex> lk(g_mu);
    Stream* s = new Stream();
    s->id = (int)g_streams.size() + 1;
    s->ready = g_host_now;
    g_streams.push_back(s);
    ++g_live_streams;
    *stream = s;
    return LG_OK;
}
int lg_stream_create_concurrent(void** stream, void* other, int* verified) {
    if (!stream || !other) return LG_ERR_INVALID;
    if (verified) *verified = 1;  // virtual streams always overlap
    return lg_stream_create(stream);
}
int lg_stream_create_cu_mask(void** stream, const unsigned* cu_mask, int mask_words) {
    if (!stream || !cu_mask || mask_words <= 0) return LG_ERR_INVALID;
    int cus = 0;
    for (int b = 0; b < mask_words * 32 && b < 256; ++b) cus += (cu_mask[b >> 5] >> (b & 31)) & 1u;
    if (cus == 0) return LG_ERR_INVALID;
    if (g_fail_cu_mask_after == 0) { *stream = nullptr; return LG_ERR_LAUNCH; }
    if (g_fail_cu_mask_after > 0) --g_fail_cu_mask_after;
    const int rc = lg_stream_create(stream);
    ++g_cu_mask_created;
    Stream* s = (Stream*)*stream;
    s->cus = cus;
    for (int w = 0; w < 8; ++w) s->mask[w] = w < mask_words ? cu_mask[w] : 0u;
    return rc;
}
int lg_streams_run_concurrently(void* a, void* b, int* concurrent) {
    if (!a || !b || a == b || !concurrent) return LG_ERR_INVALID;
    std::lock_guard<std::mutex> lk(g_mu);
    *concurrent = g_serial_probes > 0 ? 0 : 1;   // virtual streams overlap unless a test says otherwise
    if (g_serial_probes > 0) --g_serial_probes;
    return LG_OK;
}
int lg_stream_destroy(void* stream) {
    // the object stays (traces refer to it); only the count of streams in existence goes down
    std::lock_guard<std::mutex> lk(g_mu);
    if (stream) --g_live_streams;
    return LG_OK;
}
int lg_stream_attach(void*, int cu_count) { return cu_count < 0 ? LG_ERR_INVALID : LG_OK; }
int lg_stream_detach(void*) { return LG_OK; }
int lg_stream_cu_count(void* stream) { return stream ? S(stream)->cus : 256; }
int lg_stream_synchronize(void* stream) { std::lock_guard<std::mutex> lk(g_mu); g_host_now = std::max(g_host_now, S(stream)->ready); return LG_OK; }
int lg_stream_wait_event(void* stream, void* event) {
    std::lock_guard<std::mutex> lk(g_mu);
    Event* e = (Event*)event;
    if (e->recorded) S(stream)->ready = std::max(S(stream)->ready, e->time);
    return LG_OK;
}
int lg_event_create(void** event) { *event = new Event(); return LG_OK; }
int lg_event_destroy(void* event) { delete (Event*)event; return LG_OK; }
int lg_event_record(void* event, void* stream) {
    std::lock_guard<std::mutex> lk(g_mu);
    Event* e = (Event*)event;
    e->time = std::max(S(stream)->ready, g_host_now);
    e->recorded = true;
    return LG_OK;
}
int lg_event_synchronize(void* event) {
    std::lock_guard<std::mutex> lk(g_mu);
    Event* e = (Event*)event;
    if (e->recorded) g_host_now = std::max(g_host_now, e->time);
    return LG_OK;
}
int lg_event_query(void* event) {
    std::lock_guard<std::mutex> lk(g_mu);
    Event* e = (Event*)event;
    return (!e->recorded || e->time <= g_host_now) ? LG_OK : 3;
}
int lg_event_elapsed_ms(float* ms, void* start, void* stop) { *ms = (float)(((Event*)stop)->time - ((Event*)start)->time); return LG_OK; }

int lg_fill_normal_f32(float*, int64_t, uint64_t, uint64_t, float, float, void*) { return LG_OK; }
int lg_fill_normal_f16(void*, int64_t, uint64_t, uint64_t, float, float, void*) { return LG_OK; }
int lg_fill_const_f32(float*, int64_t, float, void*) { return LG_OK; }
int lg_fill_const_f16(void*, int64_t, float, void*) { return LG_OK; }
int lg_fill_causal_mask_f32(float*, int, int, void*) { return LG_OK; }
int lg_fill_causal_mask_f16(void*, int, int, void*) { return LG_OK; }

// ---- kernels -------------------------------------------------------------------------------------------------------------
#define EW(name, m, n, es, passes, p0, p1, p2) launch(stream, name, m, n, 0, p0, p1, p2, mem_cost((double)(passes) * (m) * (n) * (es)))
int lg_layer_norm_f32(const float* in, const float* g, const float*, float* out, int m, int n, void* stream) { return EW("layer_norm", m, n, 4, 2, in, g, out); }
int lg_layer_norm_f16(const void* in, const void* g, const void*, void* out, int m, int n, void* stream) { return EW("layer_norm", m, n, 2, 2, in, g, out); }
int lg_add_bias_act_f32(float* out, const float* b, int m, int n, void* stream) { return EW("add_bias_act", m, n, 4, 2, out, b, out); }
int lg_add_bias_act_f16(void* out, const void* b, int m, int n, void* stream) { return EW("add_bias_act", m, n, 2, 2, out, b, out); }
int lg_add_bias_geglu_f32(float* out, const float* in, const float* b, int m, int f, void* stream) { return EW("add_bias_geglu", m, f, 4, 3, in, b, out); }
int lg_add_bias_geglu_f16(void* out, const void* in, const void* b, int m, int f, void* stream) { return EW("add_bias_geglu", m, f, 2, 3, in, b, out); }
int lg_add_bias_input_layernorm_f32(float* out, const float* in, const float*, const float*, const float*, int m, int n, void* stream) { return EW("add_bias_input_layernorm", m, n, 4, 3, in, nullptr, out); }
int lg_add_bias_input_layernorm_f16(void* out, const void* in, const void*, const void*, const void*, int m, int n, void* stream) { return EW("add_bias_input_layernorm", m, n, 2, 3, in, nullptr, out); }
int lg_add_bias_input_layernorm_2_f32(const float* in, const float*, const float*, const float*, float* o, float* no, int m, int n, void* stream) { return EW("add_bias_input_layernorm_2", m, n, 4, 4, in, o, no); }
int lg_add_bias_input_layernorm_2_f16(const void* in, const void*, const void*, const void*, void* o, void* no, int m, int n, void* stream) { return EW("add_bias_input_layernorm_2", m, n, 2, 4, in, o, no); }
int lg_add_bias_input_f32(float* o, const float*, const float* in, int m, int n, void* stream) { return EW("add_bias_input", m, n, 4, 3, in, nullptr, o); }
int lg_add_bias_input_f16(void* o, const void*, const void* in, int m, int n, void* stream) { return EW("add_bias_input", m, n, 2, 3, in, nullptr, o); }
int lg_add_qkv_bias_transpose_f32(float* q, float*, float*, const float* Q, const float*, const float*, const float*, const float*, const float*, int b, int s, int h, int d, void* stream) { return EW("add_qkv_bias_transpose", (long long)b * s, (long long)h * d, 4, 6, Q, nullptr, q); }
int lg_add_qkv_bias_transpose_f16(void* q, void*, void*, const void* Q, const void*, const void*, const void*, const void*, const void*, int b, int s, int h, int d, void* stream) { return EW("add_qkv_bias_transpose", (long long)b * s, (long long)h * d, 2, 6, Q, nullptr, q); }
int lg_add_fused_qkv_bias_transpose_f32(float* q, float*, float*, const float* X, const float*, int b, int s, int h, int d, void* stream) { return EW("add_fused_qkv_bias_transpose", (long long)b * s, (long long)h * d, 4, 6, X, nullptr, q); }
int lg_add_fused_qkv_bias_transpose_f16(void* q, void*, void*, const void* X, const void*, int b, int s, int h, int d, void* stream) { return EW("add_fused_qkv_bias_transpose", (long long)b * s, (long long)h * d, 2, 6, X, nullptr, q); }
int lg_attn_softmax_f32(float* buf, const float* m, int b, int s, int h, float, void* stream) { return EW("attn_softmax", (long long)b * h * s, s, 4, 2, buf, m, buf); }
int lg_attn_softmax_f16(void* buf, const void* m, int b, int s, int h, float, void* stream) { return EW("attn_softmax", (long long)b * h * s, s, 2, 2, buf, m, buf); }
int lg_transpose_f32(float* dst, const float* src, int b, int s, int h, int d, void* stream) { return EW("transpose", (long long)b * s, (long long)h * d, 4, 2, src, nullptr, dst); }
int lg_transpose_f16(void* dst, const void* src, int b, int s, int h, int d, void* stream) { return EW("transpose", (long long)b * s, (long long)h * d, 2, 2, src, nullptr, dst); }

int lg_gemm_f32(int, int, int m, int n, int k, const float* A, int, const float* B, int, float* C, int, void* stream) { return launch(stream, "gemm", m, n, k, A, B, C, gemm_cost(m, n, k)); }
int lg_gemm_f16(int, int, int m, int n, int k, const void* A, int, const void* B, int, void* C, int, void* stream) { return launch(stream, "gemm", m, n, k, A, B, C, gemm_cost(m, n, k)); }
int lg_gemm_strided_batched_f32(int, int, int m, int n, int k, const float* A, int, int64_t, const float* B, int, int64_t, float* C, int, int64_t, int batch, void* stream) { return launch(stream, "gemm_batched", m, n, k, A, B, C, gemm_cost((long long)m * batch, n, k)); }
int lg_gemm_strided_batched_f16(int, int, int m, int n, int k, const void* A, int, int64_t, const void* B, int, int64_t, void* C, int, int64_t, int batch, void* stream) { return launch(stream, "gemm_batched", m, n, k, A, B, C, gemm_cost((long long)m * batch, n, k)); }
int lg_gemm_fused_f16(int, int m, int n, int k, const void* A, int, const void* B, int, void* C, int, int, const void*, int, int, int, void* stream) { return launch(stream, "gemm_fused", m, n, k, A, B, C, gemm_cost(m, n, k)); }
int lg_gemm_fused_grouped_f16(int, int m, int n, int k, int count, const void* const* A, int, const void* B, int, void* const* C, const int*, int, const void* const*, int, int, int, void* stream) { return launch(stream, "gemm_fused_grouped", (long long)m * count, n, k, A[0], B, C[0], gemm_cost((long long)m * count, n, k)); }
int lg_gemm_fused_grouped_rows_f16(int, int m, int n, int k, int count, const void* const* A, int, const void* B, int, void* const* C, const int*, const void* const*, int, int, const int*, const int* slot, const int*, void* stream) {
    (void)slot;
    return launch(stream, "gemm_fused_grouped_rows", (long long)m * count, n, k, A[0], B, C[0], gemm_cost((long long)m * count, n, k));
}
int lg_attn_prefill_f16(const void* q, const void* k, const void*, const void*, void* out, int b, int s, int h, int d, int, float, int, int, void* stream) { return launch(stream, "attn_prefill", (long long)b * h, s, d, q, k, out, gemm_cost((long long)b * h * s, s, 2 * d)); }
int lg_attn_prefill_past_f16(const void* q, const void* k, const void*, void* out, int b, int s, int past, int h, int d, int, float, int, int, void* stream) { return launch(stream, "attn_prefill_past", (long long)b * h, s, past, q, k, out, gemm_cost((long long)b * h * s, past + s, 2 * d)); }
size_t lg_attn_decode_workspace_bytes(int, int, int, int) { return 1024; }
int lg_attn_decode_f16(const void* q, const void* kc, const void*, void* out, void*, int b, int h, int d, int len, int, float, void* stream) { return launch(stream, "attn_decode", (long long)b * h, len, d, q, kc, out, mem_cost(4.0 * b * h * len * d)); }
int lg_attn_decode_static_f16(const void* q, const void* kc, const void*, void* out, int b, int h, int d, int len, int, float, void* stream) { return launch(stream, "attn_decode", (long long)b * h, len, d, q, kc, out, mem_cost(4.0 * b * h * len * d)); }
int lg_attn_decode_varlen_f16(const void* q, const void* kc, const void*, void* out, void*, int b, int h, int d, const int* slot, const int* len, int, float, void* stream) {
    long long keys = 0;
    for (int i = 0; i < b; ++i) keys += len[i];
    return launch(stream, "attn_decode_varlen", (long long)b * h, keys, slot ? slot[0] : 0, q, kc, out, mem_cost(4.0 * h * keys * d));
}
int lg_kv_append_varlen_f16(void* q, void* kc, void*, const void* Q, const void*, const void*, const void*, const void*, const void*, int b, int h, int d, const int* slot, const int* pos, int, void* stream) {
    return launch(stream, "kv_append_varlen", (long long)b * h, pos ? pos[0] : 0, slot ? slot[0] : 0, Q, kc, q, mem_cost(12.0 * b * h * d));
}
int lg_kv_append_f16(void* q, void* kc, void*, const void* Q, const void*, const void*, const void*, const void*, const void*, int b, int h, int d, int pos, int, void* stream) { return launch(stream, "kv_append", (long long)b * h, pos, d, Q, kc, q, mem_cost(12.0 * b * h * d)); }
int lg_weight_tile_f16(void* t, const void* p, int f, int k, int, int, void* stream) { return launch(stream, "weight_tile", f, k, 0, p, nullptr, t, mem_cost(4.0 * f * k)); }
int lg_weight_untile_f16(void* p, const void* t, int f, int k, int, int, void* stream) { return launch(stream, "weight_untile", f, k, 0, t, nullptr, p, mem_cost(4.0 * f * k)); }
// the measuring entries report the backend's own rates
int lg_probe_mfma_f16(const void* operands, int64_t n, void* scratch, size_t, int iters, float* ms, float* tflops, float* ghz, void*) {
    if (!operands || !scratch || iters <= 0 || !ms || n < 106504) return LG_ERR_INVALID;
    const double flop = 1024.0 * 8.0 * iters * 32.0 * 16384.0;
    *ms = (float)(flop / g_mfma_rate);
    if (tflops) *tflops = (float)(g_mfma_rate / 1e9);
    if (ghz) *ghz = 2.4f;
    return LG_OK;
}
int lg_probe_mfma_stream_f16(const void* operands, int64_t n, void* scratch, size_t sb, int iters, int loads, int reads, float* ms, float* tflops,
                             float* ghz, void* st) {
    if ((loads != 0 && loads != 4 && loads != 8) || (reads != 0 && reads != 6 && reads != 12)) return LG_ERR_INVALID;
    const int rc = lg_probe_mfma_f16(operands, n, scratch, sb, iters, ms, tflops, ghz, st);
    if (rc == LG_OK) *ms *= 2.f;   // twice the matrix instructions per round
    return rc;
}
int lg_probe_read(const void* src, size_t bytes, void* scratch, int passes, int, float* ms, float* gbps, void*) {
    if (!src || !scratch || passes <= 0 || !ms || bytes < (1u << 20)) return LG_ERR_INVALID;
    *ms = (float)((double)bytes / g_hbm_rate);
    if (gbps) *gbps = (float)(g_hbm_rate / 1e6);
    return LG_OK;
}

}  // extern "C"
