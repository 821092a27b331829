// runtime.hip -- error state, thin HIP runtime wrappers and synthetic-data fill kernels.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <unordered_map>

#include "common.hpp"

namespace lg {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: %s", what, hipGetErrorString(e));
        return LG_ERR_LAUNCH;
    }
    return LG_OK;
}

static int rt(hipError_t e, const char* what) {
    if (e == hipSuccess) return LG_OK;
    set_error("%s: %s", what, hipGetErrorString(e));
    return LG_ERR_LAUNCH;
}

// ---- stream registry -----------------------------------------------------------------------------------------------------------
// What the launchers need to know about the stream they are handed: how many compute units its kernels may run on (a CU-masked
// stream has fewer than the device, and grids are sized for what is there) and where its split-K workspace is.  The workspace is
// allocated when a stream is created or attached, never on the launch path (the counterpart of the workspace a cuBLAS handle
// owns: context.h:20-29 binds one handle per stream).
static std::mutex g_streams_mu;
static std::unordered_map<void*, StreamInfo> g_streams;

int device_cu_count() {
    static int cached = 0;
    if (cached > 0) return cached;
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
        cached = n;
    return cached > 0 ? cached : 256;
}

StreamInfo stream_info(hipStream_t stream) {
    {
        std::lock_guard<std::mutex> lk(g_streams_mu);
        auto it = g_streams.find((void*)stream);
        if (it != g_streams.end()) return it->second;
    }
    return StreamInfo{device_cu_count(), nullptr, 0};
}

static int register_stream(void* stream, int cus) {
    StreamInfo info{cus > 0 ? cus : device_cu_count(), nullptr, 0};
    {
        std::lock_guard<std::mutex> lk(g_streams_mu);
        auto it = g_streams.find(stream);
        if (it != g_streams.end()) {  // already known: only an explicit CU count changes anything
            if (cus > 0) it->second.cus = cus;
            return LG_OK;
        }
    }
    // hipMalloc may synchronise the device, so it runs outside the lock; two threads that attach the same stream at the same
    // time both get here, and the one that finds the stream registered when it comes back frees its block again
    void* p = nullptr;
    const int rc = rt(hipMalloc(&p, LG_SPLITK_WORKSPACE_BYTES), "hipMalloc (split-K workspace)");
    if (rc) return rc;
    info.ws = (float*)p;
    info.ws_bytes = LG_SPLITK_WORKSPACE_BYTES;
    {
        std::lock_guard<std::mutex> lk(g_streams_mu);
        auto it = g_streams.find(stream);
        if (it == g_streams.end()) {
            g_streams[stream] = info;
            return LG_OK;
        }
        if (cus > 0) it->second.cus = cus;
    }
    return rt(hipFree(p), "hipFree (split-K workspace of a stream registered twice)");
}

static int unregister_stream(void* stream) {
    StreamInfo info{0, nullptr, 0};
    {
        std::lock_guard<std::mutex> lk(g_streams_mu);
        auto it = g_streams.find(stream);
        if (it == g_streams.end()) return LG_OK;
        info = it->second;
        g_streams.erase(it);
    }
    if (!info.ws) return LG_OK;
    // launches on the stream may still read the workspace
    int rc = rt(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
    const int rc2 = rt(hipFree(info.ws), "hipFree (split-K workspace)");
    return rc ? rc : rc2;
}

// ---- counter-based Irwin-Hall(8) generator; integer work + two rounded fp32 ops --------------------
__device__ __forceinline__ uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
static uint64_t splitmix64_host(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
__device__ __forceinline__ uint32_t sum16x4(uint64_t r) {
    return (uint32_t)(r & 0xffffu) + (uint32_t)((r >> 16) & 0xffffu) + (uint32_t)((r >> 32) & 0xffffu) +
           (uint32_t)(r >> 48);
}

template <typename T>
__global__ void fill_normal_kernel(T* out, int64_t n, uint64_t key, float mean, float stddev) {
#pragma clang fp contract(off)  // the multiply and the add must round separately to match the CPU generator
    const float inv_sigma = 0x1.3988e2p-16f;  // 1/sqrt(8*(65536^2-1)/12)
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        uint64_t a = splitmix64(key + 2ull * (uint64_t)i);
        uint64_t b = splitmix64(key + 2ull * (uint64_t)i + 1ull);
        int32_t s = (int32_t)(sum16x4(a) + sum16x4(b)) - 262140;
        const float z = (float)s * inv_sigma;
        float v = stddev * z;
        v = v + mean;
        out[i] = (T)v;
    }
}

template <typename T>
__global__ void fill_const_kernel(T* out, int64_t n, float value) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        out[i] = (T)value;
}

template <typename T>
__global__ void fill_causal_mask_kernel(T* mask, int batch, int seq) {
    const int64_t n = (int64_t)batch * seq * seq;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const int col = (int)(i % seq);
        const int row = (int)((i / seq) % seq);
        mask[i] = (T)(col <= row ? 1.0f : 0.0f);
    }
}

static int grid_for(int64_t n, int block) {
    int64_t g = (n + block - 1) / block;
    if (g > 65536) g = 65536;
    if (g < 1) g = 1;
    return (int)g;
}

template <typename T>
static int fill_normal(T* out, int64_t n, uint64_t seed, uint64_t tensor_id, float mean, float stddev, void* stream) {
    if (n < 0 || (n > 0 && !out)) { set_error("fill_normal: bad arguments"); return LG_ERR_INVALID; }
    if (n == 0) return LG_OK;
    const uint64_t key = splitmix64_host(seed * 0x100000001B3ull + tensor_id);
    hipLaunchKernelGGL(fill_normal_kernel<T>, dim3(grid_for(n, 256)), dim3(256), 0, (hipStream_t)stream, out, n, key,
                       mean, stddev);
    return check_launch("fill_normal");
}
template <typename T>
static int fill_const(T* out, int64_t n, float value, void* stream) {
    if (n < 0 || (n > 0 && !out)) { set_error("fill_const: bad arguments"); return LG_ERR_INVALID; }
    if (n == 0) return LG_OK;
    hipLaunchKernelGGL(fill_const_kernel<T>, dim3(grid_for(n, 256)), dim3(256), 0, (hipStream_t)stream, out, n, value);
    return check_launch("fill_const");
}
template <typename T>
static int fill_causal(T* mask, int batch, int seq, void* stream) {
    if (batch <= 0 || seq <= 0 || !mask) { set_error("fill_causal_mask: bad arguments"); return LG_ERR_INVALID; }
    const int64_t n = (int64_t)batch * seq * seq;
    hipLaunchKernelGGL(fill_causal_mask_kernel<T>, dim3(grid_for(n, 256)), dim3(256), 0, (hipStream_t)stream, mask,
                       batch, seq);
    return check_launch("fill_causal_mask");
}

}  // namespace lg

using namespace lg;

extern "C" {

const char* lg_last_error(void) { return lg::g_err; }
const char* lg_version(void) { return "liger-hip 0.1 (gfx950)"; }

int lg_device_info(char* name, int name_len, int* cu_count, int* clock_khz, int* mem_clock_khz, int* bus_width_bits,
                   size_t* total_mem) {
    int dev = 0;
    int rc = rt(hipGetDevice(&dev), "hipGetDevice");
    if (rc) return rc;
    hipDeviceProp_t p;
    rc = rt(hipGetDeviceProperties(&p, dev), "hipGetDeviceProperties");
    if (rc) return rc;
    if (name && name_len > 0) {
        strncpy(name, p.gcnArchName, (size_t)name_len - 1);
        name[name_len - 1] = 0;
    }
    if (cu_count) *cu_count = p.multiProcessorCount;
    if (clock_khz) *clock_khz = p.clockRate;
    if (mem_clock_khz) *mem_clock_khz = p.memoryClockRate;
    if (bus_width_bits) *bus_width_bits = p.memoryBusWidth;
    if (total_mem) *total_mem = p.totalGlobalMem;
    return LG_OK;
}

int lg_malloc(void** ptr, size_t bytes) { return rt(hipMalloc(ptr, bytes), "hipMalloc"); }
int lg_free(void* ptr) { return rt(hipFree(ptr), "hipFree"); }
int lg_memcpy_h2d(void* dst, const void* src, size_t bytes) {
    return rt(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice), "hipMemcpy h2d");
}
int lg_memcpy_d2h(void* dst, const void* src, size_t bytes) {
    return rt(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost), "hipMemcpy d2h");
}
int lg_memcpy_d2d_async(void* dst, const void* src, size_t bytes, void* stream) {
    return rt(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream), "hipMemcpyAsync d2d");
}
int lg_memset_async(void* dst, int value, size_t bytes, void* stream) {
    return rt(hipMemsetAsync(dst, value, bytes, (hipStream_t)stream), "hipMemsetAsync");
}
int lg_device_synchronize(void) { return rt(hipDeviceSynchronize(), "hipDeviceSynchronize"); }
int lg_stream_create(void** stream) {
    if (!stream) { set_error("lg_stream_create: null argument"); return LG_ERR_INVALID; }
    hipStream_t s = nullptr;
    int rc = rt(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreateWithFlags");
    *stream = (void*)s;
    return rc ? rc : register_stream((void*)s, 0);
}
int lg_stream_attach(void* stream, int cu_count) {
    if (cu_count < 0) { set_error("lg_stream_attach: negative CU count"); return LG_ERR_INVALID; }
    return register_stream(stream, cu_count);
}
int lg_stream_detach(void* stream) { return unregister_stream(stream); }
int lg_stream_cu_count(void* stream) { return stream_info((hipStream_t)stream).cus; }
__global__ void lg_stream_first_use_kernel(int* sink) {
    if (sink && threadIdx.x == 1024) *sink = 1;  // never true: an empty kernel
}
int lg_stream_create_cu_mask(void** stream, const unsigned* cu_mask, int mask_words) {
    if (!stream || !cu_mask || mask_words <= 0) { set_error("lg_stream_create_cu_mask: bad arguments"); return LG_ERR_INVALID; }
    // Bit i of the mask selects a compute unit of accelerator die i mod 8 (the dies take the bits in turn).  A mask that leaves
    // a die without any unit is refused: the runtime fails on the host for such a stream.
    const int total = device_cu_count();
    const int dies = total >= 64 ? 8 : 1;
    int cus = 0, per_die[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int b = 0; b < mask_words * 32 && b < total; ++b)
        if (cu_mask[b >> 5] & (1u << (b & 31))) { ++cus; ++per_die[b % dies]; }
    for (int x = 0; x < dies; ++x)
        if (per_die[x] == 0) { set_error("lg_stream_create_cu_mask: the mask selects no compute unit on die %d (bit i belongs to die i mod %d)", x, dies); return LG_ERR_INVALID; }
    hipStream_t s = nullptr;
    int rc = rt(hipExtStreamCreateWithCUMask(&s, (uint32_t)mask_words, cu_mask), "hipExtStreamCreateWithCUMask");
    *stream = (void*)s;
    if (rc) return rc;
    // The runtime sets a stream's hardware queue up at its first submission.  A CU-masked stream that is destroyed without ever
    // having run anything has been seen to block in hipStreamDestroy (about one time in four), so every such stream runs one
    // empty kernel here, at creation, where waiting is allowed.
    hipLaunchKernelGGL(lg_stream_first_use_kernel, dim3(1), dim3(64), 0, s, (int*)nullptr);
    rc = rt(hipGetLastError(), "first kernel on a CU-masked stream");
    if (!rc) rc = rt(hipStreamSynchronize(s), "hipStreamSynchronize");
    if (rc) { (void)hipStreamDestroy(s); *stream = nullptr; return rc; }
    return register_stream((void*)s, cus);
}
// ---- a second stream that really runs next to the first ----------------------------------------------------------------------
// HIP multiplexes streams onto a few hardware queues (4 per process by default) and hands a new stream the least used one,
// so two streams of one process can land on the same hardware queue, where their kernels run strictly one after the other.
// Whether that happened cannot be queried, but it can be measured: one wave spins for a fixed time on `other` while a
// one-wave kernel is launched on the candidate; on separate queues the second finishes long before the first.
__global__ void lg_probe_spin_kernel(long long ticks, int* sink) {
    const long long t0 = wall_clock64();  // constant-rate counter: the loop ends after `ticks` whatever else happens
    while (wall_clock64() - t0 < ticks) {}
    if (sink && threadIdx.x == 1024) *sink = 1;  // never true: keeps the loop observable
}
__global__ void lg_probe_touch_kernel(int* sink) {
    if (sink && threadIdx.x == 1024) *sink = 1;
}
static bool runs_concurrently(hipStream_t a, hipStream_t b, bool* ok) {
    *ok = false;
    int rate_khz = 0;
    int dev = 0;
    (void)hipGetDevice(&dev);
    if (hipDeviceGetAttribute(&rate_khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || rate_khz <= 0) rate_khz = 100000;
    const double spin_ms = 0.4;
    hipEvent_t ea = nullptr, eb = nullptr;
    if (hipEventCreate(&ea) != hipSuccess || hipEventCreate(&eb) != hipSuccess) return false;
    bool concurrent = false;
    // warm both kernels up first (code upload), then the timed pair
    for (int pass = 0; pass < 2; ++pass) {
        hipLaunchKernelGGL(lg_probe_spin_kernel, dim3(1), dim3(64), 0, a, (long long)(pass ? spin_ms * rate_khz : 1), (int*)nullptr);
        if (hipEventRecord(ea, a) != hipSuccess) break;
        hipLaunchKernelGGL(lg_probe_touch_kernel, dim3(1), dim3(64), 0, b, (int*)nullptr);
        if (hipEventRecord(eb, b) != hipSuccess) break;
        if (hipStreamSynchronize(a) != hipSuccess || hipStreamSynchronize(b) != hipSuccess) break;
        if (pass == 1) {
            float ms = 0.f;  // from the end of the touch kernel on b to the end of the spin on a
            if (hipEventElapsedTime(&ms, eb, ea) != hipSuccess) break;
            concurrent = ms > 0.5f * (float)spin_ms;
            *ok = true;
        }
    }
    (void)hipEventDestroy(ea);
    (void)hipEventDestroy(eb);
    return concurrent;
}
int lg_stream_create_concurrent(void** stream, void* other, int* verified) {
    if (!stream || !other) { set_error("lg_stream_create_concurrent: bad arguments"); return LG_ERR_INVALID; }
    if (verified) *verified = 0;
    constexpr int TRIES = 8;
    hipStream_t cand[TRIES];
    int n = 0, pick = -1;
    for (; n < TRIES && pick < 0; ++n) {
        // rejected candidates stay alive until the end, so that the next one is handed another hardware queue
        if (rt(hipStreamCreateWithFlags(&cand[n], hipStreamNonBlocking), "hipStreamCreateWithFlags") != LG_OK) break;
        bool ok = false;
        const bool conc = runs_concurrently((hipStream_t)other, cand[n], &ok);
        if (!ok) { ++n; set_error("lg_stream_create_concurrent: the concurrency probe failed"); break; }
        if (conc) pick = n;
    }
    if (pick < 0 && n > 0) pick = 0;  // none verified: the caller still gets a working stream
    else if (pick >= 0 && verified) *verified = 1;
    for (int i = 0; i < n; ++i)
        if (i != pick) (void)hipStreamDestroy(cand[i]);
    if (pick < 0) return LG_ERR_LAUNCH;
    *stream = (void*)cand[pick];
    return register_stream(*stream, 0);
}
int lg_streams_run_concurrently(void* a, void* b, int* concurrent) {
    if (!a || !b || a == b || !concurrent) { set_error("lg_streams_run_concurrently: needs two different created streams"); return LG_ERR_INVALID; }
    bool ok = false;
    const bool conc = runs_concurrently((hipStream_t)a, (hipStream_t)b, &ok);
    if (!ok) { set_error("lg_streams_run_concurrently: the concurrency probe failed"); return LG_ERR_LAUNCH; }
    *concurrent = conc ? 1 : 0;
    return LG_OK;
}
int lg_stream_destroy(void* stream) {
    const int rc = unregister_stream(stream);
    const int rc2 = rt(hipStreamDestroy((hipStream_t)stream), "hipStreamDestroy");
    return rc ? rc : rc2;
}
int lg_stream_synchronize(void* stream) { return rt(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize"); }
int lg_stream_wait_event(void* stream, void* event) {
    return rt(hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)event, 0), "hipStreamWaitEvent");
}
int lg_event_create(void** event) {
    hipEvent_t e = nullptr;
    int rc = rt(hipEventCreate(&e), "hipEventCreate");
    *event = (void*)e;
    return rc;
}
int lg_event_destroy(void* event) { return rt(hipEventDestroy((hipEvent_t)event), "hipEventDestroy"); }
int lg_event_record(void* event, void* stream) {
    return rt(hipEventRecord((hipEvent_t)event, (hipStream_t)stream), "hipEventRecord");
}
int lg_event_synchronize(void* event) { return rt(hipEventSynchronize((hipEvent_t)event), "hipEventSynchronize"); }
int lg_event_query(void* event) {
    hipError_t e = hipEventQuery((hipEvent_t)event);
    if (e == hipSuccess) return LG_OK;
    if (e == hipErrorNotReady) return 3;
    return rt(e, "hipEventQuery");
}
int lg_event_elapsed_ms(float* ms, void* start, void* stop) {
    return rt(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop), "hipEventElapsedTime");
}

int lg_fill_normal_f32(float* out, int64_t n, uint64_t seed, uint64_t tensor_id, float mean, float stddev, void* stream) {
    return fill_normal<float>(out, n, seed, tensor_id, mean, stddev, stream);
}
int lg_fill_normal_f16(void* out, int64_t n, uint64_t seed, uint64_t tensor_id, float mean, float stddev, void* stream) {
    return fill_normal<half_t>((half_t*)out, n, seed, tensor_id, mean, stddev, stream);
}
int lg_fill_const_f32(float* out, int64_t n, float value, void* stream) { return fill_const<float>(out, n, value, stream); }
int lg_fill_const_f16(void* out, int64_t n, float value, void* stream) {
    return fill_const<half_t>((half_t*)out, n, value, stream);
}
int lg_fill_causal_mask_f32(float* mask, int batch, int seq, void* stream) { return fill_causal<float>(mask, batch, seq, stream); }
int lg_fill_causal_mask_f16(void* mask, int batch, int seq, void* stream) {
    return fill_causal<half_t>((half_t*)mask, batch, seq, stream);
}

}  // extern "C"
