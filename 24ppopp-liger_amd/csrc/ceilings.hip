// ceilings.hip -- two measuring kernels that put a number on what this GPU sustains, next to the published peaks.
//
// No reference counterpart (the reference measures nothing about its device).  The roofline fractions the bench prints
// divide by the published peaks (2.5 PFLOP/s dense fp16, 8 TB/s); these probes say how much of those a kernel that does
// nothing else can reach on the same device in the same process:
//   * lg_probe_mfma_f16: every wave keeps 8 + 4 operand fragments in registers and issues v_mfma_f32_16x16x32_f16 back to
//     back on a 128 x 64 wave tile (the pipelined GEMM's wave tile: 32 accumulator tiles, so no dependent MFMAs follow each
//     other), no loads, no LDS.  The operands come from a caller's buffer: with the GEMM's data distribution the matrix
//     pipes draw more power than with zeros and the clock settles lower, which is the ceiling a GEMM on that data has.
//   * lg_probe_read: every byte of a caller's buffer is read once per pass with 16-byte loads, 8 in flight per lane,
//     1 KiB contiguous per wave instruction.  On a buffer much larger than the caches this is the memory read ceiling.
// Both entries time their kernel themselves (two events on the stream they are given) and therefore block: they are
// measurement calls for a bench, not launch-path entries.
#include "common.hpp"

namespace lg {

// out[0] = shader clock ticks, out[1] = constant-rate ticks spent by block 0's first thread
__global__ __launch_bounds__(512) void probe_mfma_kernel(float* sink, long long* clocks, const half_t* in, int64_t in_elems, int iters) {
    const long long c0 = clock64(), w0 = wall_clock64();
    half8_t a[8], b[4];
    // fragments from different places of the buffer for different lanes and blocks; in_elems >= 12 * 8192 + 1024 is checked
    const int64_t span = in_elems - (12 * 8192 + 8 * 1024);
    const int64_t base = ((int64_t)blockIdx.x * 1237 * 8) % (span > 0 ? span : 1);
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] = *(const half8_t*)(in + base + (int64_t)threadIdx.x * 8 + i * 8192);
#pragma unroll
    for (int j = 0; j < 4; ++j) b[j] = *(const half8_t*)(in + base + (int64_t)threadIdx.x * 8 + (8 + j) * 8192);
    float4_t acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b[j], a[i], acc[i][j], 0, 0, 0);
        // rotate the row fragments: consecutive iterations multiply different data, as the k-loop of a GEMM does
        const half8_t t = a[0];
#pragma unroll
        for (int i = 0; i < 7; ++i) a[i] = a[i + 1];
        a[7] = t;
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) s += acc[i][j][0] + acc[i][j][3];
    if (s == 12345.678f) sink[0] = s;   // keeps the loop alive; practically never true
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        clocks[0] = clock64() - c0;
        clocks[1] = wall_clock64() - w0;
    }
}

// One pass over `chunks` 16-byte pieces: a block owns runs of 8 x 256 pieces (32 KiB), a wave instruction reads 1 KiB.
template <bool NT>
__global__ __launch_bounds__(256) void probe_read_kernel(const float4_t* src, int64_t chunks, float* sink) {
    float s = 0.f;
    const int64_t per_block = 8 * 256;
    for (int64_t base = (int64_t)blockIdx.x * per_block; base < chunks; base += (int64_t)gridDim.x * per_block) {
        float4_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            int64_t i = base + u * 256 + threadIdx.x;
            if (i >= chunks) i = chunks - 1;
            v[u] = NT ? __builtin_nontemporal_load(src + i) : src[i];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u][0] + v[u][3];
    }
    if (s == 12345.678f) sink[0] = s;
}

}  // namespace lg

using namespace lg;

extern "C" {

int lg_probe_mfma_f16(const void* operands, int64_t operand_elems, void* scratch, size_t scratch_bytes, int iters, float* ms,
                      float* tflops, float* shader_ghz, void* stream) {
    constexpr int GRID = 1024, BLOCK = 512;
    if (!operands || !scratch || iters <= 0 || !ms || operand_elems < 12 * 8192 + 8 * 1024 + 8 || scratch_bytes < 64 || !aligned16(operands) ||
        (reinterpret_cast<uintptr_t>(scratch) & 7u)) {
        set_error("lg_probe_mfma_f16: needs >= 106504 fp16 operands (16-byte aligned), 64 bytes of scratch and iters > 0");
        return LG_ERR_INVALID;
    }
    hipStream_t st = (hipStream_t)stream;
    long long* clocks = (long long*)scratch;
    float* sink = (float*)((char*)scratch + 32);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) { set_error("lg_probe_mfma_f16: hipEventCreate failed"); return LG_ERR_LAUNCH; }
    int rc = LG_OK;
    float t = 0.f;
    long long h[2] = {0, 0};
    // one short untimed launch (code upload, clocks), then the timed one
    hipLaunchKernelGGL(probe_mfma_kernel, dim3(GRID), dim3(BLOCK), 0, st, sink, clocks, (const half_t*)operands, operand_elems, iters / 8 + 1);
    if (hipEventRecord(e0, st) != hipSuccess) rc = LG_ERR_LAUNCH;
    hipLaunchKernelGGL(probe_mfma_kernel, dim3(GRID), dim3(BLOCK), 0, st, sink, clocks, (const half_t*)operands, operand_elems, iters);
    if (!rc) rc = check_launch("lg_probe_mfma_f16");
    if (!rc && (hipEventRecord(e1, st) != hipSuccess || hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&t, e0, e1) != hipSuccess ||
                hipMemcpy(h, clocks, sizeof(h), hipMemcpyDeviceToHost) != hipSuccess)) {
        set_error("lg_probe_mfma_f16: timing failed: %s", hipGetErrorString(hipGetLastError()));
        rc = LG_ERR_LAUNCH;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc) return rc;
    *ms = t;
    // per block and iteration: 8 waves x 32 MFMAs x (16 x 16 x 32 x 2) flop
    const double flop = (double)GRID * 8.0 * (double)iters * 32.0 * 16384.0;
    if (tflops) *tflops = (float)(flop / ((double)t * 1e9));
    if (shader_ghz) {
        int rate_khz = 0, dev = 0;
        (void)hipGetDevice(&dev);
        if (hipDeviceGetAttribute(&rate_khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || rate_khz <= 0) rate_khz = 100000;
        *shader_ghz = h[1] > 0 ? (float)((double)h[0] / ((double)h[1] / ((double)rate_khz * 1e3)) / 1e9) : 0.f;
    }
    return LG_OK;
}

int lg_probe_read(const void* src, size_t bytes, void* scratch, int passes, int nontemporal, float* ms, float* gbps, void* stream) {
    if (!src || !scratch || bytes < (1u << 20) || passes <= 0 || !ms || !aligned16(src)) {
        set_error("lg_probe_read: needs a 16-byte aligned buffer of at least 1 MiB, 4 bytes of scratch and passes > 0");
        return LG_ERR_INVALID;
    }
    hipStream_t st = (hipStream_t)stream;
    const int64_t chunks = (int64_t)(bytes / 16);
    const int grid = stream_info(st).cus * 8;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) { set_error("lg_probe_read: hipEventCreate failed"); return LG_ERR_LAUNCH; }
    int rc = LG_OK;
    float t = 0.f;
    auto kernel = nontemporal ? probe_read_kernel<true> : probe_read_kernel<false>;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), 0, st, (const float4_t*)src, chunks, (float*)scratch);
    if (hipEventRecord(e0, st) != hipSuccess) rc = LG_ERR_LAUNCH;
    for (int p = 0; p < passes; ++p)
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), 0, st, (const float4_t*)src, chunks, (float*)scratch);
    if (!rc) rc = check_launch("lg_probe_read");
    if (!rc && (hipEventRecord(e1, st) != hipSuccess || hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&t, e0, e1) != hipSuccess)) {
        set_error("lg_probe_read: timing failed: %s", hipGetErrorString(hipGetLastError()));
        rc = LG_ERR_LAUNCH;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc) return rc;
    *ms = t / (float)passes;
    if (gbps) *gbps = (float)((double)chunks * 16.0 * (double)passes / ((double)t * 1e6));
    return LG_OK;
}

}  // extern "C"
