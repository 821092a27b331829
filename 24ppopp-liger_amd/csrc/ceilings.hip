// ceilings.hip -- two measuring kernels that put a number on what this GPU sustains, next to the published peaks.
//
// No reference counterpart (the reference measures nothing about its device).  The roofline fractions the bench prints
// divide by the published peaks (2.5 PFLOP/s dense fp16, 8 TB/s); these probes say how much of those a kernel that does
// nothing else can reach on the same device in the same process:
//   * lg_probe_mfma_f16: every wave keeps 8 + 4 operand fragments in registers and issues v_mfma_f32_16x16x32_f16 back to
//     back on a 128 x 64 wave tile (the pipelined GEMM's wave tile: 32 accumulator tiles, so no dependent MFMAs follow each
//     other), no loads, no LDS.  The operands come from a caller's buffer: with the GEMM's data distribution the matrix
//     pipes draw more power than with zeros and the clock settles lower, which is the ceiling a GEMM on that data has.
//   * lg_probe_mfma_stream_f16: the same wave tile and instruction, but with the data movement of the pipelined GEMM's k-loop
//     and nothing else of it: per 64 MFMAs a wave copies 8 KiB from global memory (a region that stays in L2) to LDS with
//     direct-to-LDS loads and reads 24 operand fragments of 1 KiB from LDS (two slots of 64 KiB), fragments double-buffered in
//     registers.  No barrier and no wait for a particular tile (the values multiplied are the source region's either way),
//     no epilogue, no stores, no traffic beyond L2: an upper bound for any k-loop that moves its operands
//     L2 -> LDS -> registers at the GEMM's rate, whatever its synchronisation costs on top.
//   * lg_probe_read: every byte of a caller's buffer is read once per pass with 16-byte loads, 8 in flight per lane,
//     1 KiB contiguous per wave instruction.  On a buffer much larger than the caches this is the memory read ceiling.
// Both entries time their kernel themselves (two events on the stream they are given) and therefore block: they are
// measurement calls for a bench, not launch-path entries.
#include "gemm_common.hpp"

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

// The k-loop of the pipelined GEMM reduced to its data movement: 8 waves, wave tile 128 x 64, k-tile 64 (two k-steps of 32).
// LDS: two slots of [256 rows][64] X + [256 rows][64] W halves (64 KiB each).  Per iteration every wave sends 8 direct-to-LDS
// loads of 1 KiB into one slot, reads its 2 x (8 + 4) fragments and issues 64 MFMAs; see the loop for what is left out.
// GL: direct-to-LDS loads per wave and iteration (8 = the GEMM's; 4, 0 = what half / none of that traffic would leave);
// RD: LDS fragment reads per k-step (12 = the GEMM's; 6, 0).  Fragments that are not re-read keep their first values.
template <int GL, int RD>
__global__ __launch_bounds__(512) void probe_mfma_stream_kernel(float* sink, long long* clocks, const half_t* in, int64_t in_elems, int iters) {
    extern __shared__ __align__(16) unsigned char probe_smem[];
    half_t* lds = (half_t*)probe_smem;
    constexpr int SLOT = 2 * 256 * 64;   // halves per slot
    const long long c0 = clock64(), w0 = wall_clock64();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wm = wave >> 2, wn = wave & 3;
    // the source region: a power-of-two number of 1 KiB pieces (indices wrap with a mask: no division in the loop)
    int piece_mask = 1;
    while ((int64_t)(piece_mask * 2) * 512 <= in_elems) piece_mask *= 2;
    piece_mask -= 1;
    // fragment addresses inside a slot (bytes): row r, 16-byte chunk c of a [rows][64] tile at (r * 64 + (c ^ ((r >> 1) & 7)) * 8) halves
    const int fr = lane & 15, fc = lane >> 4;
    unsigned a_addr[2], b_addr[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        const int ra = wm * 128 + fr, rb = wn * 64 + fr;
        a_addr[ks] = lds_address(lds) + 2u * (unsigned)(ra * 64 + (((ks * 4 + fc) ^ ((ra >> 1) & 7)) * 8));
        b_addr[ks] = lds_address(lds) + 2u * (unsigned)(256 * 64 + rb * 64 + (((ks * 4 + fc) ^ ((rb >> 1) & 7)) * 8));
    }
    auto issue_loads = [&](int it, int n) {
        half_t* dst = lds + (it & 1) * SLOT + wave * 8 * 512;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (u >= n) break;
            const int piece = (it * 64 + wave * 8 + u + (int)blockIdx.x * 7) & piece_mask;
            load_lds16(in + (int64_t)piece * 512 + lane * 8, dst + u * 512);
        }
    };
    float4_t acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    issue_loads(0, 8);
    issue_loads(1, 8);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    barrier_keep_loads_in_flight();
    // fragments double-buffered in registers: while the matrix instructions of one k-step run, the reads of the next are in
    // flight.  Nothing waits for a particular tile: the loads of an iteration only have to have left the queue two iterations
    // later (vmcnt(8)), there is no barrier, and the reads take whatever the slot holds (every value is one of the source
    // region's): the data movement is all there, the synchronisation a real k-loop needs on top is not.
    half8_t a[2][8], b[2][4];
    static_for<2>([&](auto s) {
        static_for<8>([&](auto i) { lds_read16_issue_at<i.value * 2048>(a[s.value][i.value], a_addr[s.value]); });
        static_for<4>([&](auto q) { lds_read16_issue_at<q.value * 2048>(b[s.value][q.value], b_addr[s.value]); });
    });
    // Every destination of a hand-issued read is named by a wait before anything else may use its registers: the compiler
    // does not know that they are written when the read lands, and would hand the registers of a read whose result it
    // believes dead to the next computation (an address, say) while the read is still in flight.
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[0][0]), "+v"(a[0][1]), "+v"(a[0][2]), "+v"(a[0][3]), "+v"(a[0][4]), "+v"(a[0][5]),
                                          "+v"(a[0][6]), "+v"(a[0][7]), "+v"(b[0][0]), "+v"(b[0][1]), "+v"(b[0][2]), "+v"(b[0][3]));
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[1][0]), "+v"(a[1][1]), "+v"(a[1][2]), "+v"(a[1][3]), "+v"(a[1][4]), "+v"(a[1][5]),
                                          "+v"(a[1][6]), "+v"(a[1][7]), "+v"(b[1][0]), "+v"(b[1][1]), "+v"(b[1][2]), "+v"(b[1][3]));
    for (int it = 0; it < iters; ++it) {
        issue_loads(it + 1, GL);
        const unsigned so = (unsigned)((it & 1) * SLOT * 2), sn = (unsigned)(((it + 1) & 1) * SLOT * 2);
        static_for<2>([&](auto ks) {
            constexpr int cur = ks.value, nxt = 1 - ks.value;
            // the fragments of this k-step have arrived (they were issued a k-step ago); the next k-step's go out now
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a[cur][0]), "+v"(a[cur][1]), "+v"(a[cur][2]), "+v"(a[cur][3]), "+v"(a[cur][4]), "+v"(a[cur][5]),
                                                  "+v"(a[cur][6]), "+v"(a[cur][7]), "+v"(b[cur][0]), "+v"(b[cur][1]), "+v"(b[cur][2]), "+v"(b[cur][3]));
            const unsigned base_a = a_addr[nxt] + (nxt == 1 ? so : sn), base_b = b_addr[nxt] + (nxt == 1 ? so : sn);
            if (RD >= 6) {
                static_for<4>([&](auto i) { lds_read16_issue_at<i.value * 2048>(a[nxt][i.value], base_a); });
                static_for<2>([&](auto q) { lds_read16_issue_at<q.value * 2048>(b[nxt][q.value], base_b); });
            }
            if (RD >= 12) {
                static_for<4>([&](auto i) { lds_read16_issue_at<(i.value + 4) * 2048>(a[nxt][i.value + 4], base_a); });
                static_for<2>([&](auto q) { lds_read16_issue_at<(q.value + 2) * 2048>(b[nxt][q.value + 2], base_b); });
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) acc[i][q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b[cur][q], a[cur][i], acc[i][q], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        });
        if (GL > 0) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" : "+v"(a[0][0]), "+v"(a[0][1]), "+v"(a[0][2]), "+v"(a[0][3]), "+v"(a[0][4]), "+v"(a[0][5]), "+v"(a[0][6]),
                                                   "+v"(a[0][7]), "+v"(b[0][0]), "+v"(b[0][1]), "+v"(b[0][2]), "+v"(b[0][3]) :: "memory");
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

// both matrix probes: `stream_operands` selects the kernel with the GEMM's data movement; flop per block and iteration differ
typedef void (*probe_kernel_t)(float*, long long*, const half_t*, int64_t, int);
static probe_kernel_t stream_kernel(int loads, int reads) {
    switch (loads * 100 + reads) {
        case 812: return probe_mfma_stream_kernel<8, 12>;
        case 806: return probe_mfma_stream_kernel<8, 6>;
        case 800: return probe_mfma_stream_kernel<8, 0>;
        case 412: return probe_mfma_stream_kernel<4, 12>;
        case 406: return probe_mfma_stream_kernel<4, 6>;
        case 400: return probe_mfma_stream_kernel<4, 0>;
        case 12: return probe_mfma_stream_kernel<0, 12>;
        case 6: return probe_mfma_stream_kernel<0, 6>;
        case 0: return probe_mfma_stream_kernel<0, 0>;
    }
    return nullptr;
}
static int probe_mfma(bool stream_operands, int loads, int reads, const void* operands, int64_t operand_elems, void* scratch, size_t scratch_bytes, int iters,
                      float* ms, float* tflops, float* shader_ghz, void* stream) {
    constexpr int GRID = 1024, BLOCK = 512;
    const size_t smem = stream_operands ? 2 * 2 * 256 * 64 * sizeof(half_t) : 0;   // two slots of 64 KiB
    probe_kernel_t kernel = stream_operands ? stream_kernel(loads, reads) : probe_mfma_kernel;
    if (!kernel) { set_error("lg_probe_mfma_stream_f16: loads_per_round is 0, 4 or 8 and reads_per_step 0, 6 or 12"); return LG_ERR_INVALID; }
    if (stream_operands && hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) {
        set_error("lg_probe_mfma_stream_f16: cannot reserve %zu bytes of LDS", smem);
        return LG_ERR_LAUNCH;
    }
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
    hipLaunchKernelGGL(kernel, dim3(GRID), dim3(BLOCK), smem, st, sink, clocks, (const half_t*)operands, operand_elems, iters / 8 + 1);
    if (hipEventRecord(e0, st) != hipSuccess) rc = LG_ERR_LAUNCH;
    hipLaunchKernelGGL(kernel, dim3(GRID), dim3(BLOCK), smem, st, sink, clocks, (const half_t*)operands, operand_elems, iters);
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
    // per block and iteration: 8 waves x 32 (with streamed operands: 64) MFMAs x (16 x 16 x 32 x 2) flop
    const double flop = (double)GRID * 8.0 * (double)iters * (stream_operands ? 64.0 : 32.0) * 16384.0;
    if (tflops) *tflops = (float)(flop / ((double)t * 1e9));
    if (shader_ghz) {
        int rate_khz = 0, dev = 0;
        (void)hipGetDevice(&dev);
        if (hipDeviceGetAttribute(&rate_khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || rate_khz <= 0) rate_khz = 100000;
        *shader_ghz = h[1] > 0 ? (float)((double)h[0] / ((double)h[1] / ((double)rate_khz * 1e3)) / 1e9) : 0.f;
    }
    return LG_OK;
}

int lg_probe_mfma_f16(const void* operands, int64_t operand_elems, void* scratch, size_t scratch_bytes, int iters, float* ms,
                      float* tflops, float* shader_ghz, void* stream) {
    return probe_mfma(false, 0, 0, operands, operand_elems, scratch, scratch_bytes, iters, ms, tflops, shader_ghz, stream);
}
int lg_probe_mfma_stream_f16(const void* operands, int64_t operand_elems, void* scratch, size_t scratch_bytes, int iters, int loads_per_round,
                             int reads_per_step, float* ms, float* tflops, float* shader_ghz, void* stream) {
    return probe_mfma(true, loads_per_round, reads_per_step, operands, operand_elems, scratch, scratch_bytes, iters, ms, tflops, shader_ghz, stream);
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
