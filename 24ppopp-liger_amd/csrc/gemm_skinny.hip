// gemm_skinny.hip -- weight-streaming fp16 GEMM for few tokens (decode: M <= 64) on gfx950.
//
//   Y[M, N] = X[M, K] * W^T with W stored [N, K] (both operands K-contiguous), M <= 64.
// With a handful of token rows every weight byte is used for 2*M flops only, so the kernel is a pure HBM stream of W
// (1.4 GB per GLM-130B TP=2 layer shard) and is organised like one:
//   * a block = 4 waves x 32 output features; the grid is (N / 128) x S with S K-slices chosen so that >= ~1000 blocks
//     keep >= 16 waves per CU streaming;
//   * W fragments go from global memory straight into MFMA operand registers (a lane owns 8 consecutive k of one output
//     feature: exactly the B operand of v_mfma_f32_16x16x32_f16) in a rolling pipeline that keeps 16 independent
//     16-byte loads in flight per lane at all times;
//   * the few X rows are staged once per 256-wide k-chunk in LDS (double buffered) and shared by the block's waves;
//   * K-slices are summed in fp32 through a per-stream workspace and a small second kernel that also applies the
//     epilogue (bias / GELU / head-transposed store), so results match the single-pass kernels' rounding.
#include <mutex>
#include <unordered_map>

#include "gemm_common.cuh"

namespace lg {

constexpr int SK_BN = 128;      // output features per block
constexpr int SK_KC = 256;      // k-chunk staged in LDS
constexpr int SK_XS = SK_KC + 8;  // LDS row stride of the X chunk (halves)

// MT = number of 16-row token tiles (M <= 16*MT)
template <int MT>
__global__ __launch_bounds__(256) void gemm_skinny_nk_kernel(GemmArgs g, int kslice, float* partial, int nsplit) {
    __shared__ __attribute__((aligned(16))) half_t xs[2][16 * MT * SK_XS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, lk = lane >> 4;
    const int n0 = blockIdx.x * SK_BN + wave * 32;
    const int split = blockIdx.y;
    const int k_begin = split * kslice;
    const int nchunks = (min(g.K, k_begin + kslice) - k_begin) / SK_KC;  // whole chunks only

    // The loop below is branch-free (the launcher guarantees K-slices made of whole 256-wide chunks): rows beyond M are
    // read from row M-1 (they only feed accumulator rows that are never stored) and the chunk after the last one is the
    // last one again, so that every load is unconditional and the compiler can count outstanding loads exactly.
    // X chunk [16*MT rows][256 k]: global -> registers -> LDS buffer
    constexpr int XV = 16 * MT * (SK_KC / 8) / 256;  // 16-byte vectors per thread and chunk
    const half_t* xsrc[XV];
#pragma unroll
    for (int u = 0; u < XV; ++u) {
        const int v = tid + u * 256;
        const int row = min(v / (SK_KC / 8), g.M - 1), c = v % (SK_KC / 8);
        xsrc[u] = g.X + (int64_t)row * g.ldx + k_begin + c * 8;
    }
    auto load_x = [&](int chunk, half8_t (&xr)[XV]) {
#pragma unroll
        for (int u = 0; u < XV; ++u) xr[u] = *reinterpret_cast<const half8_t*>(xsrc[u] + chunk * SK_KC);
    };
    auto store_x = [&](int buf, const half8_t (&xr)[XV]) {
#pragma unroll
        for (int u = 0; u < XV; ++u) {
            const int v = tid + u * 256;
            const int row = v / (SK_KC / 8), c = v % (SK_KC / 8);
            *reinterpret_cast<half8_t*>(&xs[buf][row * SK_XS + c * 8]) = xr[u];
        }
    };

    float4_t acc[MT][2];
#pragma unroll
    for (int i = 0; i < MT; ++i) { acc[i][0] = float4_t{0.f, 0.f, 0.f, 0.f}; acc[i][1] = float4_t{0.f, 0.f, 0.f, 0.f}; }

    // this lane's two weight rows (output features n0 + l16 and n0 + 16 + l16); rows beyond N are clamped and never stored
    const int r0 = min(n0 + l16, g.N - 1), r1 = min(n0 + 16 + l16, g.N - 1);
    const half_t* w0 = g.W + (int64_t)r0 * g.ldw + k_begin + lk * 8;
    const half_t* w1 = g.W + (int64_t)r1 * g.ldw + k_begin + lk * 8;

    // Rolling pipeline: the 16 weight fragments of a chunk live in registers; as soon as fragment s of chunk ch has been
    // multiplied its registers are reloaded with fragment s of chunk ch+1, so every lane keeps 16 loads in flight all the
    // time.  The next X chunk is fetched at the start of a chunk (it queues behind weight loads that are consumed during
    // the chunk anyway) and written to the other LDS buffer at its end.
    half8_t b0[8], b1[8], xr[XV];
    load_x(0, xr);
    store_x(0, xr);
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        b0[s] = *reinterpret_cast<const half8_t*>(w0 + s * 32);
        b1[s] = *reinterpret_cast<const half8_t*>(w1 + s * 32);
    }
    __syncthreads();
    for (int ch = 0; ch < nchunks; ++ch) {
        const int buf = ch & 1;
        const int next = min(ch + 1, nchunks - 1);
        load_x(next, xr);
#pragma unroll
        for (int s = 0; s < 8; ++s) {
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const half8_t a = *reinterpret_cast<const half8_t*>(&xs[buf][(i * 16 + l16) * SK_XS + s * 32 + lk * 8]);
                // operands swapped: acc[i][j][r] = Y[m = 16 i + l16][n = n0 + 16 j + 4 lk + r]
                acc[i][0] = mfma16(b0[s], a, acc[i][0]);
                acc[i][1] = mfma16(b1[s], a, acc[i][1]);
            }
            b0[s] = *reinterpret_cast<const half8_t*>(w0 + next * SK_KC + s * 32);
            b1[s] = *reinterpret_cast<const half8_t*>(w1 + next * SK_KC + s * 32);
        }
        store_x(buf ^ 1, xr);
        __syncthreads();
    }

    // fp32 partials [split][M][N]; with a single slice the reduce kernel still applies the epilogue
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int m = i * 16 + l16, n = n0 + j * 16 + 4 * lk;
            if (m < g.M && n < g.N) {
                float* p = partial + ((int64_t)split * g.M + m) * g.N + n;
                if (n + 3 < g.N) {
                    *reinterpret_cast<float4_t*>(p) = acc[i][j];
                } else {
                    for (int r = 0; r < 4 && n + r < g.N; ++r) p[r] = acc[i][j][r];
                }
            }
        }
    (void)nsplit;
}

// sums the K-slices and applies the epilogue; one thread per 4 consecutive output columns
template <int EPI>
__global__ __launch_bounds__(256) void gemm_skinny_reduce_kernel(GemmArgs g, const float* partial, int nsplit) {
    const int64_t quads = (int64_t)g.M * ((g.N + 3) / 4);
    for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < quads; q += (int64_t)gridDim.x * blockDim.x) {
        const int nq = (g.N + 3) / 4;
        const int m = (int)(q / nq), n = (int)(q % nq) * 4;
        float4_t s = float4_t{0.f, 0.f, 0.f, 0.f};
        for (int sp = 0; sp < nsplit; ++sp) {
            const float* p = partial + ((int64_t)sp * g.M + m) * g.N + n;
            if (n + 3 < g.N) {
                s += *reinterpret_cast<const float4_t*>(p);
            } else {
                for (int r = 0; r < 4 && n + r < g.N; ++r) s[r] += p[r];
            }
        }
        epilogue_store4<EPI>(g, g.Y, m, n, s, true);
    }
}

// ---- per-stream workspace (the counterpart of a cuBLAS handle's workspace: context.h:20-29 binds one handle per stream) ----
struct SkinnyWs { float* ptr; size_t bytes; };
static std::mutex g_ws_mu;
static std::unordered_map<void*, SkinnyWs> g_ws;

float* splitk_workspace(hipStream_t stream, size_t bytes) {
    std::lock_guard<std::mutex> lk(g_ws_mu);
    SkinnyWs& w = g_ws[(void*)stream];
    if (w.bytes < bytes) {
        // grows only; the old block is kept alive because earlier launches on this stream may still read it
        float* p = nullptr;
        size_t want = bytes < ((size_t)32 << 20) ? ((size_t)32 << 20) : bytes;
        if (hipMalloc((void**)&p, want) != hipSuccess) return nullptr;
        w.ptr = p;
        w.bytes = want;
    }
    return w.ptr;
}

void launch_splitk_reduce(const GemmArgs& g, const float* partial, int nsplit, hipStream_t stream) {
    const dim3 block(256);
    const int64_t quads = (int64_t)g.M * ((g.N + 3) / 4);
    int rgrid = (int)((quads + 255) / 256);
    if (rgrid > 4096) rgrid = 4096;
    switch (g.epi.kind) {
        case LG_EPI_NONE: hipLaunchKernelGGL((gemm_skinny_reduce_kernel<LG_EPI_NONE>), dim3(rgrid), block, 0, stream, g, partial, nsplit); break;
        case LG_EPI_BIAS: hipLaunchKernelGGL((gemm_skinny_reduce_kernel<LG_EPI_BIAS>), dim3(rgrid), block, 0, stream, g, partial, nsplit); break;
        case LG_EPI_BIAS_GELU: hipLaunchKernelGGL((gemm_skinny_reduce_kernel<LG_EPI_BIAS_GELU>), dim3(rgrid), block, 0, stream, g, partial, nsplit); break;
        default: hipLaunchKernelGGL((gemm_skinny_reduce_kernel<LG_EPI_BIAS_HEADS>), dim3(rgrid), block, 0, stream, g, partial, nsplit); break;
    }
}

int launch_gemm_skinny_f16(const GemmArgs& g, int wlayout, int batch, hipStream_t stream, bool* handled) {
    *handled = false;
    if (batch != 1 || wlayout != W_NK) return LG_OK;
    if (g.M <= 0 || g.M > 64 || g.N < 512 || g.K < 1024 || (g.K % SK_KC) || (g.N % 4)) return LG_OK;
    if (!aligned16(g.X) || !aligned16(g.W) || !aligned16(g.Y) || (g.ldx % 8) || (g.ldw % 8)) return LG_OK;
    if (g.epi.kind == LG_EPI_BIAS_HEADS ? (g.epi.d % 4 != 0) : (g.ldy % 4 != 0)) return LG_OK;
    const int nblk = (g.N + SK_BN - 1) / SK_BN;
    // K-slices: enough blocks for ~4 per CU, slices are multiples of the 256-wide chunk
    int nsplit = 1;
    while (nblk * nsplit < 1024 && (g.K / (nsplit * 2)) >= 2 * SK_KC && nsplit < 32) nsplit *= 2;
    int kslice = ((g.K + nsplit - 1) / nsplit + SK_KC - 1) / SK_KC * SK_KC;
    nsplit = (g.K + kslice - 1) / kslice;
    const size_t bytes = (size_t)nsplit * g.M * g.N * sizeof(float);
    float* ws = splitk_workspace(stream, bytes);
    if (!ws) { set_error("gemm_skinny: cannot allocate the %zu-byte split-K workspace", bytes); *handled = true; return LG_ERR_LAUNCH; }
    *handled = true;
    const dim3 grid(nblk, nsplit), block(256);
    const int mt = (g.M + 15) / 16;
    switch (mt) {
        case 1: hipLaunchKernelGGL((gemm_skinny_nk_kernel<1>), grid, block, 0, stream, g, kslice, ws, nsplit); break;
        case 2: hipLaunchKernelGGL((gemm_skinny_nk_kernel<2>), grid, block, 0, stream, g, kslice, ws, nsplit); break;
        case 3: hipLaunchKernelGGL((gemm_skinny_nk_kernel<3>), grid, block, 0, stream, g, kslice, ws, nsplit); break;
        default: hipLaunchKernelGGL((gemm_skinny_nk_kernel<4>), grid, block, 0, stream, g, kslice, ws, nsplit); break;
    }
    launch_splitk_reduce(g, ws, nsplit, stream);
    return check_launch("gemm_f16_skinny");
}

}  // namespace lg
