// gemm.hip -- hand-written GEMMs for gfx950: the cuBLAS calls of the reference's launch vector.
//
//   gemm_f16_generic   128x128x32 tiles, 4 waves (2x2), MFMA 16x16x32 f16 -> fp32, any shape / stride /
//                      alignment, both weight layouts, optional fused epilogue.  Correctness workhorse
//                      (edge tiles, decomposed sub-ranges, attention GEMMs, small models).
//   gemm_f32_mfma      128x128x16 tiles on v_mfma_f32_32x32x2_f32 for the fp32 instantiation (any shape, both layouts);
//   gemm_f32_generic   64x64x16 VALU tiles, kept as a cross-check.
// The large aligned prefill shapes are routed to the pipelined kernels in gemm_fast.hip.
#include <stdlib.h>

#include "gemm_common.hpp"

namespace lg {

int launch_gemm_fast_f16(const GemmArgs& g, const GemmGroup& grp, int wlayout, int batch, hipStream_t stream, bool* handled);
int launch_gemm_skinny_f16(const GemmArgs& g, const GemmGroup& grp, const RowMap* rows, int wlayout, int batch, hipStream_t stream, bool* handled);
int launch_gemv_f16(const GemmArgs& g, const GemmGroup& grp, const RowMap* rows, int wlayout, int batch, hipStream_t stream, bool* handled);
int launch_gemm_skinny_kn_f16(const GemmArgs& g, const RowMap* rows, int wlayout, int batch, hipStream_t stream, bool* handled);

// ---------------------------------------------------------------------------------------------------
// fp16 generic kernel
// ---------------------------------------------------------------------------------------------------
constexpr int GB_M = 128, GB_N = 128, GB_K = 32;
constexpr int GA_STRIDE = GB_K + 8;    // halves per row of the [rows][k] tiles (80 B: conflict-light b128 reads)
constexpr int GBKN_STRIDE = GB_N + 8;  // halves per row of the [k][n] tile

// loads 8 consecutive halves p[0..7] with per-element bound `valid` (0..8); ALIGNED -> one 16-byte load
template <bool ALIGNED>
__device__ __forceinline__ half8_t load8(const half_t* p, int valid) {
    half8_t r = {0, 0, 0, 0, 0, 0, 0, 0};
    if (valid <= 0) return r;
    if (ALIGNED) {
        if (valid >= 8) return *reinterpret_cast<const half8_t*>(p);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
        if (i < valid) r[i] = p[i];
    return r;
}

template <int WL, int EPI, bool ALIGNED>
__global__ __launch_bounds__(256) void gemm_f16_generic(GemmArgs g) {
    __shared__ __attribute__((aligned(16))) half_t As[GB_M * GA_STRIDE];
    __shared__ __attribute__((aligned(16))) half_t Bs[(WL == W_KN) ? GB_K * GBKN_STRIDE : GB_N * GA_STRIDE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;  // 2x2 waves, 64x64 each
    const int m0 = blockIdx.y * GB_M, n0 = blockIdx.x * GB_N;
    const half_t* X = g.X + (int64_t)blockIdx.z * g.strideX;
    const half_t* W = g.W + (int64_t)blockIdx.z * g.strideW;
    half_t* Y = g.Y + (int64_t)blockIdx.z * g.strideY;

    float4_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

    half8_t ra[2], rb[2];
    auto gload = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int v = tid + 256 * i;
            {   // X tile: 128 rows x 4 k-vectors
                const int row = v >> 2, kv = v & 3;
                const int m = m0 + row, k = k0 + kv * 8;
                ra[i] = load8<ALIGNED>(X + (int64_t)m * g.ldx + k, (m < g.M) ? (g.K - k) : 0);
            }
            if (WL == W_TILED) {  // W tile: 8 fragment blocks (16 features x 32 k each), one lane's 16 bytes per thread
                const int blk = v >> 6, ln = v & 63;
                const int n = n0 + blk * 16;   // N % 16 == 0 and K % 32 == 0: a block is there as a whole or not at all
                rb[i] = load8<true>(W + ((int64_t)(n >> 4) * (g.K >> 5) + (k0 >> 5)) * 512 + ln * 8, (n < g.N) ? 8 : 0);
            } else if (WL == W_NK) {  // W tile: 128 n-rows x 4 k-vectors
                const int row = v >> 2, kv = v & 3;
                const int n = n0 + row, k = k0 + kv * 8;
                rb[i] = load8<ALIGNED>(W + (int64_t)n * g.ldw + k, (n < g.N) ? (g.K - k) : 0);
            } else {           // W tile: 32 k-rows x 16 n-vectors
                const int row = v >> 4, nv = v & 15;
                const int k = k0 + row, n = n0 + nv * 8;
                rb[i] = load8<ALIGNED>(W + (int64_t)k * g.ldw + n, (k < g.K) ? (g.N - n) : 0);
            }
        }
    };
    auto lstore = [&]() {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int v = tid + 256 * i;
            *reinterpret_cast<half8_t*>(&As[(v >> 2) * GA_STRIDE + (v & 3) * 8]) = ra[i];
            if (WL == W_TILED)
                *reinterpret_cast<half8_t*>(&Bs[v * 8]) = rb[i];   // block v / 64 keeps its register order
            else if (WL == W_NK)
                *reinterpret_cast<half8_t*>(&Bs[(v >> 2) * GA_STRIDE + (v & 3) * 8]) = rb[i];
            else
                *reinterpret_cast<half8_t*>(&Bs[(v >> 4) * GBKN_STRIDE + (v & 15) * 8]) = rb[i];
        }
    };

    const int l16 = lane & 15, lk = lane >> 4;  // row inside a 16-row MFMA tile, k-chunk (8 halves) index
    gload(0);
    for (int k0 = 0; k0 < g.K; k0 += GB_K) {
        __syncthreads();  // previous tile fully consumed
        lstore();
        __syncthreads();
        if (k0 + GB_K < g.K) gload(k0 + GB_K);

        half8_t a[4], b[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            a[i] = *reinterpret_cast<const half8_t*>(&As[(wm * 64 + i * 16 + l16) * GA_STRIDE + lk * 8]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (WL == W_TILED) {
                b[j] = *reinterpret_cast<const half8_t*>(&Bs[((wn * 4 + j) * 64 + lane) * 8]);
            } else if (WL == W_NK) {
                b[j] = *reinterpret_cast<const half8_t*>(&Bs[(wn * 64 + j * 16 + l16) * GA_STRIDE + lk * 8]);
            } else {
                const int col = wn * 64 + j * 16 + 4 * (l16 & 3);
                const int krow = lk * 8 + (l16 >> 2);
                half4_t lo = lds_read_tr4(&Bs[krow * GBKN_STRIDE + col]);
                half4_t hi = lds_read_tr4(&Bs[(krow + 4) * GBKN_STRIDE + col]);
                b[j] = half8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
        }
        // operands swapped so that each lane owns 4 consecutive output columns (n) of one row (m):
        //   acc[i][j][r] = Y[m_tile(i) + lane%16][n_tile(j) + 4*(lane/16) + r]
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = mfma16(b[j], a[i], acc[i][j]);
    }

    const bool vec_ok = ALIGNED && (EPI == LG_EPI_BIAS_HEADS ? (g.epi.d % 4 == 0) : (g.ldy % 4 == 0));
    if (EPI == LG_EPI_BIAS_GEGLU) {
        // a wave's four 16-feature tiles are two (gate, up) pairs (N % 32 == 0, tiles start at multiples of 64)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; j += 2)
                epilogue_geglu4(g, Y, m0 + wm * 64 + i * 16 + l16, n0 + wn * 64 + j * 16 + 4 * lk, acc[i][j], acc[i][j + 1], vec_ok);
        return;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = m0 + wm * 64 + i * 16 + l16;
            const int n = n0 + wn * 64 + j * 16 + 4 * lk;
            switch (EPI) {
                case LG_EPI_NONE: epilogue_store4<LG_EPI_NONE>(g, Y, m, n, acc[i][j], vec_ok); break;
                case LG_EPI_BIAS: epilogue_store4<LG_EPI_BIAS>(g, Y, m, n, acc[i][j], vec_ok); break;
                case LG_EPI_BIAS_GELU: epilogue_store4<LG_EPI_BIAS_GELU>(g, Y, m, n, acc[i][j], vec_ok); break;
                default: epilogue_store4<LG_EPI_BIAS_HEADS>(g, Y, m, n, acc[i][j], vec_ok); break;
            }
        }
}

template <int WL, bool ALIGNED>
static void launch_generic_epi(const GemmArgs& g, dim3 grid, hipStream_t stream) {
    switch (g.epi.kind) {
        case LG_EPI_NONE: hipLaunchKernelGGL((gemm_f16_generic<WL, LG_EPI_NONE, ALIGNED>), grid, dim3(256), 0, stream, g); break;
        case LG_EPI_BIAS: hipLaunchKernelGGL((gemm_f16_generic<WL, LG_EPI_BIAS, ALIGNED>), grid, dim3(256), 0, stream, g); break;
        case LG_EPI_BIAS_GELU: hipLaunchKernelGGL((gemm_f16_generic<WL, LG_EPI_BIAS_GELU, ALIGNED>), grid, dim3(256), 0, stream, g); break;
        case LG_EPI_BIAS_GEGLU: hipLaunchKernelGGL((gemm_f16_generic<WL, LG_EPI_BIAS_GEGLU, ALIGNED>), grid, dim3(256), 0, stream, g); break;
        default: hipLaunchKernelGGL((gemm_f16_generic<WL, LG_EPI_BIAS_HEADS, ALIGNED>), grid, dim3(256), 0, stream, g); break;
    }
}

static int gemm_f16_dispatch(GemmArgs g, int wlayout, int batch, hipStream_t stream) {
    if (g.M == 0 || g.N == 0 || batch == 0) return LG_OK;
    if (g.K == 0) { set_error("gemm: k == 0 is not supported"); return LG_ERR_INVALID; }
    bool handled = false;
    const GemmGroup one = single_group(g);
    int rc = launch_gemm_fast_f16(g, one, wlayout, batch, stream, &handled);
    if (handled) return rc;
    rc = launch_gemv_f16(g, one, nullptr, wlayout, batch, stream, &handled);
    if (handled) return rc;
    rc = launch_gemm_skinny_f16(g, one, nullptr, wlayout, batch, stream, &handled);
    if (handled) return rc;
    rc = launch_gemm_skinny_kn_f16(g, nullptr, wlayout, batch, stream, &handled);
    if (handled) return rc;
    const bool aligned = aligned16(g.X) && aligned16(g.W) && aligned16(g.Y) && (g.ldx % 8 == 0) && (g.ldw % 8 == 0) &&
                         (g.strideX % 8 == 0) && (g.strideW % 8 == 0) && (g.strideY % 4 == 0) &&
                         (g.K % 8 == 0) && (wlayout == W_NK || g.N % 8 == 0) &&
                         (g.epi.kind == LG_EPI_BIAS_HEADS || (((uintptr_t)g.Y & 7u) == 0));
    dim3 grid((g.N + GB_N - 1) / GB_N, (g.M + GB_M - 1) / GB_M, batch);
    if (grid.y > 65535 || grid.z > 65535) { set_error("gemm: problem too large for the generic grid"); return LG_ERR_INVALID; }
    if (wlayout == W_TILED) {
        if (aligned) launch_generic_epi<W_TILED, true>(g, grid, stream); else launch_generic_epi<W_TILED, false>(g, grid, stream);
    } else if (wlayout == W_NK) {
        if (aligned) launch_generic_epi<W_NK, true>(g, grid, stream); else launch_generic_epi<W_NK, false>(g, grid, stream);
    } else {
        if (aligned) launch_generic_epi<W_KN, true>(g, grid, stream); else launch_generic_epi<W_KN, false>(g, grid, stream);
    }
    return check_launch("gemm_f16");
}

// ---------------------------------------------------------------------------------------------------
// fp32 generic kernel (plumbing configuration): 64x64x16 tiles, 256 threads, 4x4 outputs per thread
// ---------------------------------------------------------------------------------------------------
struct GemmArgsF32 {
    int M, N, K;
    const float* X; int64_t ldx; int64_t strideX;
    const float* W; int64_t ldw; int64_t strideW;
    float* Y;       int64_t ldy; int64_t strideY;
};

template <int WL>
__global__ __launch_bounds__(256) void gemm_f32_generic(GemmArgsF32 g) {
    __shared__ float As[16][64 + 4];  // [k][m]
    __shared__ float Bs[16][64 + 4];  // [k][n]
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;  // 16x16 threads, 4x4 outputs each
    const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
    const float* X = g.X + (int64_t)blockIdx.z * g.strideX;
    const float* W = g.W + (int64_t)blockIdx.z * g.strideW;
    float* Y = g.Y + (int64_t)blockIdx.z * g.strideY;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < g.K; k0 += 16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid + 256 * i;  // 1024 elements per tile
            {
                const int r = e >> 4, kk = e & 15;  // X: 64 rows x 16 k, k fastest
                const int m = m0 + r, k = k0 + kk;
                As[kk][r] = (m < g.M && k < g.K) ? X[(int64_t)m * g.ldx + k] : 0.f;
            }
            if (WL == W_NK) {
                const int r = e >> 4, kk = e & 15;
                const int n = n0 + r, k = k0 + kk;
                Bs[kk][r] = (n < g.N && k < g.K) ? W[(int64_t)n * g.ldw + k] : 0.f;
            } else {
                const int kk = e >> 6, c = e & 63;  // W: 16 k x 64 n, n fastest
                const int n = n0 + c, k = k0 + kk;
                Bs[kk][c] = (n < g.N && k < g.K) ? W[(int64_t)k * g.ldw + n] : 0.f;
            }
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
            if (m < g.M && n < g.N) Y[(int64_t)m * g.ldy + n] = acc[i][j];
        }
}

// ---------------------------------------------------------------------------------------------------
// fp32 on the matrix cores: 128 x 128 x 16 tiles, 4 waves (2 x 2), v_mfma_f32_32x32x2_f32
// ---------------------------------------------------------------------------------------------------
// The reference instantiates every layer for float through cublasGemmEx(..., CUDA_R_32F, ...) (context.h:49-55,
// linear.h:47-49,99-101).  A wave owns 64 x 64 outputs = 2 x 2 MFMA tiles (64 accumulator registers); operands are swapped as
// in the fp16 kernels (the weight tile is the A operand), so a lane ends up with 4 consecutive output features of one token
// row: acc[i][j][v] = Y[token 32 i + lane % 32][feature 32 j + 8 (v / 4) + 4 (lane / 32) + v % 4].  Both tiles sit in LDS
// k-major ([16][128 + 32] floats): a wave-wide operand read is two runs of 32 consecutive floats, 32 banks apart.
typedef float float16v_t __attribute__((ext_vector_type(16)));
constexpr int SB_M = 128, SB_N = 128, SB_K = 16, SB_PITCH = 128 + 32;

template <int WL, bool ALIGNED>
__global__ __launch_bounds__(256) void gemm_f32_mfma(GemmArgsF32 g) {
    __shared__ __attribute__((aligned(16))) float Xs[SB_K * SB_PITCH];
    __shared__ __attribute__((aligned(16))) float Ws[SB_K * SB_PITCH];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * SB_M, n0 = blockIdx.x * SB_N;
    const float* X = g.X + (int64_t)blockIdx.z * g.strideX;
    const float* W = g.W + (int64_t)blockIdx.z * g.strideW;
    float* Y = g.Y + (int64_t)blockIdx.z * g.strideY;

    float16v_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // 8 consecutive floats p[0..7] with `valid` of them inside the matrix
    auto load8f = [](const float* p, int valid, float (&r)[8]) {
        if (ALIGNED && valid >= 8) {
            const float4_t a = *reinterpret_cast<const float4_t*>(p), b = *reinterpret_cast<const float4_t*>(p + 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) { r[i] = a[i]; r[4 + i] = b[i]; }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) r[i] = i < valid ? p[i] : 0.f;
        }
    };
    float rx[8], rw[8];
    auto gload = [&](int k0) {
        {   // X tile: 128 token rows x 16 k; thread = (row, half of the k range)
            const int row = tid >> 1, kh = (tid & 1) * 8;
            const int m = m0 + row, k = k0 + kh;
            load8f(X + (int64_t)m * g.ldx + k, m < g.M ? g.K - k : 0, rx);
        }
        if (WL == W_NK) {
            const int row = tid >> 1, kh = (tid & 1) * 8;
            const int n = n0 + row, k = k0 + kh;
            load8f(W + (int64_t)n * g.ldw + k, n < g.N ? g.K - k : 0, rw);
        } else {  // [K, N]: 16 k-rows x 128 features; thread = (k, 8 consecutive features)
            const int kr = tid >> 4, ns = (tid & 15) * 8;
            const int k = k0 + kr, n = n0 + ns;
            load8f(W + (int64_t)k * g.ldw + n, k < g.K ? g.N - n : 0, rw);
        }
    };
    auto lstore = [&]() {
        {
            const int row = tid >> 1, kh = (tid & 1) * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) Xs[(kh + i) * SB_PITCH + row] = rx[i];
        }
        if (WL == W_NK) {
            const int row = tid >> 1, kh = (tid & 1) * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) Ws[(kh + i) * SB_PITCH + row] = rw[i];
        } else {
            const int kr = tid >> 4, ns = (tid & 15) * 8;
            *reinterpret_cast<float4_t*>(&Ws[kr * SB_PITCH + ns]) = float4_t{rw[0], rw[1], rw[2], rw[3]};
            *reinterpret_cast<float4_t*>(&Ws[kr * SB_PITCH + ns + 4]) = float4_t{rw[4], rw[5], rw[6], rw[7]};
        }
    };

    const int l32 = lane & 31, lh = lane >> 5;
    gload(0);
    for (int k0 = 0; k0 < g.K; k0 += SB_K) {
        __syncthreads();
        lstore();
        __syncthreads();
        if (k0 + SB_K < g.K) gload(k0 + SB_K);
#pragma unroll
        for (int ks = 0; ks < SB_K / 2; ++ks) {
            float a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) a[i] = Xs[(ks * 2 + lh) * SB_PITCH + wm * 64 + i * 32 + l32];
#pragma unroll
            for (int j = 0; j < 2; ++j) b[j] = Ws[(ks * 2 + lh) * SB_PITCH + wn * 64 + j * 32 + l32];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[j], a[i], acc[i][j], 0, 0, 0);
        }
    }
    const bool vec_ok = ALIGNED && (g.ldy % 4 == 0);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int m = m0 + wm * 64 + i * 32 + l32;
        if (m >= g.M) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = n0 + wn * 64 + j * 32 + 8 * q + 4 * lh;
                float* p = Y + (int64_t)m * g.ldy + n;
                if (vec_ok && n + 3 < g.N) {
                    *reinterpret_cast<float4_t*>(p) = float4_t{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (n + r < g.N) p[r] = acc[i][j][4 * q + r];
                }
            }
    }
}

static int gemm_f32_dispatch(const GemmArgsF32& g, int wlayout, int batch, hipStream_t stream) {
    if (g.M == 0 || g.N == 0 || batch == 0) return LG_OK;
    if (g.K == 0) { set_error("gemm: k == 0 is not supported"); return LG_ERR_INVALID; }
    // LG_GEMM_F32_VALU=1 in the environment (read once) selects the vector-ALU tile kernel instead: a cross-check for tests
    static const bool valu = [] { const char* e = getenv("LG_GEMM_F32_VALU"); return e && atoi(e) != 0; }();
    if (!valu) {
        dim3 grid((g.N + SB_N - 1) / SB_N, (g.M + SB_M - 1) / SB_M, batch);
        if (grid.y > 65535 || grid.z > 65535) { set_error("gemm: problem too large for the grid"); return LG_ERR_INVALID; }
        const bool aligned = aligned16(g.X) && aligned16(g.W) && aligned16(g.Y) && (g.ldx % 4 == 0) && (g.ldw % 4 == 0) &&
                             (g.strideX % 4 == 0) && (g.strideW % 4 == 0) && (g.strideY % 4 == 0);
        if (wlayout == W_NK) {
            if (aligned) hipLaunchKernelGGL((gemm_f32_mfma<W_NK, true>), grid, dim3(256), 0, stream, g);
            else hipLaunchKernelGGL((gemm_f32_mfma<W_NK, false>), grid, dim3(256), 0, stream, g);
        } else {
            if (aligned) hipLaunchKernelGGL((gemm_f32_mfma<W_KN, true>), grid, dim3(256), 0, stream, g);
            else hipLaunchKernelGGL((gemm_f32_mfma<W_KN, false>), grid, dim3(256), 0, stream, g);
        }
        return check_launch("gemm_f32");
    }
    dim3 grid((g.N + 63) / 64, (g.M + 63) / 64, batch);
    if (grid.y > 65535 || grid.z > 65535) { set_error("gemm: problem too large for the generic grid"); return LG_ERR_INVALID; }
    if (wlayout == W_NK) hipLaunchKernelGGL((gemm_f32_generic<W_NK>), grid, dim3(256), 0, stream, g);
    else hipLaunchKernelGGL((gemm_f32_generic<W_KN>), grid, dim3(256), 0, stream, g);
    return check_launch("gemm_f32");
}

// cuBLAS column-major arguments -> row-major problem; returns LG_OK or sets the error text
static int check_blas_args(const char* what, int transa, int transb, int m, int n, int k, const void* A, int lda,
                           const void* B, int ldb, const void* C, int ldc, int batch) {
    if (transb != 0 || (transa != 0 && transa != 1 && transa != LG_OP_TILED)) { set_error("%s: only (N,N), (T,N) and (tiled,N) are supported", what); return LG_ERR_INVALID; }
    if (m < 0 || n < 0 || k < 0 || batch < 0) { set_error("%s: negative dimension", what); return LG_ERR_INVALID; }
    if (m == 0 || n == 0 || batch == 0) return LG_OK;
    if (!A || !B || !C) { set_error("%s: null pointer", what); return LG_ERR_INVALID; }
    if (transa == LG_OP_TILED && (m % 16 != 0 || k % 32 != 0 || lda != k || batch > 1 || ((uintptr_t)A & 15u))) {
        set_error("%s: tiled weights need features %% 16 == 0, k %% 32 == 0, lda == k, a 16-byte aligned pointer and no batch (m=%d k=%d lda=%d)", what, m, k, lda);
        return LG_ERR_INVALID;
    }
    const int min_lda = transa ? k : m;
    if (lda < (min_lda > 1 ? min_lda : 1) || ldb < (k > 1 ? k : 1) || ldc < (m > 1 ? m : 1)) {
        set_error("%s: leading dimension too small (lda=%d ldb=%d ldc=%d for m=%d n=%d k=%d)", what, lda, ldb, ldc, m, n, k);
        return LG_ERR_INVALID;
    }
    return LG_OK;
}

}  // namespace lg

using namespace lg;

extern "C" {

int lg_gemm_strided_batched_f16(int transa, int transb, int m, int n, int k, const void* A, int lda, int64_t strideA,
                                const void* B, int ldb, int64_t strideB, void* C, int ldc, int64_t strideC, int batch,
                                void* stream) {
    int rc = check_blas_args("gemm_f16", transa, transb, m, n, k, A, lda, B, ldb, C, ldc, batch);
    if (rc) return rc;
    GemmArgs g;
    g.M = n; g.N = m; g.K = k;
    g.X = (const half_t*)B; g.ldx = ldb; g.strideX = strideB;
    g.W = (const half_t*)A; g.ldw = lda; g.strideW = strideA;
    g.Y = (half_t*)C; g.ldy = ldc; g.strideY = strideC;
    g.epi = Epilogue{LG_EPI_NONE, nullptr, 0, 0, 0, 0};
    return gemm_f16_dispatch(g, transa == LG_OP_TILED ? W_TILED : (transa ? W_NK : W_KN), batch, (hipStream_t)stream);
}

int lg_gemm_f16(int transa, int transb, int m, int n, int k, const void* A, int lda, const void* B, int ldb, void* C,
                int ldc, void* stream) {
    return lg_gemm_strided_batched_f16(transa, transb, m, n, k, A, lda, 0, B, ldb, 0, C, ldc, 0, 1, stream);
}

int lg_gemm_fused_f16(int transa, int m, int n, int k, const void* A, int lda, const void* B, int ldb, void* C, int ldc,
                      int epilogue, const void* bias, int epi_arg0, int epi_arg1, int epi_arg2, void* stream) {
    int rc = check_blas_args("gemm_fused_f16", transa, 0, m, n, k, A, lda, B, ldb, C,
                             epilogue == LG_EPI_BIAS_HEADS ? (m > 1 ? m : 1) : (epilogue == LG_EPI_BIAS_GEGLU ? (ldc < m / 2 ? 0 : m) : ldc), 1);
    if (rc) return rc;
    if (epilogue != LG_EPI_BIAS_GEGLU && (epilogue < LG_EPI_NONE || epilogue > LG_EPI_BIAS_HEADS)) { set_error("gemm_fused_f16: unknown epilogue %d", epilogue); return LG_ERR_INVALID; }
    if (epilogue != LG_EPI_NONE && !bias) { set_error("gemm_fused_f16: epilogue needs a bias"); return LG_ERR_INVALID; }
    if (epilogue == LG_EPI_BIAS_GEGLU && m % 32 != 0) { set_error("gemm_fused_f16: the GeGLU epilogue needs features %% 32 == 0 (gate and up interleaved in groups of 16)"); return LG_ERR_INVALID; }
    if (epilogue == LG_EPI_BIAS_HEADS) {
        const int seq = epi_arg0, d = epi_arg1;
        if (seq <= 0 || d <= 0 || m % d != 0 || n % seq != 0 || d % 4 != 0 || ldc < seq ||
            (epi_arg2 != 0 && epi_arg2 < m / d)) {
            set_error("gemm_fused_f16: heads epilogue needs seq | tokens, size_per_head | features, size_per_head %% 4 == 0, "
                      "ldc (rows per head slot) >= seq, heads_total >= features / size_per_head");
            return LG_ERR_INVALID;
        }
        if (epi_arg2 == 0) epi_arg2 = m / d;
    }
    GemmArgs g;
    g.M = n; g.N = m; g.K = k;
    g.X = (const half_t*)B; g.ldx = ldb; g.strideX = 0;
    g.W = (const half_t*)A; g.ldw = lda; g.strideW = 0;
    g.Y = (half_t*)C; g.ldy = ldc; g.strideY = 0;
    g.epi = Epilogue{epilogue, (const half_t*)bias, epi_arg0, epi_arg1, epi_arg2, 0};
    return gemm_f16_dispatch(g, transa == LG_OP_TILED ? W_TILED : (transa ? W_NK : W_KN), 1, (hipStream_t)stream);
}

// mode: -1 = choose the plan, 1 = one launch if the kernels allow it (a sub-group of a plan), 0 = member by member
static int gemm_fused_grouped_f16_impl(int mode, int transa, int m, int n, int k, int count, const void* const* A, int lda, const void* B, int ldb,
                                       void* const* C, const int* ldc, int epilogue, const void* const* bias, int epi_arg0, int epi_arg1,
                                       int epi_arg2, void* stream) {
    if (count < 1 || count > LG_MAX_GROUP || !A || !C || !ldc || (epilogue != LG_EPI_NONE && !bias)) {
        set_error("gemm_fused_grouped_f16: count must be 1..%d and the pointer arrays non-null", LG_MAX_GROUP);
        return LG_ERR_INVALID;
    }
    // the pipelined kernel (many token rows, either weight layout) and the weight-streaming kernels (few token rows, weights
    // [out, in]) run the whole group as one launch; every other case is `count` plain calls
    GemmGroup grp{};
    grp.count = count;
    bool one_launch = m > 0 && n > 0 && k > 0 && count > 1 && B != nullptr;
    for (int i = 0; i < count; ++i) {
        grp.W[i] = (const half_t*)A[i];
        grp.Y[i] = (half_t*)C[i];
        grp.bias[i] = epilogue != LG_EPI_NONE ? (const half_t*)bias[i] : nullptr;
        grp.ldy[i] = ldc[i];
        if (!A[i] || !C[i] || (epilogue != LG_EPI_NONE && !bias[i])) one_launch = false;  // the plain call reports it
    }
    if (one_launch && n > 256) {
        // Many token rows (the pipelined kernel's regime): one launch or member by member?  The members' tiles side by side may
        // fill a round of workgroups that one member alone leaves half empty (384-768 token rows x 6144 features: one launch is
        // 7-13 % faster per layer), or they may end in a mostly empty last round that three launches with a narrower tile avoid
        // (1024 rows: 6 % slower).  What decides is rounds of workgroups x tile width for the best width either way, the
        // quantity the pipelined kernel's launcher minimises; ties go to separate launches.  Both ways give the same bits.
        const int cus = stream_info((hipStream_t)stream).cus;
        const int tiles_m = (n + 255) / 256;
        auto round_widths = [&](int members) {
            long best = -1;
            for (int nj = 4; nj >= 2; --nj) {
                if (m % (64 * nj)) continue;
                const long tiles = (long)tiles_m * (m / (64 * nj)) * members;
                const long u = ((tiles + cus - 1) / cus) * nj;
                if (best < 0 || u < best) best = u;
            }
            return best;
        };
        const long together = round_widths(count), apart = round_widths(1);
        if (together > 0 && apart > 0 && together >= (long)count * apart) one_launch = false;
        // A third plan for groups that are many full rounds plus a remainder (Q, K, V of 4096 rows x 6144 features: 72 columns
        // of 256-wide tiles, 16 columns to a round of 256 workgroups, 8 left over): the members before the last as one launch
        // of whole rounds of the widest tile, the last member's leading features as whole rounds too, and its remaining features
        // as one round of 128-wide tiles -- instead of six rounds of 192-wide tiles either way (4.6-6.6 % faster, measured).
        // Only taken when every launch but the last is whole rounds; pieces are addressed like any feature sub-range.
        int split_at = 0;   // feature at which the last member is cut (0: no such plan)
        const bool range_ok = epilogue == LG_EPI_NONE || epilogue == LG_EPI_BIAS || epilogue == LG_EPI_BIAS_GELU ||
                              (epilogue == LG_EPI_BIAS_HEADS && epi_arg1 > 0 && 256 % epi_arg1 == 0);
        if (mode < 0 && range_ok && m % 256 == 0 && cus % tiles_m == 0 && (transa != LG_OP_TILED || lda == k)) {
            const int cols = m / 256, per_round = cus / tiles_m, rem = (count * cols) % per_round;
            if (rem > 0 && rem < cols && ((count - 1) * cols) % per_round == 0 && (cols - rem) % per_round == 0 && 2 * rem * tiles_m <= cus)
                split_at = (cols - rem) * 256;
        }
        // LG_GEMM_GROUP=1|0 in the environment (read once) forces one launch / member by member: a measurement knob
        static const int forced = [] { const char* e = getenv("LG_GEMM_GROUP"); return e ? atoi(e) : -1; }();
        if (forced == 0) { one_launch = false; split_at = 0; }
        else if (forced == 1) { one_launch = true; split_at = 0; }
        if (mode == 0) one_launch = false;
        else if (mode == 1) one_launch = true;
        if (split_at > 0) {
            int rc = count - 1 > 1 ? gemm_fused_grouped_f16_impl(1, transa, m, n, k, count - 1, A, lda, B, ldb, C, ldc, epilogue, bias, epi_arg0, epi_arg1,
                                                                 epilogue == LG_EPI_BIAS_HEADS && epi_arg2 == 0 ? m / epi_arg1 : epi_arg2, stream)
                                   : lg_gemm_fused_f16(transa, m, n, k, A[0], lda, B, ldb, C[0], ldc[0], epilogue, epilogue != LG_EPI_NONE ? bias[0] : nullptr,
                                                       epi_arg0, epi_arg1, epi_arg2, stream);
            if (rc) return rc;
            const int last = count - 1;
            const int heads_total = epilogue == LG_EPI_BIAS_HEADS ? (epi_arg2 ? epi_arg2 : m / epi_arg1) : epi_arg2;
            const int cut[3] = {0, split_at, m};
            for (int piece = 0; piece < 2; ++piece) {
                const int f0 = cut[piece], f1 = cut[piece + 1];
                // features [f0, f1) of the last member: rows f0.. of an [out, in] weight (row-major or in fragment blocks, where
                // feature tile t starts 16 t k elements in), columns f0.. of an [in, out] one; heads f0 / d .. of a
                // head-transposed destination, columns f0.. of a plain one
                const int64_t w_off = transa == 0 ? (int64_t)f0 : (int64_t)f0 * (transa == LG_OP_TILED ? k : lda);
                const int64_t c_off = epilogue == LG_EPI_BIAS_HEADS ? (int64_t)(f0 / epi_arg1) * ldc[last] * epi_arg1 : (int64_t)f0;
                rc = lg_gemm_fused_f16(transa, f1 - f0, n, k, (const half_t*)A[last] + w_off, lda, B, ldb, (half_t*)C[last] + c_off, ldc[last], epilogue,
                                       epilogue != LG_EPI_NONE ? (const void*)((const half_t*)bias[last] + f0) : nullptr, epi_arg0, epi_arg1, heads_total, stream);
                if (rc) return rc;
            }
            return LG_OK;
        }
    }
    if (one_launch) {
        // same argument checks as the plain entry, member by member, before anything is launched
        for (int i = 0; i < count; ++i) {
            int rc = check_blas_args("gemm_fused_grouped_f16", transa, 0, m, n, k, A[i], lda, B, ldb, C[i],
                                     epilogue == LG_EPI_BIAS_HEADS ? (m > 1 ? m : 1) : ldc[i], 1);
            if (rc) return rc;
        }
        if (epilogue < LG_EPI_NONE || epilogue > LG_EPI_BIAS_HEADS) { set_error("gemm_fused_grouped_f16: unknown epilogue %d", epilogue); return LG_ERR_INVALID; }
        int heads_total = epi_arg2;
        bool ok = true;
        if (epilogue == LG_EPI_BIAS_HEADS) {
            const int seq = epi_arg0, d = epi_arg1;
            ok = seq > 0 && d > 0 && m % d == 0 && n % seq == 0 && d % 4 == 0 && (epi_arg2 == 0 || epi_arg2 >= m / d);
            for (int i = 0; i < count && ok; ++i) ok = ldc[i] >= seq;
            if (ok && heads_total == 0) heads_total = m / d;
        }
        if (ok) {
            GemmArgs g;
            g.M = n; g.N = m; g.K = k;
            g.X = (const half_t*)B; g.ldx = ldb; g.strideX = 0;
            g.W = grp.W[0]; g.ldw = lda; g.strideW = 0;
            g.Y = grp.Y[0]; g.ldy = grp.ldy[0]; g.strideY = 0;
            g.epi = Epilogue{epilogue, grp.bias[0], epi_arg0, epi_arg1, heads_total, 0};
            bool handled = false;
            const int wl = transa == LG_OP_TILED ? W_TILED : (transa ? W_NK : W_KN);
            int rc = launch_gemm_fast_f16(g, grp, wl, 1, (hipStream_t)stream, &handled);
            if (handled) return rc;
            if (transa != 0) {
                rc = launch_gemv_f16(g, grp, nullptr, wl, 1, (hipStream_t)stream, &handled);
                if (handled) return rc;
                rc = launch_gemm_skinny_f16(g, grp, nullptr, wl, 1, (hipStream_t)stream, &handled);
                if (handled) return rc;
            }
        }
    }
    for (int i = 0; i < count; ++i) {
        int rc = lg_gemm_fused_f16(transa, m, n, k, A[i], lda, B, ldb, C[i], ldc[i], epilogue, epilogue != LG_EPI_NONE ? bias[i] : nullptr,
                                   epi_arg0, epi_arg1, epi_arg2, stream);
        if (rc) return rc;
    }
    return LG_OK;
}

int lg_gemm_fused_grouped_f16(int transa, int m, int n, int k, int count, const void* const* A, int lda, const void* B, int ldb,
                              void* const* C, const int* ldc, int epilogue, const void* const* bias, int epi_arg0, int epi_arg1,
                              int epi_arg2, void* stream) {
    return gemm_fused_grouped_f16_impl(-1, transa, m, n, k, count, A, lda, B, ldb, C, ldc, epilogue, bias, epi_arg0, epi_arg1, epi_arg2, stream);
}

int lg_gemm_fused_grouped_rows_f16(int transa, int m, int n, int k, int count, const void* const* A, int lda, const void* B, int ldb,
                                   void* const* C, const int* ldc, const void* const* bias, int size_per_head, int heads_total,
                                   const int* use_rows, const int* slot, const int* pos, void* stream) {
    const int d = size_per_head;
    if (count < 1 || count > LG_MAX_GROUP || !A || !C || !ldc || !bias || !use_rows) {
        set_error("gemm_fused_grouped_rows_f16: count must be 1..%d and the pointer arrays non-null", LG_MAX_GROUP);
        return LG_ERR_INVALID;
    }
    if (m < 0 || n < 0 || k < 0 || n > LG_ROWMAP_MAX) { set_error("gemm_fused_grouped_rows_f16: at most %d token rows (n = %d)", LG_ROWMAP_MAX, n); return LG_ERR_INVALID; }
    if (m == 0 || n == 0) return LG_OK;
    if (d <= 0 || m % d != 0 || d % 4 != 0 || heads_total < m / d) {
        set_error("gemm_fused_grouped_rows_f16: size_per_head must divide the features and be a multiple of 4, heads_total >= features / size_per_head");
        return LG_ERR_INVALID;
    }
    bool any_rows = false;
    for (int i = 0; i < count; ++i) any_rows = any_rows || use_rows[i] != 0;
    if (any_rows && (!slot || !pos)) { set_error("gemm_fused_grouped_rows_f16: null slot / pos array"); return LG_ERR_INVALID; }
    RowMap rm{};
    for (int r = 0; r < n && any_rows; ++r) {
        if (slot[r] < 0 || pos[r] < 0) { set_error("gemm_fused_grouped_rows_f16: token row %d: slot %d, pos %d", r, slot[r], pos[r]); return LG_ERR_INVALID; }
        rm.slot[r] = slot[r];
        rm.pos[r] = pos[r];
    }
    GemmGroup grp{};
    grp.count = count;
    for (int i = 0; i < count; ++i) {
        int rc = check_blas_args("gemm_fused_grouped_rows_f16", transa, 0, m, n, k, A[i], lda, B, ldb, C[i], m > 1 ? m : 1, 1);
        if (rc) return rc;
        if (!bias[i]) { set_error("gemm_fused_grouped_rows_f16: null bias"); return LG_ERR_INVALID; }
        if (ldc[i] < 1) { set_error("gemm_fused_grouped_rows_f16: ldc (rows per head slot) must be >= 1"); return LG_ERR_INVALID; }
        for (int r = 0; r < n && use_rows[i]; ++r)
            if (pos[r] >= ldc[i]) { set_error("gemm_fused_grouped_rows_f16: token row %d: pos %d outside the %d rows of a head slot", r, pos[r], ldc[i]); return LG_ERR_INVALID; }
        grp.W[i] = (const half_t*)A[i];
        grp.Y[i] = (half_t*)C[i];
        grp.bias[i] = (const half_t*)bias[i];
        grp.ldy[i] = ldc[i];
        grp.rows[i] = use_rows[i] ? 1 : 0;
    }
    if (transa != 0) {
        GemmArgs g;
        g.M = n; g.N = m; g.K = k;
        g.X = (const half_t*)B; g.ldx = ldb; g.strideX = 0;
        g.W = grp.W[0]; g.ldw = lda; g.strideW = 0;
        g.Y = grp.Y[0]; g.ldy = grp.ldy[0]; g.strideY = 0;
        g.epi = Epilogue{LG_EPI_BIAS_HEADS_ROWS, grp.bias[0], 1, d, heads_total, grp.rows[0]};
        const int wl = transa == LG_OP_TILED ? W_TILED : W_NK;
        bool handled = false;
        int rc = launch_gemv_f16(g, grp, &rm, wl, 1, (hipStream_t)stream, &handled);
        if (handled) return rc;
        rc = launch_gemm_skinny_f16(g, grp, &rm, wl, 1, (hipStream_t)stream, &handled);
        if (handled) return rc;
    }
    if (transa == 0) {
        // weights stored [in, out]: one launch of the LDS-transposing weight-streaming kernel per member
        bool all = true;
        for (int i = 0; i < count && all; ++i) {
            GemmArgs g;
            g.M = n; g.N = m; g.K = k;
            g.X = (const half_t*)B; g.ldx = ldb; g.strideX = 0;
            g.W = grp.W[i]; g.ldw = lda; g.strideW = 0;
            g.Y = grp.Y[i]; g.ldy = grp.ldy[i]; g.strideY = 0;
            g.epi = Epilogue{LG_EPI_BIAS_HEADS_ROWS, grp.bias[i], 1, d, heads_total, grp.rows[i]};
            bool handled = false;
            int rc = launch_gemm_skinny_kn_f16(g, &rm, W_KN, 1, (hipStream_t)stream, &handled);
            if (rc) return rc;
            all = handled;
            if (!handled && i > 0) { set_error("gemm_fused_grouped_rows_f16: members of one group must take the same kernel"); return LG_ERR_INVALID; }
        }
        if (all) return LG_OK;
    }
    // anything the weight-streaming kernels do not take: plain calls, one per member -- and one per token row for a member
    // whose rows go to their own places
    for (int i = 0; i < count; ++i) {
        if (!use_rows[i]) {
            int rc = lg_gemm_fused_f16(transa, m, n, k, A[i], lda, B, ldb, C[i], ldc[i], LG_EPI_BIAS_HEADS, bias[i], 1, d, heads_total, stream);
            if (rc) return rc;
            continue;
        }
        for (int r = 0; r < n; ++r) {
            half_t* dst = (half_t*)C[i] + ((int64_t)slot[r] * heads_total * ldc[i] + pos[r]) * d;
            int rc = lg_gemm_fused_f16(transa, m, 1, k, A[i], lda, (const half_t*)B + (int64_t)r * ldb, ldb, dst, ldc[i], LG_EPI_BIAS_HEADS,
                                       bias[i], 1, d, heads_total, stream);
            if (rc) return rc;
        }
    }
    return LG_OK;
}

int lg_gemm_strided_batched_f32(int transa, int transb, int m, int n, int k, const float* A, int lda, int64_t strideA,
                                const float* B, int ldb, int64_t strideB, float* C, int ldc, int64_t strideC, int batch,
                                void* stream) {
    if (transa == LG_OP_TILED) { set_error("gemm_f32: tiled weights are an fp16 layout"); return LG_ERR_INVALID; }
    int rc = check_blas_args("gemm_f32", transa, transb, m, n, k, A, lda, B, ldb, C, ldc, batch);
    if (rc) return rc;
    GemmArgsF32 g;
    g.M = n; g.N = m; g.K = k;
    g.X = B; g.ldx = ldb; g.strideX = strideB;
    g.W = A; g.ldw = lda; g.strideW = strideA;
    g.Y = C; g.ldy = ldc; g.strideY = strideC;
    return gemm_f32_dispatch(g, transa ? W_NK : W_KN, batch, (hipStream_t)stream);
}

int lg_gemm_f32(int transa, int transb, int m, int n, int k, const float* A, int lda, const float* B, int ldb, float* C,
                int ldc, void* stream) {
    return lg_gemm_strided_batched_f32(transa, transb, m, n, k, A, lda, 0, B, ldb, 0, C, ldc, 0, 1, stream);
}

}  // extern "C"
