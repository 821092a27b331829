// gemv.hip -- weight-streaming fp16 matrix-vector kernel for one to four token rows (batch-1 decode) on gfx950.
//
//   Y[M, N] = X[M, K] * W^T with W stored [N, K], M <= 4.
// Every weight byte is used for 2*M flops, so the kernel is nothing but an HBM stream of W with the arithmetic on the
// vector ALUs (v_dot2_f32_f16); what matters is how the stream is issued:
//   * a wave owns 4 consecutive output features and walks their weight rows along k: one wave instruction reads 1 KiB of
//     ONE row (64 lanes x 16 bytes, fully contiguous), 16 such loads (4 rows x 4 k-steps) are kept in flight per lane in a
//     rolling pipeline (a fragment's registers are reloaded as soon as it has been multiplied);
//   * a block (4 waves = 16 features) covers the whole of K, so there are no K-slices, no fp32 partials and no second
//     kernel: lanes accumulate in fp32, one butterfly sum per output at the end, epilogue (bias / GELU / head-transposed
//     store) applied in place;
//   * the M token rows are staged once per block in LDS (M * K * 2 bytes) and shared by the 4 weight rows of every wave;
//     the first weight loads are issued before that staging so that the stream starts at once.
// Each output is one fixed-order fp32 sum (per-lane partial sums over k in an order fixed by the output's position, then a
// butterfly), independent of the other token rows.
#include "gemm_common.hpp"

namespace lg {

constexpr int GV_ROWS = 4;          // weight rows (output features) per wave
constexpr int GV_U = 4;             // k-steps in flight per row
constexpr int GV_KSTEP = 512;       // halves per wave instruction and row (64 lanes x 8)
constexpr int GV_MAX_LDS = 65536;   // bytes of staged X per block

__device__ __forceinline__ float dot8(half8_t w, half8_t x, float acc) {
#pragma unroll
    for (int p = 0; p < 4; ++p)
        acc = __builtin_amdgcn_fdot2(half2_t{w[2 * p], w[2 * p + 1]}, half2_t{x[2 * p], x[2 * p + 1]}, acc, false);
    return acc;
}

// MR = staged token rows (1, 2 or 4; rows >= M are zero)
template <int MR, int EPI>
__global__ __launch_bounds__(256) void gemv_nk_kernel(GemmArgs g, GemmGroup members, RowMap rm) {
    extern __shared__ __attribute__((aligned(16))) half_t xs[];  // [MR][K]
    select_group(g, members);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n0 = (blockIdx.x * 4 + wave) * GV_ROWS;
    const int K = g.K;
    const int ksteps = K / GV_KSTEP;  // the launcher guarantees K % (GV_KSTEP * GV_U) == 0

    // weight rows of this wave (rows beyond N are clamped and never stored)
    const half_t* wrow[GV_ROWS];
#pragma unroll
    for (int r = 0; r < GV_ROWS; ++r) wrow[r] = g.W + (int64_t)min(n0 + r, g.N - 1) * g.ldw + lane * 8;

    // Every wave walks k in groups of GV_U k-steps, starting at its own group and wrapping around: with a power-of-two row
    // pitch (K = 16384) rows that are walked in phase would all hit the same memory channels at the same time.
    const int groups = ksteps / GV_U;
    int grp = (blockIdx.x * 4 + wave) % groups;

    // the stream starts before X is staged
    half8_t wv[GV_U][GV_ROWS];
#pragma unroll
    for (int u = 0; u < GV_U; ++u)
#pragma unroll
        for (int r = 0; r < GV_ROWS; ++r) wv[u][r] = *reinterpret_cast<const half8_t*>(wrow[r] + (int64_t)(grp * GV_U + u) * GV_KSTEP);

    for (int v = tid; v < MR * (K / 8); v += 256) {
        const int row = v / (K / 8), c = v % (K / 8);
        half8_t val = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        if (row < g.M) val = *reinterpret_cast<const half8_t*>(g.X + (int64_t)row * g.ldx + c * 8);
        *reinterpret_cast<half8_t*>(&xs[row * K + c * 8]) = val;
    }
    __syncthreads();

    float acc[GV_ROWS][MR];
#pragma unroll
    for (int r = 0; r < GV_ROWS; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) acc[r][m] = 0.f;

    for (int it = 0; it < groups; ++it) {
        // the group after the last one is the last one again: every load is unconditional
        const int next = (it + 1 < groups) ? (grp + 1 == groups ? 0 : grp + 1) : grp;
#pragma unroll
        for (int u = 0; u < GV_U; ++u) {
            half8_t xv[MR];
#pragma unroll
            for (int m = 0; m < MR; ++m) xv[m] = *reinterpret_cast<const half8_t*>(&xs[m * K + (grp * GV_U + u) * GV_KSTEP + lane * 8]);
#pragma unroll
            for (int r = 0; r < GV_ROWS; ++r) {
#pragma unroll
                for (int m = 0; m < MR; ++m) acc[r][m] = dot8(wv[u][r], xv[m], acc[r][m]);
                wv[u][r] = *reinterpret_cast<const half8_t*>(wrow[r] + (int64_t)(next * GV_U + u) * GV_KSTEP);
            }
        }
        grp = next;
    }

#pragma unroll
    for (int m = 0; m < MR; ++m) {
#pragma unroll
        for (int q = 0; q < GV_ROWS / 4; ++q) {
            float4_t out;
#pragma unroll
            for (int r = 0; r < 4; ++r) out[r] = wave_sum(acc[q * 4 + r][m]);
            if (lane == 0 && m < g.M) epilogue_store4<EPI>(g, g.Y, m, n0 + q * 4, out, true, &rm);
        }
    }
}

int launch_gemv_f16(const GemmArgs& g, const GemmGroup& grp, const RowMap* rows, int wlayout, int batch, hipStream_t stream, bool* handled) {
    *handled = false;
    if (batch != 1 || wlayout != W_NK) return LG_OK;
    if (g.M <= 0 || g.M > 4 || g.N < 256 || (g.N % 4) || g.K < GV_KSTEP * GV_U || (g.K % (GV_KSTEP * GV_U))) return LG_OK;
    const int mr = g.M == 1 ? 1 : (g.M == 2 ? 2 : 4);
    const size_t smem = (size_t)mr * g.K * sizeof(half_t);
    if (smem > (size_t)GV_MAX_LDS) return LG_OK;
    if (!aligned16(g.X) || (g.ldx % 8) || (g.ldw % 8) || !group_aligned(g, grp)) return LG_OK;
    if (g.epi.kind == LG_EPI_BIAS_HEADS_ROWS && (!rows || g.M > LG_ROWMAP_MAX)) return LG_OK;
    if (g.epi.kind == LG_EPI_BIAS_GEGLU) return LG_OK;  // pairs features 16 apart: left to the sliced kernel and its reduce step
    *handled = true;
    const RowMap rm = rows ? *rows : RowMap{};
    const dim3 grid((g.N + 4 * GV_ROWS - 1) / (4 * GV_ROWS), grp.count), block(256);
#define LG_GV(MR_, E_)                                                                                              \
    do {                                                                                                            \
        /* set once per instantiation; the initialisation of a function-local static is thread-safe */              \
        static const hipError_t attr_rc = hipFuncSetAttribute((const void*)gemv_nk_kernel<MR_, E_>, hipFuncAttributeMaxDynamicSharedMemorySize, GV_MAX_LDS); \
        (void)attr_rc;                                                                                              \
        hipLaunchKernelGGL((gemv_nk_kernel<MR_, E_>), grid, block, smem, stream, g, grp, rm);                              \
    } while (0)
#define LG_GV_MR(E_)                                 \
    switch (mr) {                                    \
        case 1: LG_GV(1, E_); break;                 \
        case 2: LG_GV(2, E_); break;                 \
        default: LG_GV(4, E_); break;                \
    }
    switch (g.epi.kind) {
        case LG_EPI_NONE: LG_GV_MR(LG_EPI_NONE); break;
        case LG_EPI_BIAS: LG_GV_MR(LG_EPI_BIAS); break;
        case LG_EPI_BIAS_GELU: LG_GV_MR(LG_EPI_BIAS_GELU); break;
        case LG_EPI_BIAS_HEADS_ROWS: LG_GV_MR(LG_EPI_BIAS_HEADS_ROWS); break;
        default: LG_GV_MR(LG_EPI_BIAS_HEADS); break;
    }
#undef LG_GV_MR
#undef LG_GV
    return check_launch("gemv_f16");
}

}  // namespace lg
