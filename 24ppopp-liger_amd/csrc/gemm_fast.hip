// gemm_fast.hip -- pipelined 256x256x64 fp16 GEMM for gfx950 (the prefill shapes of the launch vector).
//
//   Y[M, N] = X[M, K] * W,  W row-major [K, N] (the reference's layout) or [N, K];  fp32 accumulate, optional fused
//   epilogue.  Requires M % 256 == 0, N % 256 == 0, K % 64 == 0 and 16-byte aligned operands; everything else goes to
//   the generic kernel in gemm.hip.
//
// Structure (one workgroup = 8 waves = one 256x256 output tile, one workgroup per CU):
//   * global -> LDS with direct-to-LDS loads (global_load_lds_dwordx4): no VGPR staging, each wave instruction fills
//     1 KiB of LDS; two LDS stages (2 x 64 KiB);
//   * software pipeline with ONE barrier per k-tile, placed between the tile's two k-steps: fragments are double
//     buffered in registers, so when a wave reaches the barrier the whole of tile t is already in its registers.  After
//     the barrier tile t's stage is free and is refilled with tile t+2 (a full iteration ahead of its use), the first
//     fragments of tile t+1 stream in under the MFMAs of tile t's second k-step, and tile t+1's second-step fragments
//     under its first-step MFMAs.  MFMA, LDS-read and global-load issue are interleaved explicitly
//     (sched_group_barrier) so that the matrix pipe never waits for a block of LDS reads;
//   * LDS layouts are XOR-swizzled through the *global* address each lane loads from (the LDS position of a lane's
//     16 bytes is fixed by the instruction), so that both the 16-byte fragment reads of X and the transposed 8-byte
//     reads of a [K, N] weight tile are spread over the banks;
//   * wave grid 2 (M) x 4 (N): each wave owns 128 x 64 outputs = 8 x 4 MFMA 16x16x32 tiles, 128 fp32 accumulators;
//     operands are swapped in the MFMA so that a lane ends up with 4 consecutive output columns of one row;
//   * workgroup ids are remapped so that the 32 workgroups resident on one XCD (ids congruent mod 8) form a compact
//     4 x 8 block of tiles and share their X / W panels in that XCD's L2.
#include "gemm_common.cuh"

namespace lg {

constexpr int FB_M = 256, FB_K = 64;
constexpr int F_THREADS = 512;
// The tile is 256 x (64 * NJ) outputs: NJ = 4 -> 256 x 256, NJ = 3 -> 256 x 192 (used when it needs fewer rounds of 256
// workgroups, e.g. N = 6144: 512 tiles = 2 full rounds instead of 384 tiles = 1.5 rounds)
constexpr int stage_halves(int NJ) { return FB_M * FB_K + FB_K * 64 * NJ; }  // X tile + W tile per stage

typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(1))) const void gbl_void_t;

__device__ __forceinline__ void load_lds16(const half_t* gptr, half_t* lds_wave_base) {
    // every lane supplies its own global address; the 64 x 16 bytes land contiguously at lds_wave_base
    __builtin_amdgcn_global_load_lds((gbl_void_t*)gptr, (lds_void_t*)lds_wave_base, 16, 0, 0);
}

// swizzles: position (in 16-byte chunks) of logical chunk c in row r of the [rows][64] tiles; block (32 bytes) of
// logical block b in row k of the [64][256] tile
__device__ __forceinline__ int swz_a(int row, int c) { return c ^ ((row >> 1) & 7); }
// the 32 lanes served together by one transposed read touch rows k0..k0+3 and k0+8..k0+11: eight distinct XOR values
__device__ __forceinline__ int swz_b(int k, int blk) { return blk ^ ((k & 3) | ((k >> 1) & 4)); }

template <int WL, int EPI, int NJ>
__global__ __launch_bounds__(F_THREADS) void gemm_f16_fast(GemmArgs g, int tiles_m, int tiles_n) {
    constexpr int FB_N = 64 * NJ;
    constexpr int F_STAGE_HALVES = stage_halves(NJ);
    constexpr int WCH = (FB_K * FB_N) / 512 / 8;  // 1 KiB chunks of the W tile per wave (= NJ)
    static_assert(WL == W_NK || NJ == 4, "the [in, out] weight tile layout is written for 256-wide tiles");
    extern __shared__ __attribute__((aligned(16))) half_t smem[];  // 2 stages x (X tile, W tile)

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 2, wn = wave & 3;  // 2 x 4 waves; each 128 (M) x 16*NJ (N)
    const int l16 = lane & 15, lk = lane >> 4;

    // ---- XCD-aware tile mapping --------------------------------------------------------------------------------
    int tm, tn;
    {
        const int bid = blockIdx.x;
        const int ntiles = tiles_m * tiles_n;
        if ((tiles_m % 4 == 0) && (tiles_n % 8 == 0) && (ntiles % 256 == 0)) {
            const int xcd = bid & 7, slot = bid >> 3;          // slot: order of arrival on this XCD
            const int chunk = (slot >> 5) * 8 + xcd;          // blocks of 32 tiles (4 x 8)
            const int in = slot & 31;
            const int chunks_n = tiles_n >> 3;
            tm = (chunk / chunks_n) * 4 + (in & 3);
            tn = (chunk % chunks_n) * 8 + (in >> 2);
        } else {
            tm = bid % tiles_m;
            tn = bid / tiles_m;
        }
    }
    const int m0 = tm * FB_M, n0 = tn * FB_N;
    const half_t* X = g.X + (int64_t)m0 * g.ldx;
    const half_t* W = (WL == W_KN) ? g.W + n0 : g.W + (int64_t)n0 * g.ldw;

    // ---- per-lane global offsets of the 8 direct-to-LDS loads of one k-tile ---------------------------------------------
    // X tile (and W tile when [N, K]): 32 chunks of 1 KiB = 8 rows x 128 B; wave w fills chunks w, w+8, w+16, w+24.
    int xoff[4], woff[WCH];  // element offsets inside the tile; the launcher guarantees they fit 31 bits
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int q = i * 8 + wave;
        const int row = q * 8 + (lane >> 3), pos = lane & 7;
        const int c = swz_a(row, pos);  // XOR is an involution: the chunk stored at `pos` is logical chunk pos ^ f(row)
        xoff[i] = row * (int)g.ldx + c * 8;
        if (i >= WCH) continue;
        if (WL == W_NK) {
            woff[i] = row * (int)g.ldw + c * 8;
        } else {
            // W tile [64 k][256 n]: chunk q = k-rows 2q, 2q+1 (512 B each)
            const int k = q * 2 + (lane >> 5), p = lane & 31;
            const int blk = swz_b(k, p >> 1);
            woff[i] = k * (int)g.ldw + (blk * 2 + (p & 1)) * 8;
        }
    }
    const int64_t wstep = (WL == W_KN) ? (int64_t)FB_K * g.ldw : FB_K;

    auto issue = [&](int kt, int stage) {
        half_t* xs = smem + stage * F_STAGE_HALVES;
        half_t* ws = xs + FB_M * FB_K;
        const half_t* xg = X + (int64_t)kt * FB_K;
        const half_t* wg = W + (int64_t)kt * wstep;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int q = i * 8 + wave;
            load_lds16(xg + xoff[i], xs + q * 512);
            if (i < WCH) load_lds16(wg + woff[i], ws + q * 512);
        }
    };

    float4_t acc[8][NJ];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

    // fragments of k-step ks of the tile in `stage`: 8 row tiles of X, NJ column tiles of W
    auto read_frags = [&](int stage, int ks, half8_t (&a)[8], half8_t (&b)[NJ]) {
        const half_t* xs = smem + stage * F_STAGE_HALVES;
        const half_t* ws = xs + FB_M * FB_K;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int row = wm * 128 + i * 16 + l16;
            a[i] = *reinterpret_cast<const half8_t*>(&xs[row * FB_K + swz_a(row, ks * 4 + lk) * 8]);
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            if (WL == W_NK) {
                const int row = wn * (16 * NJ) + j * 16 + l16;
                b[j] = *reinterpret_cast<const half8_t*>(&ws[row * FB_K + swz_a(row, ks * 4 + lk) * 8]);
            } else {
                const int blk = wn * 4 + j;                      // 32-byte block = 16 output columns
                const int k = ks * 32 + lk * 8 + (l16 >> 2);     // this lane's source row of the first 4x16 read
                const half4_t lo = lds_read_tr4(&ws[k * FB_N + swz_b(k, blk) * 16 + (l16 & 3) * 4]);
                const half4_t hi = lds_read_tr4(&ws[(k + 4) * FB_N + swz_b(k + 4, blk) * 16 + (l16 & 3) * 4]);
                b[j] = half8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
        }
    };
    // operands swapped so that each lane owns 4 consecutive output columns of one row
    auto do_mfma = [&](half8_t (&a)[8], half8_t (&b)[NJ]) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j) acc[i][j] = mfma16(b[j], a[i], acc[i][j]);
    };
    constexpr int NDS = (WL == W_NK) ? 8 + NJ : 8 + 2 * NJ;  // LDS read instructions per k-step
    constexpr int NMFMA = 8 * NJ;                             // MFMAs per k-step
    constexpr int NLOAD = 4 + WCH;                            // global -> LDS loads per k-tile and thread

    const int ktiles = g.K / FB_K;
    issue(0, 0);
    if (ktiles > 1) issue(1, 1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    half8_t a0[8], b0[NJ], a1[8], b1[NJ];
    read_frags(0, 0, a0, b0);

    for (int kt = 0; kt < ktiles; ++kt) {
        const int stage = kt & 1;
        // first k-step multiplies while the second k-step's fragments stream in
        read_frags(stage, 1, a1, b1);
        do_mfma(a0, b0);
#pragma unroll
        for (int i = 0; i < NDS; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // 2 MFMA
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // 1 LDS read
        }
        __builtin_amdgcn_sched_group_barrier(0x008, NMFMA - 2 * NDS, 0);
        __builtin_amdgcn_sched_barrier(0);
        // this wave's loads of tile kt+1 have landed and all of tile kt is in its registers
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __syncthreads();
        // every wave is past tile kt: its stage takes tile kt+2; tile kt+1's first fragments stream in under the MFMAs
        if (kt + 2 < ktiles) issue(kt + 2, stage);
        if (kt + 1 < ktiles) read_frags(stage ^ 1, 0, a0, b0);
        do_mfma(a1, b1);
#pragma unroll
        for (int i = 0; i < NLOAD; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // global -> LDS load
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // LDS read
        }
#pragma unroll
        for (int i = 0; i < NDS - NLOAD; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, NMFMA - 2 * NDS, 0);
        __builtin_amdgcn_sched_barrier(0);
    }

    // ---- epilogue: acc[i][j][r] = Y[m0 + wm*128 + i*16 + l16][n0 + wn*16*NJ + j*16 + 4*lk + r] -----------------------------
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
            epilogue_store4<EPI>(g, g.Y, m0 + wm * 128 + i * 16 + l16, n0 + wn * (16 * NJ) + j * 16 + 4 * lk, acc[i][j], true);
}

template <int WL, int NJ>
static void launch_fast_epi(const GemmArgs& g, int tiles_m, int tiles_n, hipStream_t stream) {
    const dim3 grid(tiles_m * tiles_n), block(F_THREADS);
    const size_t smem = 2 * stage_halves(NJ) * sizeof(half_t);
#define LG_FAST(E)                                                                                                  \
    do {                                                                                                            \
        static bool attr_set = false;                                                                               \
        if (!attr_set) {                                                                                            \
            (void)hipFuncSetAttribute((const void*)gemm_f16_fast<WL, E, NJ>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
            attr_set = true;                                                                                        \
        }                                                                                                           \
        hipLaunchKernelGGL((gemm_f16_fast<WL, E, NJ>), grid, block, smem, stream, g, tiles_m, tiles_n);             \
    } while (0)
    switch (g.epi.kind) {
        case LG_EPI_NONE: LG_FAST(LG_EPI_NONE); break;
        case LG_EPI_BIAS: LG_FAST(LG_EPI_BIAS); break;
        case LG_EPI_BIAS_GELU: LG_FAST(LG_EPI_BIAS_GELU); break;
        default: LG_FAST(LG_EPI_BIAS_HEADS); break;
    }
#undef LG_FAST
}

int launch_gemm_fast_f16(const GemmArgs& g, int wlayout, int batch, hipStream_t stream, bool* handled) {
    *handled = false;
    if (batch != 1) return LG_OK;
    if (g.M % FB_M || g.K % FB_K || g.M <= 0 || g.N <= 0 || g.K <= 0) return LG_OK;
    if (!aligned16(g.X) || !aligned16(g.W) || !aligned16(g.Y) || (g.ldx % 8) || (g.ldw % 8)) return LG_OK;
    if (g.ldx >= (1 << 22) || g.ldw >= (1 << 22)) return LG_OK;  // 256 rows x ld must fit the 31-bit tile offsets
    if (g.epi.kind == LG_EPI_BIAS_HEADS ? (g.epi.d % 4 != 0) : (g.ldy % 4 != 0)) return LG_OK;
    // tile width: the one that needs the least work-rounds on 256 CUs (rounds x tile width); ties go to the wider tile
    const int tiles_m = g.M / FB_M;
    int best_nj = 0;
    long best_cost = 0;
    for (int nj = 4; nj >= 3; --nj) {
        if (g.N % (64 * nj)) continue;
        if (nj == 3 && wlayout != W_NK) continue;
        const long tiles = (long)tiles_m * (g.N / (64 * nj));
        const long cost = ((tiles + 255) / 256) * nj;
        if (!best_nj || cost < best_cost) { best_nj = nj; best_cost = cost; }
    }
    if (!best_nj) return LG_OK;
    *handled = true;
    const int tiles_n = g.N / (64 * best_nj);
    if (wlayout == W_NK) {
        if (best_nj == 4) launch_fast_epi<W_NK, 4>(g, tiles_m, tiles_n, stream);
        else launch_fast_epi<W_NK, 3>(g, tiles_m, tiles_n, stream);
    } else {
        launch_fast_epi<W_KN, 4>(g, tiles_m, tiles_n, stream);
    }
    return check_launch("gemm_f16_fast");
}

}  // namespace lg
