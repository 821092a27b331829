// gemm_skinny_kn.hip -- weight-streaming fp16 GEMM for few tokens (decode: M <= 64) with weights stored [in, out].
//
//   Y[M, N] = X[M, K] * W with W row-major [K, N]: the layout the reference's (N,N) cuBLAS call implies (linear.h:47-49,99-101).
// As in gemm_skinny.hip every weight byte is used for 2*M flops only, so the kernel is an HBM stream of W.  Here a lane's natural
// 16-byte load holds 8 consecutive output features of ONE k, while the MFMA wants 8 consecutive k of one feature, so the stream
// goes through LDS and comes back out through the gfx950 transposed LDS read:
//   * global -> LDS with direct-to-LDS loads (no VGPR staging): a workgroup of 4 waves owns 128 output features and a K-slice and
//     (256 where N allows) walks it in k-tiles of 64; a W tile is [64 k][128 or 256 n] = 16 or 32 KiB, every wave instruction
//     fills 1 KiB = 4 k-rows x 256 bytes or 2 k-rows x 512 bytes;
//   * a ring of NS tiles (X tile beside it): NS - 1 tiles = 48 .. 96 KiB of weight loads are in flight per CU at all times, one
//     barrier per k-tile; the loop is branch-free (tile indices are clamped), so the outstanding-load counts are exact;
//   * LDS positions are XOR-swizzled through the global address each lane loads from, as in the pipelined kernel, so the
//     transposed 8-byte reads (ds_read_b64_tr_b16) and the 16-byte reads of the token rows are spread over the banks;
//   * K is sliced over the grid until the stream's compute units are filled (N / 128 workgroups per slice); the fp32 partials
//     go to the stream's workspace and the shared reduce kernel sums them in slice order and applies the epilogue.
#include "gemm_common.hpp"

namespace lg {

constexpr int KN_KT = 64;    // k-tile
constexpr int KN_THREADS = 256;

// KN_BN = output features per workgroup (128 or 256); ring depth: as many tiles as the 160 KiB of LDS hold comfortably
template <int MT, int KN_BN> constexpr int kn_stages() { return KN_BN == 128 ? (MT <= 2 ? 6 : 4) : (MT <= 2 ? 4 : 3); }
template <int MT, int KN_BN> constexpr int kn_lds_halves() { return kn_stages<MT, KN_BN>() * (KN_KT * KN_BN + 16 * MT * KN_KT); }

// MT = number of 16-row token tiles (M <= 16 * MT)
template <int MT, int KN_BN>
__global__ __launch_bounds__(KN_THREADS) void gemm_skinny_kn_kernel(GemmArgs g, int kslice, float* partial) {
    constexpr int NS = kn_stages<MT, KN_BN>();
    constexpr int WL = (KN_KT * KN_BN) / 512 / 4;      // W loads per wave and k-tile (1 KiB each)
    constexpr int LPR = KN_BN / 8;                     // lanes per k-row of the W tile
    constexpr int RPC = 64 / LPR;                      // k-rows per 1 KiB chunk
    constexpr int NU = KN_BN / 64;                     // 16-feature MFMA tiles per wave
    constexpr int W_TILE = KN_KT * KN_BN;              // halves per ring slot
    constexpr int X_TILE = 16 * MT * KN_KT;
    constexpr int XCH = 2 * MT;                        // 1 KiB chunks of an X tile (8 rows x 128 bytes each)
    constexpr int XL = (XCH + 3) / 4;                  // X loads per wave and k-tile (chunks wrap around: a few are fetched twice)
    constexpr int LPS = WL + XL;                       // loads per thread and k-tile
    extern __shared__ __attribute__((aligned(16))) half_t smem[];
    half_t* const wring = smem;
    half_t* const xring = smem + NS * W_TILE;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, lk = lane >> 4;
    const int n0 = blockIdx.x * KN_BN;
    const int split = blockIdx.y;
    const int k_begin = split * kslice;
    const int ktiles = (min(g.K, k_begin + kslice) - k_begin) / KN_KT;

    // per-lane byte offsets of this thread's loads inside a k-tile
    unsigned woff[WL], xoff[XL];
    int xchunk[XL];
#pragma unroll
    for (int i = 0; i < WL; ++i) {
        const int q = i * 4 + wave;                    // chunk: k-rows RPC q .. RPC q + RPC - 1
        const int k = q * RPC + lane / LPR, p = lane % LPR;
        const int blk = swz_b(k, p >> 1);
        woff[i] = (unsigned)(k * (int)g.ldw + (blk * 2 + (p & 1)) * 8) * 2u;
    }
#pragma unroll
    for (int i = 0; i < XL; ++i) {
        const int c = (i * 4 + wave) % XCH;
        const int row = c * 8 + (lane >> 3), pos = lane & 7;
        const int xrow = min(row, g.M - 1);            // rows beyond M read row M-1; their results are never stored
        xoff[i] = (unsigned)(xrow * (int)g.ldx + swz_a(row, pos) * 8) * 2u;
        xchunk[i] = c;
    }
    const char* Wg = reinterpret_cast<const char*>(g.W + n0 + (int64_t)k_begin * g.ldw);
    const char* Xg = reinterpret_cast<const char*>(g.X + k_begin);
    const int64_t wstep = (int64_t)KN_KT * g.ldw * 2, xstep = KN_KT * 2;
    auto issue = [&](int t) {
        const int kt = t < ktiles ? t : ktiles - 1;    // clamped: the extra loads of the last iterations refill slots nobody reads
        const int slot = t % NS;
        half_t* ws = wring + slot * W_TILE;
        half_t* xs = xring + slot * X_TILE;
#pragma unroll
        for (int i = 0; i < WL; ++i) load_lds16(reinterpret_cast<const half_t*>(Wg + kt * wstep + woff[i]), ws + (i * 4 + wave) * 512);
#pragma unroll
        for (int i = 0; i < XL; ++i) load_lds16(reinterpret_cast<const half_t*>(Xg + kt * xstep + xoff[i]), xs + xchunk[i] * 512);
    };

    float4_t acc[MT][NU];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int u = 0; u < NU; ++u) acc[i][u] = float4_t{0.f, 0.f, 0.f, 0.f};

#pragma unroll
    for (int t = 0; t < NS - 1; ++t) issue(t);
    for (int t = 0; t < ktiles; ++t) {
        // tile t has landed when at most the loads of tiles t+1 .. t+NS-2 are outstanding
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((NS - 2) * LPS) : "memory");
        barrier_keep_loads_in_flight();  // tile t is visible to every wave, and every wave is done with tile t-1: its slot is refilled now
        issue(t + NS - 1);
        const half_t* ws = wring + (t % NS) * W_TILE;
        const half_t* xs = xring + (t % NS) * X_TILE;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            // transposed reads issued by hand (see lds_read_tr4_issue): all of the k-step's, then one wait
            half4_t blo[NU], bhi[NU];
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                const int blk = wave * NU + u;                   // 32-byte block = 16 output features
                const int k = ks * 32 + lk * 8 + (l16 >> 2);     // this lane's source row of the first 4x16 read
                lds_read_tr4_issue(blo[u], &ws[k * KN_BN + swz_b(k, blk) * 16 + (l16 & 3) * 4]);
                lds_read_tr4_issue(bhi[u], &ws[(k + 4) * KN_BN + swz_b(k + 4, blk) * 16 + (l16 & 3) * 4]);
            }
            half8_t b[NU];
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                lds_tr_wait<0>(blo[u], bhi[u]);
                b[u] = join_half4(blo[u], bhi[u]);
            }
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const int row = i * 16 + l16;
                const half8_t a = *reinterpret_cast<const half8_t*>(&xs[row * KN_KT + swz_a(row, ks * 4 + lk) * 8]);
                // operands swapped: acc[i][u][r] = Y[16 i + l16][n0 + 16 NU wave + 16 u + 4 lk + r]
#pragma unroll
                for (int u = 0; u < NU; ++u) acc[i][u] = mfma16(b[u], a, acc[i][u]);
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the clamped refills of the last iterations

#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int m = i * 16 + l16;
        if (m >= g.M) continue;
        float* prow = partial + ((int64_t)split * g.M + m) * g.N + n0 + wave * (16 * NU) + 4 * lk;
#pragma unroll
        for (int u = 0; u < NU; ++u) *reinterpret_cast<float4_t*>(prow + 16 * u) = acc[i][u];
    }
}

template <int MT, int BN>
static void launch_kn(const GemmArgs& g, int kslice, float* ws, dim3 grid, hipStream_t stream) {
    const int smem = kn_lds_halves<MT, BN>() * (int)sizeof(half_t);
    // set once per instantiation; the initialisation of a function-local static is thread-safe
    static const hipError_t attr_rc = hipFuncSetAttribute((const void*)gemm_skinny_kn_kernel<MT, BN>, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
    (void)attr_rc;
    hipLaunchKernelGGL((gemm_skinny_kn_kernel<MT, BN>), grid, dim3(KN_THREADS), smem, stream, g, kslice, ws);
}
template <int BN>
static void launch_kn_mt(const GemmArgs& g, int kslice, float* ws, dim3 grid, hipStream_t stream) {
    switch ((g.M + 15) / 16) {
        case 1: launch_kn<1, BN>(g, kslice, ws, grid, stream); break;
        case 2: launch_kn<2, BN>(g, kslice, ws, grid, stream); break;
        case 3: launch_kn<3, BN>(g, kslice, ws, grid, stream); break;
        default: launch_kn<4, BN>(g, kslice, ws, grid, stream); break;
    }
}

int launch_gemm_skinny_kn_f16(const GemmArgs& g, const RowMap* rows, int wlayout, int batch, hipStream_t stream, bool* handled) {
    *handled = false;
    if (batch != 1 || wlayout != W_KN) return LG_OK;
    if (g.M <= 0 || g.M > 64 || g.N < 512 || (g.N % 128) || g.K < 512 || (g.K % KN_KT)) return LG_OK;
    if (!aligned16(g.X) || !aligned16(g.W) || (g.ldx % 8) || (g.ldw % 8) || (reinterpret_cast<uintptr_t>(g.Y) & 7u)) return LG_OK;
    if (g.ldx >= (1 << 22) || g.ldw >= (1 << 22)) return LG_OK;  // 64 rows x ld must fit the 31-bit tile offsets
    const bool heads = g.epi.kind == LG_EPI_BIAS_HEADS || g.epi.kind == LG_EPI_BIAS_HEADS_ROWS;
    if (heads ? (g.epi.d % 4 != 0) : (g.ldy % 4 != 0)) return LG_OK;
    if (g.epi.kind == LG_EPI_BIAS_HEADS_ROWS && !rows) return LG_OK;
    const StreamInfo si = stream_info(stream);
    if (!si.ws) return LG_OK;   // the K-slices need the stream's workspace
    // 256 features per workgroup where N allows: 512-byte row pieces per load instead of 256 (the six GEMMs of a decode step at
    // 32 token rows: 350 us against 378 us)
    const int BN = (g.N % 256) ? 128 : 256;
    const int nblk = g.N / BN, ktiles = g.K / KN_KT;
    // as few K-slices as fill the stream's compute units (one workgroup per CU keeps 48 .. 80 KiB of loads in flight), each
    // at least 8 k-tiles long, and no more than the workspace holds
    int nsplit = si.cus / nblk;   // one workgroup per compute unit, or as close below as the slice length allows
    if (nsplit > ktiles / 8) nsplit = ktiles / 8;
    if (nsplit > 32) nsplit = 32;
    if (nsplit < 1) nsplit = 1;
    const size_t slice_bytes = (size_t)g.M * g.N * sizeof(float);
    while (nsplit > 1 && (size_t)nsplit * slice_bytes > si.ws_bytes) nsplit /= 2;
    if (slice_bytes > si.ws_bytes) return LG_OK;
    int kt_per = (ktiles + nsplit - 1) / nsplit;
    nsplit = (ktiles + kt_per - 1) / kt_per;
    const int kslice = kt_per * KN_KT;
    *handled = true;
    const dim3 grid(nblk, nsplit);
    if (BN == 256) launch_kn_mt<256>(g, kslice, si.ws, grid, stream);
    else launch_kn_mt<128>(g, kslice, si.ws, grid, stream);
    launch_splitk_reduce(g, si.ws, nsplit, stream, rows);
    return check_launch("gemm_f16_skinny_kn");
}

}  // namespace lg
