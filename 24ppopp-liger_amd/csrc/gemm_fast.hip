// gemm_fast.hip -- pipelined 256x256x64 fp16 GEMM for gfx950 (the prefill shapes of the launch vector).
//
//   Y[M, N] = X[M, K] * W,  W row-major [K, N] (the reference's layout) or [N, K];  fp32 accumulate, optional fused
//   epilogue.  Requires N % 128 == 0 (or % 192), K % 64 == 0, M > 64 (any M; a partial last row of tiles is padded) and 16-byte aligned operands; everything else goes to
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
#include <stdlib.h>

#include "gemm_common.hpp"
#include <type_traits>

namespace lg {

constexpr int FB_M = 256, FB_K = 64;
constexpr int F_THREADS = 512;
// The tile is 256 x (64 * NJ) outputs: NJ = 4 -> 256 x 256, NJ = 3 -> 256 x 192, NJ = 2 -> 256 x 128 (used when it needs fewer rounds of 256
// workgroups, e.g. N = 6144: 512 tiles = 2 full rounds instead of 384 tiles = 1.5 rounds)
// LDS: a ring of 3 X tiles and a ring of 2 W tiles (256-wide: 96 + 64 KiB = the whole 160 KiB of a CU)
constexpr int X_STAGES = 3, W_STAGES = 2;
constexpr int lds_halves(int NJ) { return X_STAGES * FB_M * FB_K + W_STAGES * FB_K * 64 * NJ; }

// [64 k][64 NJ n] weight tile: which logical 32-byte block sits at block position `pos` of row k (swz_kn), and at which position
// logical block `blk` sits (unswz_kn).  Power-of-two widths XOR (an involution); the 192-wide tile has 12 blocks to a row and
// rotates instead: its rows are 96 dwords apart, so rows k and k + 2 (and k + 8, k + 10: the other half of the 32 lanes that one
// transposed read serves together) would share banks, and a rotation by ((k >> 1) & 1) + 2 ((k >> 3) & 1) blocks separates them.
template <int NJ> __device__ __forceinline__ int swz_kn(int k, int pos) {
    if (NJ == 3) { const int b = pos + ((k >> 1) & 1) + 2 * ((k >> 3) & 1); return b >= 12 ? b - 12 : b; }
    return swz_b(k, pos);
}
template <int NJ> __device__ __forceinline__ int unswz_kn(int k, int blk) {
    if (NJ == 3) { const int p = blk - ((k >> 1) & 1) - 2 * ((k >> 3) & 1); return p < 0 ? p + 12 : p; }
    return swz_b(k, blk);
}

template <int WL, int EPI, int NJ>
__global__ __launch_bounds__(F_THREADS) void gemm_f16_fast(GemmArgs g, GemmGroup grp, int tiles_m, int tiles_n, float* partial, int kt_per_split, int cus, int wide_store) {
    constexpr int FB_N = 64 * NJ;
    constexpr int X_TILE = FB_M * FB_K, W_TILE = FB_K * FB_N;  // halves per ring slot
    constexpr int WCH = (FB_K * FB_N) / 512 / 8;  // 1 KiB chunks of the W tile per wave (= NJ)
    extern __shared__ __attribute__((aligned(16))) half_t smem[];  // X ring (3 tiles), then W ring (2 tiles)
    half_t* const xring = smem;
    half_t* const wring = smem + X_STAGES * X_TILE;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: LDS bases stay in scalar registers
    const int wm = wave >> 2, wn = wave & 3;  // 2 x 4 waves; each 128 (M) x 16*NJ (N)
    const int l16 = lane & 15, lk = lane >> 4;

    // ---- XCD-aware tile mapping --------------------------------------------------------------------------------
    int tm, tn;
    {
        const int bid = blockIdx.x;
        const int ntiles = tiles_m * tiles_n;
        // The workgroups that run at the same time ("a round": one per compute unit of the stream, P = cus / 8 on each XCD; 256
        // and 32 on the whole chip) cover an RM x RN region of tiles, each XCD a compact 4 x P/4 block of it (its L2 then serves
        // 4 + P/4 operand panels to P tiles).  A round reads RM X panels and RN W panels from memory, so the region is made as
        // square as the tile counts allow: on the whole chip 16 x 16 (32 panels; FFN-1 1346 -> 1412 TFLOP/s against rounds of
        // 4 x 64), else 8 x 32.
        const int P = cus >> 3, pw = P >> 2;  // pw: width of an XCD's block in tiles
        int RM = 0;
        if (pw >= 1 && (P & 3) == 0) {
            if ((tiles_m % 16 == 0) && (tiles_n % (2 * pw) == 0) && tiles_n >= 6 * pw) RM = 16;
            else if ((tiles_m % 8 == 0) && (tiles_n % (4 * pw) == 0)) RM = 8;
        }
        if (RM) {
            const int RN = (8 * P) / RM, xcols = RN / pw;      // XCD blocks per region row
            const int xcd = bid & 7, slot = bid >> 3;          // slot: order of arrival on this XCD
            const int round = slot / P, in = slot % P;
            const int regions_n = tiles_n / RN;
            tm = (round / regions_n) * RM + (xcd / xcols) * 4 + (in & 3);
            tn = (round % regions_n) * RN + (xcd % xcols) * pw + (in >> 2);
        } else if (pw >= 1 && (P & 3) == 0 && (tiles_m % 4 == 0) && (tiles_n % pw == 0) && (ntiles % (8 * P) == 0)) {
            const int xcd = bid & 7, slot = bid >> 3;
            const int chunk = (slot / P) * 8 + xcd;           // blocks of P tiles (4 x P/4)
            const int in = slot % P;
            const int chunks_n = tiles_n / pw;
            tm = (chunk / chunks_n) * 4 + (in & 3);
            tn = (chunk % chunks_n) * pw + (in >> 2);
        } else {
            tm = bid % tiles_m;
            tn = bid / tiles_m;
        }
    }
    // a group (problems that share X and the shape: the Q, K and V projections) lays its members' tile columns side by side;
    // from here on g is the member's problem and n0 a feature index inside it
    if (grp.count > 1) {
        const int per = tiles_n / grp.count;
        const int member = tn / per;
        tn -= member * per;
        g.W = grp.W[member];
        g.Y = grp.Y[member];
        g.epi.bias = grp.bias[member];
        g.ldy = grp.ldy[member];
    }
    const int m0 = tm * FB_M, n0 = tn * FB_N;
    // K-slice of this workgroup (blockIdx.y; the whole K when the launch is not split): k-tiles [kt0, kt0 + ktiles)
    const int split = blockIdx.y;
    const int kt0 = split * kt_per_split;
    const int ktiles = min(g.K / FB_K - kt0, kt_per_split);
    const half_t* X = g.X + (int64_t)m0 * g.ldx + (int64_t)kt0 * FB_K;
    // tiled weights: feature tile n0 / 16 starts n0 * K elements in, and a k-tile of 64 is two consecutive 512-element blocks
    const half_t* W = (WL == W_KN)   ? g.W + n0 + (int64_t)kt0 * FB_K * g.ldw
                      : (WL == W_NK) ? g.W + (int64_t)n0 * g.ldw + (int64_t)kt0 * FB_K
                                     : g.W + (int64_t)n0 * g.ldw + (int64_t)kt0 * 1024;

    // ---- per-lane global offsets of the 8 direct-to-LDS loads of one k-tile ---------------------------------------------
    // X tile (and W tile when [N, K]): 32 chunks of 1 KiB = 8 rows x 128 B; wave w fills chunks w, w+8, w+16, w+24.
    unsigned xoff[4], woff[WCH];  // byte offsets inside the tile; the launcher guarantees they fit 32 bits
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int q = i * 8 + wave;
        const int row = q * 8 + (lane >> 3), pos = lane & 7;
        const int c = swz_a(row, pos);  // XOR is an involution: the chunk stored at `pos` is logical chunk pos ^ f(row)
        // token rows beyond M (last, partial row of tiles) are read from row M-1; their results are never stored
        const int xrow = min(row, g.M - 1 - m0);
        xoff[i] = (unsigned)(xrow * (int)g.ldx + c * 8) * 2u;
        if (i >= WCH) continue;
        if (WL == W_TILED) {
            // chunk q of the W tile = fragment block (feature tile q / 2, k-step q % 2): one contiguous KiB in memory that lands
            // as one contiguous KiB of LDS, each lane's 16 bytes where the lane will read them back
            woff[i] = ((unsigned)(q >> 1) * (unsigned)(g.K >> 5) * 512u + (unsigned)(q & 1) * 512u + (unsigned)lane * 8u) * 2u;
        } else if (WL == W_NK) {
            woff[i] = (unsigned)(row * (int)g.ldw + c * 8) * 2u;
        } else {
            // W tile [64 k][FB_N n]: a k-row is FB_N / 8 lanes wide, chunk q = 64 / (FB_N / 8) consecutive k-rows
            // (the 192-wide tile has 24 lanes to a k-row, so a chunk's lanes straddle rows: every lane finds its own row and place)
            constexpr int LPR = FB_N / 8;
            const int f = q * 64 + lane;
            const int k = f / LPR, p = f % LPR;
            const int blk = swz_kn<NJ>(k, p >> 1);
            woff[i] = (unsigned)(k * (int)g.ldw + (blk * 2 + (p & 1)) * 8) * 2u;
        }
    }
    const int64_t wstep = (WL == W_KN) ? (int64_t)FB_K * g.ldw : (WL == W_NK ? FB_K : 1024);

    // tile index clamped to the last one: the loop body is branch-free, the extra loads of the last iterations
    // refill slots nobody reads any more
    auto x_tile = [&](int kt) { return reinterpret_cast<const char*>(X + (int64_t)(kt < ktiles ? kt : ktiles - 1) * FB_K); };
    auto w_tile = [&](int kt) { return reinterpret_cast<const char*>(W + (int64_t)(kt < ktiles ? kt : ktiles - 1) * wstep); };
    // load l of a k-tile: l < WCH -> chunk l of the W tile, else chunk l - WCH of the X tile (W first: it is needed first)
    auto issue_one = [&](int l, const char* xg, const char* wg, half_t* xs, half_t* ws) {
        if (l < WCH) load_lds16(reinterpret_cast<const half_t*>(wg + woff[l]), ws + (l * 8 + wave) * 512);
        else load_lds16(reinterpret_cast<const half_t*>(xg + xoff[l - WCH]), xs + ((l - WCH) * 8 + wave) * 512);
    };

    float4_t acc[8][NJ];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

    // LDS read unit u of k-step ks: u < NJ -> W fragment u, else X fragment u - NJ (W first: every MFMA row needs all of b)
    // [K, N] weights: the two transposed 8-byte reads of a W fragment are issued by hand (lds_read_tr4_issue) into blo / bhi
    // [set][u] and joined into the fragment at the start of the phase that multiplies it (finish_b)
    half4_t blo[2][NJ], bhi[2][NJ];
    int wfrag[NJ];   // [K, N] weights: offset (halves) inside a W tile of this lane's first transposed read of fragment u at ks = 0
#pragma unroll
    for (int u = 0; u < NJ; ++u) {
        const int blk = wn * NJ + u;             // 32-byte block = 16 output columns
        const int k = lk * 8 + (l16 >> 2);       // this lane's source row of the first 4x16 read
        wfrag[u] = k * FB_N + unswz_kn<NJ>(k, blk) * 16 + (l16 & 3) * 4;
    }
    auto read_unit = [&](const half_t* xs, const half_t* ws, int ks, int u, half8_t (&a)[8], half8_t (&b)[NJ], int set) {
        if (u >= NJ) {
            const int i = u - NJ;
            const int row = wm * 128 + i * 16 + l16;
            a[i] = *reinterpret_cast<const half8_t*>(&xs[row * FB_K + swz_a(row, ks * 4 + lk) * 8]);
        } else if (WL == W_TILED) {
            b[u] = *reinterpret_cast<const half8_t*>(&ws[(((wn * NJ + u) * 2 + ks) * 64 + lane) * 8]);
        } else if (WL == W_NK) {
            const int row = wn * (16 * NJ) + u * 16 + l16;
            b[u] = *reinterpret_cast<const half8_t*>(&ws[row * FB_K + swz_a(row, ks * 4 + lk) * 8]);
        } else {
            // rows k and k + 4 of the tile, k = 32 ks + 8 lk + l16 / 4; neither ks nor the + 4 changes a block's position in its
            // row (the swizzles look at bits 0, 1 and 3 of k only), so both are plain offsets from the lane's base for ks = 0
            lds_read_tr4_issue(blo[set][u], ws + wfrag[u] + ks * 32 * FB_N);
            lds_read_tr4_issue(bhi[set][u], ws + wfrag[u] + (ks * 32 + 4) * FB_N);
        }
    };
    auto finish_b = [&](half8_t (&b)[NJ], int set) {
        if (WL != W_KN) return;
#pragma unroll
        for (int u = 0; u < NJ; ++u) {
            lds_tr_wait<0>(blo[set][u], bhi[set][u]);
            b[u] = join_half4(blo[set][u], bhi[set][u]);
        }
    };
    constexpr int NDS = 8 + NJ;       // LDS read units per k-step
    constexpr int NMFMA = 8 * NJ;     // MFMAs per k-step
    constexpr int NLOAD = 4 + WCH;    // global -> LDS loads per k-tile and thread
    constexpr int DS_SPAN = NMFMA * 3 / 4;  // the reads of a phase are issued under its first 3/4 MFMAs
    constexpr int W_SPAN = NMFMA / 2;       // the W loads (needed first) go under the first half of the second k-step's
                                            // MFMAs, the X loads under the second half
    // One phase = the NMFMA MFMAs of one k-step (fragments ma, mb) with the LDS reads of the next k-step (into ra, rb)
    // and, if LOADS, the global -> LDS loads of a later k-tile placed between them in exactly this order: the
    // scheduling fence after every MFMA keeps the compiler from regrouping them.  Operands are swapped in the MFMA so
    // that each lane owns 4 consecutive output columns of one row.
    auto phase = [&](auto with_loads, auto mset_c, half8_t (&ma)[8], half8_t (&mb)[NJ], half8_t (&ra)[8], half8_t (&rb)[NJ],
                     const half_t* rxs, const half_t* rws, int rks, const char* xg, const char* wg, half_t* lxs,
                     half_t* lws) {
        constexpr bool LOADS = decltype(with_loads)::value;
        constexpr int MSET = decltype(mset_c)::value;   // which blo / bhi set holds mb's halves; the reads go to the other
        finish_b(mb, MSET);
#pragma unroll
        for (int m = 0; m < NMFMA; ++m) {
            const int i = m / NJ, j = m % NJ;
            acc[i][j] = mfma16(mb[j], ma[i], acc[i][j]);
            if (LOADS) {
#pragma unroll
                for (int l = 0; l < NLOAD; ++l) {
                    const int at = l < WCH ? l * W_SPAN / WCH : W_SPAN + (l - WCH) * (NMFMA - W_SPAN) / 4;
                    if (at == m) issue_one(l, xg, wg, lxs, lws);
                }
            }
#pragma unroll
            for (int u = 0; u < NDS; ++u) {
                // [N, K] weights: one read unit every DS_SPAN / NDS MFMAs.  [K, N] weights: the W units (two transposed
                // reads each) go under the first NJ MFMAs, the X units are spread over the rest (measured: 8 % faster)
                const int at = (WL != W_KN) ? (u * DS_SPAN + DS_SPAN - 1) / NDS : (u < NJ ? u : NJ + (u - NJ) * (DS_SPAN - NJ) / 8);
                if (at == m) read_unit(rxs, rws, rks, u, ra, rb, MSET ^ 1);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // prologue: X0 W0 X1 W1 X2; everything but X2 must have landed before the first fragments are read
    for (int t = 0; t < 3; ++t) {
#pragma unroll
        for (int l = (t < 2 ? 0 : WCH); l < NLOAD; ++l)
            issue_one(l, x_tile(t), w_tile(t), xring + t * X_TILE, wring + (t & 1) * W_TILE);
    }
    asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    __syncthreads();
    half8_t a0[8], b0[NJ], a1[8], b1[NJ];
#pragma unroll
    for (int u = 0; u < NDS; ++u) read_unit(xring, wring, 0, u, a0, b0, 0);

    int xslot = 0, xnext = 1;  // kt % 3, (kt + 1) % 3
    for (int kt = 0; kt < ktiles; ++kt) {
        const int wslot = kt & 1;
        half_t* const xs = xring + xslot * X_TILE;
        half_t* const ws = wring + wslot * W_TILE;
        // first k-step multiplies while the second k-step's fragments stream in
        phase(std::false_type{}, std::integral_constant<int, 0>{}, a0, b0, a1, b1, xs, ws, 1, nullptr, nullptr, nullptr, nullptr);
        // all of tile kt is in this wave's registers; its loads of X(kt+1) and W(kt+1) have landed, the four loads of
        // X(kt+2) issued last may stay in flight across the barrier
        asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
        __syncthreads();
        // every wave is past tile kt: its W slot takes W(kt+2), its X slot X(kt+3); tile kt+1's first fragments stream
        // in under the MFMAs of the second k-step
        phase(std::true_type{}, std::integral_constant<int, 1>{}, a1, b1, a0, b0, xring + xnext * X_TILE, wring + (wslot ^ 1) * W_TILE, 0, x_tile(kt + 3),
              w_tile(kt + 2), xs, ws);
        xslot = xnext;
        xnext = (xnext == X_STAGES - 1) ? 0 : xnext + 1;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the clamped refills of the last iterations
    if (WL == W_KN) {
        // the last phase has issued the transposed reads of a tile that is never multiplied: they are waited for and named
        // here, so that nothing may reuse their registers while they can still land (hand-issued reads are invisible to
        // the compiler's own bookkeeping)
#pragma unroll
        for (int u = 0; u < NJ; ++u) lds_tr_wait<0>(blo[0][u], bhi[0][u]);
    }

    // ---- epilogue: acc[i][j][r] = Y[m0 + wm*128 + i*16 + l16][n0 + wn*16*NJ + j*16 + 4*lk + r] -----------------------------
    // Everything that depends only on the column (bias, head offset) or only on the row (batch / position split) is
    // computed once, so the 8 x NJ stores of a lane are not separated by dependent loads or integer divisions.
    if (EPI == LG_EPI_PARTIAL) {
        // split-K: the fp32 accumulators of this K-slice go to partial[split][M][N]; a second kernel sums the slices
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int m = m0 + wm * 128 + i * 16 + l16;
            if (m >= g.M) continue;
            float* prow = partial + ((int64_t)split * g.M + m) * g.N + n0 + wn * (16 * NJ) + 4 * lk;
#pragma unroll
            for (int j = 0; j < NJ; ++j) *reinterpret_cast<float4_t*>(prow + j * 16) = acc[i][j];
        }
        return;
    }
    if (EPI == LG_EPI_BIAS_GEGLU) {
        // the wave's 16-feature tiles are (gate, up) pairs (NJ even): out[m][(n / 32) * 16 + n % 16 ..] = gelu(gate + b) * (up + b)
        float bg[NJ / 2 + 1][4], bu[NJ / 2 + 1][4];
        int col[NJ / 2 + 1];
#pragma unroll
        for (int jp = 0; jp < NJ / 2; ++jp) {
            const int n = n0 + wn * (16 * NJ) + jp * 32 + 4 * lk;
            const half4_t g4 = *reinterpret_cast<const half4_t*>(g.epi.bias + n);
            const half4_t u4 = *reinterpret_cast<const half4_t*>(g.epi.bias + n + 16);
#pragma unroll
            for (int r = 0; r < 4; ++r) { bg[jp][r] = (float)g4[r]; bu[jp][r] = (float)u4[r]; }
            col[jp] = (n >> 5) * 16 + (n & 15);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int m = m0 + wm * 128 + i * 16 + l16;
            if (m >= g.M) continue;
            half_t* yrow = g.Y + (int64_t)m * g.ldy;
#pragma unroll
            for (int jp = 0; jp < NJ / 2; ++jp) {
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] = gelu_tanh(acc[i][2 * jp][r] + bg[jp][r]) * (acc[i][(2 * jp + 1) % NJ][r] + bu[jp][r]);
                const half4_t o = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
                *reinterpret_cast<half4_t*>(yrow + col[jp]) = o;
            }
        }
        return;
    }
    float bias_v[NJ][4];
    int64_t col_off[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int n = n0 + wn * (16 * NJ) + j * 16 + 4 * lk;
        if (EPI != LG_EPI_NONE && EPI != LG_EPI_PARTIAL) {
            const half4_t bv = *reinterpret_cast<const half4_t*>(g.epi.bias + n);
#pragma unroll
            for (int r = 0; r < 4; ++r) bias_v[j][r] = (float)bv[r];
        }
        // LG_EPI_BIAS_HEADS: [M = b*seq + s, N = head*d + e] -> [b, head, s, e] with ldy rows reserved per (b, head);
        // n..n+3 stay inside one head (d % 4 == 0)
        if (EPI == LG_EPI_BIAS_HEADS) col_off[j] = (int64_t)(n / g.epi.d) * g.ldy * g.epi.d + (n % g.epi.d);
        else col_off[j] = n;
    }
    if (wide_store) {
        // The tile goes through LDS (the ring is idle now) and leaves in whole rows: in the accumulator layout a wave's store
        // instruction writes 32 bytes of 16 different rows; read back row by row, 32 lanes write 512 contiguous bytes of one
        // row.  Rows are 16 bytes apart from a multiple of 128 in LDS, so the 8-byte writes of a half-wave (16 rows x 2 lane
        // groups) and the 16-byte reads fall on distinct banks.
        constexpr int PITCH = FB_N + 8;  // halves
        __syncthreads();                 // every wave has read its last fragments
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                float v[4] = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
                if (EPI != LG_EPI_NONE) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) v[r] += bias_v[j][r];
                }
                if (EPI == LG_EPI_BIAS_GELU) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) v[r] = gelu_tanh(v[r]);
                }
                const half4_t o = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
                *reinterpret_cast<half4_t*>(&smem[(wm * 128 + i * 16 + l16) * PITCH + wn * (16 * NJ) + j * 16 + 4 * lk]) = o;
            }
        }
        __syncthreads();
        constexpr int CPR = FB_N / 8;                 // 16-byte chunks per tile row
        constexpr int ITERS = FB_M * CPR / F_THREADS;  // 16, 12 or 8
#pragma unroll 4
        for (int it = 0; it < ITERS; ++it) {
            const int c = it * F_THREADS + tid;
            const int row = c / CPR, cc = c % CPR;
            const int m = m0 + row, n = n0 + cc * 8;
            if (m >= g.M) continue;
            const half8_t o = *reinterpret_cast<const half8_t*>(&smem[row * PITCH + cc * 8]);
            int64_t off;
            if (EPI == LG_EPI_BIAS_HEADS) {
                const int b = m / g.epi.seq, sq = m % g.epi.seq;
                off = (((int64_t)b * g.epi.heads_total + n / g.epi.d) * g.ldy + sq) * (int64_t)g.epi.d + (n % g.epi.d);
            } else {
                off = (int64_t)m * g.ldy + n;
            }
            *reinterpret_cast<half8_t*>(g.Y + off) = o;
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int m = m0 + wm * 128 + i * 16 + l16;
        if (m >= g.M) continue;
        int64_t row_off;
        if (EPI == LG_EPI_BIAS_HEADS) {
            const int b = m / g.epi.seq, sq = m % g.epi.seq;
            row_off = ((int64_t)b * g.epi.heads_total * g.ldy + sq) * (int64_t)g.epi.d;
        } else {
            row_off = (int64_t)m * g.ldy;
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            float v[4] = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
            if (EPI != LG_EPI_NONE) {
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] += bias_v[j][r];
            }
            if (EPI == LG_EPI_BIAS_GELU) {
#pragma unroll
                for (int r = 0; r < 4; ++r) v[r] = gelu_tanh(v[r]);
            }
            const half4_t o = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
            *reinterpret_cast<half4_t*>(g.Y + row_off + col_off[j]) = o;
        }
    }
}

template <int WL, int NJ>
static int launch_fast_epi(const GemmArgs& g, const GemmGroup& grp, int tiles_m, int tiles_n, const StreamInfo& si, hipStream_t stream) {
    const int tiles = tiles_m * tiles_n, ktiles = g.K / FB_K;
    const int cus = si.cus;
    // At most 256 token rows (one row of tiles, the continuation of the weight-streaming kernel's regime): the time is set by
    // how fast the weights stream in, so K is split over otherwise idle CUs (slices of >= 8 k-tiles, fp32 partials in the
    // stream's workspace, summed in slice order by a second kernel that applies the epilogue; no more slices than the workspace
    // holds, none on a stream without one).  Larger M never splits K, so that a token row's result does not depend on how many
    // other rows are in the batch (each output is one sequential sum over k).
    int nsplit = 1;
    if (tiles_m == 1 && tiles <= cus / 2 && si.ws && grp.count == 1) {
        nsplit = cus / tiles;
        if (nsplit > ktiles / 8) nsplit = ktiles / 8;
        if (nsplit > 16) nsplit = 16;
        const size_t slice_bytes = (size_t)g.M * g.N * sizeof(float);
        if ((size_t)nsplit * slice_bytes > si.ws_bytes) nsplit = (int)(si.ws_bytes / slice_bytes);
        if (nsplit < 1) nsplit = 1;
    }
    int kt_per_split = (ktiles + nsplit - 1) / nsplit;
    nsplit = (ktiles + kt_per_split - 1) / kt_per_split;
    float* partial = nsplit > 1 ? si.ws : nullptr;
    const dim3 grid(tiles, nsplit), block(F_THREADS);
    const size_t smem = lds_halves(NJ) * sizeof(half_t);
    // whole-row stores through LDS need 16-byte aligned rows (heads epilogue: rows of size_per_head halves)
    static const int wide_forced = [] { const char* e = getenv("LG_GEMM_WIDE_STORE"); return e ? atoi(e) : -1; }();
    int wide = 1;
    for (int i = 0; i < grp.count; ++i)
        if (g.epi.kind == LG_EPI_BIAS_HEADS ? (g.epi.d % 8 != 0) : (grp.ldy[i] % 8 != 0)) wide = 0;
    if (wide_forced >= 0) wide = wide && wide_forced;
#define LG_FAST(E)                                                                                                  \
    do {                                                                                                            \
        /* set once per instantiation; the initialisation of a function-local static is thread-safe */              \
        static const hipError_t attr_rc = hipFuncSetAttribute((const void*)gemm_f16_fast<WL, E, NJ>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
        (void)attr_rc;                                                                                              \
        hipLaunchKernelGGL((gemm_f16_fast<WL, E, NJ>), grid, block, smem, stream, g, grp, tiles_m, tiles_n, partial, kt_per_split, cus, wide); \
    } while (0)
    if (nsplit > 1) {
        LG_FAST(LG_EPI_PARTIAL);
        launch_splitk_reduce(g, partial, nsplit, stream);
    } else {
        switch (g.epi.kind) {
            case LG_EPI_NONE: LG_FAST(LG_EPI_NONE); break;
            case LG_EPI_BIAS: LG_FAST(LG_EPI_BIAS); break;
            case LG_EPI_BIAS_GELU: LG_FAST(LG_EPI_BIAS_GELU); break;
            case LG_EPI_BIAS_GEGLU:
                if constexpr (NJ % 2 == 0) LG_FAST(LG_EPI_BIAS_GEGLU);  // the launcher picks an even tile width for it
                break;
            default: LG_FAST(LG_EPI_BIAS_HEADS); break;
        }
    }
#undef LG_FAST
    return LG_OK;
}

int launch_gemm_fast_f16(const GemmArgs& g, const GemmGroup& grp, int wlayout, int batch, hipStream_t stream, bool* handled) {
    *handled = false;
    if (batch != 1) return LG_OK;
    if (g.K % FB_K || g.M <= 0 || g.N <= 0 || g.K <= 0) return LG_OK;
    // A partial last row of tiles computes (and discards) up to 255 extra token rows.  Even so this kernel is the faster one
    // for every token count the weight-streaming kernel does not take (M = 128: 182 us vs 331 us in the generic kernel for a
    // 16384 x 12288 weight), because with few token rows the time is set by how fast the weights stream in.
    if (g.M <= 64) return LG_OK;
    if (!aligned16(g.X) || (g.ldx % 8) || (g.ldw % 8)) return LG_OK;
    if (g.ldx >= (1 << 22) || g.ldw >= (1 << 22)) return LG_OK;  // 256 rows x ld must fit the 31-bit tile offsets
    if (wlayout == W_TILED && g.ldw != g.K) return LG_OK;
    for (int i = 0; i < grp.count; ++i) {
        if (!aligned16(grp.W[i]) || !aligned16(grp.Y[i])) return LG_OK;
        if (g.epi.kind == LG_EPI_BIAS_HEADS ? (g.epi.d % 4 != 0) : (grp.ldy[i] % 4 != 0)) return LG_OK;
        if (g.epi.kind != LG_EPI_NONE && (reinterpret_cast<uintptr_t>(grp.bias[i]) & 7u)) return LG_OK;  // 8-byte bias loads
    }
    if (grp.count > 1 && g.M <= FB_M) return LG_OK;  // one row of tiles may want K-slices, which take single problems only
    // tile width: the one that needs the least work-rounds on the stream's CUs (rounds x tile width); ties go to the wider tile
    const StreamInfo si = stream_info(stream);
    const int tiles_m = (g.M + FB_M - 1) / FB_M;
    int best_nj = 0;
    long best_cost = 0;
    for (int nj = 4; nj >= 2; --nj) {
        if (g.N % (64 * nj)) continue;
        if (nj == 3 && g.epi.kind == LG_EPI_BIAS_GEGLU) continue;  // a wave must hold whole (gate, up) pairs of 16-feature tiles
        const long tiles = (long)tiles_m * (g.N / (64 * nj)) * grp.count;
        // narrower tiles move more operand bytes per flop: about 3 % / 35 % more time per unit of width (measured)
        const long cost = ((tiles + si.cus - 1) / si.cus) * nj * (nj == 4 ? 100 : nj == 3 ? 103 : 135);
        if (!best_nj || cost < best_cost) { best_nj = nj; best_cost = cost; }
    }
    // LG_GEMM_TILE_WIDTH=2|3|4 in the environment (read once) overrides the choice where that width divides N: a measurement knob
    // (256 x 128 tiles leave registers and LDS for a second kernel's waves on the same compute unit)
    static const int forced_nj = [] { const char* e = getenv("LG_GEMM_TILE_WIDTH"); return e ? atoi(e) : 0; }();
    if (forced_nj >= 2 && forced_nj <= 4 && g.N % (64 * forced_nj) == 0 && !(forced_nj == 3 && g.epi.kind == LG_EPI_BIAS_GEGLU)) best_nj = forced_nj;
    if (!best_nj) return LG_OK;
    *handled = true;
    const int tiles_n = g.N / (64 * best_nj) * grp.count;
    int rc;
    if (wlayout == W_TILED) {
        if (best_nj == 4) rc = launch_fast_epi<W_TILED, 4>(g, grp, tiles_m, tiles_n, si, stream);
        else if (best_nj == 3) rc = launch_fast_epi<W_TILED, 3>(g, grp, tiles_m, tiles_n, si, stream);
        else rc = launch_fast_epi<W_TILED, 2>(g, grp, tiles_m, tiles_n, si, stream);
    } else if (wlayout == W_NK) {
        if (best_nj == 4) rc = launch_fast_epi<W_NK, 4>(g, grp, tiles_m, tiles_n, si, stream);
        else if (best_nj == 3) rc = launch_fast_epi<W_NK, 3>(g, grp, tiles_m, tiles_n, si, stream);
        else rc = launch_fast_epi<W_NK, 2>(g, grp, tiles_m, tiles_n, si, stream);
    } else {
        if (best_nj == 4) rc = launch_fast_epi<W_KN, 4>(g, grp, tiles_m, tiles_n, si, stream);
        else if (best_nj == 3) rc = launch_fast_epi<W_KN, 3>(g, grp, tiles_m, tiles_n, si, stream);
        else rc = launch_fast_epi<W_KN, 2>(g, grp, tiles_m, tiles_n, si, stream);
    }
    return rc != LG_OK ? rc : check_launch("gemm_f16_fast");
}

}  // namespace lg
