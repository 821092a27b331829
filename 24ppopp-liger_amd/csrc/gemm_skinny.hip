// gemm_skinny.hip -- weight-streaming fp16 GEMM for few tokens (decode: M <= 64) on gfx950.
//
//   Y[M, N] = X[M, K] * W^T with W stored [N, K] (both operands K-contiguous), M <= 64.
// With a handful of token rows every weight byte is used for 2*M flops only, so the kernel is a pure HBM stream of W
// (1.4 GB per GLM-130B TP=2 layer shard) and is organised like one:
//   * as few blocks as fill the chip (one block of 4 waves keeps 64 KiB of weight loads in flight, enough for one CU; more
//     blocks mean more K-slices, fp32 partials and reduce work).  If N alone gives >= 192 blocks of 64 (or 32) features, a
//     block walks the whole of K and applies the epilogue itself; otherwise a block = 4 waves x 32 features, the grid is
//     (N / 128) x S with the fewest K-slices S that give >= 192 blocks, and a second kernel sums the slices;
//   * W fragments go from global memory straight into MFMA operand registers (a lane owns 8 consecutive k of one output
//     feature: exactly the B operand of v_mfma_f32_16x16x32_f16) in a rolling pipeline that keeps 16 independent
//     16-byte loads in flight per lane at all times;
//   * the few X rows are staged once per 256-wide k-chunk in LDS (double buffered) and shared by the block's waves;
//   * K-slices (when there are any) are summed in fp32 through the stream's workspace and a small second kernel that also
//     applies the epilogue (bias / GELU / head-transposed store), so results match the single-pass kernels' rounding.
#include "gemm_common.hpp"

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
    // Blocks walk their chunks in rotated order (block b starts at chunk b mod nchunks and wraps around): with a
    // power-of-two row pitch (K = 16384) the blocks of a K-slice, which run in step, would otherwise all touch the same
    // memory channels at the same time (12288 x 16384 weight, 32 token rows: 97 -> 84 us).
    const int rot = blockIdx.x % nchunks;
    auto chunk_at = [&](int i) { const int c = rot + i; return c >= nchunks ? c - nchunks : c; };

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
    load_x(rot, xr);
    store_x(0, xr);
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        b0[s] = *reinterpret_cast<const half8_t*>(w0 + rot * SK_KC + s * 32);
        b1[s] = *reinterpret_cast<const half8_t*>(w1 + rot * SK_KC + s * 32);
    }
    __syncthreads();
    for (int ch = 0; ch < nchunks; ++ch) {
        const int buf = ch & 1;
        const int next = chunk_at(ch + 1 < nchunks ? ch + 1 : ch);
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

// ---- whole K in one block ------------------------------------------------------------------------------------------------
// When N alone gives enough work K is not sliced at all: a wave owns one 16-feature MFMA tile and walks the whole of K for it,
// the epilogue is applied to the accumulators, and there are no fp32 partials and no second kernel.  The 16-feature tiles of the
// problem (of all members of a group, which share X) are dealt out in runs of consecutive tiles to a grid of exactly one block per
// compute unit, NWV = ceil(tiles / CUs) waves a block, with the last wave having a tile only in the first blocks.  Every wave streams the same number of bytes, and one block per compute unit measured
// fastest (32 token rows, 256 CUs: 12288 features as 256 blocks of 3 waves 75.7 us at K = 16384 and 25.8 us at K = 6144, as 192
// blocks of 4 waves 86.1 and 29.7 us).
// A wave's rolling pipeline is DEPTH chunks deep (8 loads per chunk): two chunks for blocks of 3 to 8 waves, four chunks for the
// 2-wave block, which then keeps the 64 KiB of a 4-wave block in flight.
// TILED: the weights are stored as 16 x 32 fragment blocks (W_TILED): a wave's fragments are consecutive KiBs of one sequential
// stream, every load instruction covers whole 128-byte lines, and the loads are marked non-temporal (the weights of a decode
// step are read once per step and are far larger than any cache).  On the [N, K] layout the same hint costs 15-40 %: there a
// fragment is half a line per row, and a line that is not kept is fetched twice.  12288 x 16384 weight at 32 rows: 76.8 -> 63.0 us.
template <int MT, int EPI, int NWV, int DEPTH, bool TILED>
__global__ __launch_bounds__(64 * NWV) void gemm_skinny_direct_kernel(GemmArgs g, GemmGroup grp, RowMap rm, int tiles_per_member) {
    constexpr int THREADS = 64 * NWV;
    __shared__ __attribute__((aligned(16))) half_t xs[2][16 * MT * SK_XS];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, lk = lane >> 4;
    // the tiles of all members, laid end to end, are dealt out in runs of consecutive tiles: the first `full` blocks take NWV
    // tiles each, the others NWV - 1; a wave without a tile keeps the block's loads, barriers and arithmetic but reads one and
    // the same weight chunk over and over (cache hits) and stores nothing
    const int tiles = tiles_per_member * grp.count;
    const int full = tiles - (NWV - 1) * (int)gridDim.x;  // 1 .. gridDim.x (the launcher's choice of grid and NWV)
    const int b = blockIdx.x;
    const int tile = b * (NWV - 1) + min(b, full) + wave;
    const bool active = wave < NWV - 1 || b < full;
    const int member = min(tile / tiles_per_member, grp.count - 1);
    const int n0 = active ? (tile - member * tiles_per_member) * 16 : 0;
    const int wstep = active ? SK_KC : 0;
    if (grp.count > 1) {
        g.W = grp.W[member];
        g.Y = grp.Y[member];
        g.epi.bias = grp.bias[member];
        g.ldy = grp.ldy[member];
        g.epi.rows = grp.rows[member];
    }
    const int nchunks = g.K / SK_KC;  // a multiple of DEPTH (the launcher checks)
    const int rot = blockIdx.x % nchunks;  // rotated chunk order, see gemm_skinny_nk_kernel
    auto chunk_at = [&](int i) { int c = rot + i; while (c >= nchunks) c -= nchunks; return c; };

    // X chunk = 16 MT rows x 32 vectors of 8 halves, spread over the block's threads; when that does not divide evenly (6
    // waves) the last threads fetch and store the last vector once more, which keeps every load unconditional
    constexpr int XTOT = 16 * MT * (SK_KC / 8);
    constexpr int XV = (XTOT + THREADS - 1) / THREADS;
    const half_t* xsrc[XV];
#pragma unroll
    for (int u = 0; u < XV; ++u) {
        const int v = min(tid + u * THREADS, XTOT - 1);
        const int row = min(v / (SK_KC / 8), g.M - 1), c = v % (SK_KC / 8);
        xsrc[u] = g.X + (int64_t)row * g.ldx + c * 8;
    }
    auto load_x = [&](int chunk, half8_t (&xr)[XV]) {
#pragma unroll
        for (int u = 0; u < XV; ++u) xr[u] = *reinterpret_cast<const half8_t*>(xsrc[u] + chunk * SK_KC);
    };
    auto store_x = [&](int buf, const half8_t (&xr)[XV]) {
#pragma unroll
        for (int u = 0; u < XV; ++u) {
            const int v = min(tid + u * THREADS, XTOT - 1);
            const int row = v / (SK_KC / 8), c = v % (SK_KC / 8);
            *reinterpret_cast<half8_t*>(&xs[buf][row * SK_XS + c * 8]) = xr[u];
        }
    };

    float4_t acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};

    // [N, K]: this lane's weight row (rows beyond N are clamped, never stored), fragments 32 halves apart, chunks 256 apart;
    // tiled: this lane's 16 bytes of the feature tile's first block, fragments one block (512 halves) apart, chunks 8 blocks
    const half_t* w0 = TILED ? g.W + (int64_t)n0 * g.ldw + lane * 8 : g.W + (int64_t)min(n0 + l16, g.N - 1) * g.ldw + lk * 8;
    constexpr int FSTEP = TILED ? 512 : 32, CMUL = TILED ? 16 : 1;
    auto wload = [](const half_t* p) {
        return TILED ? __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(p)) : *reinterpret_cast<const half8_t*>(p);
    };

    // bf[d]: the weight fragments of chunks d, d + DEPTH, ...; xq[p]: token rows on their way to LDS, fetched two chunks
    // ahead (loads complete in order: waiting for rows fetched only one chunk ahead would also wait for all but the last 8
    // weight loads, i.e. drain the pipeline at every chunk)
    half8_t bf[DEPTH][8], xq[2][XV];
    // the prologue issues its loads in the order the loop would have (W(c) DEPTH chunks and X(c) two chunks before chunk c),
    // so that the compiler's count of outstanding loads at the loop head is exact
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        if (d == DEPTH - 2) load_x(chunk_at(0), xq[0]);
        if (d == DEPTH - 1) load_x(chunk_at(1), xq[1]);
#pragma unroll
        for (int s = 0; s < 8; ++s) bf[d][s] = wload(w0 + chunk_at(d) * wstep * CMUL + s * FSTEP);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    }
    store_x(0, xq[0]);
    __syncthreads();
    // one chunk: multiply its 8 fragments (registers b) with the X chunk in LDS buffer `buf`, reloading each pair of
    // fragments' registers with the chunk DEPTH ahead as soon as both have been used; at its end the X chunk fetched one chunk ago goes
    // to the other LDS buffer.  Chunks past the
    // end wrap around to valid addresses and are never multiplied.
    auto do_chunk = [&](int ch, int buf, half8_t (&b)[8]) {
        load_x(chunk_at(ch + 2), xq[buf]);
        const half_t* wn = w0 + chunk_at(ch + DEPTH) * wstep * CMUL;
        // compiler-only fences keep every load where it is written (left alone, the compiler moves the X loads to the end
        // of the chunk, right in front of the LDS stores that wait for them)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < 8; ++s) {
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const half8_t a = *reinterpret_cast<const half8_t*>(&xs[buf][(i * 16 + l16) * SK_XS + s * 32 + lk * 8]);
                acc[i] = mfma16(b[s], a, acc[i]);  // operands swapped: acc[i][r] = Y[16 i + l16][n0 + 4 lk + r]
            }
            // a fragment is one 64-byte half of a 128-byte weight line per row: both halves are requested back to back,
            // after the second has been used (requested a fragment apart they reach the L2 as two separate half-line reads)
            if (s & 1) {
                b[s - 1] = wload(wn + (s - 1) * FSTEP);
                b[s] = wload(wn + s * FSTEP);
            }
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
        }
        store_x(buf ^ 1, xq[buf ^ 1]);
        __syncthreads();
    };
    for (int ch = 0; ch < nchunks; ch += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) do_chunk(ch + d, d & 1, bf[d]);
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
        if (active) epilogue_store4<EPI>(g, g.Y, i * 16 + l16, n0 + 4 * lk, acc[i], true, &rm);
}

template <int MT, int NWV, int DEPTH, bool TILED>
static void launch_direct(const GemmArgs& g, const GemmGroup& grp, const RowMap& rm, int nblocks, hipStream_t stream) {
    const dim3 grid(nblocks), block(64 * NWV);
    const int tpm = (g.N + 15) / 16;
    switch (g.epi.kind) {
        case LG_EPI_NONE: hipLaunchKernelGGL((gemm_skinny_direct_kernel<MT, LG_EPI_NONE, NWV, DEPTH, TILED>), grid, block, 0, stream, g, grp, rm, tpm); break;
        case LG_EPI_BIAS: hipLaunchKernelGGL((gemm_skinny_direct_kernel<MT, LG_EPI_BIAS, NWV, DEPTH, TILED>), grid, block, 0, stream, g, grp, rm, tpm); break;
        case LG_EPI_BIAS_GELU: hipLaunchKernelGGL((gemm_skinny_direct_kernel<MT, LG_EPI_BIAS_GELU, NWV, DEPTH, TILED>), grid, block, 0, stream, g, grp, rm, tpm); break;
        case LG_EPI_BIAS_HEADS_ROWS: hipLaunchKernelGGL((gemm_skinny_direct_kernel<MT, LG_EPI_BIAS_HEADS_ROWS, NWV, DEPTH, TILED>), grid, block, 0, stream, g, grp, rm, tpm); break;
        default: hipLaunchKernelGGL((gemm_skinny_direct_kernel<MT, LG_EPI_BIAS_HEADS, NWV, DEPTH, TILED>), grid, block, 0, stream, g, grp, rm, tpm); break;
    }
}
template <int NWV, int DEPTH, bool TILED>
static void launch_direct_mt(const GemmArgs& g, const GemmGroup& grp, const RowMap& rm, int nblocks, hipStream_t stream) {
    switch ((g.M + 15) / 16) {
        case 1: launch_direct<1, NWV, DEPTH, TILED>(g, grp, rm, nblocks, stream); break;
        case 2: launch_direct<2, NWV, DEPTH, TILED>(g, grp, rm, nblocks, stream); break;
        case 3: launch_direct<3, NWV, DEPTH, TILED>(g, grp, rm, nblocks, stream); break;
        default: launch_direct<4, NWV, DEPTH, TILED>(g, grp, rm, nblocks, stream); break;
    }
}
template <bool TILED>
static void launch_direct_nwv(int nwv, const GemmArgs& g, const GemmGroup& grp, const RowMap& rm, int nblocks, hipStream_t stream) {
    switch (nwv) {
        case 2: launch_direct<1, 2, 4, TILED>(g, grp, rm, nblocks, stream); break;
        case 3: launch_direct_mt<3, 2, TILED>(g, grp, rm, nblocks, stream); break;
        case 4: launch_direct_mt<4, 2, TILED>(g, grp, rm, nblocks, stream); break;
        case 5: launch_direct_mt<5, 2, TILED>(g, grp, rm, nblocks, stream); break;
        case 6: launch_direct_mt<6, 2, TILED>(g, grp, rm, nblocks, stream); break;
        default: launch_direct_mt<8, 2, TILED>(g, grp, rm, nblocks, stream); break;
    }
}

// sums the K-slices and applies the epilogue; one thread per 4 consecutive output columns
template <int EPI>
__global__ __launch_bounds__(256) void gemm_skinny_reduce_kernel(GemmArgs g, const float* partial, int nsplit, RowMap rm) {
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
        epilogue_store4<EPI>(g, g.Y, m, n, s, true, &rm);
    }
}

// GeGLU: one thread per 4 consecutive OUTPUT columns; it sums the slices of the gate quad and of the up quad 16 features on
__global__ __launch_bounds__(256) void gemm_skinny_reduce_geglu_kernel(GemmArgs g, const float* partial, int nsplit) {
    const int nq = g.N / 8;  // output quads per token row (N % 32 == 0)
    const int64_t quads = (int64_t)g.M * nq;
    for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < quads; q += (int64_t)gridDim.x * blockDim.x) {
        const int m = (int)(q / nq), c = (int)(q % nq) * 4;
        const int n = (c >> 4) * 32 + (c & 15);
        float4_t sg = float4_t{0.f, 0.f, 0.f, 0.f}, su = float4_t{0.f, 0.f, 0.f, 0.f};
        for (int sp = 0; sp < nsplit; ++sp) {
            const float* p = partial + ((int64_t)sp * g.M + m) * g.N + n;
            sg += *reinterpret_cast<const float4_t*>(p);
            su += *reinterpret_cast<const float4_t*>(p + 16);
        }
        epilogue_geglu4(g, g.Y, m, n, sg, su, (g.ldy % 4 == 0) && aligned_dev16(g.Y));
    }
}

void launch_splitk_reduce(const GemmArgs& g, const float* partial, int nsplit, hipStream_t stream, const RowMap* rows) {
    const dim3 block(256);
    if (g.epi.kind == LG_EPI_BIAS_GEGLU) {
        const int64_t gq = (int64_t)g.M * (g.N / 8);
        int gg = (int)((gq + 255) / 256);
        if (gg > 4096) gg = 4096;
        hipLaunchKernelGGL(gemm_skinny_reduce_geglu_kernel, dim3(gg), block, 0, stream, g, partial, nsplit);
        return;
    }
    const int64_t quads = (int64_t)g.M * ((g.N + 3) / 4);
    int rgrid = (int)((quads + 255) / 256);
    if (rgrid > 4096) rgrid = 4096;
    const RowMap rm = rows ? *rows : RowMap{};
    switch (g.epi.kind) {
        case LG_EPI_NONE: hipLaunchKernelGGL((gemm_skinny_reduce_kernel<LG_EPI_NONE>), dim3(rgrid), block, 0, stream, g, partial, nsplit, rm); break;
        case LG_EPI_BIAS: hipLaunchKernelGGL((gemm_skinny_reduce_kernel<LG_EPI_BIAS>), dim3(rgrid), block, 0, stream, g, partial, nsplit, rm); break;
        case LG_EPI_BIAS_GELU: hipLaunchKernelGGL((gemm_skinny_reduce_kernel<LG_EPI_BIAS_GELU>), dim3(rgrid), block, 0, stream, g, partial, nsplit, rm); break;
        case LG_EPI_BIAS_HEADS_ROWS: hipLaunchKernelGGL((gemm_skinny_reduce_kernel<LG_EPI_BIAS_HEADS_ROWS>), dim3(rgrid), block, 0, stream, g, partial, nsplit, rm); break;
        default: hipLaunchKernelGGL((gemm_skinny_reduce_kernel<LG_EPI_BIAS_HEADS>), dim3(rgrid), block, 0, stream, g, partial, nsplit, rm); break;
    }
}

// grp.count > 1: handled only if the unsliced kernels apply (the caller then falls back to one launch per member)
int launch_gemm_skinny_f16(const GemmArgs& g, const GemmGroup& grp, const RowMap* rows, int wlayout, int batch, hipStream_t stream, bool* handled) {
    *handled = false;
    if (batch != 1 || (wlayout != W_NK && wlayout != W_TILED)) return LG_OK;
    if (g.M <= 0 || g.M > 64 || g.N < 512 || g.K < 1024 || (g.K % SK_KC) || (g.N % 4)) return LG_OK;
    if (wlayout == W_TILED && ((g.N % 16) || g.ldw != g.K)) return LG_OK;
    if (!aligned16(g.X) || (g.ldx % 8) || (g.ldw % 8) || !group_aligned(g, grp)) return LG_OK;
    if (g.epi.kind == LG_EPI_BIAS_HEADS_ROWS && !rows) return LG_OK;
    const RowMap rm = rows ? *rows : RowMap{};
    const int mt = (g.M + 15) / 16;
    // GeGLU pairs features 16 apart, which sit in different waves of the unsliced kernel: such problems take the sliced kernel
    // below (one slice when N alone fills the chip), whose reduce step forms the product
    const bool geglu = g.epi.kind == LG_EPI_BIAS_GEGLU;
    const StreamInfo si = stream_info(stream);
    const int cus = si.cus;  // compute units this stream's kernels run on: "one round of blocks" means this many
    // Unsliced: the 16-feature tiles are dealt to one block per compute unit of the stream, 2 to 8 waves a block (the partly
    // filled last wave sits in the first blocks only).  That needs enough tiles to give most compute units two waves, whole
    // pipeline depths of chunks, and for the 2-wave block (four chunks deep) registers for one row tile only.  Problems with more
    // tiles than 8 waves a block take many rounds of 4-wave blocks, where the partial last round no longer matters.
    {
        const int tiles = (g.N + 15) / 16 * grp.count;
        int nwv = (tiles + cus - 1) / cus, nblocks = cus;
        if (nwv > 8 && tiles >= 16 * cus) { nwv = 4; nblocks = (tiles + 3) / 4; }
        if (nwv == 7) { nwv = 8; nblocks = (tiles + 7) / 8; }
        const bool deep = nwv == 2;
        if (!geglu && nwv >= 2 && nwv <= 8 && tiles >= cus * 3 / 2 && g.K % ((deep ? 4 : 2) * SK_KC) == 0 && (!deep || mt == 1) &&
            (int64_t)(nwv - 1) * nblocks < tiles && tiles <= (int64_t)nwv * nblocks) {  // what the kernel's dealing assumes
            *handled = true;
            if (wlayout == W_TILED) launch_direct_nwv<true>(nwv, g, grp, rm, nblocks, stream);
            else launch_direct_nwv<false>(nwv, g, grp, rm, nblocks, stream);
            return check_launch("gemm_f16_skinny");
        }
    }
    if (wlayout == W_TILED) return LG_OK;  // the K-sliced kernel below reads [N, K] rows
    if (grp.count > 1 || g.epi.kind == LG_EPI_BIAS_HEADS_ROWS) return LG_OK;  // the sliced kernels take plain single problems only
    const int nblk = (g.N + SK_BN - 1) / SK_BN;
    // K-slices: as few as fill the chip.  One block of 4 waves keeps 64 KiB of weight loads in flight, which is enough for one
    // CU; more slices only add fp32 partials and reduce work (six GEMMs of a decode step at 32 token rows on 256 CUs: 344 us
    // with >= 1024 blocks, 315 us with >= 256, 289 us with >= 192, 336 us with >= 128).  Slices are multiples of the 256-wide
    // chunk, and no more than the stream's workspace holds; a stream without a workspace leaves the problem to the generic kernel.
    if (!si.ws) return LG_OK;
    int nsplit = 1;
    while (nblk * nsplit < cus * 3 / 4 && (g.K / (nsplit * 2)) >= 2 * SK_KC && nsplit < 32) nsplit *= 2;
    const size_t slice_bytes = (size_t)g.M * g.N * sizeof(float);
    while (nsplit > 1 && (size_t)nsplit * slice_bytes > si.ws_bytes) nsplit /= 2;
    if (slice_bytes > si.ws_bytes) return LG_OK;
    int kslice = ((g.K + nsplit - 1) / nsplit + SK_KC - 1) / SK_KC * SK_KC;
    nsplit = (g.K + kslice - 1) / kslice;
    float* ws = si.ws;
    *handled = true;
    const dim3 grid(nblk, nsplit), block(256);
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
