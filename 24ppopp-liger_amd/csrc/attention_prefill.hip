// attention_prefill.hip -- fused LDS-tiled prefill attention for gfx950 (flash-style, online softmax).
//
// Replaces the reference's qk_gemm -> attn_softmax -> qkv_gemm (-> transpose) sequence (bert_layer.h:145-168) and
// keeps its softmax semantics: t = q.k * scalar + (1 - mask) * (-10000), p = exp(t - max t), out = sum p v / (sum p +
// 1e-6).  The S x S score matrix never touches HBM.
//
// Work split: one block = 32 NW queries of one (batch, head), NW waves x 32 queries (NW = 4; blocks of 8 waves halve the tile
// loads per query and measure the same).  K and V tiles of 64 keys go from global
// memory straight into LDS (direct-to-LDS loads, no VGPR staging) into a ring of two tiles each: the loads of tile t+1 are
// issued right after the barrier that publishes tile t and run under tile t's MFMAs, one barrier per tile.  The LDS position of a
// lane's 16 bytes is fixed by the load instruction, so the tiles are made bank-conflict-free by rotating, through the global
// address each lane loads from, the 16-byte chunks (K) or 32-byte blocks (V) of row r by r places: the 16 rows that one
// fragment read touches then fall into 16 different bank groups.  Rows beyond the sequence are read from its last row and
// masked out of the softmax.  Everything is computed transposed so that no cross-lane data movement is needed between the two GEMMs:
//   S^T[key, q] = K[key, :] . Q[q, :]      A = K tile (16-byte LDS reads), B = Q (registers, loaded once)
//   O^T[d, q]  += V^T[d, key] * P^T[key, q] A = V tile through the gfx950 transposed LDS read, B = P^T, which is
//                                           exactly the accumulator layout S^T came out in (4 consecutive keys per
//                                           lane), so the probabilities go from MFMA result to MFMA operand in place.
// Softmax statistics are per query = per (lane % 16); the four 16-lane groups hold different keys and are combined
// with two row swaps per tile.
#include "gemm_common.hpp"

namespace lg {

constexpr int PF_BC = 64;   // keys per LDS tile

// max(x, x of lane ^ 16) and max(x, x of lane ^ 32) through the gfx950 row-swap instructions: with both operands holding
// x, v_permlane16_swap leaves {row 0, row 0, row 2, row 2} in the first and {row 1, row 1, row 3, row 3} in the second
// (rows of 16 lanes), v_permlane32_swap {low half, low half} and {high half, high half}.  Plain VALU operations: no trip
// through the LDS crossbar (ds_bpermute) in the middle of the softmax's dependent chain.
typedef unsigned uint2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float max_of_swapped(uint2_t r) {
    float m;
    asm("v_max_f32 %0, %1, %2" : "=v"(m) : "v"(r[0]), "v"(r[1]));  // by hand: fmaxf would first canonicalise both bit-cast inputs
    return m;
}
__device__ __forceinline__ float max_xor16(float x) {
    const unsigned u = __float_as_uint(x);
    return max_of_swapped(__builtin_amdgcn_permlane16_swap(u, u, false, false));
}
__device__ __forceinline__ float max_xor32(float x) {
    const unsigned u = __float_as_uint(x);
    return max_of_swapped(__builtin_amdgcn_permlane32_swap(u, u, false, false));
}

template <int D, int NW, bool CAUSAL, bool HAS_MASK>
// two waves per SIMD (at most 256 registers): the softmax arithmetic of one wave runs under the MFMAs of the other
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void attn_prefill_kernel(const half_t* __restrict__ q_buf, const half_t* __restrict__ k_buf,
                                                           const half_t* __restrict__ v_buf, const half_t* __restrict__ mask,
                                                           half_t* out, int seq, int head_num, int kv_rows, float scalar,
                                                           int out_layout, int q_off) {
    constexpr int DC = D / 32;      // 32-wide d chunks (k steps of the S^T GEMM)
    constexpr int DT = D / 16;      // 16-wide d tiles (rows of O^T)
    constexpr int CPR = D / 8;      // 16-byte chunks per row
    constexpr int BPR = D / 16;     // 32-byte blocks per row
    constexpr int TILE = PF_BC * D; // halves per tile
    constexpr int PF_BQ = 32 * NW;  // queries per block
    constexpr int LPT = TILE / 8 / (64 * NW);  // direct-to-LDS loads per thread and tile (K and V each)
    static_assert(TILE % (8 * 64 * NW) == 0, "a tile must be a whole number of 1 KiB wave loads per wave");
    __shared__ __attribute__((aligned(16))) half_t Ks[2][TILE];
    __shared__ __attribute__((aligned(16))) half_t Vs[2][TILE];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, g = lane >> 4;
    // Workgroups are handed to the 8 XCDs round-robin by their linear id.  All query blocks of one (batch, head) go to ONE
    // XCD: without a causal mask one after the other (they read the same K/V rows, which that XCD's L2 then serves); with it,
    // ordered by their length (below), which costs the L2 re-use (K/V are then fetched about 2.5 times, from the memory-side
    // cache) and gains an even finish.
    int bh = blockIdx.y, qblk = blockIdx.x;    // bh = b * head_num + head
    if ((gridDim.y & 7) == 0) {
        const int lin = blockIdx.x + gridDim.x * blockIdx.y;
        const int xcd = lin & 7, slot = lin >> 3;
        if (CAUSAL) {
            // a causal query block's work grows with its position: every XCD starts the last (longest) query block of all its
            // heads first, then the one before, ... so that the blocks still running at the end are the short ones
            const int per_xcd = (int)gridDim.y >> 3;
            bh = (slot % per_xcd) * 8 + xcd;
            qblk = (int)gridDim.x - 1 - slot / per_xcd;
        } else {
            bh = (slot / (int)gridDim.x) * 8 + xcd;
            qblk = slot % (int)gridDim.x;
        }
    }
    const int b = bh / head_num, head = bh % head_num;
    const int q0 = qblk * PF_BQ;               // first query of the block
    const int qw = q0 + wave * 32;             // first query of the wave
    // q_off > 0: the `seq` queries are positions q_off .. q_off + seq - 1 of a sequence whose first q_off keys and values are
    // already in k_buf / v_buf (a prefill continued in chunks over a KV cache); keys 0 .. kv_len - 1 exist
    const int kv_len = q_off + seq;
    const int qwa = q_off + qw;                // absolute position of the wave's first query

    const half_t* Q = q_buf + (int64_t)bh * seq * D;
    const half_t* K = k_buf + (int64_t)bh * kv_rows * D;
    const half_t* V = v_buf + (int64_t)bh * kv_rows * D;

    // position of logical chunk c (K) / block blk (V) in row r of a tile
    constexpr bool P2 = (CPR & (CPR - 1)) == 0;   // power-of-two row: 16 rows further on the rotation is the same again
    auto kpos = [](int r, int c) { return P2 ? ((c + r) & (CPR - 1)) : (c + r) % CPR; };
    auto vpos = [](int r, int blk) { return P2 ? ((blk + r) & (BPR - 1)) : (blk + r) % BPR; };
    // LDS offsets (in halves) of this lane's fragment reads.  With a power-of-two row the rotation of rows r and r + 16 is the
    // same, so one offset per d-chunk serves every 16-row group (the group's distance folds into the instruction's offset field).
    constexpr int KG = P2 ? 1 : 4, VG = P2 ? 1 : 4;
    int kfrag[KG][DC], vfrag[VG][DT];
#pragma unroll
    for (int kt = 0; kt < KG; ++kt)
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) kfrag[kt][dc] = (kt * 16 + l16) * D + kpos(kt * 16 + l16, dc * 4 + g) * 8;
#pragma unroll
    for (int vg = 0; vg < VG; ++vg)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const int row = vg * 16 + 4 * g + (l16 >> 2);
            vfrag[vg][dt] = row * D + vpos(row, dt) * 16 + 4 * (l16 & 3);
        }

    // this thread's loads of one tile: LDS chunk f = (i * 4 + wave) * 64 + lane sits in row f / CPR at position f % CPR and must
    // receive the logical chunk that belongs there
    int lrow[LPT];
    unsigned koff[LPT], voff[LPT];
#pragma unroll
    for (int i = 0; i < LPT; ++i) {
        const int f = (i * NW + wave) * 64 + lane;
        const int r = f / CPR, p = f % CPR;
        lrow[i] = r;
        const int kc = (p - r % CPR + CPR) % CPR;                       // kpos(r, kc) == p
        const int vb = ((p >> 1) - r % BPR + BPR) % BPR;                // vpos(r, vb) == p >> 1
        koff[i] = (unsigned)(kc * 8);
        voff[i] = (unsigned)((vb * 2 + (p & 1)) * 8);
    }
    auto issue = [&](int k0, int buf) {
#pragma unroll
        for (int i = 0; i < LPT; ++i) {
            const int64_t row = min(k0 + lrow[i], kv_len - 1);          // rows beyond the sequence: its last row, masked later
            load_lds16(K + row * D + koff[i], &Ks[buf][(i * NW + wave) * 512]);
            load_lds16(V + row * D + voff[i], &Vs[buf][(i * NW + wave) * 512]);
        }
    };

    // Q fragments: qf[qt][dc] = Q[qw + qt*16 + l16][dc*32 + 8g .. +8]
    half8_t qf[2][DC];
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        const int q = qw + qt * 16 + l16;
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) {
            if (q < seq) qf[qt][dc] = *reinterpret_cast<const half8_t*>(Q + (int64_t)q * D + dc * 32 + g * 8);
            else qf[qt][dc] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        }
    }

    float4_t o[DT][2];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) o[dt][qt] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_run[2] = {-1e30f, -1e30f};
    float l_run[2] = {0.f, 0.f};  // per-lane partial sums (this lane's keys only)

    const float sl2 = scalar * 1.4426950408889634f;            // scores in log2 units
    constexpr float MASK_L2 = -10000.0f * 1.4426950408889634f;  // the reference's additive mask term, in the same units
    const int kv_end = CAUSAL ? min(kv_len, q_off + q0 + PF_BQ) : kv_len;
    issue(0, 0);
    for (int k0 = 0, t = 0; k0 < kv_end; k0 += PF_BC, ++t) {
        const int buf = t & 1;
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // this thread's part of tile t has landed
        barrier_keep_loads_in_flight();  // tile t is visible to every wave, and every wave is done with tile t-1: its buffer is refilled now
        if (k0 + PF_BC < kv_end) issue(k0 + PF_BC, buf ^ 1);
        // a wave whose queries all lie before this key tile has nothing to do here (causal), but keeps loading and hitting
        // the barrier, so only the math is skipped
        if (CAUSAL && k0 > qwa + 31) continue;
        const half_t* ks = Ks[buf];
        const half_t* vs = Vs[buf];

        // ---- S^T = K Q^T ------------------------------------------------------------------------------------
        // The LDS reads of this loop are issued by hand (lds_read16_issue / lds_read_tr4_issue): the compiler would put a wait
        // for the loads of the NEXT tile, issued just above, in front of every read of THIS tile.  The fragments of key tile
        // kt + 1 are requested before the MFMAs of key tile kt.
        float4_t s[4][2];
        half8_t kf[2][DC];
        // one address register per d-chunk when the row is a power of two (the key tile's distance goes into the instruction)
        unsigned kbase[DC];
#pragma unroll
        for (int dc = 0; dc < DC; ++dc) kbase[dc] = lds_address(ks + kfrag[0][dc]);
        auto kissue = [&](auto ktc, int slot) {
            constexpr int kt = decltype(ktc)::value;
#pragma unroll
            for (int dc = 0; dc < DC; ++dc) {
                if constexpr (P2) lds_read16_issue_at<kt * 16 * D * 2>(kf[slot][dc], kbase[dc]);
                else lds_read16_issue(kf[slot][dc], &ks[kfrag[kt % KG][dc]]);
            }
        };
        kissue(std::integral_constant<int, 0>{}, 0);
        static_for<4>([&](auto ktc) {
            constexpr int kt = decltype(ktc)::value;
            constexpr int slot = kt & 1;
            if constexpr (kt + 1 < 4) kissue(std::integral_constant<int, kt + 1>{}, slot ^ 1);
            s[kt][0] = float4_t{0.f, 0.f, 0.f, 0.f};
            s[kt][1] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int dc = 0; dc < DC; ++dc) {
                if constexpr (kt + 1 < 4) lds_read16_wait<DC>(kf[slot][dc]);   // the DC reads of the next key tile may be outstanding
                else lds_read16_wait<0>(kf[slot][dc]);
                s[kt][0] = mfma16(kf[slot][dc], qf[0][dc], s[kt][0]);
                s[kt][1] = mfma16(kf[slot][dc], qf[1][dc], s[kt][1]);
            }
        });
        // ---- scale, mask, online softmax (per query column) -----------------------------------------------------
        // Scores are kept in log2 units (scale folded with log2 e: exp(t - m) = exp2(t' - m')), so that a score costs one
        // multiply, one max, one subtract, one exp2 and one add.  The causal comparison is only made on tiles that reach above
        // the diagonal of the wave's first query, the end-of-sequence test only on the last tile (both wave-uniform).
        const bool diag = CAUSAL && (k0 + PF_BC - 1 > qwa);
        const bool tail = k0 + PF_BC > kv_len;
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
            const int q = qw + qt * 16 + l16;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r) s[kt][qt][r] *= sl2;
            if (HAS_MASK) {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt) {
                    const int key = k0 + kt * 16 + 4 * g;
                    if (q < seq) {
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (key + r < seq) s[kt][qt][r] += (1.0f - (float)mask[((int64_t)b * seq + q) * seq + key + r]) * MASK_L2;
                    }
                }
            }
            if (diag) {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (k0 + kt * 16 + 4 * g + r > q_off + q) s[kt][qt][r] += MASK_L2;
            }
            if (tail) {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (k0 + kt * 16 + 4 * g + r >= kv_len) s[kt][qt][r] = -1e30f;  // beyond the sequence: not part of the row at all
            }
            float mx = -1e30f;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r) mx = fmaxf(mx, s[kt][qt][r]);
            mx = max_xor16(mx);
            mx = max_xor32(mx);
            const float m_new = fmaxf(m_run[qt], mx);
            const float corr = __builtin_amdgcn_exp2f(m_run[qt] - m_new);
            m_run[qt] = m_new;
            float ls = 0.f;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float p = __builtin_amdgcn_exp2f(s[kt][qt][r] - m_new);
                    s[kt][qt][r] = p;
                    ls += p;
                }
            l_run[qt] = l_run[qt] * corr + ls;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) o[dt][qt] *= corr;
        }
        // ---- O^T += V^T P^T ---------------------------------------------------------------------------------------
        unsigned vbase[DT];   // as for K: one address register per d-tile when the row is a power of two
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vbase[dt] = lds_address(vs + vfrag[0][dt]);
        static_for<2>([&](auto jc) {  // two k-steps of 32 keys: key tiles 2j and 2j+1
            constexpr int j = decltype(jc)::value;
            half8_t pf[2];
#pragma unroll
            for (int qt = 0; qt < 2; ++qt) {
                const float4_t lo = s[2 * j][qt], hi = s[2 * j + 1][qt];
                pf[qt] = half8_t{(half_t)lo[0], (half_t)lo[1], (half_t)lo[2], (half_t)lo[3],
                                 (half_t)hi[0], (half_t)hi[1], (half_t)hi[2], (half_t)hi[3]};
            }
            // The transposed reads are issued by hand (the builtin would make the compiler wait for the
            // loads of the NEXT tile, issued above, before every read), a group of VGRP fragments ahead of the MFMAs that use
            // them: logical 32-byte block dt of rows 32 j + 4 g + l16 / 4 and 16 rows further on, this lane's 8 bytes inside it.
            constexpr int VGRP = 2;
            static_assert(DT % VGRP == 0, "head size must be a multiple of 32");
            half4_t vlo[2][VGRP], vhi[2][VGRP];
            auto vissue = [&](int grp, int slot) {
#pragma unroll
                for (int i = 0; i < VGRP; ++i) {
                    const int dt = grp * VGRP + i;
                    if constexpr (P2) {
                        lds_read_tr4_issue_at<(2 * j) * 16 * D * 2>(vlo[slot][i], vbase[dt]);
                        lds_read_tr4_issue_at<(2 * j + 1) * 16 * D * 2>(vhi[slot][i], vbase[dt]);
                    } else {
                        lds_read_tr4_issue(vlo[slot][i], &vs[vfrag[(2 * j) % VG][dt]]);
                        lds_read_tr4_issue(vhi[slot][i], &vs[vfrag[(2 * j + 1) % VG][dt]]);
                    }
                }
            };
            vissue(0, 0);
#pragma unroll
            for (int grp = 0; grp < DT / VGRP; ++grp) {
                const int slot = grp & 1;
                if (grp + 1 < DT / VGRP) vissue(grp + 1, slot ^ 1);
#pragma unroll
                for (int i = 0; i < VGRP; ++i) {
                    // the reads of the next group (2 VGRP of them) may still be outstanding
                    if (grp + 1 < DT / VGRP) lds_tr_wait<2 * VGRP>(vlo[slot][i], vhi[slot][i]);
                    else lds_tr_wait<0>(vlo[slot][i], vhi[slot][i]);
                    const half8_t a = join_half4(vlo[slot][i], vhi[slot][i]);
                    const int dt = grp * VGRP + i;
                    o[dt][0] = mfma16(a, pf[0], o[dt][0]);
                    o[dt][1] = mfma16(a, pf[1], o[dt][1]);
                }
            }
        });
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // ---- normalise and store ----------------------------------------------------------------------------------------
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
        float l = l_run[qt];
        l += __shfl_xor(l, 16, 64);
        l += __shfl_xor(l, 32, 64);
        const float inv = 1.0f / (l + 1e-6f);
        const int q = qw + qt * 16 + l16;
        if (q >= seq) continue;
        half_t* dst = (out_layout == 1) ? out + (((int64_t)b * seq + q) * head_num + head) * D
                                        : out + ((int64_t)bh * seq + q) * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const float4_t v = o[dt][qt];
            const half4_t h = {(half_t)(v[0] * inv), (half_t)(v[1] * inv), (half_t)(v[2] * inv), (half_t)(v[3] * inv)};
            *reinterpret_cast<half4_t*>(dst + dt * 16 + 4 * g) = h;
        }
    }
}

template <int D, int NW>
static void launch_prefill(const half_t* q, const half_t* k, const half_t* v, const half_t* mask, half_t* out, int batch,
                           int seq, int head_num, int kv_rows, float scalar, int causal, int out_layout, int q_off, hipStream_t st) {
    constexpr int BQ = 32 * NW;
    dim3 grid((seq + BQ - 1) / BQ, batch * head_num), block(64 * NW);
    if (causal)
        hipLaunchKernelGGL((attn_prefill_kernel<D, NW, true, false>), grid, block, 0, st, q, k, v, mask, out, seq, head_num, kv_rows, scalar, out_layout, q_off);
    else if (mask)
        hipLaunchKernelGGL((attn_prefill_kernel<D, NW, false, true>), grid, block, 0, st, q, k, v, mask, out, seq, head_num, kv_rows, scalar, out_layout, q_off);
    else
        hipLaunchKernelGGL((attn_prefill_kernel<D, NW, false, false>), grid, block, 0, st, q, k, v, mask, out, seq, head_num, kv_rows, scalar, out_layout, q_off);
}

}  // namespace lg

using namespace lg;

static int attn_prefill_entry(const char* what, const void* q_buf, const void* k_buf, const void* v_buf, const void* attr_mask,
                              void* out, int batch, int seq, int past, int head_num, int size_per_head, int kv_rows,
                              float scalar, int causal, int out_layout, void* stream) {
    if (batch < 0 || seq < 0 || past < 0 || head_num <= 0 || (int64_t)past + seq > kv_rows || (out_layout != 0 && out_layout != 1)) {
        set_error("%s: bad shape (seq=%d past=%d kv_rows=%d)", what, seq, past, kv_rows);
        return LG_ERR_INVALID;
    }
    if (past > 0 && attr_mask) { set_error("%s: an explicit mask covers [seq, seq] positions only; past > 0 needs causal or no mask", what); return LG_ERR_INVALID; }
    if (size_per_head != 64 && size_per_head != 96 && size_per_head != 128) { set_error("%s: size_per_head must be 64, 96 or 128", what); return LG_ERR_INVALID; }
    if (batch == 0 || seq == 0) return LG_OK;
    if (!q_buf || !k_buf || !v_buf || !out) { set_error("%s: null pointer", what); return LG_ERR_INVALID; }
    if (!aligned16(q_buf) || !aligned16(k_buf) || !aligned16(v_buf) || !aligned16(out)) {
        set_error("%s: pointers must be 16-byte aligned", what);
        return LG_ERR_INVALID;
    }
    if ((int64_t)batch * head_num > 65535) { set_error("%s: batch * head_num > 65535", what); return LG_ERR_INVALID; }
    scalar = (float)(half_t)scalar;
    if (size_per_head == 128)
        launch_prefill<128, 4>((const half_t*)q_buf, (const half_t*)k_buf, (const half_t*)v_buf, (const half_t*)attr_mask,
                            (half_t*)out, batch, seq, head_num, kv_rows, scalar, causal, out_layout, past, (hipStream_t)stream);
    else if (size_per_head == 96)
        launch_prefill<96, 4>((const half_t*)q_buf, (const half_t*)k_buf, (const half_t*)v_buf, (const half_t*)attr_mask,
                           (half_t*)out, batch, seq, head_num, kv_rows, scalar, causal, out_layout, past, (hipStream_t)stream);
    else
        launch_prefill<64, 4>((const half_t*)q_buf, (const half_t*)k_buf, (const half_t*)v_buf, (const half_t*)attr_mask,
                           (half_t*)out, batch, seq, head_num, kv_rows, scalar, causal, out_layout, past, (hipStream_t)stream);
    return check_launch(what);
}

extern "C" int lg_attn_prefill_f16(const void* q_buf, const void* k_buf, const void* v_buf, const void* attr_mask,
                                   void* out, int batch, int seq, int head_num, int size_per_head, int kv_rows,
                                   float scalar, int causal, int out_layout, void* stream) {
    return attn_prefill_entry("attn_prefill", q_buf, k_buf, v_buf, attr_mask, out, batch, seq, 0, head_num, size_per_head, kv_rows, scalar,
                              causal, out_layout, stream);
}

extern "C" int lg_attn_prefill_past_f16(const void* q_buf, const void* k_buf, const void* v_buf, void* out, int batch, int seq,
                                        int past, int head_num, int size_per_head, int kv_rows, float scalar, int causal,
                                        int out_layout, void* stream) {
    return attn_prefill_entry("attn_prefill_past", q_buf, k_buf, v_buf, nullptr, out, batch, seq, past, head_num, size_per_head, kv_rows,
                              scalar, causal, out_layout, stream);
}
