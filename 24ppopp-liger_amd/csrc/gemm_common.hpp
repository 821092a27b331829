// gemm_common.hpp -- operand descriptors, epilogues and MFMA helpers shared by the GEMM kernels.
//
// All kernels here use the row-major view of the reference's column-major cuBLAS calls:
//     Y[M, N] (ldy) = X[M, K] (ldx) * W,      W given either as [K, N] (W_KN) or as [N, K] (W_NK).
// M = tokens, N = output features, K = reduction.
#pragma once
#include <utility>

#include "common.hpp"

namespace lg {

// W_TILED: the [N, K] matrix cut into 16-feature x 32-k blocks, each stored as the 1 KiB an MFMA B operand of
// v_mfma_f32_16x16x32_f16 occupies in a wave's registers: lane l (feature l % 16, k-group l / 16) owns bytes [16 l, 16 l + 16)
// of its block = W[16 t + l % 16][32 c + 8 (l / 16) .. + 8); block (t, c) is block number t * (K / 32) + c.  A wave-wide
// 16-byte load of one block is one contiguous KiB, and the blocks a feature tile needs along k follow each other in memory:
// a weight-streaming kernel reads its weights as one sequential stream per wave (which is what lets it mark the loads
// non-temporal), a tile kernel copies blocks to LDS and reads fragments back without any swizzle.  Feature tile t starts
// 16 t * K elements into the matrix, exactly where row 16 t of the [N, K] layout starts, so sub-ranges and packed row blocks
// keep the pointer arithmetic of W_NK as long as they start at multiples of 16 features.  Needs N % 16 == 0, K % 32 == 0.
enum WLayout { W_KN = 0, W_NK = 1, W_TILED = 2 };
__host__ __device__ __forceinline__ int64_t tiled_offset(int n, int k, int64_t K) {
    return ((int64_t)(n >> 4) * (K >> 5) + (k >> 5)) * 512 + ((((k >> 3) & 3) << 4) + (n & 15)) * 8 + (k & 7);
}

struct Epilogue {
    int kind;             // LG_EPI_*
    const half_t* bias;   // [N] or nullptr
    int seq;              // LG_EPI_BIAS_HEADS: tokens per sequence
    int d;                // LG_EPI_BIAS_HEADS: size_per_head
    int heads_total;      // LG_EPI_BIAS_HEADS: heads per batch entry in the destination (>= N / d)
    int rows;             // LG_EPI_BIAS_HEADS_ROWS: 1 = token row m goes to (slot[m], pos[m]) of the RowMap, 0 = to (m, 0)
};

// kernel-internal epilogue: LG_EPI_BIAS_HEADS for one token per sequence, where every token row has its own destination
// (batch entry, position) -- the K and V rows of decode steps of different requests batched into one launch
constexpr int LG_EPI_BIAS_HEADS_ROWS = 4;
constexpr int LG_ROWMAP_MAX = LG_ATTN_DECODE_MAX_SEQS;
struct RowMap {  // passed by value with the launch
    int slot[LG_ROWMAP_MAX];
    int pos[LG_ROWMAP_MAX];
};

struct GemmArgs {
    int M, N, K;
    const half_t* X; int64_t ldx; int64_t strideX;
    const half_t* W; int64_t ldw; int64_t strideW;
    half_t* Y;       int64_t ldy; int64_t strideY;
    Epilogue epi;
};

// Up to three problems that share X and the shape and differ in weight, bias and destination (the Q, K and V projections of a
// decode step): the weight-streaming kernels run them as one launch, blockIdx.y selecting the problem.
constexpr int LG_MAX_GROUP = 3;
struct GemmGroup {
    int count;  // 1 = plain launch (the GemmArgs' own W / Y / bias / ldy are used)
    const half_t* W[LG_MAX_GROUP];
    half_t* Y[LG_MAX_GROUP];
    const half_t* bias[LG_MAX_GROUP];
    int64_t ldy[LG_MAX_GROUP];
    int rows[LG_MAX_GROUP];  // LG_EPI_BIAS_HEADS_ROWS: whether the member's token rows follow the RowMap
};
__device__ __forceinline__ void select_group(GemmArgs& g, const GemmGroup& grp) {
    if (grp.count > 1) {
        const int gi = blockIdx.y;
        g.W = grp.W[gi];
        g.Y = grp.Y[gi];
        g.epi.bias = grp.bias[gi];
        g.ldy = grp.ldy[gi];
        g.epi.rows = grp.rows[gi];
    }
}

// host side: a plain launch seen as a group of one
inline GemmGroup single_group(const GemmArgs& g) {
    GemmGroup grp{};
    grp.count = 1;
    grp.W[0] = g.W; grp.Y[0] = g.Y; grp.bias[0] = g.epi.bias; grp.ldy[0] = g.ldy; grp.rows[0] = g.epi.rows;
    return grp;
}
// what the vectorised loads and stores of the weight-streaming kernels need of every member of the group
inline bool group_aligned(const GemmArgs& g, const GemmGroup& grp) {
    for (int i = 0; i < grp.count; ++i) {
        if (!aligned16(grp.W[i]) || !aligned16(grp.Y[i])) return false;
        if ((g.epi.kind == LG_EPI_BIAS_HEADS || g.epi.kind == LG_EPI_BIAS_HEADS_ROWS) ? (g.epi.d % 4 != 0) : (grp.ldy[i] % 4 != 0)) return false;
    }
    return true;
}

__device__ __forceinline__ float4_t mfma16(half8_t a, half8_t b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

typedef __attribute__((address_space(3))) short4_t lds_short4_t;

// Transposed 4x16 LDS read (gfx950 ds_read_b64_tr_b16).  Within each group of 16 lanes, source lane s
// supplies the address of 4 consecutive halves; destination lane j = 4a + c receives, for r = 0..3, element c
// of source lane (a + 4r).  With source lane s pointing at row (s/4), columns 4*(s%4).. of a [k][n] tile,
// lane j ends up with tile[k0..k0+3][j]: four consecutive k for one n -- the MFMA operand order.
__device__ __forceinline__ half4_t lds_read_tr4(const half_t* p) {
    short4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_t*)p);
    return __builtin_bit_cast(half4_t, r);
}

// The same read issued as inline assembly, for kernels that fill their LDS tiles with direct-to-LDS loads (load_lds16): the
// compiler cannot tell which outstanding direct-to-LDS load the builtin's read may alias and puts an s_waitcnt vmcnt(0) in front
// of it, which drains the load pipeline of a ring of tiles at every read.  The kernels order tiles and reads themselves (their
// own vmcnt wait + barrier before a tile is read), so the read is hidden from that analysis.  The compiler then does not know
// that `dst` arrives late either: nothing may touch dst before lds_tr_wait has named it.
__device__ __forceinline__ void lds_read_tr4_issue(half4_t& dst, const half_t* p) {
    const unsigned addr = (unsigned)(uintptr_t)p;  // a pointer into LDS: its low 32 bits are the LDS address
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(dst) : "v"(addr));
}
// waits until at most PENDING LDS operations issued after the reads of lo / hi are outstanding, and makes every later use of
// lo / hi depend on that wait
template <int PENDING = 0>
__device__ __forceinline__ void lds_tr_wait(half4_t& lo, half4_t& hi) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(lo), "+v"(hi) : "n"(PENDING));
}
// the plain 16-byte LDS read and its wait, issued by hand for the same reason
__device__ __forceinline__ void lds_read16_issue(half8_t& dst, const half_t* p) {
    const unsigned addr = (unsigned)(uintptr_t)p;
    asm volatile("ds_read_b128 %0, %1" : "=v"(dst) : "v"(addr));
}
template <int PENDING = 0>
__device__ __forceinline__ void lds_read16_wait(half8_t& v) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(v) : "n"(PENDING));
}
// Both reads at LDS byte address `addr` plus a compile-time byte offset that travels in the instruction (16-bit field): a lane
// that reads the same position of several rows groups or ring slots needs one address register for all of them.
template <int OFF>
__device__ __forceinline__ void lds_read16_issue_at(half8_t& dst, unsigned addr) {
    static_assert(OFF >= 0 && OFF < 65536, "the offset field of an LDS instruction holds 16 bits");
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
template <int OFF>
__device__ __forceinline__ void lds_read_tr4_issue_at(half4_t& dst, unsigned addr) {
    static_assert(OFF >= 0 && OFF < 65536, "the offset field of an LDS instruction holds 16 bits");
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
__device__ __forceinline__ unsigned lds_address(const half_t* p) { return (unsigned)(uintptr_t)p; }

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a compile-time constant in its body
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

__device__ __forceinline__ half8_t join_half4(half4_t lo, half4_t hi) {
    return half8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

// Workgroup barrier for loops that keep direct-to-LDS loads in flight across it.  __syncthreads() carries a fence for which the
// compiler waits for ALL such loads (s_waitcnt vmcnt(0)): a ring of tiles would drain at every barrier.  Here the caller waits
// for exactly the loads and LDS operations it needs (s_waitcnt vmcnt(n) lgkmcnt(0) in front of the call); the empty assembly
// statements keep the compiler from moving memory accesses across the barrier instruction.
__device__ __forceinline__ void barrier_keep_loads_in_flight() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// ---- direct-to-LDS loads and the bank-conflict swizzles of the LDS-tiled kernels -------------------------------------------
typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(1))) const void gbl_void_t;

__device__ __forceinline__ void load_lds16(const half_t* gptr, half_t* lds_wave_base) {
    // every lane supplies its own global address; the 64 x 16 bytes land contiguously at lds_wave_base
    __builtin_amdgcn_global_load_lds((gbl_void_t*)gptr, (lds_void_t*)lds_wave_base, 16, 0, 0);
}

// swizzles: position (in 16-byte chunks) of logical chunk c in row r of the [rows][64] tiles; block (32 bytes) of
// logical block b in row k of a [64][128 or 256] weight tile
__device__ __forceinline__ int swz_a(int row, int c) { return c ^ ((row >> 1) & 7); }
// the 32 lanes served together by one transposed read touch rows k0..k0+3 and k0+8..k0+11: eight distinct XOR values
__device__ __forceinline__ int swz_b(int k, int blk) { return blk ^ ((k & 3) | ((k >> 1) & 4)); }

// Applies the epilogue to 4 consecutive output columns n..n+3 of token row m and stores them.
template <int EPI>
__device__ __forceinline__ void epilogue_store4(const GemmArgs& g, half_t* Yb, int m, int n, float4_t acc, bool vec_ok,
                                                const RowMap* rm = nullptr) {
    if (m >= g.M || n >= g.N) return;
    float v[4] = {acc[0], acc[1], acc[2], acc[3]};
    if (EPI != LG_EPI_NONE) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (n + r < g.N) v[r] += (float)g.epi.bias[n + r];
    }
    if (EPI == LG_EPI_BIAS_GELU) {
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = gelu_tanh(v[r]);
    }
    int64_t base;
    if (EPI == LG_EPI_BIAS_HEADS_ROWS) {
        // one token per sequence: row m -> [slot, head, pos, e] with ldy rows reserved per (slot, head)
        const int b = g.epi.rows ? rm->slot[m] : m, s = g.epi.rows ? rm->pos[m] : 0;
        const int head = n / g.epi.d, e = n % g.epi.d;
        base = (((int64_t)b * g.epi.heads_total + head) * g.ldy + s) * (int64_t)g.epi.d + e;
    } else if (EPI == LG_EPI_BIAS_HEADS) {
        // [M = b*seq + s, N = head*d + e]  ->  [b, head, s, e] with ldy rows reserved per (b, head)
        const int b = m / g.epi.seq, s = m % g.epi.seq;
        const int head = n / g.epi.d, e = n % g.epi.d;
        base = (((int64_t)b * g.epi.heads_total + head) * g.ldy + s) * (int64_t)g.epi.d + e;  // n..n+3 stay inside one head (d % 4 == 0)
    } else {
        base = (int64_t)m * g.ldy + n;
    }
    if (vec_ok && n + 3 < g.N) {
        half4_t o = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
        *reinterpret_cast<half4_t*>(Yb + base) = o;
    } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (n + r < g.N) Yb[base + r] = (half_t)v[r];
    }
}

// LG_EPI_BIAS_GEGLU: `gate` holds features n..n+3 of token row m (n % 32 < 16: a gate group), `up` features n+16..n+19 (the up
// columns of the same indices); the product goes to columns (n / 32) * 16 + n % 16 .. + 3 of the [M, N / 2] output.
__device__ __forceinline__ void epilogue_geglu4(const GemmArgs& g, half_t* Yb, int m, int n, float4_t gate, float4_t up, bool vec_ok) {
    if (m >= g.M || n >= g.N) return;
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
        v[r] = gelu_tanh(gate[r] + (float)g.epi.bias[n + r]) * (up[r] + (float)g.epi.bias[n + 16 + r]);
    const int64_t base = (int64_t)m * g.ldy + (n >> 5) * 16 + (n & 15);
    if (vec_ok) {
        half4_t o = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
        *reinterpret_cast<half4_t*>(Yb + base) = o;
    } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) Yb[base + r] = (half_t)v[r];
    }
}

// ---- split-K support shared by the weight-streaming and the pipelined kernel (gemm_skinny.hip) --------------------------
constexpr int LG_EPI_PARTIAL = 100;  // kernel-internal: store the fp32 accumulators of K-slice `split` to partial[split][M][N]
// The fp32 partials live in the stream's workspace (StreamInfo::ws, allocated when the stream was created or attached); a
// launcher never allocates: with no workspace, or one that is too small, it slices K less or not at all.
// Y = epilogue(sum over the nsplit K-slices in slice order) of the fp32 partials [nsplit][M][N]
void launch_splitk_reduce(const GemmArgs& g, const float* partial, int nsplit, hipStream_t stream, const RowMap* rows = nullptr);

}  // namespace lg
