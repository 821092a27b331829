// attention.hip -- decode attention over a KV cache (HBM streaming) and the KV append, for gfx950.
//
// Decode attention is a pure bandwidth problem: every K and V byte of the cache is read exactly once and
// used for ~1 flop.  The kernel therefore keeps the data path as short as possible:
//   * 16-byte global loads straight into registers, no LDS staging;
//   * a key row (d halves) is spread over d/8 adjacent lanes, so one wave-wide load covers 64*8/d keys and
//     every load instruction touches whole 256-byte rows;
//   * q.k partial sums are reduced inside the d/8-lane group with shuffles, so every lane of the group ends
//     up holding the score of "its" key and can scale the matching V vector without any exchange;
//   * each lane group runs its own online softmax (running max / sum / weighted V) and the groups, waves
//     and KV splits are merged once at the end;
//   * a thread block is 4 waves; with >= 4 blocks per CU there are 16+ waves per CU, each with 2*UNROLL
//     independent 1 KiB loads in flight.
// Softmax semantics are the reference's (attention_kernels.cu:480-519): p = exp(t - max t) / (sum + 1e-6),
// t = q.k * scalar, all positions < len unmasked.
#include <stdlib.h>
#include <mutex>

#include "common.hpp"

namespace lg {

// Sequences of one launch that do not share a length or do not sit in consecutive cache slots (decode steps of different
// requests batched into one launch): per-sequence cache slot and valid length, passed by value with the launch.
constexpr int DEC_MAX_SEQS = LG_ATTN_DECODE_MAX_SEQS;
struct DecodeSeqs {
    int slot[DEC_MAX_SEQS];
    int len[DEC_MAX_SEQS];
};

// partial result of one (b, head, split): max, sum, weighted V (fp32)
//   workspace layout: [B*h][nsplit][2 + D] floats
// A key row of D halves is D/8 16-byte chunks; lane `sub` of an LPK-lane group holds chunks sub, sub + LPK, ... (CPL of
// them), so one wave-wide load covers 64 / LPK keys with LPK * 16 contiguous bytes of each (D = 128: LPK 16, whole rows;
// D = 64: LPK 8; D = 96: LPK 4 x 3 chunks).
// NT: the K / V loads are marked non-temporal.  Every load instruction covers whole 128-byte lines and every byte is used once,
// so nothing is lost by not keeping the lines; the launcher sets it when the keys and values of the launch exceed what the
// memory-side cache could hold for the next step anyway.
template <int D, int LPK, int UNROLL, bool VARLEN, bool NT>
__global__ __launch_bounds__(256) void attn_decode_kernel(const half_t* __restrict__ q, const half_t* __restrict__ kc,
                                                          const half_t* __restrict__ vc, half_t* out, float* ws,
                                                          int len, int max_len, int nsplit, float scalar, int head_num,
                                                          DecodeSeqs seqs) {
    constexpr int CPL = D / (8 * LPK);  // 16-byte chunks per lane and key
    constexpr int KPL = 64 / LPK;       // keys per wave-wide load
    static_assert(CPL * LPK * 8 == D, "D must be LPK * CPL * 8");
    __shared__ float s_m[4 * KPL], s_l[4 * KPL];
    __shared__ float s_acc[4 * KPL][D];

    const int bh = blockIdx.x, split = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int grp = lane / LPK, sub = lane % LPK;
    int64_t cache_row = bh;  // (cache slot, head) row of the caches
    if (VARLEN) {
        const int b = bh / head_num, head = bh % head_num;
        len = seqs.len[b];
        cache_row = (int64_t)seqs.slot[b] * head_num + head;
    }

    // key range of this block, then of this wave (contiguous quarters)
    const int per_split = (len + nsplit - 1) / nsplit;
    const int s_begin = min(len, split * per_split);
    const int s_end = min(len, s_begin + per_split);
    const int per_wave = (s_end - s_begin + 3) / 4;
    const int w_begin = min(s_end, s_begin + wave * per_wave);
    const int w_end = min(s_end, w_begin + per_wave);

    float qf[CPL][8];
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
        half8_t qv = *reinterpret_cast<const half8_t*>(q + (int64_t)bh * D + (c * LPK + sub) * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) qf[c][j] = (float)qv[j] * scalar;
    }
    const half_t* kbase = kc + cache_row * max_len * D + sub * 8;
    const half_t* vbase = vc + cache_row * max_len * D + sub * 8;

    float m_run = -1e30f, l_run = 0.f;
    float acc[CPL][8];
#pragma unroll
    for (int c = 0; c < CPL; ++c)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[c][j] = 0.f;

    for (int base = w_begin; base < w_end; base += KPL * UNROLL) {
        half8_t kv[UNROLL][CPL], vv[UNROLL][CPL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int key = base + u * KPL + grp;
#pragma unroll
            for (int c = 0; c < CPL; ++c) {
                if (key < w_end) {
                    const half8_t* kp = reinterpret_cast<const half8_t*>(kbase + (int64_t)key * D + c * LPK * 8);
                    const half8_t* vp = reinterpret_cast<const half8_t*>(vbase + (int64_t)key * D + c * LPK * 8);
                    kv[u][c] = NT ? __builtin_nontemporal_load(kp) : *kp;
                    vv[u][c] = NT ? __builtin_nontemporal_load(vp) : *vp;
                } else {
                    kv[u][c] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
                    vv[u][c] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
                }
            }
        }
        float s[UNROLL];
        float m_new = m_run;
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            float p = 0.f;
#pragma unroll
            for (int c = 0; c < CPL; ++c)
#pragma unroll
                for (int j = 0; j < 8; ++j) p = fmaf(qf[c][j], (float)kv[u][c][j], p);
#pragma unroll
            for (int o = LPK / 2; o > 0; o >>= 1) p += __shfl_xor(p, o, 64);
            const int key = base + u * KPL + grp;
            s[u] = (key < w_end) ? p : -1e30f;
            m_new = fmaxf(m_new, s[u]);
        }
        const float corr = __expf(m_run - m_new);
        l_run *= corr;
#pragma unroll
        for (int c = 0; c < CPL; ++c)
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[c][j] *= corr;
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int key = base + u * KPL + grp;
            const float p = (key < w_end) ? __expf(s[u] - m_new) : 0.f;
            l_run += p;
#pragma unroll
            for (int c = 0; c < CPL; ++c)
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[c][j] = fmaf(p, (float)vv[u][c][j], acc[c][j]);
        }
        m_run = m_new;
    }

    // merge the 4*KPL lane groups of the block through LDS
    const int slot = wave * KPL + grp;
    if (sub == 0) { s_m[slot] = m_run; s_l[slot] = l_run; }
#pragma unroll
    for (int c = 0; c < CPL; ++c)
#pragma unroll
        for (int j = 0; j < 8; ++j) s_acc[slot][(c * LPK + sub) * 8 + j] = acc[c][j];
    __syncthreads();
    if (threadIdx.x < D) {
        float m = -1e30f;
        for (int i = 0; i < 4 * KPL; ++i) m = fmaxf(m, s_m[i]);
        float l = 0.f, o = 0.f;
        for (int i = 0; i < 4 * KPL; ++i) {
            const float c = __expf(s_m[i] - m);
            l += s_l[i] * c;
            o += s_acc[i][threadIdx.x] * c;
        }
        if (nsplit == 1) {
            out[(int64_t)bh * D + threadIdx.x] = (half_t)(o / (l + 1e-6f));
        } else {
            float* w = ws + ((int64_t)bh * nsplit + split) * (2 + D);
            if (threadIdx.x == 0) { w[0] = m; w[1] = l; }
            w[2 + threadIdx.x] = o;
        }
    }
}

template <int D>
__global__ void attn_decode_merge_kernel(const float* __restrict__ ws, half_t* out, int nsplit) {
    const int bh = blockIdx.x, t = threadIdx.x;  // blockDim = D
    const float* w = ws + (int64_t)bh * nsplit * (2 + D);
    float m = -1e30f;
    for (int i = 0; i < nsplit; ++i) m = fmaxf(m, w[i * (2 + D)]);
    float l = 0.f, o = 0.f;
    for (int i = 0; i < nsplit; ++i) {
        const float c = __expf(w[i * (2 + D)] - m);
        l += w[i * (2 + D) + 1] * c;
        o += w[i * (2 + D) + 2 + t] * c;
    }
    out[(int64_t)bh * D + t] = (half_t)(o / (l + 1e-6f));
}

// Split-KV partial slots (b, head, split) any launch can need.  decode_nsplit only doubles the split count while
// bh * ns < 1024, so whenever partials are used at all (ns > 1) there are fewer than 2048 of them -- whatever the batch.
constexpr int DEC_MAX_SLOTS = 2048;
constexpr int DEC_MAX_D = 128;

static int decode_nsplit(int bh, int len) {
    // aim for >= 1024 blocks (4 per CU on 256 CUs) while keeping >= 128 keys per block
    int ns = 1;
    while (bh * ns < 1024 && (len / (ns * 2)) >= 128 && ns < 64) ns *= 2;
    return ns;
}

template <int D, int LPK, int UNROLL>
static void launch_decode(const half_t* q, const half_t* kc, const half_t* vc, half_t* out, float* ws, int bh, int head_num,
                          int len, int max_len, int ns, float scalar, const DecodeSeqs* seqs, hipStream_t st) {
    const dim3 grid(bh, ns);
    // more keys and values than half the 256 MB memory-side cache: the next step would not find them there anyway
    static const int nt_forced = [] { const char* e = getenv("LG_ATTN_DECODE_NT"); return e ? atoi(e) : -1; }();
    const bool nt = nt_forced >= 0 ? nt_forced != 0 : (int64_t)bh * len * D * 4 > ((int64_t)128 << 20);
    if (seqs) {
        if (nt) hipLaunchKernelGGL((attn_decode_kernel<D, LPK, UNROLL, true, true>), grid, dim3(256), 0, st, q, kc, vc, out, ws, len, max_len, ns, scalar, head_num, *seqs);
        else hipLaunchKernelGGL((attn_decode_kernel<D, LPK, UNROLL, true, false>), grid, dim3(256), 0, st, q, kc, vc, out, ws, len, max_len, ns, scalar, head_num, *seqs);
    } else {
        if (nt) hipLaunchKernelGGL((attn_decode_kernel<D, LPK, UNROLL, false, true>), grid, dim3(256), 0, st, q, kc, vc, out, ws, len, max_len, ns, scalar, head_num, DecodeSeqs{});
        else hipLaunchKernelGGL((attn_decode_kernel<D, LPK, UNROLL, false, false>), grid, dim3(256), 0, st, q, kc, vc, out, ws, len, max_len, ns, scalar, head_num, DecodeSeqs{});
    }
    if (ns > 1) hipLaunchKernelGGL((attn_decode_merge_kernel<D>), dim3(bh), dim3(D), 0, st, (const float*)ws, out, ns);
}

// Argument checks and launch shared by the three entry points.  `seqs` = per-sequence slots and lengths or nullptr (all
// sequences `len` long, sequence b in cache slot b); ws_capacity_slots = partial slots the workspace holds.
static int attn_decode_common(const char* what, const void* q, const void* k_cache, const void* v_cache, void* out, float* ws,
                              int64_t ws_capacity_slots, int batch, int head_num, int size_per_head, int len, int max_len,
                              float scalar, const DecodeSeqs* seqs, hipStream_t st) {
    if (batch < 0 || head_num <= 0 || len <= 0 || max_len < len) { set_error("%s: bad shape (len=%d max_len=%d)", what, len, max_len); return LG_ERR_INVALID; }
    if (size_per_head != 64 && size_per_head != 96 && size_per_head != 128) { set_error("%s: size_per_head must be 64, 96 or 128", what); return LG_ERR_INVALID; }
    if (batch == 0) return LG_OK;
    if (!q || !k_cache || !v_cache || !out) { set_error("%s: null pointer", what); return LG_ERR_INVALID; }
    if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache)) { set_error("%s: pointers must be 16-byte aligned", what); return LG_ERR_INVALID; }
    if ((int64_t)batch * head_num > 0x7fffffff) { set_error("%s: batch * head_num too large", what); return LG_ERR_INVALID; }
    const int bh = batch * head_num;
    const int ns = decode_nsplit(bh, len);
    if (ns > 1 && !ws) { set_error("%s: workspace required", what); return LG_ERR_INVALID; }
    if (ns > 1 && (int64_t)bh * ns > ws_capacity_slots) {
        set_error("%s: %d x %d split-KV partials exceed the workspace's %lld slots", what, bh, ns, (long long)ws_capacity_slots);
        return LG_ERR_INVALID;
    }
    scalar = (float)(half_t)scalar;
    const half_t *qh = (const half_t*)q, *kh = (const half_t*)k_cache, *vh = (const half_t*)v_cache;
    if (size_per_head == 128) launch_decode<128, 16, 8>(qh, kh, vh, (half_t*)out, ws, bh, head_num, len, max_len, ns, scalar, seqs, st);
    else if (size_per_head == 96) launch_decode<96, 4, 4>(qh, kh, vh, (half_t*)out, ws, bh, head_num, len, max_len, ns, scalar, seqs, st);
    else launch_decode<64, 8, 8>(qh, kh, vh, (half_t*)out, ws, bh, head_num, len, max_len, ns, scalar, seqs, st);
    return check_launch(what);
}

// ---- split-KV partials in device memory that belongs to the library (lg_attn_decode_static_f16) ---------------------------
// One array per GPU, held until the process ends; every call on a GPU uses that GPU's array.
static __device__ __align__(256) float scratch[DEC_MAX_SLOTS * (2 + DEC_MAX_D)];
constexpr int DEC_MAX_DEVICES = 64;
static std::mutex g_scratch_mu;
static float* g_scratch_ptr[DEC_MAX_DEVICES] = {};

// Device address of this GPU's `scratch` (the array's name is only a host-side stand-in for it): looked up once per device,
// with that device current.
static int scratch_address(float** ptr) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { set_error("attn_decode_static: hipGetDevice: %s", hipGetErrorString(e)); return LG_ERR_LAUNCH; }
    if (dev < 0 || dev >= DEC_MAX_DEVICES) { set_error("attn_decode_static: device %d not supported", dev); return LG_ERR_INVALID; }
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) { set_error("attn_decode_static: hipGetSymbolAddress: %s", hipGetErrorString(e)); return LG_ERR_LAUNCH; }
        g_scratch_ptr[dev] = (float*)p;
    }
    *ptr = g_scratch_ptr[dev];
    return LG_OK;
}

// q_out[b,head,:] = Q[b, head*d ..] + bq;  caches[slot_b,head,pos_b,:] = K/V + bias.  VARLEN: slot_b, pos_b come per sequence
// (seqs.slot / seqs.len), otherwise slot_b = b and pos_b = pos.
template <bool VARLEN>
__global__ __launch_bounds__(256) void kv_append_kernel(half_t* q_out, half_t* kc, half_t* vc, const half_t* __restrict__ Q,
                                                        const half_t* __restrict__ bq, const half_t* __restrict__ K,
                                                        const half_t* __restrict__ bk, const half_t* __restrict__ V,
                                                        const half_t* __restrict__ bv, int head_num, int d, int pos,
                                                        int max_len, int64_t total_vec, DecodeSeqs seqs) {
    const int dv = d / 8, nv = head_num * dv;
    for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < total_vec; v += (int64_t)gridDim.x * blockDim.x) {
        const int64_t b = v / nv;
        const int c = (int)(v % nv), head = c / dv, e = c % dv;
        const int64_t si = b * (int64_t)head_num * d + (int64_t)c * 8;
        const int64_t row = VARLEN ? seqs.slot[b] : b;
        const int p = VARLEN ? seqs.len[b] : pos;
        const int64_t ci = ((row * head_num + head) * (int64_t)max_len + p) * d + (int64_t)e * 8;
        typedef Vec16<half_t> Vh;
        Vh a, bb, o;
        a = *reinterpret_cast<const Vh*>(Q + si); bb = *reinterpret_cast<const Vh*>(bq + (int64_t)c * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) o.set(j, a.get(j) + bb.get(j));
        *reinterpret_cast<Vh*>(q_out + si) = o;
        a = *reinterpret_cast<const Vh*>(K + si); bb = *reinterpret_cast<const Vh*>(bk + (int64_t)c * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) o.set(j, a.get(j) + bb.get(j));
        *reinterpret_cast<Vh*>(kc + ci) = o;
        a = *reinterpret_cast<const Vh*>(V + si); bb = *reinterpret_cast<const Vh*>(bv + (int64_t)c * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) o.set(j, a.get(j) + bb.get(j));
        *reinterpret_cast<Vh*>(vc + ci) = o;
    }
}

static int kv_append_common(const char* what, void* q_out, void* k_cache, void* v_cache, const void* Q, const void* bias_Q,
                            const void* K, const void* bias_K, const void* V, const void* bias_V, int batch, int head_num,
                            int size_per_head, int pos, int max_len, const DecodeSeqs* seqs, hipStream_t st) {
    if (batch < 0 || head_num <= 0 || size_per_head <= 0 || size_per_head % 8 != 0 || pos < 0 || pos >= max_len) {
        set_error("%s: bad shape (pos=%d max_len=%d d=%d)", what, pos, max_len, size_per_head);
        return LG_ERR_INVALID;
    }
    if (batch == 0) return LG_OK;
    const void* ptrs[9] = {q_out, k_cache, v_cache, Q, bias_Q, K, bias_K, V, bias_V};
    for (const void* p : ptrs)
        if (!p || !aligned16(p)) { set_error("%s: null or unaligned pointer", what); return LG_ERR_INVALID; }
    const int64_t total = (int64_t)batch * head_num * size_per_head / 8;
    int64_t grid = (total + 255) / 256;
    if (grid > 4096) grid = 4096;
    if (seqs)
        hipLaunchKernelGGL(kv_append_kernel<true>, dim3((int)grid), dim3(256), 0, st, (half_t*)q_out, (half_t*)k_cache,
                           (half_t*)v_cache, (const half_t*)Q, (const half_t*)bias_Q, (const half_t*)K, (const half_t*)bias_K,
                           (const half_t*)V, (const half_t*)bias_V, head_num, size_per_head, pos, max_len, total, *seqs);
    else
        hipLaunchKernelGGL(kv_append_kernel<false>, dim3((int)grid), dim3(256), 0, st, (half_t*)q_out, (half_t*)k_cache,
                           (half_t*)v_cache, (const half_t*)Q, (const half_t*)bias_Q, (const half_t*)K, (const half_t*)bias_K,
                           (const half_t*)V, (const half_t*)bias_V, head_num, size_per_head, pos, max_len, total, DecodeSeqs{});
    return check_launch(what);
}

}  // namespace lg

using namespace lg;

extern "C" {

size_t lg_attn_decode_workspace_bytes(int batch, int head_num, int size_per_head, int max_len) {
    if (batch <= 0 || head_num <= 0 || size_per_head <= 0 || max_len <= 0) return 0;
    // an upper bound for every batch and length (a smaller batch may split its keys further than a larger one)
    return (size_t)DEC_MAX_SLOTS * (2 + (size_t)size_per_head) * sizeof(float);
}

int lg_attn_decode_f16(const void* q, const void* k_cache, const void* v_cache, void* out, void* workspace, int batch,
                       int head_num, int size_per_head, int len, int max_len, float scalar, void* stream) {
    return attn_decode_common("attn_decode", q, k_cache, v_cache, out, (float*)workspace, DEC_MAX_SLOTS, batch, head_num,
                              size_per_head, len, max_len, scalar, nullptr, (hipStream_t)stream);
}

int lg_attn_decode_varlen_f16(const void* q, const void* k_cache, const void* v_cache, void* out, void* workspace, int batch,
                              int head_num, int size_per_head, const int* slot, const int* len, int max_len, float scalar,
                              void* stream) {
    if (batch < 0 || batch > DEC_MAX_SEQS) { set_error("attn_decode_varlen: batch must be 0..%d", DEC_MAX_SEQS); return LG_ERR_INVALID; }
    if (batch == 0) return LG_OK;
    if (!slot || !len) { set_error("attn_decode_varlen: null slot / len array"); return LG_ERR_INVALID; }
    DecodeSeqs seqs{};
    int longest = 0;
    for (int b = 0; b < batch; ++b) {
        if (slot[b] < 0 || len[b] <= 0 || len[b] > max_len) { set_error("attn_decode_varlen: sequence %d: slot %d, len %d (max_len %d)", b, slot[b], len[b], max_len); return LG_ERR_INVALID; }
        seqs.slot[b] = slot[b];
        seqs.len[b] = len[b];
        longest = len[b] > longest ? len[b] : longest;
    }
    return attn_decode_common("attn_decode_varlen", q, k_cache, v_cache, out, (float*)workspace, DEC_MAX_SLOTS, batch, head_num,
                              size_per_head, longest, max_len, scalar, &seqs, (hipStream_t)stream);
}

int lg_attn_decode_static_f16(const void* q, const void* k_cache, const void* v_cache, void* out, int batch, int head_num,
                              int size_per_head, int len, int max_len, float scalar, void* stream) {
    if (size_per_head > DEC_MAX_D) { set_error("attn_decode_static: size_per_head %d exceeds the maximum %d", size_per_head, DEC_MAX_D); return LG_ERR_INVALID; }
    float* ws = nullptr;
    const int rc = scratch_address(&ws);
    if (rc != LG_OK) return rc;
    return attn_decode_common("attn_decode_static", q, k_cache, v_cache, out, ws, DEC_MAX_SLOTS, batch, head_num, size_per_head, len,
                              max_len, scalar, nullptr, (hipStream_t)stream);
}

int lg_kv_append_f16(void* q_out, void* k_cache, void* v_cache, const void* Q, const void* bias_Q, const void* K,
                     const void* bias_K, const void* V, const void* bias_V, int batch, int head_num, int size_per_head,
                     int pos, int max_len, void* stream) {
    return kv_append_common("kv_append", q_out, k_cache, v_cache, Q, bias_Q, K, bias_K, V, bias_V, batch, head_num, size_per_head,
                            pos, max_len, nullptr, (hipStream_t)stream);
}

int lg_kv_append_varlen_f16(void* q_out, void* k_cache, void* v_cache, const void* Q, const void* bias_Q, const void* K,
                            const void* bias_K, const void* V, const void* bias_V, int batch, int head_num, int size_per_head,
                            const int* slot, const int* pos, int max_len, void* stream) {
    if (batch < 0 || batch > DEC_MAX_SEQS) { set_error("kv_append_varlen: batch must be 0..%d", DEC_MAX_SEQS); return LG_ERR_INVALID; }
    if (batch == 0) return LG_OK;
    if (!slot || !pos) { set_error("kv_append_varlen: null slot / pos array"); return LG_ERR_INVALID; }
    DecodeSeqs seqs{};
    for (int b = 0; b < batch; ++b) {
        if (slot[b] < 0 || pos[b] < 0 || pos[b] >= max_len) { set_error("kv_append_varlen: sequence %d: slot %d, pos %d (max_len %d)", b, slot[b], pos[b], max_len); return LG_ERR_INVALID; }
        seqs.slot[b] = slot[b];
        seqs.len[b] = pos[b];
    }
    return kv_append_common("kv_append_varlen", q_out, k_cache, v_cache, Q, bias_Q, K, bias_K, V, bias_V, batch, head_num,
                            size_per_head, 0, max_len, &seqs, (hipStream_t)stream);
}

}  // extern "C"
