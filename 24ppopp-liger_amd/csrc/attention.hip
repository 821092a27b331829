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
#include "common.cuh"

namespace lg {

constexpr int DEC_UNROLL = 8;

// partial result of one (b, head, split): max, sum, weighted V (fp32)
//   workspace layout: [B*h][nsplit][2 + D] floats
template <int D>
__global__ __launch_bounds__(256) void attn_decode_kernel(const half_t* __restrict__ q, const half_t* __restrict__ kc,
                                                          const half_t* __restrict__ vc, half_t* out, float* ws,
                                                          int len, int max_len, int nsplit, float scalar) {
    constexpr int LPK = D / 8;        // lanes per key row
    constexpr int KPL = 64 / LPK;     // keys per wave-wide load
    __shared__ float s_m[4 * KPL], s_l[4 * KPL];
    __shared__ float s_acc[4 * KPL][D];

    const int bh = blockIdx.x, split = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int grp = lane / LPK, sub = lane % LPK;

    // key range of this block, then of this wave (contiguous quarters)
    const int per_split = (len + nsplit - 1) / nsplit;
    const int s_begin = split * per_split;
    const int s_end = min(len, s_begin + per_split);
    const int per_wave = (s_end - s_begin + 3) / 4;
    const int w_begin = s_begin + wave * per_wave;
    const int w_end = min(s_end, w_begin + per_wave);

    float qf[8];
    {
        half8_t qv = *reinterpret_cast<const half8_t*>(q + (int64_t)bh * D + sub * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) qf[j] = (float)qv[j] * scalar;
    }
    const half_t* kbase = kc + (int64_t)bh * max_len * D + sub * 8;
    const half_t* vbase = vc + (int64_t)bh * max_len * D + sub * 8;

    float m_run = -1e30f, l_run = 0.f;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    for (int base = w_begin; base < w_end; base += KPL * DEC_UNROLL) {
        half8_t kv[DEC_UNROLL], vv[DEC_UNROLL];
#pragma unroll
        for (int u = 0; u < DEC_UNROLL; ++u) {
            const int key = base + u * KPL + grp;
            if (key < w_end) {
                kv[u] = *reinterpret_cast<const half8_t*>(kbase + (int64_t)key * D);
                vv[u] = *reinterpret_cast<const half8_t*>(vbase + (int64_t)key * D);
            } else {
                kv[u] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
                vv[u] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
            }
        }
        float s[DEC_UNROLL];
        float m_new = m_run;
#pragma unroll
        for (int u = 0; u < DEC_UNROLL; ++u) {
            float p = 0.f;
#pragma unroll
            for (int j = 0; j < 8; ++j) p = fmaf(qf[j], (float)kv[u][j], p);
#pragma unroll
            for (int o = LPK / 2; o > 0; o >>= 1) p += __shfl_xor(p, o, 64);
            const int key = base + u * KPL + grp;
            s[u] = (key < w_end) ? p : -1e30f;
            m_new = fmaxf(m_new, s[u]);
        }
        const float corr = __expf(m_run - m_new);
        l_run *= corr;
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] *= corr;
#pragma unroll
        for (int u = 0; u < DEC_UNROLL; ++u) {
            const int key = base + u * KPL + grp;
            const float p = (key < w_end) ? __expf(s[u] - m_new) : 0.f;
            l_run += p;
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = fmaf(p, (float)vv[u][j], acc[j]);
        }
        m_run = m_new;
    }

    // merge the 4*KPL lane groups of the block through LDS
    const int slot = wave * KPL + grp;
    if (sub == 0) { s_m[slot] = m_run; s_l[slot] = l_run; }
#pragma unroll
    for (int j = 0; j < 8; ++j) s_acc[slot][sub * 8 + j] = acc[j];
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

static int decode_nsplit(int bh, int len) {
    // aim for >= 1024 blocks (4 per CU on 256 CUs) while keeping >= 128 keys per block
    int ns = 1;
    while (bh * ns < 1024 && (len / (ns * 2)) >= 128 && ns < 64) ns *= 2;
    return ns;
}

// q_out[b,head,:] = Q[b, head*d ..] + bq;  caches[b,head,pos,:] = K/V + bias
__global__ __launch_bounds__(256) void kv_append_kernel(half_t* q_out, half_t* kc, half_t* vc, const half_t* __restrict__ Q,
                                                        const half_t* __restrict__ bq, const half_t* __restrict__ K,
                                                        const half_t* __restrict__ bk, const half_t* __restrict__ V,
                                                        const half_t* __restrict__ bv, int head_num, int d, int pos,
                                                        int max_len, int64_t total_vec) {
    const int dv = d / 8, nv = head_num * dv;
    for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < total_vec; v += (int64_t)gridDim.x * blockDim.x) {
        const int64_t b = v / nv;
        const int c = (int)(v % nv), head = c / dv, e = c % dv;
        const int64_t si = b * (int64_t)head_num * d + (int64_t)c * 8;
        const int64_t ci = ((b * head_num + head) * (int64_t)max_len + pos) * d + (int64_t)e * 8;
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

}  // namespace lg

using namespace lg;

extern "C" {

size_t lg_attn_decode_workspace_bytes(int batch, int head_num, int size_per_head, int max_len) {
    if (batch <= 0 || head_num <= 0 || size_per_head <= 0 || max_len <= 0) return 0;
    const int bh = batch * head_num;
    return (size_t)bh * decode_nsplit(bh, max_len) * (2 + (size_t)size_per_head) * sizeof(float);
}

int lg_attn_decode_f16(const void* q, const void* k_cache, const void* v_cache, void* out, void* workspace, int batch,
                       int head_num, int size_per_head, int len, int max_len, float scalar, void* stream) {
    if (batch < 0 || head_num <= 0 || len <= 0 || max_len < len) { set_error("attn_decode: bad shape (len=%d max_len=%d)", len, max_len); return LG_ERR_INVALID; }
    if (size_per_head != 64 && size_per_head != 128) { set_error("attn_decode: size_per_head must be 64 or 128"); return LG_ERR_INVALID; }
    if (batch == 0) return LG_OK;
    if (!q || !k_cache || !v_cache || !out) { set_error("attn_decode: null pointer"); return LG_ERR_INVALID; }
    if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache)) { set_error("attn_decode: pointers must be 16-byte aligned"); return LG_ERR_INVALID; }
    const int bh = batch * head_num;
    const int ns = decode_nsplit(bh, len);
    if (ns > 1 && !workspace) { set_error("attn_decode: workspace required"); return LG_ERR_INVALID; }
    scalar = (float)(half_t)scalar;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid(bh, ns);
    if (size_per_head == 128) {
        hipLaunchKernelGGL((attn_decode_kernel<128>), grid, dim3(256), 0, st, (const half_t*)q, (const half_t*)k_cache,
                           (const half_t*)v_cache, (half_t*)out, (float*)workspace, len, max_len, ns, scalar);
        if (ns > 1) hipLaunchKernelGGL((attn_decode_merge_kernel<128>), dim3(bh), dim3(128), 0, st, (const float*)workspace, (half_t*)out, ns);
    } else {
        hipLaunchKernelGGL((attn_decode_kernel<64>), grid, dim3(256), 0, st, (const half_t*)q, (const half_t*)k_cache,
                           (const half_t*)v_cache, (half_t*)out, (float*)workspace, len, max_len, ns, scalar);
        if (ns > 1) hipLaunchKernelGGL((attn_decode_merge_kernel<64>), dim3(bh), dim3(64), 0, st, (const float*)workspace, (half_t*)out, ns);
    }
    return check_launch("attn_decode");
}

int lg_kv_append_f16(void* q_out, void* k_cache, void* v_cache, const void* Q, const void* bias_Q, const void* K,
                     const void* bias_K, const void* V, const void* bias_V, int batch, int head_num, int size_per_head,
                     int pos, int max_len, void* stream) {
    if (batch < 0 || head_num <= 0 || size_per_head <= 0 || size_per_head % 8 != 0 || pos < 0 || pos >= max_len) {
        set_error("kv_append: bad shape (pos=%d max_len=%d d=%d)", pos, max_len, size_per_head);
        return LG_ERR_INVALID;
    }
    if (batch == 0) return LG_OK;
    const void* ptrs[9] = {q_out, k_cache, v_cache, Q, bias_Q, K, bias_K, V, bias_V};
    for (const void* p : ptrs)
        if (!p || !aligned16(p)) { set_error("kv_append: null or unaligned pointer"); return LG_ERR_INVALID; }
    const int64_t total = (int64_t)batch * head_num * size_per_head / 8;
    int64_t grid = (total + 255) / 256;
    if (grid > 4096) grid = 4096;
    hipLaunchKernelGGL(kv_append_kernel, dim3((int)grid), dim3(256), 0, (hipStream_t)stream, (half_t*)q_out, (half_t*)k_cache,
                       (half_t*)v_cache, (const half_t*)Q, (const half_t*)bias_Q, (const half_t*)K, (const half_t*)bias_K,
                       (const half_t*)V, (const half_t*)bias_V, head_num, size_per_head, pos, max_len, total);
    return check_launch("kv_append");
}

}  // extern "C"
