// attention_prefill.hip -- fused LDS-tiled prefill attention for gfx950 (flash-style, online softmax).
//
// Replaces the reference's qk_gemm -> attn_softmax -> qkv_gemm (-> transpose) sequence (bert_layer.h:145-168) and
// keeps its softmax semantics: t = q.k * scalar + (1 - mask) * (-10000), p = exp(t - max t), out = sum p v / (sum p +
// 1e-6).  The S x S score matrix never touches HBM.
//
// Work split: one block = 128 queries of one (batch, head); 4 waves x 32 queries.  K and V tiles of 64 keys are staged
// in LDS.  Everything is computed transposed so that no cross-lane data movement is needed between the two GEMMs:
//   S^T[key, q] = K[key, :] . Q[q, :]      A = K tile (16-byte LDS reads), B = Q (registers, loaded once)
//   O^T[d, q]  += V^T[d, key] * P^T[key, q] A = V tile through the gfx950 transposed LDS read, B = P^T, which is
//                                           exactly the accumulator layout S^T came out in (4 consecutive keys per
//                                           lane), so the probabilities go from MFMA result to MFMA operand in place.
// Softmax statistics are per query = per (lane % 16); the four 16-lane groups hold different keys and are combined
// with two shuffles per tile.
#include "gemm_common.cuh"

namespace lg {

constexpr int PF_BQ = 128;  // queries per block
constexpr int PF_BC = 64;   // keys per LDS tile

template <int D, bool CAUSAL, bool HAS_MASK>
__global__ __launch_bounds__(256) void attn_prefill_kernel(const half_t* __restrict__ q_buf, const half_t* __restrict__ k_buf,
                                                           const half_t* __restrict__ v_buf, const half_t* __restrict__ mask,
                                                           half_t* out, int seq, int head_num, int kv_rows, float scalar,
                                                           int out_layout) {
    constexpr int KS = D + 8;       // LDS row stride in halves
    constexpr int DC = D / 32;      // 32-wide d chunks (k steps of the S^T GEMM)
    constexpr int DT = D / 16;      // 16-wide d tiles (rows of O^T)
    __shared__ __attribute__((aligned(16))) half_t Ks[PF_BC * KS];
    __shared__ __attribute__((aligned(16))) half_t Vs[PF_BC * KS];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    const int bh = blockIdx.y;                 // b * head_num + head
    const int b = bh / head_num, head = bh % head_num;
    const int q0 = blockIdx.x * PF_BQ;         // first query of the block
    const int qw = q0 + wave * 32;             // first query of the wave

    const half_t* Q = q_buf + (int64_t)bh * seq * D;
    const half_t* K = k_buf + (int64_t)bh * kv_rows * D;
    const half_t* V = v_buf + (int64_t)bh * kv_rows * D;

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

    const int kv_end = CAUSAL ? min(seq, q0 + PF_BQ) : seq;
    for (int k0 = 0; k0 < kv_end; k0 += PF_BC) {
        __syncthreads();  // previous tile fully consumed
        // stage K and V tiles: 64 rows x D halves each; rows beyond seq are zero-filled
        constexpr int VPR = D / 8;               // 16-byte vectors per row
        constexpr int NVEC = PF_BC * VPR;        // per tile
#pragma unroll
        for (int i = 0; i < NVEC / 256; ++i) {
            const int v = tid + 256 * i;
            const int row = v / VPR, c = v % VPR;
            half8_t kk = half8_t{0, 0, 0, 0, 0, 0, 0, 0}, vv = kk;
            if (k0 + row < seq) {
                kk = *reinterpret_cast<const half8_t*>(K + (int64_t)(k0 + row) * D + c * 8);
                vv = *reinterpret_cast<const half8_t*>(V + (int64_t)(k0 + row) * D + c * 8);
            }
            *reinterpret_cast<half8_t*>(&Ks[row * KS + c * 8]) = kk;
            *reinterpret_cast<half8_t*>(&Vs[row * KS + c * 8]) = vv;
        }
        __syncthreads();
        // a wave whose queries all lie before this key tile has nothing to do here (causal), but must keep hitting the
        // barriers above, so only the math is skipped
        if (CAUSAL && k0 > qw + 31) continue;

        // ---- S^T = K Q^T ------------------------------------------------------------------------------------
        float4_t s[4][2];
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
            s[kt][0] = float4_t{0.f, 0.f, 0.f, 0.f};
            s[kt][1] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int dc = 0; dc < DC; ++dc) {
                const half8_t a = *reinterpret_cast<const half8_t*>(&Ks[(kt * 16 + l16) * KS + dc * 32 + g * 8]);
                s[kt][0] = mfma16(a, qf[0][dc], s[kt][0]);
                s[kt][1] = mfma16(a, qf[1][dc], s[kt][1]);
            }
        }
        // ---- scale, mask, online softmax (per query column) -----------------------------------------------------
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
            const int q = qw + qt * 16 + l16;
            float mx = -1e30f;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) {
                float mterm[4] = {0.f, 0.f, 0.f, 0.f};
                if (HAS_MASK) {
                    const int key = k0 + kt * 16 + 4 * g;
                    if (q < seq) {
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (key + r < seq) mterm[r] = (1.0f - (float)mask[((int64_t)b * seq + q) * seq + key + r]) * -10000.0f;
                    }
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int key = k0 + kt * 16 + 4 * g + r;
                    float t = s[kt][qt][r] * scalar + mterm[r];
                    if (CAUSAL && key > q) t += -10000.0f;
                    if (key >= seq) t = -1e30f;  // beyond the sequence: not part of the row at all
                    s[kt][qt][r] = t;
                    mx = fmaxf(mx, t);
                }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_run[qt], mx);
            const float corr = __expf(m_run[qt] - m_new);
            m_run[qt] = m_new;
            float ls = 0.f;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float p = __expf(s[kt][qt][r] - m_new);
                    s[kt][qt][r] = p;
                    ls += p;
                }
            l_run[qt] = l_run[qt] * corr + ls;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) o[dt][qt] *= corr;
        }
        // ---- O^T += V^T P^T ---------------------------------------------------------------------------------------
#pragma unroll
        for (int j = 0; j < 2; ++j) {  // two k-steps of 32 keys: key tiles 2j and 2j+1
            half8_t pf[2];
#pragma unroll
            for (int qt = 0; qt < 2; ++qt) {
                const float4_t lo = s[2 * j][qt], hi = s[2 * j + 1][qt];
                pf[qt] = half8_t{(half_t)lo[0], (half_t)lo[1], (half_t)lo[2], (half_t)lo[3],
                                 (half_t)hi[0], (half_t)hi[1], (half_t)hi[2], (half_t)hi[3]};
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int col = dt * 16 + 4 * (l16 & 3);
                const int row = (2 * j) * 16 + 4 * g + (l16 >> 2);
                const half4_t lo = lds_read_tr4(&Vs[row * KS + col]);
                const half4_t hi = lds_read_tr4(&Vs[(row + 16) * KS + col]);
                const half8_t a = half8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                o[dt][0] = mfma16(a, pf[0], o[dt][0]);
                o[dt][1] = mfma16(a, pf[1], o[dt][1]);
            }
        }
    }

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

template <int D>
static void launch_prefill(const half_t* q, const half_t* k, const half_t* v, const half_t* mask, half_t* out, int batch,
                           int seq, int head_num, int kv_rows, float scalar, int causal, int out_layout, hipStream_t st) {
    dim3 grid((seq + PF_BQ - 1) / PF_BQ, batch * head_num);
    if (causal)
        hipLaunchKernelGGL((attn_prefill_kernel<D, true, false>), grid, dim3(256), 0, st, q, k, v, mask, out, seq, head_num, kv_rows, scalar, out_layout);
    else if (mask)
        hipLaunchKernelGGL((attn_prefill_kernel<D, false, true>), grid, dim3(256), 0, st, q, k, v, mask, out, seq, head_num, kv_rows, scalar, out_layout);
    else
        hipLaunchKernelGGL((attn_prefill_kernel<D, false, false>), grid, dim3(256), 0, st, q, k, v, mask, out, seq, head_num, kv_rows, scalar, out_layout);
}

}  // namespace lg

using namespace lg;

extern "C" int lg_attn_prefill_f16(const void* q_buf, const void* k_buf, const void* v_buf, const void* attr_mask,
                                   void* out, int batch, int seq, int head_num, int size_per_head, int kv_rows,
                                   float scalar, int causal, int out_layout, void* stream) {
    if (batch < 0 || seq < 0 || head_num <= 0 || kv_rows < seq || (out_layout != 0 && out_layout != 1)) {
        set_error("attn_prefill: bad shape (seq=%d kv_rows=%d)", seq, kv_rows);
        return LG_ERR_INVALID;
    }
    if (size_per_head != 64 && size_per_head != 96 && size_per_head != 128) { set_error("attn_prefill: size_per_head must be 64, 96 or 128"); return LG_ERR_INVALID; }
    if (batch == 0 || seq == 0) return LG_OK;
    if (!q_buf || !k_buf || !v_buf || !out) { set_error("attn_prefill: null pointer"); return LG_ERR_INVALID; }
    if (!aligned16(q_buf) || !aligned16(k_buf) || !aligned16(v_buf) || !aligned16(out)) {
        set_error("attn_prefill: pointers must be 16-byte aligned");
        return LG_ERR_INVALID;
    }
    if ((int64_t)batch * head_num > 65535) { set_error("attn_prefill: batch * head_num > 65535"); return LG_ERR_INVALID; }
    scalar = (float)(half_t)scalar;
    if (size_per_head == 128)
        launch_prefill<128>((const half_t*)q_buf, (const half_t*)k_buf, (const half_t*)v_buf, (const half_t*)attr_mask,
                            (half_t*)out, batch, seq, head_num, kv_rows, scalar, causal, out_layout, (hipStream_t)stream);
    else if (size_per_head == 96)
        launch_prefill<96>((const half_t*)q_buf, (const half_t*)k_buf, (const half_t*)v_buf, (const half_t*)attr_mask,
                           (half_t*)out, batch, seq, head_num, kv_rows, scalar, causal, out_layout, (hipStream_t)stream);
    else
        launch_prefill<64>((const half_t*)q_buf, (const half_t*)k_buf, (const half_t*)v_buf, (const half_t*)attr_mask,
                           (half_t*)out, batch, seq, head_num, kv_rows, scalar, causal, out_layout, (hipStream_t)stream);
    return check_launch("attn_prefill");
}
