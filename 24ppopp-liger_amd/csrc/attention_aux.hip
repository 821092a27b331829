// attention_aux.hip -- the reference-shaped helper kernels around the attention GEMMs:
// Q/K/V bias + head transpose, scale+mask+softmax (in place), transpose back.
// All are pure HBM streaming; 16-byte accesses, one wave64 per softmax row.
#include "common.hpp"

namespace lg {

// ---- buf[b,head,s,:] = X[b,s,head,:] + bias[head,:]   (attention_kernels.cu:79-224) -----------------
template <typename T>
struct QkvPtrs {
    const T* src[3];
    const T* bias[3];
    T* dst[3];
};

// FUSED = false: three separate [M, n] inputs; true: one packed [M, 3, n] input with bias [3, n].
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void qkv_bias_transpose_kernel(QkvPtrs<T> p, int seq, int head_num, int d,
                                                                 int64_t src_row_stride, int64_t total) {
    constexpr int VN = VEC ? Vec16<T>::N : 1;
    const int t = blockIdx.y;
    const T* __restrict__ src = p.src[t];
    const T* __restrict__ bias = p.bias[t];
    T* dst = p.dst[t];
    const int n = head_num * d;
    const int nv = n / VN;   // vectors per token row
    const int dv = d / VN;   // vectors per head
    for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < total; v += (int64_t)gridDim.x * blockDim.x) {
        const int64_t tok = v / nv;          // b*seq + s
        const int c = (int)(v % nv);         // vector column inside the row
        const int head = c / dv, e = c % dv;
        const int64_t b = tok / seq;
        const int s = (int)(tok % seq);
        const int64_t si = tok * src_row_stride + (int64_t)c * VN;
        const int64_t di = (((b * head_num + head) * seq + s) * (int64_t)d) + (int64_t)e * VN;
        if (VEC) {
            typedef Vec16<T> V;
            V a = *reinterpret_cast<const V*>(src + si);
            V bb = *reinterpret_cast<const V*>(bias + (int64_t)c * VN);
            V o;
#pragma unroll
            for (int j = 0; j < V::N; ++j) o.set(j, a.get(j) + bb.get(j));
            *reinterpret_cast<V*>(dst + di) = o;
        } else {
            stf(dst + di, ldf(src + si) + ldf(bias + c));
        }
    }
}

template <typename T>
static int launch_qkv(const QkvPtrs<T>& p, int batch, int seq, int head_num, int d, int64_t src_row_stride,
                      hipStream_t stream, const char* what) {
    if (batch < 0 || seq < 0 || head_num <= 0 || d <= 0) { set_error("%s: bad shape", what); return LG_ERR_INVALID; }
    for (int t = 0; t < 3; ++t)
        if (!p.src[t] || !p.bias[t] || !p.dst[t]) { set_error("%s: null pointer", what); return LG_ERR_INVALID; }
    const int64_t M = (int64_t)batch * seq;
    if (M == 0) return LG_OK;
    constexpr int VN = Vec16<T>::N;
    bool vec = (d % VN == 0) && (src_row_stride % VN == 0);
    for (int t = 0; t < 3; ++t) vec = vec && aligned16(p.src[t]) && aligned16(p.bias[t]) && aligned16(p.dst[t]);
    const int64_t total = M * head_num * d / (vec ? VN : 1);
    int64_t grid = (total + 255) / 256;
    if (grid > 32768) grid = 32768;
    if (vec)
        hipLaunchKernelGGL((qkv_bias_transpose_kernel<T, true>), dim3((int)grid, 3), dim3(256), 0, stream, p, seq,
                           head_num, d, src_row_stride, total);
    else
        hipLaunchKernelGGL((qkv_bias_transpose_kernel<T, false>), dim3((int)grid, 3), dim3(256), 0, stream, p, seq,
                           head_num, d, src_row_stride, total);
    return check_launch(what);
}

// ---- dst[b,s,head,:] = src[b,head,s,:]   (attention_kernels.cu:682-742) -----------------------------
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void transpose_back_kernel(T* dst, const T* __restrict__ src, int seq, int head_num,
                                                             int d, int64_t total) {
    constexpr int VN = VEC ? Vec16<T>::N : 1;
    const int dv = d / VN;
    for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < total; v += (int64_t)gridDim.x * blockDim.x) {
        // v enumerates dst in [b, s, head, e] order
        const int e = (int)(v % dv);
        const int64_t r = v / dv;
        const int head = (int)(r % head_num);
        const int64_t tok = r / head_num;
        const int64_t b = tok / seq;
        const int s = (int)(tok % seq);
        const int64_t si = (((b * head_num + head) * seq + s) * (int64_t)d) + (int64_t)e * VN;
        const int64_t di = v * VN;
        if (VEC) {
            typedef Vec16<T> V;
            *reinterpret_cast<V*>(dst + di) = *reinterpret_cast<const V*>(src + si);
        } else {
            dst[di] = src[si];
        }
    }
}

template <typename T>
static int launch_transpose(T* dst, const T* src, int batch, int seq, int head_num, int d, hipStream_t stream) {
    if (batch < 0 || seq < 0 || head_num <= 0 || d <= 0 || !dst || !src) { set_error("transpose: bad arguments"); return LG_ERR_INVALID; }
    const int64_t n = (int64_t)batch * seq * head_num * d;
    if (n == 0) return LG_OK;
    constexpr int VN = Vec16<T>::N;
    const bool vec = (d % VN == 0) && aligned16(dst) && aligned16(src);
    const int64_t total = n / (vec ? VN : 1);
    int64_t grid = (total + 255) / 256;
    if (grid > 32768) grid = 32768;
    if (vec)
        hipLaunchKernelGGL((transpose_back_kernel<T, true>), dim3((int)grid), dim3(256), 0, stream, dst, src, seq, head_num, d, total);
    else
        hipLaunchKernelGGL((transpose_back_kernel<T, false>), dim3((int)grid), dim3(256), 0, stream, dst, src, seq, head_num, d, total);
    return check_launch("transpose");
}

// ---- softmax (attention_kernels.cu:395-680) -----------------------------------------------------------
//   t = qk*scalar + (1 - mask)*(-10000);  p = exp(t - max t);  out = p / (sum p + 1e-6)
// One wave64 per row, the row held in registers as NC 16-byte vectors per lane.
template <typename T, int NC>
__global__ __launch_bounds__(256) void softmax_wave_kernel(T* buf, const T* __restrict__ mask, int seq, int head_num,
                                                           int64_t rows, float scalar) {
    typedef Vec16<T> V;
    constexpr int VN = V::N;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int64_t b = row / ((int64_t)head_num * seq);
    const int sq = (int)(row % seq);
    T* p = buf + row * seq;
    const T* mrow = mask + (b * seq + sq) * (int64_t)seq;
    const int nvec = seq / VN;
    float t[NC][VN];
    float mx = -1e20f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int v = lane + c * 64;
        if (v < nvec) {
            V a = *reinterpret_cast<const V*>(p + (int64_t)v * VN);
            V m = *reinterpret_cast<const V*>(mrow + (int64_t)v * VN);
#pragma unroll
            for (int j = 0; j < VN; ++j) {
                t[c][j] = a.get(j) * scalar + (1.0f - m.get(j)) * -10000.0f;
                mx = fmaxf(mx, t[c][j]);
            }
        } else {
#pragma unroll
            for (int j = 0; j < VN; ++j) t[c][j] = -1e20f;
        }
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int v = lane + c * 64;
        if (v < nvec) {
#pragma unroll
            for (int j = 0; j < VN; ++j) {
                t[c][j] = __expf(t[c][j] - mx);
                sum += t[c][j];
            }
        }
    }
    sum = wave_sum(sum);
    const float inv = 1.0f / (sum + 1e-6f);
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int v = lane + c * 64;
        if (v < nvec) {
            V o;
#pragma unroll
            for (int j = 0; j < VN; ++j) o.set(j, t[c][j] * inv);
            *reinterpret_cast<V*>(p + (int64_t)v * VN) = o;
        }
    }
}

// any seq / alignment: one block per row, three passes
template <typename T>
__global__ __launch_bounds__(256) void softmax_scalar_kernel(T* buf, const T* mask, int seq, int head_num, float scalar) {
    __shared__ float scratch[16];
    const int64_t row = blockIdx.x;
    const int64_t b = row / ((int64_t)head_num * seq);
    const int sq = (int)(row % seq);
    T* p = buf + row * seq;
    const T* mrow = mask + (b * seq + sq) * (int64_t)seq;
    float mx = -1e20f;
    for (int i = threadIdx.x; i < seq; i += blockDim.x)
        mx = fmaxf(mx, ldf(p + i) * scalar + (1.0f - ldf(mrow + i)) * -10000.0f);
    mx = block_max(mx, scratch);
    float sum = 0.f;
    for (int i = threadIdx.x; i < seq; i += blockDim.x)
        sum += __expf(ldf(p + i) * scalar + (1.0f - ldf(mrow + i)) * -10000.0f - mx);
    sum = block_sum(sum, scratch);
    const float inv = 1.0f / (sum + 1e-6f);
    for (int i = threadIdx.x; i < seq; i += blockDim.x)
        stf(p + i, __expf(ldf(p + i) * scalar + (1.0f - ldf(mrow + i)) * -10000.0f - mx) * inv);
}

template <typename T>
static int launch_softmax(T* buf, const T* mask, int batch, int seq, int head_num, float scalar, hipStream_t stream) {
    if (batch < 0 || seq < 0 || head_num <= 0 || !buf || !mask) { set_error("attn_softmax: bad arguments"); return LG_ERR_INVALID; }
    const int64_t rows = (int64_t)batch * head_num * seq;
    if (rows == 0) return LG_OK;
    scalar = (float)(T)scalar;  // the reference keeps the scalar as T (bert_layer.h:94)
    constexpr int VN = Vec16<T>::N;
    const bool vec = (seq % VN == 0) && aligned16(buf) && aligned16(mask);
    const int nvec = seq / VN;
    if (vec && nvec <= 64 * 8) {
        const int nc = (nvec + 63) / 64;
        const int64_t grid = (rows + 3) / 4;
        if (grid > 0x7fffffff) { set_error("attn_softmax: too many rows"); return LG_ERR_INVALID; }
#define LG_SM_LAUNCH(NCC)                                                                                          \
    hipLaunchKernelGGL((softmax_wave_kernel<T, NCC>), dim3((unsigned)grid), dim3(256), 0, stream, buf, mask, seq,   \
                       head_num, rows, scalar)
        if (nc <= 1) LG_SM_LAUNCH(1);
        else if (nc <= 2) LG_SM_LAUNCH(2);
        else if (nc <= 4) LG_SM_LAUNCH(4);
        else LG_SM_LAUNCH(8);
#undef LG_SM_LAUNCH
    } else {
        if (rows > 0x7fffffff) { set_error("attn_softmax: too many rows"); return LG_ERR_INVALID; }
        hipLaunchKernelGGL((softmax_scalar_kernel<T>), dim3((unsigned)rows), dim3(256), 0, stream, buf, mask, seq, head_num, scalar);
    }
    return check_launch("attn_softmax");
}

}  // namespace lg

using namespace lg;

extern "C" {

int lg_add_qkv_bias_transpose_f32(float* q_buf, float* k_buf, float* v_buf, const float* Q, const float* bias_Q,
                                  const float* K, const float* bias_K, const float* V, const float* bias_V, int batch,
                                  int seq, int head_num, int size_per_head, void* stream) {
    QkvPtrs<float> p = {{Q, K, V}, {bias_Q, bias_K, bias_V}, {q_buf, k_buf, v_buf}};
    return launch_qkv<float>(p, batch, seq, head_num, size_per_head, (int64_t)head_num * size_per_head,
                             (hipStream_t)stream, "add_qkv_bias_transpose");
}
int lg_add_qkv_bias_transpose_f16(void* q_buf, void* k_buf, void* v_buf, const void* Q, const void* bias_Q,
                                  const void* K, const void* bias_K, const void* V, const void* bias_V, int batch,
                                  int seq, int head_num, int size_per_head, void* stream) {
    QkvPtrs<half_t> p = {{(const half_t*)Q, (const half_t*)K, (const half_t*)V},
                         {(const half_t*)bias_Q, (const half_t*)bias_K, (const half_t*)bias_V},
                         {(half_t*)q_buf, (half_t*)k_buf, (half_t*)v_buf}};
    return launch_qkv<half_t>(p, batch, seq, head_num, size_per_head, (int64_t)head_num * size_per_head,
                              (hipStream_t)stream, "add_qkv_bias_transpose");
}
int lg_add_fused_qkv_bias_transpose_f32(float* q_buf, float* k_buf, float* v_buf, const float* QKV, const float* qkv_bias,
                                        int batch, int seq, int head_num, int size_per_head, void* stream) {
    if (!QKV || !qkv_bias) { set_error("add_fused_qkv_bias_transpose: null pointer"); return LG_ERR_INVALID; }
    const int64_t n = (int64_t)head_num * size_per_head;
    QkvPtrs<float> p = {{QKV, QKV + n, QKV + 2 * n}, {qkv_bias, qkv_bias + n, qkv_bias + 2 * n}, {q_buf, k_buf, v_buf}};
    return launch_qkv<float>(p, batch, seq, head_num, size_per_head, 3 * n, (hipStream_t)stream,
                             "add_fused_qkv_bias_transpose");
}
int lg_add_fused_qkv_bias_transpose_f16(void* q_buf, void* k_buf, void* v_buf, const void* QKV, const void* qkv_bias,
                                        int batch, int seq, int head_num, int size_per_head, void* stream) {
    if (!QKV || !qkv_bias) { set_error("add_fused_qkv_bias_transpose: null pointer"); return LG_ERR_INVALID; }
    const int64_t n = (int64_t)head_num * size_per_head;
    const half_t* x = (const half_t*)QKV;
    const half_t* b = (const half_t*)qkv_bias;
    QkvPtrs<half_t> p = {{x, x + n, x + 2 * n}, {b, b + n, b + 2 * n}, {(half_t*)q_buf, (half_t*)k_buf, (half_t*)v_buf}};
    return launch_qkv<half_t>(p, batch, seq, head_num, size_per_head, 3 * n, (hipStream_t)stream,
                              "add_fused_qkv_bias_transpose");
}
int lg_attn_softmax_f32(float* buffer, const float* attr_mask, int batch, int seq, int head_num, float scalar, void* stream) {
    return launch_softmax<float>(buffer, attr_mask, batch, seq, head_num, scalar, (hipStream_t)stream);
}
int lg_attn_softmax_f16(void* buffer, const void* attr_mask, int batch, int seq, int head_num, float scalar, void* stream) {
    return launch_softmax<half_t>((half_t*)buffer, (const half_t*)attr_mask, batch, seq, head_num, scalar, (hipStream_t)stream);
}
int lg_transpose_f32(float* dst, const float* src, int batch, int seq, int head_num, int size_per_head, void* stream) {
    return launch_transpose<float>(dst, src, batch, seq, head_num, size_per_head, (hipStream_t)stream);
}
int lg_transpose_f16(void* dst, const void* src, int batch, int seq, int head_num, int size_per_head, void* stream) {
    return launch_transpose<half_t>((half_t*)dst, (const half_t*)src, batch, seq, head_num, size_per_head, (hipStream_t)stream);
}

}  // extern "C"
