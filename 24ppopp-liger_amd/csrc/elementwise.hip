// elementwise.hip -- bias+GELU, bias+residual and the LayerNorm family for gfx950.
//
// All of these are HBM-bound.  The vector kernels move 16 bytes per lane per access, keep one row
// in registers (one HBM read, one HBM write per element) and reduce with wave64 shuffles; statistics
// are two-pass in fp32 exactly as the reference computes them (cuda_kernels.cu:463-508):
//   mean = sum(x)/n,  var = sum((x-mean)^2)/n,  y = (x-mean) * rsqrt(var + 1e-6) * gamma + beta.
#include "common.hpp"

namespace lg {

enum LnMode { LN_PLAIN = 0, LN_ADD_INPLACE = 1, LN_ADD_STORE = 2 };

// One row per block, row cached in registers as NV 16-byte vectors per thread.
//   LN_PLAIN        x = src                                   dst = LN(x)
//   LN_ADD_INPLACE  x = src + add + bias        (fp32)        dst = LN(x)          (dst may alias src)
//   LN_ADD_STORE    x = T(add + src + bias); sum_out = x      dst = LN(x)          (sum_out may alias src)
//                   with the mean taken over the unrounded fp32 sums and the variance and output over the stored x,
//                   as the reference kernel does (cuda_kernels.cu:377-408)
template <typename T, int MODE, int NV>
__global__ __launch_bounds__(256) void ln_vec_kernel(const T* __restrict__ src, const T* __restrict__ add,
                                                     const T* __restrict__ bias, const T* __restrict__ gamma,
                                                     const T* __restrict__ beta, T* sum_out, T* dst, int n) {
    typedef Vec16<T> V;
    constexpr int VN = V::N;
    __shared__ float scratch[16];
    const int nvec = n / VN;
    const int64_t row = (int64_t)blockIdx.x * n;
    float x[NV][VN];
    float local = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = threadIdx.x + i * blockDim.x;
        if (v < nvec) {
            V a = *reinterpret_cast<const V*>(src + row + (int64_t)v * VN);
            if (MODE != LN_PLAIN) {
                V r = *reinterpret_cast<const V*>(add + row + (int64_t)v * VN);
                V b = *reinterpret_cast<const V*>(bias + (int64_t)v * VN);
                V s;
#pragma unroll
                for (int j = 0; j < VN; ++j) {
                    float t = r.get(j) + a.get(j) + b.get(j);
                    local += t;  // the mean sums the unrounded value in every mode
                    if (MODE == LN_ADD_STORE) {
                        s.set(j, t);
                        t = s.get(j);  // variance and output use the stored (rounded) value
                    }
                    x[i][j] = t;
                }
                if (MODE == LN_ADD_STORE) *reinterpret_cast<V*>(sum_out + row + (int64_t)v * VN) = s;
            } else {
#pragma unroll
                for (int j = 0; j < VN; ++j) {
                    x[i][j] = a.get(j);
                    local += x[i][j];
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < VN; ++j) x[i][j] = 0.f;
        }
    }
    const float mean = block_sum(local, scratch) / (float)n;
    float lv = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = threadIdx.x + i * blockDim.x;
        if (v < nvec) {
#pragma unroll
            for (int j = 0; j < VN; ++j) {
                const float d = x[i][j] - mean;
                lv += d * d;
            }
        }
    }
    const float var = block_sum(lv, scratch) / (float)n;
    const float rstd = rsqrtf(var + 1e-6f);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int v = threadIdx.x + i * blockDim.x;
        if (v < nvec) {
            V g = *reinterpret_cast<const V*>(gamma + (int64_t)v * VN);
            V b = *reinterpret_cast<const V*>(beta + (int64_t)v * VN);
            V o;
#pragma unroll
            for (int j = 0; j < VN; ++j) o.set(j, ((x[i][j] - mean) * rstd) * g.get(j) + b.get(j));
            *reinterpret_cast<V*>(dst + row + (int64_t)v * VN) = o;
        }
    }
}

// Any n, any alignment: three passes over the row with scalar accesses (the reference's own shape).
template <typename T, int MODE>
__global__ __launch_bounds__(256) void ln_scalar_kernel(const T* src, const T* add, const T* bias, const T* gamma,
                                                        const T* beta, T* sum_out, T* dst, int n) {
    __shared__ float scratch[16];
    const int64_t row = (int64_t)blockIdx.x * n;
    // pass 1: form x (stored to sum_out for LN_ADD_STORE) and sum
    float local = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float t = ldf(src + row + i);
        if (MODE != LN_PLAIN) t = ldf(add + row + i) + t + ldf(bias + i);
        if (MODE == LN_ADD_STORE) stf(sum_out + row + i, t);  // the mean still sums the unrounded t
        local += t;
    }
    const float mean = block_sum(local, scratch) / (float)n;
    float lv = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float t;
        if (MODE == LN_PLAIN) t = ldf(src + row + i);
        else if (MODE == LN_ADD_STORE) t = ldf(sum_out + row + i);
        else t = ldf(add + row + i) + ldf(src + row + i) + ldf(bias + i);
        const float d = t - mean;
        lv += d * d;
    }
    const float var = block_sum(lv, scratch) / (float)n;
    const float rstd = rsqrtf(var + 1e-6f);
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float t;
        if (MODE == LN_PLAIN) t = ldf(src + row + i);
        else if (MODE == LN_ADD_STORE) t = ldf(sum_out + row + i);
        else t = ldf(add + row + i) + ldf(src + row + i) + ldf(bias + i);
        // LN_ADD_INPLACE: dst aliases src, but element i is read and written by this thread only
        stf(dst + row + i, ((t - mean) * rstd) * ldf(gamma + i) + ldf(beta + i));
    }
}

template <typename T, int MODE>
static int launch_ln(const T* src, const T* add, const T* bias, const T* gamma, const T* beta, T* sum_out, T* dst,
                     int m, int n, hipStream_t stream, const char* what) {
    if (m < 0 || n <= 0) { set_error("%s: bad shape m=%d n=%d", what, m, n); return LG_ERR_INVALID; }
    if (m == 0) return LG_OK;
    if (!src || !gamma || !beta || !dst || (MODE != LN_PLAIN && (!add || !bias)) || (MODE == LN_ADD_STORE && !sum_out)) {
        set_error("%s: null pointer", what);
        return LG_ERR_INVALID;
    }
    if (m == 0) return LG_OK;
    constexpr int VN = Vec16<T>::N;
    const bool vec_ok = (n % VN == 0) && aligned16(src) && aligned16(gamma) && aligned16(beta) && aligned16(dst) &&
                        (MODE == LN_PLAIN || (aligned16(add) && aligned16(bias))) &&
                        (MODE != LN_ADD_STORE || aligned16(sum_out));
    const int nvec = n / VN;
    if (vec_ok && nvec <= 256 * 16) {
        int block = ((nvec + 63) / 64) * 64;
        if (block > 256) block = 256;
        const int nv = (nvec + block - 1) / block;
#define LG_LN_LAUNCH(NVV)                                                                                             \
    hipLaunchKernelGGL((ln_vec_kernel<T, MODE, NVV>), dim3(m), dim3(block), 0, stream, src, add, bias, gamma, beta,   \
                       sum_out, dst, n)
        if (nv <= 1) LG_LN_LAUNCH(1);
        else if (nv <= 2) LG_LN_LAUNCH(2);
        else if (nv <= 4) LG_LN_LAUNCH(4);
        else if (nv <= 6) LG_LN_LAUNCH(6);
        else if (nv <= 8) LG_LN_LAUNCH(8);
        else if (nv <= 12) LG_LN_LAUNCH(12);
        else LG_LN_LAUNCH(16);
#undef LG_LN_LAUNCH
    } else {
        hipLaunchKernelGGL((ln_scalar_kernel<T, MODE>), dim3(m), dim3(256), 0, stream, src, add, bias, gamma, beta,
                           sum_out, dst, n);
    }
    return check_launch(what);
}

// ---- bias + GELU(tanh), in place -------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void bias_gelu_vec_kernel(T* out, const T* __restrict__ bias, int64_t total_vec,
                                                            int nvec_row) {
    typedef Vec16<T> V;
    for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < total_vec; v += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(v % nvec_row);
        V a = *reinterpret_cast<const V*>(out + v * V::N);
        V b = *reinterpret_cast<const V*>(bias + (int64_t)c * V::N);
        V o;
#pragma unroll
        for (int j = 0; j < V::N; ++j) o.set(j, gelu_tanh(a.get(j) + b.get(j)));
        *reinterpret_cast<V*>(out + v * V::N) = o;
    }
}
template <typename T>
__global__ __launch_bounds__(256) void bias_gelu_scalar_kernel(T* out, const T* bias, int64_t total, int n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x)
        stf(out + i, gelu_tanh(ldf(out + i) + ldf(bias + (i % n))));
}

template <typename T>
static int launch_bias_gelu(T* out, const T* bias, int m, int n, hipStream_t stream) {
    if (m < 0 || n <= 0) { set_error("add_bias_act: bad shape m=%d n=%d", m, n); return LG_ERR_INVALID; }
    if (m == 0) return LG_OK;
    if (!out || !bias) { set_error("add_bias_act: null pointer"); return LG_ERR_INVALID; }
    constexpr int VN = Vec16<T>::N;
    const int64_t total = (int64_t)m * n;
    if (n % VN == 0 && aligned16(out) && aligned16(bias)) {
        const int64_t tv = total / VN;
        int64_t grid = (tv + 255) / 256;
        if (grid > 256 * 32) grid = 256 * 32;
        hipLaunchKernelGGL((bias_gelu_vec_kernel<T>), dim3((int)grid), dim3(256), 0, stream, out, bias, tv, n / VN);
    } else {
        int64_t grid = (total + 255) / 256;
        if (grid > 65536) grid = 65536;
        hipLaunchKernelGGL((bias_gelu_scalar_kernel<T>), dim3((int)grid), dim3(256), 0, stream, out, bias, total, n);
    }
    return check_launch("add_bias_act");
}

// ---- GeGLU: out[m, f] = gelu_tanh(in[m, j] + bias[j]) * (in[m, f + j] + bias[f + j]),  in = [gate | up] ------------
template <typename T>
__global__ __launch_bounds__(256) void bias_geglu_vec_kernel(T* out, const T* __restrict__ in, const T* __restrict__ bias,
                                                             int64_t total_vec, int nvec_row, int f) {
    typedef Vec16<T> V;
    for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < total_vec; v += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row = v / nvec_row;
        const int c = (int)(v % nvec_row);
        const T* src = in + row * 2 * f + (int64_t)c * V::N;
        V g = *reinterpret_cast<const V*>(src);
        V u = *reinterpret_cast<const V*>(src + f);
        V bg = *reinterpret_cast<const V*>(bias + (int64_t)c * V::N);
        V bu = *reinterpret_cast<const V*>(bias + f + (int64_t)c * V::N);
        V o;
#pragma unroll
        for (int j = 0; j < V::N; ++j) o.set(j, gelu_tanh(g.get(j) + bg.get(j)) * (u.get(j) + bu.get(j)));
        *reinterpret_cast<V*>(out + v * V::N) = o;
    }
}
template <typename T>
__global__ __launch_bounds__(256) void bias_geglu_scalar_kernel(T* out, const T* in, const T* bias, int64_t total, int f) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row = i / f;
        const int j = (int)(i % f);
        const T* src = in + row * 2 * f;
        stf(out + i, gelu_tanh(ldf(src + j) + ldf(bias + j)) * (ldf(src + f + j) + ldf(bias + f + j)));
    }
}

template <typename T>
static int launch_bias_geglu(T* out, const T* in, const T* bias, int m, int f, hipStream_t stream) {
    if (m < 0 || f <= 0) { set_error("add_bias_geglu: bad shape m=%d f=%d", m, f); return LG_ERR_INVALID; }
    if (m == 0) return LG_OK;
    if (!out || !in || !bias) { set_error("add_bias_geglu: null pointer"); return LG_ERR_INVALID; }
    constexpr int VN = Vec16<T>::N;
    const int64_t total = (int64_t)m * f;
    if (f % VN == 0 && aligned16(out) && aligned16(in) && aligned16(bias)) {
        const int64_t tv = total / VN;
        int64_t grid = (tv + 255) / 256;
        if (grid > 256 * 32) grid = 256 * 32;
        hipLaunchKernelGGL((bias_geglu_vec_kernel<T>), dim3((int)grid), dim3(256), 0, stream, out, in, bias, tv, f / VN, f);
    } else {
        int64_t grid = (total + 255) / 256;
        if (grid > 65536) grid = 65536;
        hipLaunchKernelGGL((bias_geglu_scalar_kernel<T>), dim3((int)grid), dim3(256), 0, stream, out, in, bias, total, f);
    }
    return check_launch("add_bias_geglu");
}

// ---- output = output + input + bias -----------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void add_bias_input_vec_kernel(T* output, const T* __restrict__ input,
                                                                 const T* __restrict__ bias, int64_t total_vec,
                                                                 int nvec_row) {
    typedef Vec16<T> V;
    for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < total_vec; v += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(v % nvec_row);
        V a = *reinterpret_cast<const V*>(output + v * V::N);
        V r = *reinterpret_cast<const V*>(input + v * V::N);
        V b = *reinterpret_cast<const V*>(bias + (int64_t)c * V::N);
        V o;
#pragma unroll
        for (int j = 0; j < V::N; ++j) o.set(j, a.get(j) + r.get(j) + b.get(j));
        *reinterpret_cast<V*>(output + v * V::N) = o;
    }
}
template <typename T>
__global__ __launch_bounds__(256) void add_bias_input_scalar_kernel(T* output, const T* input, const T* bias,
                                                                    int64_t total, int n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x)
        stf(output + i, ldf(output + i) + ldf(input + i) + ldf(bias + (i % n)));
}
template <typename T>
static int launch_add_bias_input(T* output, const T* bias, const T* input, int m, int n, hipStream_t stream) {
    if (m < 0 || n <= 0) { set_error("add_bias_input: bad shape m=%d n=%d", m, n); return LG_ERR_INVALID; }
    if (m == 0) return LG_OK;
    if (!output || !bias || !input) { set_error("add_bias_input: null pointer"); return LG_ERR_INVALID; }
    constexpr int VN = Vec16<T>::N;
    const int64_t total = (int64_t)m * n;
    if (n % VN == 0 && aligned16(output) && aligned16(bias) && aligned16(input)) {
        const int64_t tv = total / VN;
        int64_t grid = (tv + 255) / 256;
        if (grid > 256 * 32) grid = 256 * 32;
        hipLaunchKernelGGL((add_bias_input_vec_kernel<T>), dim3((int)grid), dim3(256), 0, stream, output, input, bias, tv, n / VN);
    } else {
        int64_t grid = (total + 255) / 256;
        if (grid > 65536) grid = 65536;
        hipLaunchKernelGGL((add_bias_input_scalar_kernel<T>), dim3((int)grid), dim3(256), 0, stream, output, input, bias, total, n);
    }
    return check_launch("add_bias_input");
}

}  // namespace lg

using namespace lg;

extern "C" {

int lg_layer_norm_f32(const float* in, const float* gamma, const float* beta, float* out, int m, int n, void* stream) {
    return launch_ln<float, LN_PLAIN>(in, nullptr, nullptr, gamma, beta, nullptr, out, m, n, (hipStream_t)stream, "layer_norm");
}
int lg_layer_norm_f16(const void* in, const void* gamma, const void* beta, void* out, int m, int n, void* stream) {
    return launch_ln<half_t, LN_PLAIN>((const half_t*)in, nullptr, nullptr, (const half_t*)gamma, (const half_t*)beta,
                                       nullptr, (half_t*)out, m, n, (hipStream_t)stream, "layer_norm");
}
int lg_add_bias_act_f32(float* out, const float* bias, int m, int n, void* stream) {
    return launch_bias_gelu<float>(out, bias, m, n, (hipStream_t)stream);
}
int lg_add_bias_geglu_f32(float* out, const float* in, const float* bias, int m, int f, void* stream) {
    return lg::launch_bias_geglu<float>(out, in, bias, m, f, (hipStream_t)stream);
}
int lg_add_bias_geglu_f16(void* out, const void* in, const void* bias, int m, int f, void* stream) {
    return lg::launch_bias_geglu<lg::half_t>((lg::half_t*)out, (const lg::half_t*)in, (const lg::half_t*)bias, m, f, (hipStream_t)stream);
}
int lg_add_bias_act_f16(void* out, const void* bias, int m, int n, void* stream) {
    return launch_bias_gelu<half_t>((half_t*)out, (const half_t*)bias, m, n, (hipStream_t)stream);
}
int lg_add_bias_input_layernorm_f32(float* out, const float* input, const float* bias, const float* gamma,
                                    const float* beta, int m, int n, void* stream) {
    return launch_ln<float, LN_ADD_INPLACE>(out, input, bias, gamma, beta, nullptr, out, m, n, (hipStream_t)stream,
                                            "add_bias_input_layernorm");
}
int lg_add_bias_input_layernorm_f16(void* out, const void* input, const void* bias, const void* gamma, const void* beta,
                                    int m, int n, void* stream) {
    return launch_ln<half_t, LN_ADD_INPLACE>((const half_t*)out, (const half_t*)input, (const half_t*)bias,
                                             (const half_t*)gamma, (const half_t*)beta, nullptr, (half_t*)out, m, n,
                                             (hipStream_t)stream, "add_bias_input_layernorm");
}
int lg_add_bias_input_layernorm_2_f32(const float* input, const float* gamma, const float* beta, const float* bias,
                                      float* output, float* norm_output, int m, int n, void* stream) {
    return launch_ln<float, LN_ADD_STORE>(output, input, bias, gamma, beta, output, norm_output, m, n,
                                          (hipStream_t)stream, "add_bias_input_layernorm_2");
}
int lg_add_bias_input_layernorm_2_f16(const void* input, const void* gamma, const void* beta, const void* bias,
                                      void* output, void* norm_output, int m, int n, void* stream) {
    return launch_ln<half_t, LN_ADD_STORE>((const half_t*)output, (const half_t*)input, (const half_t*)bias,
                                           (const half_t*)gamma, (const half_t*)beta, (half_t*)output,
                                           (half_t*)norm_output, m, n, (hipStream_t)stream, "add_bias_input_layernorm_2");
}
int lg_add_bias_input_f32(float* output, const float* bias, const float* input, int m, int n, void* stream) {
    return launch_add_bias_input<float>(output, bias, input, m, n, (hipStream_t)stream);
}
int lg_add_bias_input_f16(void* output, const void* bias, const void* input, int m, int n, void* stream) {
    return launch_add_bias_input<half_t>((half_t*)output, (const half_t*)bias, (const half_t*)input, m, n, (hipStream_t)stream);
}

}  // extern "C"
