// common.hpp -- shared device helpers for the gfx950 (CDNA4, wave64) kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/liger_hip.h"

namespace lg {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef short short4_t __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// thread-local error text, set by the host-side launchers
void set_error(const char* fmt, ...);
int check_launch(const char* what);

// What is known about a stream (runtime.hip): the compute units its kernels may run on (fewer than the device for a CU-masked
// stream) and its split-K workspace (nullptr for a stream the library neither created nor was told about with lg_stream_attach).
constexpr size_t LG_SPLITK_WORKSPACE_BYTES = (size_t)64 << 20;
struct StreamInfo {
    int cus;
    float* ws;
    size_t ws_bytes;
};
StreamInfo stream_info(hipStream_t stream);
int device_cu_count();

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

// Block-wide sum for up to 1024 threads (16 waves); every thread gets the result.
// `scratch` must hold 16 floats; two back-to-back calls may reuse it (barrier at entry).
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    if (nw == 1) return v;
    __syncthreads();
    if (lane == 0) scratch[wid] = v;
    __syncthreads();
    float r = (lane < nw) ? scratch[lane] : 0.f;
    return wave_sum(r);
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    v = wave_max(v);
    if (nw == 1) return v;
    __syncthreads();
    if (lane == 0) scratch[wid] = v;
    __syncthreads();
    float r = (lane < nw) ? scratch[lane] : -3.0e38f;
    return wave_max(r);
}

// scalar load/store helpers that work for both element types
template <typename T> __device__ __forceinline__ float ldf(const T* p) { return (float)(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v) { *p = (T)v; }

// 16-byte vector of T
template <typename T> struct Vec16;
template <> struct Vec16<float> {
    static constexpr int N = 4;
    float4_t v;
    __device__ __forceinline__ float get(int i) const { return v[i]; }
    __device__ __forceinline__ void set(int i, float x) { v[i] = x; }
};
template <> struct Vec16<half_t> {
    static constexpr int N = 8;
    half8_t v;
    __device__ __forceinline__ float get(int i) const { return (float)v[i]; }
    __device__ __forceinline__ void set(int i, float x) { v[i] = (half_t)x; }
};

__device__ __forceinline__ float gelu_tanh(float x) {
    // 0.5 x (1 + tanh(0.79788456 (x + 0.044715 x^3)))   (reference cuda_kernels.cu:9-15)
    // evaluated as x / (1 + exp(-2u)), the same function with one hardware exp2 and one reciprocal
    const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    const float e = __builtin_amdgcn_exp2f(-2.0f * 1.4426950408889634f * u);  // inf for very negative x: result -0
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
__device__ __forceinline__ bool aligned_dev16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace lg
