// weight_layout.hip -- re-laying a weight matrix into the tiled (fragment-block) layout and back.
//
// No reference counterpart: the reference never initialises or loads a weight, so the storage layout is private to the
// Linear_* classes (linear.h:40,92 allocate k * n / world_size elements and nothing else is said about them).  A layer
// that owns its weights re-lays them once, when they are loaded, into the layout its kernels read fastest; the GEMM entry
// points take that layout as transa = LG_OP_TILED.
#include "gemm_common.hpp"

namespace lg {

// one thread per 8 consecutive k of one feature: 16 bytes in the tiled matrix
template <bool TO_TILED>
__global__ __launch_bounds__(256) void weight_tile_kernel(half_t* dst, const half_t* src, int N, int K, int src_nk, int64_t ld) {
    const int64_t vecs = (int64_t)N * (K >> 3);
    for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < vecs; v += (int64_t)gridDim.x * blockDim.x) {
        // v enumerates the tiled matrix in storage order: consecutive threads touch consecutive 16-byte pieces of it
        const int64_t blk = v >> 6;
        const int ln = (int)(v & 63);
        const int t = (int)(blk / (K >> 5)), c = (int)(blk % (K >> 5));
        const int n = t * 16 + (ln & 15), k = c * 32 + (ln >> 4) * 8;
        half_t* tp = (TO_TILED ? dst : const_cast<half_t*>(src)) + v * 8;
        if (src_nk) {
            half_t* lp = (TO_TILED ? const_cast<half_t*>(src) : dst) + (int64_t)n * ld + k;
            if (TO_TILED) *reinterpret_cast<half8_t*>(tp) = *reinterpret_cast<const half8_t*>(lp);
            else *reinterpret_cast<half8_t*>(lp) = *reinterpret_cast<const half8_t*>(tp);
        } else {
            half_t* lp = (TO_TILED ? const_cast<half_t*>(src) : dst) + (int64_t)k * ld + n;
            if (TO_TILED) {
                half8_t r;
#pragma unroll
                for (int i = 0; i < 8; ++i) r[i] = lp[(int64_t)i * ld];
                *reinterpret_cast<half8_t*>(tp) = r;
            } else {
                const half8_t r = *reinterpret_cast<const half8_t*>(tp);
#pragma unroll
                for (int i = 0; i < 8; ++i) lp[(int64_t)i * ld] = r[i];
            }
        }
    }
}

static int relay(const char* what, bool to_tiled, void* dst, const void* src, int features, int k, int plain_transa, int ld, void* stream) {
    if (features < 0 || k < 0 || (plain_transa != 0 && plain_transa != 1)) { set_error("%s: bad arguments", what); return LG_ERR_INVALID; }
    if (features == 0 || k == 0) return LG_OK;
    if (!dst || !src || features % 16 != 0 || k % 32 != 0 || !aligned16(dst) || !aligned16(src) || dst == src) {
        set_error("%s: needs distinct 16-byte aligned matrices, features %% 16 == 0 and k %% 32 == 0 (features=%d k=%d)", what, features, k);
        return LG_ERR_INVALID;
    }
    const int min_ld = plain_transa ? k : features;
    if (ld < min_ld || (plain_transa && (ld % 8 != 0))) { set_error("%s: leading dimension %d too small or not a multiple of 8", what, ld); return LG_ERR_INVALID; }
    const int64_t vecs = (int64_t)features * (k >> 3);
    int grid = (int)((vecs + 255) / 256);
    if (grid > 65536) grid = 65536;
    if (to_tiled) hipLaunchKernelGGL(weight_tile_kernel<true>, dim3(grid), dim3(256), 0, (hipStream_t)stream, (half_t*)dst, (const half_t*)src, features, k, plain_transa, (int64_t)ld);
    else hipLaunchKernelGGL(weight_tile_kernel<false>, dim3(grid), dim3(256), 0, (hipStream_t)stream, (half_t*)dst, (const half_t*)src, features, k, plain_transa, (int64_t)ld);
    return check_launch(what);
}

}  // namespace lg

using namespace lg;

extern "C" {

int lg_weight_tile_f16(void* tiled, const void* plain, int features, int k, int plain_transa, int ld_plain, void* stream) {
    return relay("lg_weight_tile_f16", true, tiled, plain, features, k, plain_transa, ld_plain, stream);
}
int lg_weight_untile_f16(void* plain, const void* tiled, int features, int k, int plain_transa, int ld_plain, void* stream) {
    return relay("lg_weight_untile_f16", false, plain, tiled, features, k, plain_transa, ld_plain, stream);
}

}  // extern "C"
