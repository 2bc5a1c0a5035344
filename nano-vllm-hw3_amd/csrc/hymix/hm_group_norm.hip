// A float32 residual whose sublayers are normalised on their OUTPUT only, with an RMS norm taken over groups of
// channels: x <- x + group_norm(f(x)) * w, where f reads x itself.  One launch per token does the boundary between two
// sublayers: the norm of the result, the residual add, and the next reader's copy of x in the storage type (or, behind
// the last layer, the model's final norm).  With token ids the "result" is a row of the embedding table and x is
// assigned instead of added to (the model's first norm).  Also the scaling and soft cap of logits.
#include "hm_common.h"

namespace hm {

// row[0 .. W) holds the vector; every group of gs consecutive channels gets 1 / sqrt(mean(group^2) + eps) in rinv
__device__ __forceinline__ void group_rinv(const float* row, float* rinv, int W, int groups, float eps) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int gs = W / groups;
    for (int g = wave; g < groups; g += nw) {
        const float* p = row + (size_t)g * gs;
        float ss = 0.f;
        for (int i = lane; i < gs; i += 64) ss += p[i] * p[i];
        ss = wave_sum(ss);
        if (lane == 0) rinv[g] = 1.f / sqrtf(ss / (float)gs + eps);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void group_norm_residual_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                                  const int64_t* __restrict__ ids, const T* __restrict__ post_w,
                                                                  const T* __restrict__ next_w, int groups, float eps,
                                                                  T* __restrict__ h_out, int W) {
    extern __shared__ float row[];             // W floats, then `groups` reciprocal roots
    float* rinv = row + W;
    const int64_t t = blockIdx.x;
    const int gs = W / groups;
    float* xr = x + (size_t)t * W;
    if (y != nullptr) {
        const T* yr = y + (size_t)(ids ? ids[t] : t) * W;
        for (int c = threadIdx.x; c < W; c += 256) row[c] = to_f(yr[c]);
        __syncthreads();
        group_rinv(row, rinv, W, groups, eps);
        __syncthreads();
        for (int c = threadIdx.x; c < W; c += 256) {
            const float n = row[c] * rinv[c / gs] * to_f(post_w[c]);
            const float v = ids ? n : xr[c] + n;
            xr[c] = v;
            row[c] = v;
        }
    } else {
        for (int c = threadIdx.x; c < W; c += 256) row[c] = xr[c];
    }
    if (h_out == nullptr) return;
    T* hr = h_out + (size_t)t * W;
    if (next_w == nullptr) {                   // the sublayers read x itself: its copy in the storage type
        for (int c = threadIdx.x; c < W; c += 256) hr[c] = from_f<T>(row[c]);
        return;
    }
    __syncthreads();
    group_rinv(row, rinv, W, groups, eps);
    __syncthreads();
    for (int c = threadIdx.x; c < W; c += 256) hr[c] = from_f<T>(row[c] * rinv[c / gs] * to_f(next_w[c]));
}

__global__ void scale_softcap_kernel(float* __restrict__ x, int64_t n, float scale, float cap) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float v = x[i] * scale;
    x[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
}

}  // namespace hm

using namespace hm;

extern "C" int hm_group_norm_residual(int dtype, float* x, const void* y, const int64_t* ids, const void* post_w,
                                      const void* next_w, int groups, float eps, void* h_out, int64_t T, int W, void* stream) {
    if (T < 0 || W < 1 || groups < 1 || W % groups != 0 || (y && !post_w) || (ids && !y) || (next_w && !h_out) ||
        (T > 0 && !x)) {
        set_error("hm_group_norm_residual: bad argument");
        return HM_EINVAL;
    }
    const size_t lds = ((size_t)W + groups) * 4;
    if (lds > 60 * 1024) { set_error("hm_group_norm_residual: width %d does not fit the row buffer", W); return HM_ESHAPE; }
    if (T == 0) return HM_OK;
    HM_DISPATCH(dtype, "hm_group_norm_residual",
                hipLaunchKernelGGL(group_norm_residual_kernel<DT>, dim3((unsigned)T), dim3(256), lds, as_stream(stream), x,
                                   (const DT*)y, ids, (const DT*)post_w, (const DT*)next_w, groups, eps, (DT*)h_out, W));
    HM_CHECK_LAUNCH("hm_group_norm_residual");
    return HM_OK;
}

extern "C" int hm_scale_softcap(float* x, int64_t n, float scale, float cap, void* stream) {
    if (n < 0 || (n > 0 && !x)) {
        set_error("hm_scale_softcap: bad argument");
        return HM_EINVAL;
    }
    if (n == 0) return HM_OK;
    hipLaunchKernelGGL(scale_softcap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, as_stream(stream), x, n, scale, cap);
    HM_CHECK_LAUNCH("hm_scale_softcap");
    return HM_OK;
}
