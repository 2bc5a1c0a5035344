// A float32 residual whose sublayers sit between two Dynamic-Tanh norms: dyt(z) = tanh(alpha z) * w + b per channel, a
// scalar alpha and two vectors per norm, no statistics over the row.  One elementwise launch does the boundary between
// two sublayers: the norm of the result, the residual add, and the norm in front of the next sublayer (or, behind the
// last layer, the model's final norm).  With token ids the "result" is a row of the embedding table, assigned as it is.
#include "hm_common.h"

namespace hm {

template <typename T, int VEC>
__global__ __launch_bounds__(256) void dyt_residual_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                           const int64_t* __restrict__ ids, const T* __restrict__ post_w,
                                                           const T* __restrict__ post_b, const float* __restrict__ post_alpha,
                                                           const T* __restrict__ next_w, const T* __restrict__ next_b,
                                                           const float* __restrict__ next_alpha, T* __restrict__ h_out,
                                                           int64_t total, int W) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    if (i >= total) return;
    const int64_t t = i / W;
    const int c = (int)(i - t * W);            // VEC divides W: a pack stays inside a row
    struct alignas(sizeof(T) * VEC) Pack { T v[VEC]; };
    struct alignas(4 * VEC) PackF { float v[VEC]; };
    PackF xv;
    if (y != nullptr) {
        if (ids != nullptr) {
            const Pack e = *(const Pack*)(y + (size_t)ids[t] * W + c);
#pragma unroll
            for (int k = 0; k < VEC; ++k) xv.v[k] = to_f(e.v[k]);
        } else {
            const Pack yv = *(const Pack*)(y + i), w = *(const Pack*)(post_w + c), b = *(const Pack*)(post_b + c);
            const float a = post_alpha[0];
            xv = *(const PackF*)(x + i);
#pragma unroll
            for (int k = 0; k < VEC; ++k) xv.v[k] += tanhf(a * to_f(yv.v[k])) * to_f(w.v[k]) + to_f(b.v[k]);
        }
        *(PackF*)(x + i) = xv;
    } else {
        xv = *(const PackF*)(x + i);
    }
    if (h_out == nullptr) return;
    Pack out;
    if (next_w != nullptr) {
        const Pack w = *(const Pack*)(next_w + c), b = *(const Pack*)(next_b + c);
        const float a = next_alpha[0];
#pragma unroll
        for (int k = 0; k < VEC; ++k) out.v[k] = from_f<T>(tanhf(a * xv.v[k]) * to_f(w.v[k]) + to_f(b.v[k]));
    } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k) out.v[k] = from_f<T>(xv.v[k]);
    }
    *(Pack*)(h_out + i) = out;
}

}  // namespace hm

using namespace hm;

extern "C" int hm_dyt_residual(int dtype, float* x, const void* y, const int64_t* ids, const void* post_w, const void* post_b,
                               const float* post_alpha, const void* next_w, const void* next_b, const float* next_alpha,
                               void* h_out, int64_t T, int W, void* stream) {
    if (T < 0 || W < 1 || (y && !ids && (!post_w || !post_b || !post_alpha)) || (ids && !y) ||
        (next_w && (!next_b || !next_alpha || !h_out)) || (T > 0 && !x)) {
        set_error("hm_dyt_residual: bad argument");
        return HM_EINVAL;
    }
    if (T == 0) return HM_OK;
    const int64_t total = T * W;
    const uintptr_t bits = (uintptr_t)x | (uintptr_t)y | (uintptr_t)post_w | (uintptr_t)post_b | (uintptr_t)next_w |
                           (uintptr_t)next_b | (uintptr_t)h_out;
#define HM_DYT(VEC_)                                                                                                         \
    hipLaunchKernelGGL((dyt_residual_kernel<DT, VEC_>), dim3((unsigned)((total / VEC_ + 255) / 256)), dim3(256), 0,           \
                       as_stream(stream), x, (const DT*)y, ids, (const DT*)post_w, (const DT*)post_b, post_alpha,             \
                       (const DT*)next_w, (const DT*)next_b, next_alpha, (DT*)h_out, total, W)
    HM_DISPATCH(dtype, "hm_dyt_residual", if (W % 4 == 0 && bits % 16 == 0) HM_DYT(4); else HM_DYT(1));
#undef HM_DYT
    HM_CHECK_LAUNCH("hm_dyt_residual");
    return HM_OK;
}
