// Shared helpers of libseqmix (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../../include/seqmix.h"

namespace sm {

typedef __bf16 bf16_t;
typedef bf16_t bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));

void set_error(const char* fmt, ...);

template <typename T> __device__ __forceinline__ float to_f(T v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f(float v) { return (T)v; }   // bf16: round to nearest even

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

// sum over a workgroup of up to 16 waves; `red` = 16 floats of LDS; every thread gets the total
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();                      // red may still be read from a previous call
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += red[i];
    return t;
}

// what an expert applies between its two products (SM_ACT_*): the clamped GLU of a gate and an up product, or a GELU
// of the up product alone (exact, or the tanh form)
__device__ __forceinline__ float gelu_erf(float z) { return 0.5f * z * (1.f + erff(z * 0.70710678118654752f)); }
__device__ __forceinline__ float gelu_tanh(float z) {
    return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
// the gated forms: g' = min(g, limit), u' = clamp(u, +-limit), g' sigmoid(alpha g') (u' + 1) (SM_ACT_CLAMPED_GLU), or with
// SM_ACT_SILU_GLU the same without the one: silu(g) u for limit = +inf and alpha = 1
__device__ __forceinline__ float gated_act(float g, float u, float limit, float alpha, int act) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.f + __expf(-alpha * g)) * (u + (act == SM_ACT_SILU_GLU ? 0.f : 1.f));
}
__device__ __forceinline__ bool act_is_gated(int act) { return act == SM_ACT_CLAMPED_GLU || act == SM_ACT_SILU_GLU; }
__device__ __forceinline__ float plain_act(float z, int act) { return act == SM_ACT_GELU_TANH ? gelu_tanh(z) : gelu_erf(z); }

static inline hipStream_t as_stream(void* s) { return (hipStream_t)s; }

#define SM_CHECK_LAUNCH(name)                                                    \
    do {                                                                         \
        hipError_t e_ = hipGetLastError();                                       \
        if (e_ != hipSuccess) {                                                  \
            sm::set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
            return SM_ELAUNCH;                                                   \
        }                                                                        \
    } while (0)

// run `call<T>` for the storage type named by a dtype code
#define SM_DISPATCH(dtype, name, ...)                                        \
    do {                                                                     \
        if ((dtype) == SM_F32) { typedef float DT; __VA_ARGS__; }             \
        else if ((dtype) == SM_BF16) { typedef sm::bf16_t DT; __VA_ARGS__; }  \
        else { sm::set_error("%s: unknown dtype %d", name, (int)(dtype)); return SM_EINVAL; } \
    } while (0)

}  // namespace sm
