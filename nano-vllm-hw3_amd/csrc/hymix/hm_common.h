// Shared helpers of libhymix (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../../include/hymix.h"

namespace hm {

typedef __bf16 bf16_t;
typedef bf16_t bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

void set_error(const char* fmt, ...);

template <typename T> __device__ __forceinline__ float to_f(T v) { return (float)v; }
template <typename T> __device__ __forceinline__ T from_f(float v) { return (T)v; }   // bf16: round to nearest even

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
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

__device__ __forceinline__ float sigmoid_f(float v) { return 1.f / (1.f + expf(-v)); }

// Pooled blocks a query at position `pos` sees beside its window: the blocks of `pool` tokens whose last token lies at
// or before pos - window.  (Block e of a sequence is row e % pool_rows of the pooled page block_table[e / pool_rows];
// pool_rows * pool >= block_size, so that page exists as soon as the block is complete.)
__host__ __device__ __forceinline__ int pooled_seen(int pos, int window, int pool) {
    return (pool > 0 && window > 0 && pos + 1 - window > 0) ? (pos + 1 - window) / pool : 0;
}

static inline hipStream_t as_stream(void* s) { return (hipStream_t)s; }

#define HM_CHECK_LAUNCH(name)                                                    \
    do {                                                                         \
        hipError_t e_ = hipGetLastError();                                       \
        if (e_ != hipSuccess) {                                                  \
            hm::set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
            return HM_ELAUNCH;                                                   \
        }                                                                        \
    } while (0)

// run the statement with DT = the storage type named by a dtype code
#define HM_DISPATCH(dtype, name, ...)                                        \
    do {                                                                     \
        if ((dtype) == HM_F32) { typedef float DT; __VA_ARGS__; }             \
        else if ((dtype) == HM_BF16) { typedef hm::bf16_t DT; __VA_ARGS__; }  \
        else { hm::set_error("%s: unknown dtype %d", name, (int)(dtype)); return HM_EINVAL; } \
    } while (0)

}  // namespace hm
