// Latent (compressed key/value) attention: the per-token latent is RMS-normalised and stored in a paged cache, and
// queries that already carry the key up-projection ("absorbed" queries, one row of R numbers per head) attend over
// the cache rows, which serve as keys AND values.  This file holds the norm + store launch and the portable
// attention kernel (any R, f32 or bf16 storage, f32 arithmetic); the matrix-core kernels are in sm_latent_mfma.hip.
#include "sm_common.h"

namespace sm {

template <typename T>
__global__ __launch_bounds__(64) void latent_norm_store_kernel(const T* __restrict__ x, int64_t row_stride,
                                                               const T* __restrict__ w, float eps, T* __restrict__ cache,
                                                               const int32_t* __restrict__ slot_mapping, int R) {
    const int64_t t = blockIdx.x;
    const int64_t slot = slot_mapping ? slot_mapping[t] : t;        // no mapping: a dense result, row by row
    if (slot < 0) return;
    const T* xr = x + (size_t)t * row_stride;
    float ss = 0.f;
    for (int c = threadIdx.x; c < R; c += 64) {
        const float v = to_f(xr[c]);
        ss += v * v;
    }
    ss = wave_sum(ss);
    const float r = 1.f / sqrtf(ss / (float)R + eps);
    T* out = cache + (size_t)slot * R;
    for (int c = threadIdx.x; c < R; c += 64) out[c] = from_f<T>(to_f(xr[c]) * r * to_f(w[c]));
}

// The latent with a rotated key part beside it.  x rows hold [R latent | Rd key part]; the latent is RMS-normalised
// with a weight, the first rot_dims channels of the key part turn by position * inv_freq (channel 2i pairs with 2i + 1),
// and both are stored as one cache row [R + Rd].  The queries' own rotated parts (q rows hold per head [D | Rd]) turn
// the same way and land in columns R .. R + Rd of the absorbed queries qa [T, H, R + Rd].  Angles are f32.
template <typename T>
__global__ __launch_bounds__(256) void latent_rope_store_kernel(const T* __restrict__ x, int64_t x_stride, const T* __restrict__ w,
                                                                float eps, const T* __restrict__ q, int64_t q_stride,
                                                                T* __restrict__ qa, const float* __restrict__ inv_freq,
                                                                int rot_half, const int32_t* __restrict__ tok_pos,
                                                                T* __restrict__ cache, const int32_t* __restrict__ slot_mapping,
                                                                int H, int D, int R, int Rd) {
    extern __shared__ float cs[];              // rot_half cosines, then rot_half sines
    __shared__ float red[16];
    const int64_t t = blockIdx.x;
    const int tid = threadIdx.x, RK = R + Rd;
    const float pos = (float)tok_pos[t];
    for (int i = tid; i < rot_half; i += 256) sincosf(pos * inv_freq[i], cs + rot_half + i, cs + i);
    const T* xr = x + (size_t)t * x_stride;
    float ss = 0.f;
    for (int c = tid; c < R; c += 256) {
        const float v = to_f(xr[c]);
        ss += v * v;
    }
    ss = block_sum(ss, red);                   // (its barriers also publish cs)
    const float r = 1.f / sqrtf(ss / (float)R + eps);
    // queries: head hd's rotated part
    for (int e = tid; e < H * Rd; e += 256) {
        const int hd = e / Rd, c = e - hd * Rd;
        const T* qr = q + (size_t)t * q_stride + (size_t)hd * (D + Rd) + D;
        float v = to_f(qr[c]);
        if (c < 2 * rot_half) {
            const int i = c >> 1;
            const float o = to_f(qr[c ^ 1]);
            v = (c & 1) ? v * cs[i] + o * cs[rot_half + i] : v * cs[i] - o * cs[rot_half + i];
        }
        qa[((size_t)t * H + hd) * RK + R + c] = from_f<T>(v);
    }
    const int slot = slot_mapping[t];
    if (slot < 0) return;
    T* out = cache + (size_t)slot * RK;
    for (int c = tid; c < R; c += 256) out[c] = from_f<T>(to_f(xr[c]) * r * to_f(w[c]));
    for (int c = tid; c < Rd; c += 256) {
        float v = to_f(xr[R + c]);
        if (c < 2 * rot_half) {
            const int i = c >> 1;
            const float o = to_f(xr[R + (c ^ 1)]);
            v = (c & 1) ? v * cs[i] + o * cs[rot_half + i] : v * cs[i] - o * cs[rot_half + i];
        }
        out[R + c] = from_f<T>(v);
    }
}

constexpr int kRowChunk = 64;      // keys per step of the portable kernel

template <typename T>
__global__ __launch_bounds__(256) void latent_attn_rows_kernel(const T* __restrict__ q, const T* __restrict__ cache,
                                                               const int32_t* __restrict__ block_tables,
                                                               const int32_t* __restrict__ tok_seq,
                                                               const int32_t* __restrict__ tok_pos, T* __restrict__ o,
                                                               float scale, int H, int R, int block_size, int max_blocks,
                                                               int RV, int window) {
    extern __shared__ float q_lds[];                 // R floats
    __shared__ float s_lds[kRowChunk];
    __shared__ int row_lds[kRowChunk];
    const int64_t t = blockIdx.x;
    const int hd = blockIdx.y;
    const int b = tok_seq[t], n = tok_pos[t] + 1;    // keys 0 .. n-1 are visible
    const int32_t* table = block_tables + (size_t)b * max_blocks;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const T* qr = q + ((size_t)t * H + hd) * R;
    for (int c = tid; c < R; c += 256) q_lds[c] = to_f(qr[c]);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};             // channels tid, tid + 256, ... of the output row
    float m_run = -INFINITY, l_run = 0.f;
    // cache rows are R wide: all of a row is the key, its first RV columns are the value; with a window the keys start
    // at n - window
    for (int k0 = window > 0 ? max(0, n - window) : 0; k0 < n; k0 += kRowChunk) {
        __syncthreads();                             // q_lds ready / previous chunk's s_lds and row_lds consumed
        if (tid < kRowChunk) {
            const int key = k0 + tid;
            row_lds[tid] = key < n ? table[key / block_size] * block_size + key % block_size : -1;
        }
        __syncthreads();
        for (int kk = wave; kk < kRowChunk; kk += 4) {
            const int row = row_lds[kk];
            float d = 0.f;
            if (row >= 0) {
                const T* cr = cache + (size_t)row * R;
                for (int c = lane; c < R; c += 64) d += q_lds[c] * to_f(cr[c]);
            }
            d = wave_sum(d);
            if (lane == 0) s_lds[kk] = row >= 0 ? d * scale : -INFINITY;
        }
        __syncthreads();
        float mx = m_run;
        for (int kk = 0; kk < kRowChunk; ++kk) mx = fmaxf(mx, s_lds[kk]);
        const float alpha = __expf(m_run - mx);      // first chunk: exp(-inf) = 0
        float psum = 0.f;
        for (int r = 0; r < 4; ++r) acc[r] *= alpha;
        for (int kk = 0; kk < kRowChunk; ++kk) {
            const int row = row_lds[kk];
            if (row < 0) break;
            const float p = __expf(s_lds[kk] - mx);
            psum += p;
            const T* cr = cache + (size_t)row * R;
            for (int r = 0; r < 4; ++r) {
                const int c = tid + 256 * r;
                if (c < RV) acc[r] += p * to_f(cr[c]);
            }
        }
        l_run = l_run * alpha + psum;
        m_run = mx;
    }
    T* orow = o + ((size_t)t * H + hd) * RV;
    const float inv = 1.f / l_run;
    for (int r = 0; r < 4; ++r) {
        const int c = tid + 256 * r;
        if (c < RV) orow[c] = from_f<T>(acc[r] * inv);
    }
}

}  // namespace sm

using namespace sm;

extern "C" int sm_latent_norm_store(int dtype, const void* x, int64_t row_stride, const void* w, float eps, void* cache,
                                    const int32_t* slot_mapping, int64_t T, int R, void* stream) {
    if (T < 0 || R < 1 || row_stride < R || (T > 0 && (!x || !w || !cache || !slot_mapping))) {
        set_error("sm_latent_norm_store: bad argument");
        return SM_EINVAL;
    }
    if (T == 0) return SM_OK;
    SM_DISPATCH(dtype, "sm_latent_norm_store",
                hipLaunchKernelGGL(latent_norm_store_kernel<DT>, dim3((unsigned)T), dim3(64), 0, as_stream(stream), (const DT*)x,
                                   row_stride, (const DT*)w, eps, (DT*)cache, slot_mapping, R));
    SM_CHECK_LAUNCH("sm_latent_norm_store");
    return SM_OK;
}

extern "C" int sm_rms_norm_rows(int dtype, const void* x, int64_t row_stride, const void* w, float eps, void* out, int64_t T,
                                int R, void* stream) {
    if (T < 0 || R < 1 || row_stride < R || (T > 0 && (!x || !w || !out))) {
        set_error("sm_rms_norm_rows: bad argument");
        return SM_EINVAL;
    }
    if (T == 0) return SM_OK;
    SM_DISPATCH(dtype, "sm_rms_norm_rows",
                hipLaunchKernelGGL(latent_norm_store_kernel<DT>, dim3((unsigned)T), dim3(64), 0, as_stream(stream), (const DT*)x,
                                   row_stride, (const DT*)w, eps, (DT*)out, (const int32_t*)nullptr, R));
    SM_CHECK_LAUNCH("sm_rms_norm_rows");
    return SM_OK;
}

extern "C" int sm_latent_attn_rows(int dtype, const void* q, const void* cache, const int32_t* block_tables,
                                   const int32_t* tok_seq, const int32_t* tok_pos, void* o, float scale, int64_t T, int H,
                                   int R, int block_size, int max_blocks, int RV, int window, void* stream) {
    if (RV <= 0) RV = R;
    if (T < 0 || H < 1 || R < 1 || RV > R || window < 0 || block_size < 1 || max_blocks < 1 ||
        (T > 0 && (!q || !cache || !block_tables || !tok_seq || !tok_pos || !o))) {
        set_error("sm_latent_attn_rows: bad argument");
        return SM_EINVAL;
    }
    if (R > 1024 || H > 65535) { set_error("sm_latent_attn_rows: R <= 1024 and H <= 65535"); return SM_ESHAPE; }
    if (T == 0) return SM_OK;
    dim3 grid((unsigned)T, (unsigned)H);
    SM_DISPATCH(dtype, "sm_latent_attn_rows",
                hipLaunchKernelGGL(latent_attn_rows_kernel<DT>, grid, dim3(256), (size_t)R * 4, as_stream(stream), (const DT*)q,
                                   (const DT*)cache, block_tables, tok_seq, tok_pos, (DT*)o, scale, H, R, block_size, max_blocks,
                                   RV, window));
    SM_CHECK_LAUNCH("sm_latent_attn_rows");
    return SM_OK;
}

extern "C" int sm_latent_rope_store(int dtype, const void* x, int64_t x_stride, const void* w, float eps, const void* q,
                                    int64_t q_stride, void* qa, const float* inv_freq, int rot_dims, const int32_t* tok_pos,
                                    void* cache, const int32_t* slot_mapping, int64_t T, int H, int D, int R, int Rd,
                                    void* stream) {
    if (T < 0 || H < 1 || D < 0 || R < 1 || Rd < 0 || rot_dims < 0 || rot_dims % 2 || rot_dims > Rd || x_stride < R + Rd ||
        q_stride < (int64_t)H * (D + Rd) || (rot_dims > 0 && !inv_freq) ||
        (T > 0 && (!x || !w || !q || !qa || !tok_pos || !cache || !slot_mapping))) {
        set_error("sm_latent_rope_store: bad argument");
        return SM_EINVAL;
    }
    if (rot_dims > 8192) { set_error("sm_latent_rope_store: at most 8192 rotated channels"); return SM_ESHAPE; }
    if (T == 0) return SM_OK;
    SM_DISPATCH(dtype, "sm_latent_rope_store",
                hipLaunchKernelGGL(latent_rope_store_kernel<DT>, dim3((unsigned)T), dim3(256), (size_t)rot_dims * 4 + 16,
                                   as_stream(stream), (const DT*)x, x_stride, (const DT*)w, eps, (const DT*)q, q_stride, (DT*)qa,
                                   inv_freq, rot_dims / 2, tok_pos, (DT*)cache, slot_mapping, H, D, R, Rd));
    SM_CHECK_LAUNCH("sm_latent_rope_store");
    return SM_OK;
}
