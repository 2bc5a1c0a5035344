// Rotary attention over a paged key/value cache.  This file holds the per-token preparation launch (norms of q and k,
// rotation, value blending, cache store) and the portable attention kernel (any head sizes, f32 or bf16 storage, f32
// arithmetic) with the masks and sinks the layers can ask for; the matrix-core kernels are in hm_attn_mfma.hip.
#include "hm_common.h"

namespace hm {

// One workgroup per token.  q and k travel through LDS as f32: [H*D] then [G*D].  VEC consecutive channels per global
// access (VEC = 8 when every segment of the row starts and ends on a multiple of 8: 16-byte accesses for bf16).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void qkv_prepare_kernel(const T* __restrict__ qkv, int64_t row_stride, int H, int G, int D,
                                                          int V, const T* __restrict__ q_norm_w, const T* __restrict__ k_norm_w,
                                                          const T* __restrict__ q_head_w, const T* __restrict__ k_head_w,
                                                          const float* __restrict__ q_head_scale,
                                                          float eps, const float* __restrict__ inv_freq, int rot_half,
                                                          int unit_norm, const int32_t* __restrict__ tok_pos,
                                                          const int32_t* __restrict__ slot_mapping, T* __restrict__ k_cache,
                                                          T* __restrict__ v_cache, const T* __restrict__ v_first,
                                                          int64_t v_first_stride, const float* __restrict__ lam,
                                                          T* __restrict__ q_out, int interleaved, float rot_mag,
                                                          int v_unit_norm) {
    extern __shared__ float qk[];
    __shared__ float red[16];
    const int64_t t = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (k_cache == nullptr) G = 0;             // the row holds q only: keys and values come from another layer's cache
    const int nq = H * D, nk = G * D, nv = G * V;
    struct alignas(sizeof(T) * VEC) Pack { T v[VEC]; };
    const T* row = qkv + (size_t)t * row_stride;
    float sq = 0.f, sk = 0.f;
    for (int c = tid * VEC; c < nq + nk; c += 256 * VEC) {
        const Pack pk = *(const Pack*)(row + c);
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float v = to_f(pk.v[e]);
            qk[c + e] = v;
            ss += v * v;
        }
        if (c < nq) sq += ss; else sk += ss;
    }
    if (q_norm_w != nullptr) {                 // RMS norm over the whole projection, with a weight
        sq = block_sum(sq, red);
        sk = block_sum(sk, red);
        const float rq = 1.f / sqrtf(sq / (float)nq + eps), rk = 1.f / sqrtf(sk / (float)nk + eps);
        for (int c = tid; c < nq + nk; c += 256)
            qk[c] = c < nq ? qk[c] * rq * to_f(q_norm_w[c]) : qk[c] * rk * to_f(k_norm_w[c - nq]);
    }
    if (q_head_w != nullptr || q_head_scale != nullptr) {
        // every head RMS-normalised over its own channels with one weight row shared by the heads (a wave per head);
        // then the query heads times their own number
        __syncthreads();
        for (int hh = wave; hh < H + G; hh += 4) {
            float* p = qk + (size_t)hh * D;
            float r = 1.f;
            if (q_head_w != nullptr) {
                float ss = 0.f;
                for (int i = lane; i < D; i += 64) ss += p[i] * p[i];
                ss = wave_sum(ss);
                r = 1.f / sqrtf(ss / (float)D + eps);
            }
            const T* w = q_head_w == nullptr ? nullptr : (hh < H ? q_head_w : k_head_w);
            const float hs = (q_head_scale != nullptr && hh < H) ? q_head_scale[hh] : 1.f;
            for (int i = lane; i < D; i += 64) p[i] = (w ? p[i] * r * to_f(w[i]) : p[i]) * hs;
        }
    }
    // the angles depend on the channel pair alone: one sine and cosine per pair, shared by all heads
    float* cs = qk + nq + nk;
    const float pos = (float)tok_pos[t];
    for (int i = tid; i < rot_half; i += 256) {
        float sn, cn;
        sincosf(pos * inv_freq[i], &sn, &cn);
        cs[i] = cn * rot_mag;                  // (rot_mag = 1 leaves them as they are)
        cs[rot_half + i] = sn * rot_mag;
    }
    __syncthreads();
    for (int e = tid; e < (H + G) * rot_half; e += 256) {       // one thread per rotated pair
        const int hh = e / rot_half, i = e - hh * rot_half;
        const float c = cs[i], s = cs[rot_half + i];
        float* p = qk + (size_t)hh * D;
        // channel i pairs with channel i + rot_half, or (interleaved) channel 2i with channel 2i + 1
        const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + rot_half;
        const float a = p[ia], b = p[ib];
        p[ia] = a * c - b * s;
        p[ib] = b * c + a * s;
    }
    __syncthreads();
    if (unit_norm) {                           // every head divided by its RMS; one wave per head
        for (int hh = wave; hh < H + G; hh += 4) {
            float* p = qk + (size_t)hh * D;
            float ss = 0.f;
            for (int i = lane; i < D; i += 64) ss += p[i] * p[i];
            ss = wave_sum(ss);
            const float r = 1.f / sqrtf(ss / (float)D + eps);
            for (int i = lane; i < D; i += 64) p[i] *= r;
        }
        __syncthreads();
    }
    for (int c = tid * VEC; c < nq; c += 256 * VEC) {
        Pack pk;
#pragma unroll
        for (int e = 0; e < VEC; ++e) pk.v[e] = from_f<T>(qk[c + e]);
        *(Pack*)(q_out + (size_t)t * nq + c) = pk;
    }
    const int slot = slot_mapping[t];
    if (slot < 0) return;
    for (int c = tid * VEC; c < nk; c += 256 * VEC) {
        Pack pk;
#pragma unroll
        for (int e = 0; e < VEC; ++e) pk.v[e] = from_f<T>(qk[nq + c + e]);
        *(Pack*)(k_cache + (size_t)slot * nk + c) = pk;
    }
    const T* vr = row + nq + nk;
    if (v_unit_norm) {                         // every value head divided by its RMS (no weight); one wave per head
        for (int gg = wave; gg < G; gg += 4) {
            const T* p = vr + (size_t)gg * V;
            float ss = 0.f;
            for (int i = lane; i < V; i += 64) { const float v = to_f(p[i]); ss += v * v; }
            ss = wave_sum(ss);
            const float r = 1.f / sqrtf(ss / (float)V + eps);
            T* dst = v_cache + (size_t)slot * nv + (size_t)gg * V;
            for (int i = lane; i < V; i += 64) dst[i] = from_f<T>(to_f(p[i]) * r);
        }
    } else if (v_first != nullptr) {
        const float l = lam[0];
        const T* fr = v_first + (size_t)t * v_first_stride;
        for (int c = tid * VEC; c < nv; c += 256 * VEC) {
            const Pack a = *(const Pack*)(vr + c), f = *(const Pack*)(fr + c);
            Pack pk;
#pragma unroll
            for (int e = 0; e < VEC; ++e) pk.v[e] = from_f<T>((1.f - l) * to_f(a.v[e]) + l * to_f(f.v[e]));
            *(Pack*)(v_cache + (size_t)slot * nv + c) = pk;
        }
    } else {
        for (int c = tid * VEC; c < nv; c += 256 * VEC) *(Pack*)(v_cache + (size_t)slot * nv + c) = *(const Pack*)(vr + c);
    }
}

constexpr int kRowChunk = 64;      // keys per step of the portable kernel

// One workgroup per (token, head).  The keys a query at position i sees are enumerated as one list: with a window, the
// kept first tokens that lie before the window, then the window; without, all of 0..i.  The order of the sums depends on
// the position alone.
template <typename T>
__global__ __launch_bounds__(256) void attn_rows_kernel(const T* __restrict__ q, const T* __restrict__ k_cache,
                                                        const T* __restrict__ v_cache, const int32_t* __restrict__ block_tables,
                                                        const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                                                        const float* __restrict__ sink, int window, int keep_first, float scale,
                                                        T* __restrict__ o, int H, int G, int D, int V, int block_size,
                                                        int max_blocks, const T* __restrict__ kp_cache,
                                                        const T* __restrict__ vp_cache, int pool, int pool_rows, int chunk,
                                                        const float* __restrict__ head_bias, int sigmoid_w) {
    extern __shared__ float q_lds[];                 // D floats
    __shared__ float s_lds[kRowChunk];
    __shared__ int row_lds[kRowChunk];
    const int64_t t = blockIdx.x;
    const int hd = blockIdx.y, g = hd / (H / G);
    const int b = tok_seq[t], n = tok_pos[t] + 1;    // keys 0 .. n-1 are causal
    // the first visible key: the window's start, or (chunked mask) the start of the query's own chunk of positions
    const int lo = max(window > 0 ? max(0, n - window) : 0, chunk > 0 ? (n - 1) / chunk * chunk : 0);
    const int kept = window > 0 ? min(keep_first, lo) : 0;
    const int seen = pooled_seen(n - 1, window, pool);       // pooled blocks that lie wholly before the window
    const int total = seen + kept + (n - lo);
    const int32_t* table = block_tables + (size_t)b * max_blocks;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const T* qr = q + ((size_t)t * H + hd) * D;
    for (int c = tid; c < D; c += 256) q_lds[c] = to_f(qr[c]);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};             // channels tid, tid + 256, ... of the output row
    float m_run = -INFINITY, l_run = 0.f;
    for (int k0 = 0; k0 < total; k0 += kRowChunk) {
        __syncthreads();                             // q_lds ready / previous chunk's s_lds and row_lds consumed
        if (tid < kRowChunk) {
            const int e = k0 + tid;
            if (e < seen) {                          // a pooled entry: row -2 - r of the pooled caches
                row_lds[tid] = -2 - (table[e / pool_rows] * pool_rows + e % pool_rows);
            } else {
                const int f = e - seen;
                const int key = f < kept ? f : lo + (f - kept);
                row_lds[tid] = e < total ? table[key / block_size] * block_size + key % block_size : -1;
            }
        }
        __syncthreads();
        for (int kk = wave; kk < kRowChunk; kk += 4) {
            const int row = row_lds[kk];
            float d = 0.f;
            if (row != -1) {
                const T* kr = row >= 0 ? k_cache + ((size_t)row * G + g) * D : kp_cache + ((size_t)(-2 - row) * G + g) * D;
                for (int c = lane; c < D; c += 64) d += q_lds[c] * to_f(kr[c]);
            }
            d = wave_sum(d);
            if (lane == 0) s_lds[kk] = row != -1 ? d * scale : -INFINITY;
        }
        __syncthreads();
        if (sigmoid_w) {                             // independent weights sigmoid(score + bias), not normalised over keys
            const float hb = head_bias ? head_bias[hd] : 0.f;
            for (int kk = 0; kk < kRowChunk; ++kk) {
                const int row = row_lds[kk];
                if (row == -1) break;
                const float p = sigmoid_f(s_lds[kk] + hb);
                const T* vr = v_cache + ((size_t)row * G + g) * V;
                for (int r = 0; r < 4; ++r) {
                    const int c = tid + 256 * r;
                    if (c < V) acc[r] += p * to_f(vr[c]);
                }
            }
            continue;
        }
        float mx = m_run;
        for (int kk = 0; kk < kRowChunk; ++kk) mx = fmaxf(mx, s_lds[kk]);
        const float alpha = expf(m_run - mx);        // first chunk: exp(-inf) = 0
        float psum = 0.f;
        for (int r = 0; r < 4; ++r) acc[r] *= alpha;
        for (int kk = 0; kk < kRowChunk; ++kk) {
            const int row = row_lds[kk];
            if (row == -1) break;
            const float p = expf(s_lds[kk] - mx);
            psum += p;
            const T* vr = row >= 0 ? v_cache + ((size_t)row * G + g) * V : vp_cache + ((size_t)(-2 - row) * G + g) * V;
            for (int r = 0; r < 4; ++r) {
                const int c = tid + 256 * r;
                if (c < V) acc[r] += p * to_f(vr[c]);
            }
        }
        l_run = l_run * alpha + psum;
        m_run = mx;
    }
    float inv;
    if (sigmoid_w) {
        inv = 1.f;
    } else if (sink != nullptr) {                    // one more term in the denominator, no value
        const float sk = sink[hd], mx = fmaxf(m_run, sk), alpha = expf(m_run - mx);
        for (int r = 0; r < 4; ++r) acc[r] *= alpha;
        inv = 1.f / (l_run * alpha + expf(sk - mx));
    } else {
        inv = 1.f / l_run;
    }
    T* orow = o + ((size_t)t * H + hd) * V;
    for (int r = 0; r < 4; ++r) {
        const int c = tid + 256 * r;
        if (c < V) orow[c] = from_f<T>(acc[r] * inv);
    }
}

// Mean key and mean value of every block of `pool` tokens that a step completes.  Sequence b's portion covers the
// positions [seq_pos0[b], ctx_lens[b]); it completes the blocks seq_pos0[b] / pool .. ctx_lens[b] / pool - 1.  A
// workgroup owns one such block and kPoolCols packs of VEC channels of the joined [key | value] row; its 256 threads are
// 8 key lanes x 32 packs: a lane sums every 8th token of the block as the caches hold it (f32), the lanes' partial sums
// are added in lane order through LDS, so the order of the sum depends on the shapes alone.  (The grid is over blocks,
// not tokens: the tokens that end a block are a stride apart, which would put all the work on one XCD.)
constexpr int kPoolChunk = 64;     // tokens whose cache rows are looked up at a time
constexpr int kPoolCols = 32, kPoolLanes = 8;

template <typename T, int VEC>
__global__ __launch_bounds__(256) void pool_blocks_kernel(const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                                          T* __restrict__ kp_cache, T* __restrict__ vp_cache,
                                                          const int32_t* __restrict__ block_tables,
                                                          const int32_t* __restrict__ seq_pos0, const int32_t* __restrict__ ctx_lens,
                                                          int nk, int nv, int block_size, int max_blocks, int pool, int pool_rows) {
    __shared__ float part[kPoolLanes][kPoolCols][VEC];
    __shared__ int rows[kPoolChunk];
    const int b = blockIdx.y;
    const int blk = seq_pos0[b] / pool + blockIdx.x;
    if (blk >= ctx_lens[b] / pool) return;     // (uniform over the workgroup)
    const int first = blk * pool;
    const int32_t* table = block_tables + (size_t)b * max_blocks;
    const size_t prow = (size_t)table[blk / pool_rows] * pool_rows + blk % pool_rows;
    const float inv = 1.f / (float)pool;
    struct alignas(sizeof(T) * VEC) Pack { T v[VEC]; };
    const int tid = threadIdx.x, col = tid % kPoolCols, lane = tid / kPoolCols;
    const int c = (blockIdx.z * kPoolCols + col) * VEC;          // first channel of this thread's pack: a key channel if c < nk
    const bool live = c < nk + nv, is_k = c < nk;
    const T* src = is_k ? k_cache + c : v_cache + (c - nk);
    const int width = is_k ? nk : nv;
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
    for (int j0 = 0; j0 < pool; j0 += kPoolChunk) {
        __syncthreads();                       // the previous chunk's rows are consumed
        if (tid < kPoolChunk && j0 + tid < pool) {
            const int key = first + j0 + tid;
            rows[tid] = table[key / block_size] * block_size + key % block_size;
        }
        __syncthreads();
        const int n = min(kPoolChunk, pool - j0);
        if (live)
            for (int j = lane; j < n; j += kPoolLanes) {
                const Pack pk = *(const Pack*)(src + (size_t)rows[j] * width);
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[e] += to_f(pk.v[e]);
            }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) part[lane][col][e] = acc[e];
    __syncthreads();
    if (!live || lane != 0) return;
    Pack out;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        float sum = 0.f;
        for (int l = 0; l < kPoolLanes; ++l) sum += part[l][col][e];
        out.v[e] = from_f<T>(sum * inv);
    }
    if (is_k) *(Pack*)(kp_cache + prow * nk + c) = out;
    else *(Pack*)(vp_cache + prow * nv + (c - nk)) = out;
}

}  // namespace hm

using namespace hm;

extern "C" int hm_qkv_prepare(int dtype, const void* qkv, int64_t row_stride, int H, int G, int D, int V, const void* q_norm_w,
                              const void* k_norm_w, float eps, const float* inv_freq, int rot_half, int unit_norm,
                              const int32_t* tok_pos, const int32_t* slot_mapping, void* k_cache, void* v_cache,
                              const void* v_first, int64_t v_first_stride, const float* lam, void* q_out, int64_t T,
                              const void* q_head_w, const void* k_head_w, const float* q_head_scale, int interleaved,
                              float rot_mag, int v_unit_norm, void* stream) {
    const bool q_only = !k_cache && !v_cache;
    if (T < 0 || H < 1 || G < 1 || D < 1 || V < 1 || H % G != 0 || rot_half < 0 || 2 * rot_half > D ||
        row_stride < (q_only ? (int64_t)H * D : (int64_t)(H + G) * D + (int64_t)G * V) || (!q_norm_w) != (!k_norm_w) ||
        (rot_half > 0 && !inv_freq) || (v_first && (!lam || v_first_stride < (int64_t)G * V)) || (!k_cache) != (!v_cache) ||
        (q_only && (v_first || k_norm_w)) || (q_head_w && !q_only && !k_head_w) || (v_unit_norm && v_first) ||
        (T > 0 && (!qkv || !tok_pos || !slot_mapping || !q_out))) {
        set_error("hm_qkv_prepare: bad argument");
        return HM_EINVAL;
    }
    const size_t lds = ((size_t)(H + G) * D + 2 * (size_t)rot_half) * 4;
    if (lds > 60 * 1024) { set_error("hm_qkv_prepare: (heads + kv_heads) * dim = %d does not fit the row buffer", (H + G) * D); return HM_ESHAPE; }
    if (T == 0) return HM_OK;
    // packs need every segment (q, k, v, the rows themselves and the blended values' rows) on multiples of 8 elements
    if (q_only) G = 0;
    const bool wide = (H * D) % 8 == 0 && (G * D) % 8 == 0 && (G * V) % 8 == 0 && row_stride % 8 == 0 &&
                      (!v_first || v_first_stride % 8 == 0);
    const uintptr_t bits = (uintptr_t)qkv | (uintptr_t)v_first | (uintptr_t)q_out | (uintptr_t)k_cache | (uintptr_t)v_cache;
#define HM_PREP(VEC_)                                                                                                         \
    hipLaunchKernelGGL((qkv_prepare_kernel<DT, VEC_>), dim3((unsigned)T), dim3(256), lds, as_stream(stream), (const DT*)qkv,  \
                       row_stride, H, G, D, V, (const DT*)q_norm_w, (const DT*)k_norm_w, (const DT*)q_head_w,                 \
                       (const DT*)k_head_w, q_head_scale, eps, inv_freq, rot_half, unit_norm,                                 \
                       tok_pos, slot_mapping, (DT*)k_cache, (DT*)v_cache, (const DT*)v_first, v_first_stride, lam, (DT*)q_out, \
                       interleaved, rot_mag, v_unit_norm)
    HM_DISPATCH(dtype, "hm_qkv_prepare", if (wide && bits % (8 * sizeof(DT)) == 0) HM_PREP(8); else HM_PREP(1));
#undef HM_PREP
    HM_CHECK_LAUNCH("hm_qkv_prepare");
    return HM_OK;
}

extern "C" int hm_attn_rows(int dtype, const void* q, const void* k_cache, const void* v_cache, const int32_t* block_tables,
                            const int32_t* tok_seq, const int32_t* tok_pos, const float* sink, int window, int keep_first,
                            float scale, void* o, int64_t T, int H, int G, int D, int V, int block_size, int max_blocks,
                            const void* kp_cache, const void* vp_cache, int pool, int pool_rows, int chunk, const float* head_bias,
                            int sigmoid_w, void* stream) {
    if (T < 0 || H < 1 || G < 1 || H % G != 0 || D < 1 || V < 1 || block_size < 1 || max_blocks < 1 || window < 0 || keep_first < 0 ||
        chunk < 0 || (chunk > 0 && (keep_first > 0 || pool > 0)) || (sigmoid_w && (sink || pool > 0)) || (head_bias && !sigmoid_w) ||
        pool < 0 || (pool > 0 && (!kp_cache || !vp_cache || window < 1 || keep_first > 0 || pool_rows * pool < block_size)) ||
        (T > 0 && (!q || !k_cache || !v_cache || !block_tables || !tok_seq || !tok_pos || !o))) {
        set_error("hm_attn_rows: bad argument");
        return HM_EINVAL;
    }
    if (V > 1024 || D > 8192 || H > 65535) { set_error("hm_attn_rows: vdim <= 1024, dim <= 8192 and heads <= 65535"); return HM_ESHAPE; }
    if (T == 0) return HM_OK;
    dim3 grid((unsigned)T, (unsigned)H);
    HM_DISPATCH(dtype, "hm_attn_rows",
                hipLaunchKernelGGL(attn_rows_kernel<DT>, grid, dim3(256), (size_t)D * 4, as_stream(stream), (const DT*)q,
                                   (const DT*)k_cache, (const DT*)v_cache, block_tables, tok_seq, tok_pos, sink, window,
                                   keep_first, scale, (DT*)o, H, G, D, V, block_size, max_blocks, (const DT*)kp_cache,
                                   (const DT*)vp_cache, pool, pool_rows, chunk, head_bias, sigmoid_w));
    HM_CHECK_LAUNCH("hm_attn_rows");
    return HM_OK;
}

extern "C" int hm_pool_blocks(int dtype, const void* k_cache, const void* v_cache, void* kp_cache, void* vp_cache,
                              const int32_t* block_tables, const int32_t* seq_pos0, const int32_t* ctx_lens, int B, int max_q, int G,
                              int D, int V, int block_size, int max_blocks, int pool, int pool_rows, void* stream) {
    if (B < 0 || max_q < 0 || G < 1 || D < 1 || V < 1 || block_size < 1 || max_blocks < 1 || pool < 1 || pool_rows < 1 ||
        (int64_t)pool_rows * pool < block_size ||
        (B > 0 && max_q > 0 && (!k_cache || !v_cache || !kp_cache || !vp_cache || !block_tables || !seq_pos0 || !ctx_lens))) {
        set_error("hm_pool_blocks: bad argument");
        return HM_EINVAL;
    }
    if (B > 65535) { set_error("hm_pool_blocks: at most 65535 sequences"); return HM_ESHAPE; }
    if (B == 0 || max_q == 0) return HM_OK;
    // packs of 8 channels (16 bytes in bf16) when every row starts and ends on a multiple of 8
    const bool wide = (G * D) % 8 == 0 && (G * V) % 8 == 0;
    const uintptr_t bits = (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)kp_cache | (uintptr_t)vp_cache;
    const int blocks = max_q / pool + 1;       // the most blocks a portion of max_q tokens completes
#define HM_POOL(VEC_)                                                                                                      \
    hipLaunchKernelGGL((pool_blocks_kernel<DT, VEC_>),                                                                    \
                       dim3((unsigned)blocks, (unsigned)B, (unsigned)((G * (D + V) / VEC_ + kPoolCols - 1) / kPoolCols)),  \
                       dim3(256), 0, as_stream(stream), (const DT*)k_cache, (const DT*)v_cache, (DT*)kp_cache, (DT*)vp_cache, \
                       block_tables, seq_pos0, ctx_lens, G * D, G * V, block_size, max_blocks, pool, pool_rows)
    HM_DISPATCH(dtype, "hm_pool_blocks", if (wide && bits % (8 * sizeof(DT)) == 0) HM_POOL(8); else HM_POOL(1));
#undef HM_POOL
    HM_CHECK_LAUNCH("hm_pool_blocks");
    return HM_OK;
}
