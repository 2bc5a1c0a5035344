// Paged key/value attention on the matrix cores (bf16).  Two kernels around one tile loop (hm_attn_tile.h):
//   portions of any length: a workgroup of four waves owns 128 consecutive query rows of ONE (sequence, key/value head);
//     rows run token by token, query head by query head of the group, so a row's position is that of its token;
//   single-token queries (decode): the group's query heads of a sequence's one token are the rows of one wave; the tile
//     list is split over workgroups, every (sequence, split, head) leaves an unnormalised partial state {m c, l, O} in the
//     workspace, and a second launch merges the splits in order and adds the sink to the denominator.
#include "hm_attn_tile.h"

namespace hm {

template <int NBK, int NBV, bool SIG>
__global__ __launch_bounds__(256) void attn_tiles_kernel(const unsigned short* __restrict__ q, const unsigned short* __restrict__ kc,
                                                         const unsigned short* __restrict__ vc,
                                                         const int32_t* __restrict__ block_tables,
                                                         const int32_t* __restrict__ qstart, const int32_t* __restrict__ seq_pos0,
                                                         const float* __restrict__ sink, int window, int keep_first, float scale,
                                                         unsigned short* __restrict__ o, int H, int G, int D, int V, int block_size,
                                                         int max_blocks, const unsigned short* __restrict__ kp,
                                                         const unsigned short* __restrict__ vp, int pool, int pool_rows,
                                                         int chunk, const float* __restrict__ head_bias) {
    __shared__ __attribute__((aligned(16))) unsigned char lds_k[TileGeom<NBK>::LDS_BYTES];
    __shared__ __attribute__((aligned(16))) unsigned char lds_v[TileGeom<NBV>::LDS_BYTES];
    const int b = blockIdx.y, g = blockIdx.z, rep = H / G;
    const int q0 = qstart[b], rows = (qstart[b + 1] - q0) * rep;
    const int tile0 = ((int)gridDim.x - 1 - (int)blockIdx.x) * 128;            // heaviest tiles first
    if (tile0 >= rows) return;
    const int pos0 = seq_pos0[b];
    const int lane = threadIdx.x & 63, l31 = lane & 31, hi = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = tile0 + 32 * wave + l31;
    const int rc = min(r, rows - 1);
    const int tok = rc / rep, head = g * rep + rc % rep;
    const int row_pos = pos0 + tok;
    const int wave_min_pos = pos0 + min(tile0 + 32 * wave, rows - 1) / rep;
    const int n_keys = pos0 + min(tile0 + 127, rows - 1) / rep + 1;
    const TileWalk walk = make_walk(pos0 + tile0 / rep, n_keys - 1, window, keep_first, pool, chunk);
    const float c_log2 = scale * 1.4426950408889634f;
    const float bias_log2 = (SIG && head_bias) ? head_bias[head] * 1.4426950408889634f : 0.f;
    f32x16 oacc[NBV];
    float m_run, l_tot;
    kv_tile_loop<NBK, NBV, 4, SIG>(q + ((size_t)(q0 + tok) * H + head) * D, kc, vc, block_tables + (size_t)b * max_blocks, D, V, G, g,
                                   block_size, walk, 0, walk.count(n_keys), n_keys, row_pos, wave_min_pos, window, keep_first, c_log2,
                                   kp, vp, pool, pool_rows, lds_k, lds_v, oacc, m_run, l_tot, chunk, bias_log2);
    if (r >= rows) return;
    // the sink joins the denominator with its own score, which is not scaled (m_run is finite: a row sees itself);
    // sigmoid weights are not normalised
    const float den = l_tot + (sink ? expf(sink[head] - m_run * scale) : 0.f);
    const float inv = SIG ? 1.f : 1.f / den;
    unsigned short* op = o + ((size_t)(q0 + tok) * H + head) * V + 4 * hi;
#pragma unroll
    for (int d = 0; d < NBV; ++d)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
            if (32 * d + 8 * rq + 4 * hi >= V) continue;
            u16x4 o4;
#pragma unroll
            for (int e = 0; e < 4; ++e) o4[e] = __builtin_bit_cast(unsigned short, (bf16_t)(oacc[d][4 * rq + e] * inv));
            *(u16x4*)(op + 32 * d + 8 * rq) = o4;
        }
}

// floats per (sequence, split, head) in the workspace: maximum in log2 units, sum, then the padded outputs
__host__ __device__ constexpr int part_stride(int nbv) { return 32 * nbv + 2; }

template <int NBK, int NBV, bool SIG>
__global__ __launch_bounds__(64) void attn_decode_kernel(const unsigned short* __restrict__ q, const unsigned short* __restrict__ kc,
                                                         const unsigned short* __restrict__ vc,
                                                         const int32_t* __restrict__ block_tables, const int32_t* __restrict__ ctx,
                                                         int window, int keep_first, float scale, float* __restrict__ ws, int H,
                                                         int G, int D, int V, int block_size, int max_blocks, int splits,
                                                         const unsigned short* __restrict__ kp,
                                                         const unsigned short* __restrict__ vp, int pool, int pool_rows, int chunk,
                                                         const float* __restrict__ head_bias) {
    __shared__ __attribute__((aligned(16))) unsigned char lds_k[TileGeom<NBK>::LDS_BYTES];
    __shared__ __attribute__((aligned(16))) unsigned char lds_v[TileGeom<NBV>::LDS_BYTES];
    const int sp = blockIdx.x, b = blockIdx.y, g = blockIdx.z, rep = H / G;
    const int n = ctx[b];
    const TileWalk walk = make_walk(n - 1, n - 1, window, keep_first, pool, chunk);
    const int nt = walk.count(n), per = (nt + splits - 1) / splits;
    const int vt_lo = sp * per, vt_hi = min(nt, vt_lo + per);
    const int lane = threadIdx.x & 63, l31 = lane & 31, hi = lane >> 5;
    const int rc = min(l31, rep - 1), head = g * rep + rc;
    float* part = ws + (((size_t)b * splits + sp) * H + head) * part_stride(NBV);
    if (vt_lo >= vt_hi) {                                    // an empty split: the merge skips l == 0
        if (l31 < rep && hi == 0) { part[0] = -INFINITY; part[1] = 0.f; }
        return;
    }
    const float c_log2 = scale * 1.4426950408889634f;
    f32x16 oacc[NBV];
    float m_run, l_tot;
    const float bias_log2 = (SIG && head_bias) ? head_bias[head] * 1.4426950408889634f : 0.f;
    kv_tile_loop<NBK, NBV, 1, SIG>(q + ((size_t)b * H + head) * D, kc, vc, block_tables + (size_t)b * max_blocks, D, V, G, g,
                                   block_size, walk, vt_lo, vt_hi, n, n - 1, n - 1, window, keep_first, c_log2, kp, vp, pool,
                                   pool_rows, lds_k, lds_v, oacc, m_run, l_tot, chunk, bias_log2);
    if (l31 >= rep) return;
    if (hi == 0) { part[0] = l_tot > 0.f ? m_run * c_log2 : -INFINITY; part[1] = l_tot; }
#pragma unroll
    for (int d = 0; d < NBV; ++d)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq)
#pragma unroll
            for (int e = 0; e < 4; ++e) part[2 + 32 * d + 8 * rq + 4 * hi + e] = oacc[d][4 * rq + e];
}

__global__ void attn_decode_merge_kernel(const float* __restrict__ ws, const float* __restrict__ sink,
                                         unsigned short* __restrict__ o, int H, int V, int splits, int stride, int plain_sum) {
    const size_t row = blockIdx.x;                          // b * H + h
    const size_t b = row / H, h = row % H;
    if (plain_sum) {                                        // weights that are not normalised: the splits' outputs add up
        for (int c = threadIdx.x; c < V; c += blockDim.x) {
            float acc = 0.f;
            for (int s = 0; s < splits; ++s) {
                const float* p = ws + ((b * splits + s) * H + h) * stride;
                if (p[1] > 0.f) acc += p[2 + c];
            }
            o[row * V + c] = __builtin_bit_cast(unsigned short, (bf16_t)acc);
        }
        return;
    }
    const float sk = sink ? sink[h] * 1.4426950408889634f : -INFINITY;       // in log2 units, as the partial maxima
    float M = sk;
    for (int s = 0; s < splits; ++s) {
        const float* p = ws + ((b * splits + s) * H + h) * stride;
        if (p[1] > 0.f) M = fmaxf(M, p[0]);
    }
    float L = sink ? __builtin_amdgcn_exp2f(sk - M) : 0.f;
    for (int s = 0; s < splits; ++s) {
        const float* p = ws + ((b * splits + s) * H + h) * stride;
        if (p[1] > 0.f) L += __builtin_amdgcn_exp2f(p[0] - M) * p[1];
    }
    const float inv = 1.f / L;
    for (int c = threadIdx.x; c < V; c += blockDim.x) {
        float acc = 0.f;
        for (int s = 0; s < splits; ++s) {
            const float* p = ws + ((b * splits + s) * H + h) * stride;
            if (p[1] > 0.f) acc += __builtin_amdgcn_exp2f(p[0] - M) * p[2 + c];
        }
        o[row * V + c] = __builtin_bit_cast(unsigned short, (bf16_t)(acc * inv));
    }
}

static int padded_nb(int n) {
    const int nb = (n + 31) / 32;
    return nb <= 2 ? nb : 4;
}

static bool pool_args_ok(const void* kp, const void* vp, int pool, int pool_rows, int window, int keep_first, int block_size) {
    if (pool < 0) return false;
    return pool == 0 || (kp && vp && window > 0 && keep_first == 0 && pool_rows > 0 && (int64_t)pool_rows * pool >= block_size);
}

static bool shape_ok(int H, int G, int D, int V, int block_size) {
    return D % 8 == 0 && V % 8 == 0 && D <= 128 && V <= 128 && block_size % kTileKeys == 0 && H % G == 0;
}

}  // namespace hm

using namespace hm;

// run M with K_ / V_ bound to the padded head sizes ...
#define HM_BY_HEAD_SIZE_(nbk, nbv, M, S)                                          \
    do {                                                                          \
        if (nbk == 1) { if (nbv == 1) M(1, 1, S); else if (nbv == 2) M(1, 2, S); else M(1, 4, S); } \
        else if (nbk == 2) { if (nbv == 1) M(2, 1, S); else if (nbv == 2) M(2, 2, S); else M(2, 4, S); } \
        else { if (nbv == 1) M(4, 1, S); else if (nbv == 2) M(4, 2, S); else M(4, 4, S); } \
    } while (0)
// ... and S_ to the kind of weights (softmax or sigmoid)
#define HM_BY_HEAD_SIZE(nbk, nbv, sig, M)                                         \
    do { if (sig) HM_BY_HEAD_SIZE_(nbk, nbv, M, true); else HM_BY_HEAD_SIZE_(nbk, nbv, M, false); } while (0)

extern "C" int hm_attn_tiles(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_tables,
                             const int32_t* qstart, const int32_t* seq_pos0, const float* sink, int window, int keep_first,
                             float scale, void* o, int B, int max_q, int H, int G, int D, int V, int block_size, int max_blocks,
                             const void* kp_cache, const void* vp_cache, int pool, int pool_rows, int chunk,
                             const float* head_bias, int sigmoid_w, void* stream) {
    if (chunk < 0 || (chunk > 0 && (keep_first > 0 || pool > 0)) || (sigmoid_w && (sink || pool > 0)) || (head_bias && !sigmoid_w)) {
        set_error("hm_attn_tiles: a chunked mask goes without kept first tokens and pooled blocks, sigmoid weights without sink and pooled blocks");
        return HM_EINVAL;
    }
    if (B < 0 || max_q < 0 || H < 1 || G < 1 || D < 1 || V < 1 || block_size < 1 || max_blocks < 1 || window < 0 || keep_first < 0 ||
        !pool_args_ok(kp_cache, vp_cache, pool, pool_rows, window, keep_first, block_size) ||
        (B > 0 && max_q > 0 && (!q || !k_cache || !v_cache || !block_tables || !qstart || !seq_pos0 || !o))) {
        set_error("hm_attn_tiles: bad argument");
        return HM_EINVAL;
    }
    if (!shape_ok(H, G, D, V, block_size) || B > 65535 || G > 65535) {
        set_error("hm_attn_tiles: needs dim and vdim multiples of 8 up to 128, block_size %% 64 == 0, at most 65535 sequences");
        return HM_ESHAPE;
    }
    if (B == 0 || max_q == 0) return HM_OK;
    const int64_t tiles = ((int64_t)max_q * (H / G) + 127) / 128;
    dim3 grid((unsigned)tiles, (unsigned)B, (unsigned)G), block(256);
    hipStream_t s = as_stream(stream);
    const int nbk = padded_nb(D), nbv = padded_nb(V);
#define HM_TILES(K_, V_, S_)                                                                                                 \
    hipLaunchKernelGGL((attn_tiles_kernel<K_, V_, S_>), grid, block, 0, s, (const unsigned short*)q, (const unsigned short*)k_cache, \
                       (const unsigned short*)v_cache, block_tables, qstart, seq_pos0, sink, window, keep_first, scale,       \
                       (unsigned short*)o, H, G, D, V, block_size, max_blocks, (const unsigned short*)kp_cache,               \
                       (const unsigned short*)vp_cache, pool, pool_rows, chunk, head_bias)
    HM_BY_HEAD_SIZE(nbk, nbv, sigmoid_w, HM_TILES);
#undef HM_TILES
    HM_CHECK_LAUNCH("hm_attn_tiles");
    return HM_OK;
}

extern "C" size_t hm_attn_decode_workspace_bytes(int64_t B, int H, int V, int splits) {
    if (B <= 0 || H <= 0 || V <= 0 || splits <= 0) return 0;
    return (size_t)B * splits * H * part_stride(padded_nb(V)) * sizeof(float);
}

extern "C" int hm_attn_decode(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_tables,
                              const int32_t* ctx, const float* sink, int window, int keep_first, float scale, void* o, int64_t B,
                              int H, int G, int D, int V, int block_size, int max_blocks, int splits, void* workspace,
                              size_t workspace_bytes, const void* kp_cache, const void* vp_cache, int pool, int pool_rows,
                              int chunk, const float* head_bias, int sigmoid_w, void* stream) {
    if (chunk < 0 || (chunk > 0 && (keep_first > 0 || pool > 0)) || (sigmoid_w && (sink || pool > 0)) || (head_bias && !sigmoid_w)) {
        set_error("hm_attn_decode: a chunked mask goes without kept first tokens and pooled blocks, sigmoid weights without sink and pooled blocks");
        return HM_EINVAL;
    }
    if (B < 0 || H < 1 || G < 1 || D < 1 || V < 1 || block_size < 1 || max_blocks < 1 || splits < 1 || window < 0 || keep_first < 0 ||
        !pool_args_ok(kp_cache, vp_cache, pool, pool_rows, window, keep_first, block_size) ||
        (B > 0 && (!q || !k_cache || !v_cache || !block_tables || !ctx || !o || !workspace))) {
        set_error("hm_attn_decode: bad argument");
        return HM_EINVAL;
    }
    if (!shape_ok(H, G, D, V, block_size) || H / G > 32 || B > 65535 || G > 65535 || splits > 65535) {
        set_error("hm_attn_decode: needs dim and vdim multiples of 8 up to 128, block_size %% 64 == 0, at most 32 query heads per group");
        return HM_ESHAPE;
    }
    if (workspace_bytes < hm_attn_decode_workspace_bytes(B, H, V, splits)) {
        set_error("hm_attn_decode: workspace too small");
        return HM_EWORKSPACE;
    }
    if (B == 0) return HM_OK;
    dim3 grid((unsigned)splits, (unsigned)B, (unsigned)G);
    hipStream_t s = as_stream(stream);
    const int nbk = padded_nb(D), nbv = padded_nb(V);
#define HM_DEC(K_, V_, S_)                                                                                                    \
    hipLaunchKernelGGL((attn_decode_kernel<K_, V_, S_>), grid, dim3(64), 0, s, (const unsigned short*)q, (const unsigned short*)k_cache, \
                       (const unsigned short*)v_cache, block_tables, ctx, window, keep_first, scale, (float*)workspace, H, G, D, \
                       V, block_size, max_blocks, splits, (const unsigned short*)kp_cache, (const unsigned short*)vp_cache, pool, \
                       pool_rows, chunk, head_bias)
    HM_BY_HEAD_SIZE(nbk, nbv, sigmoid_w, HM_DEC);
#undef HM_DEC
    HM_CHECK_LAUNCH("hm_attn_decode");
    hipLaunchKernelGGL(attn_decode_merge_kernel, dim3((unsigned)(B * H)), dim3(64), 0, s, (const float*)workspace, sink,
                       (unsigned short*)o, H, V, splits, part_stride(nbv), sigmoid_w);
    HM_CHECK_LAUNCH("hm_attn_decode (merge)");
    return HM_OK;
}
