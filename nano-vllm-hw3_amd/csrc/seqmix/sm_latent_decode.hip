// Latent attention for single-token queries (decode) on the matrix cores.  The H heads of a sequence's one token are
// the query rows (they all see the same keys); the keys are split over workgroups in whole tiles, every
// (sequence, split) leaves an unnormalised partial state {m * c, l, O} in the workspace, and a second launch merges
// the splits in order.  The split count is the caller's and does not depend on the sequences' lengths.
#include "sm_latent_tile.h"

namespace sm {

// floats per (sequence, split, head) in the workspace: scaled maximum, sum, RP outputs
__host__ __device__ constexpr int part_stride(int nb) { return 32 * nb + 2; }

template <int NB, int NBV, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void latent_attn_decode_kernel(const unsigned short* __restrict__ q,
                                                                        const unsigned short* __restrict__ cache,
                                                                        const int32_t* __restrict__ block_tables,
                                                                        const int32_t* __restrict__ ctx, float* __restrict__ ws,
                                                                        float c_log2, int H, int R, int block_size,
                                                                        int max_blocks, int splits, int window) {
    typedef TileGeom<NB> G;
    __shared__ __attribute__((aligned(16))) unsigned char lds[G::LDS_BYTES];
    const int sp = blockIdx.x, b = blockIdx.y;
    const int n = ctx[b];
    // the visible keys start at the tile that holds key n - window; whole tiles per split
    const int first = window > 0 ? max(0, n - window) / kTileKeys * kTileKeys : 0;
    const int per = ((n - first + kTileKeys - 1) / kTileKeys + splits - 1) / splits * kTileKeys;
    const int k_lo = first + sp * per, k_hi = min(n, k_lo + per);
    const int lane = threadIdx.x & 63, l31 = lane & 31, hi = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = 32 * wave + l31;
    float* part = ws + (((size_t)b * splits + sp) * H + min(r, H - 1)) * part_stride(NBV);
    if (k_lo >= k_hi) {                                      // an empty split: the merge skips l == 0
        if (r < H && hi == 0) { part[0] = -INFINITY; part[1] = 0.f; }
        return;
    }
    const int rc = min(r, H - 1);
    f32x16 oacc[NBV];
    float m_run, l_tot;
    latent_tile_loop<NB, NBV, WAVES>(q + ((size_t)b * H + rc) * R, cache, block_tables + (size_t)b * max_blocks, R, block_size,
                                     k_lo, k_hi, n - 1, n - 1, c_log2, window, lds, oacc, m_run, l_tot);
    if (r >= H) return;
    if (hi == 0) { part[0] = l_tot > 0.f ? m_run * c_log2 : -INFINITY; part[1] = l_tot; }
#pragma unroll
    for (int d = 0; d < NBV; ++d)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq)
#pragma unroll
            for (int e = 0; e < 4; ++e) part[2 + 32 * d + 8 * rq + 4 * hi + e] = oacc[d][4 * rq + e];
}

__global__ void latent_decode_merge_kernel(const float* __restrict__ ws, unsigned short* __restrict__ o, int H, int R, int splits,
                                           int stride) {
    const size_t row = blockIdx.x;                          // b * H + h
    const size_t b = row / H, h = row % H;
    float M = -INFINITY;
    for (int s = 0; s < splits; ++s) {
        const float* p = ws + ((b * splits + s) * H + h) * stride;
        if (p[1] > 0.f) M = fmaxf(M, p[0]);
    }
    float L = 0.f;
    for (int s = 0; s < splits; ++s) {
        const float* p = ws + ((b * splits + s) * H + h) * stride;
        if (p[1] > 0.f) L += __builtin_amdgcn_exp2f(p[0] - M) * p[1];
    }
    const float inv = 1.f / L;
    for (int c = threadIdx.x; c < R; c += blockDim.x) {
        float acc = 0.f;
        for (int s = 0; s < splits; ++s) {
            const float* p = ws + ((b * splits + s) * H + h) * stride;
            if (p[1] > 0.f) acc += __builtin_amdgcn_exp2f(p[0] - M) * p[2 + c];
        }
        o[row * R + c] = __builtin_bit_cast(unsigned short, (bf16_t)(acc * inv));
    }
}

// the padded value width the kernel SM_BY_LATENT_SIZE picks for (R, RV)
static int padded_nbv(int R, int RV) {
    const int nb = (R + 31) / 32, nbv = (RV + 31) / 32;
    int got = 0;
#define SM_PICK(NB_, NBV_) got = NBV_
    SM_BY_LATENT_SIZE(nb, nbv, SM_PICK);
#undef SM_PICK
    return got;
}

}  // namespace sm

using namespace sm;

extern "C" size_t sm_latent_decode_workspace_bytes(int64_t B, int H, int R, int splits) {
    if (B <= 0 || H <= 0 || R <= 0 || splits <= 0) return 0;
    return (size_t)B * splits * H * part_stride(padded_nbv(R, R)) * sizeof(float);       // (a narrower value part needs less)
}

extern "C" int sm_latent_attn_decode(const void* q, const void* cache, const int32_t* block_tables, const int32_t* ctx, void* o,
                                     float scale, int64_t B, int H, int R, int block_size, int max_blocks, int splits,
                                     void* workspace, size_t workspace_bytes, int RV, int window, void* stream) {
    if (RV <= 0) RV = R;
    if (B < 0 || H < 1 || R < 1 || RV > R || window < 0 || block_size < 1 || max_blocks < 1 || splits < 1 ||
        (B > 0 && (!q || !cache || !block_tables || !ctx || !o || !workspace))) {
        set_error("sm_latent_attn_decode: bad argument");
        return SM_EINVAL;
    }
    if (R % 8 || RV % 4 || R > 256 || block_size % 64 || H > 128 || B > 65535 || splits > 65535) {
        set_error("sm_latent_attn_decode: needs R %% 8 == 0, R <= 256, block_size %% 64 == 0, H <= 128");
        return SM_ESHAPE;
    }
    if (workspace_bytes < sm_latent_decode_workspace_bytes(B, H, R, splits)) {
        set_error("sm_latent_attn_decode: workspace too small");
        return SM_EWORKSPACE;
    }
    if (B == 0) return SM_OK;
    const int nb = (R + 31) / 32, nbv = (RV + 31) / 32, waves = H <= 32 ? 1 : (H <= 64 ? 2 : 4);
    dim3 grid((unsigned)splits, (unsigned)B);
    const float c = scale * 1.4426950408889634f;
    hipStream_t s = as_stream(stream);
#define SM_DEC(NB_, NBV_, W_)                                                                                              \
    hipLaunchKernelGGL((latent_attn_decode_kernel<NB_, NBV_, W_>), grid, dim3(64 * W_), 0, s, (const unsigned short*)q,    \
                       (const unsigned short*)cache, block_tables, ctx, (float*)workspace, c, H, R, block_size, max_blocks, \
                       splits, window)
#define SM_DEC_W(NB_, NBV_) do { if (waves == 1) SM_DEC(NB_, NBV_, 1); else if (waves == 2) SM_DEC(NB_, NBV_, 2); else SM_DEC(NB_, NBV_, 4); } while (0)
    SM_BY_LATENT_SIZE(nb, nbv, SM_DEC_W);
#undef SM_DEC_W
#undef SM_DEC
    SM_CHECK_LAUNCH("sm_latent_attn_decode");
    hipLaunchKernelGGL(latent_decode_merge_kernel, dim3((unsigned)(B * H)), dim3(64), 0, s, (const float*)workspace,
                       (unsigned short*)o, H, RV, splits, part_stride(padded_nbv(R, RV)));
    SM_CHECK_LAUNCH("sm_latent_attn_decode (merge)");
    return SM_OK;
}
