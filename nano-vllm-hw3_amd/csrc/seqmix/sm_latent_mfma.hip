// Latent attention on the matrix cores, portions of any length: a workgroup of four waves owns 128 consecutive
// query rows of ONE sequence's portion (rows run token by token, head by head, so a row's last visible key is the
// position of its token) and walks the cache tiles up to the last row's position.
#include "sm_latent_tile.h"

namespace sm {

template <int NB, int NBV>
__global__ __launch_bounds__(256) void latent_attn_tiles_kernel(const unsigned short* __restrict__ q,
                                                                const unsigned short* __restrict__ cache,
                                                                const int32_t* __restrict__ block_tables,
                                                                const int32_t* __restrict__ qstart,
                                                                const int32_t* __restrict__ seq_pos0,
                                                                unsigned short* __restrict__ o, float c_log2, int H, int R,
                                                                int block_size, int max_blocks, int RV, int window) {
    typedef TileGeom<NB> G;
    __shared__ __attribute__((aligned(16))) unsigned char lds[G::LDS_BYTES];
    const int b = blockIdx.y;
    const int q0 = qstart[b], rows = (qstart[b + 1] - q0) * H;
    const int tile0 = ((int)gridDim.x - 1 - (int)blockIdx.x) * 128;            // heaviest tiles first
    if (tile0 >= rows) return;
    const int pos0 = seq_pos0[b];
    const int lane = threadIdx.x & 63, l31 = lane & 31, hi = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = tile0 + 32 * wave + l31;
    const int rc = min(r, rows - 1);
    const int row_pos = pos0 + rc / H;
    const int wave_min_pos = pos0 + min(tile0 + 32 * wave, rows - 1) / H;
    const int k_hi = pos0 + min(tile0 + 127, rows - 1) / H + 1;
    // with a window the walk starts at the tile that holds the first key the workgroup's first row sees
    const int k_lo = window > 0 ? max(0, pos0 + tile0 / H - window + 1) / kTileKeys * kTileKeys : 0;
    f32x16 oacc[NBV];
    float m_run, l_tot;
    latent_tile_loop<NB, NBV, 4>(q + ((size_t)q0 * H + rc) * R, cache, block_tables + (size_t)b * max_blocks, R, block_size, k_lo,
                                 k_hi, row_pos, wave_min_pos, c_log2, window, lds, oacc, m_run, l_tot);
    if (r >= rows) return;
    const float inv = 1.f / l_tot;
    unsigned short* op = o + ((size_t)q0 * H + r) * RV + 4 * hi;
#pragma unroll
    for (int d = 0; d < NBV; ++d)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
            if (32 * d + 8 * rq + 4 * hi >= RV) continue;
            u16x4 o4;
#pragma unroll
            for (int e = 0; e < 4; ++e) o4[e] = __builtin_bit_cast(unsigned short, (bf16_t)(oacc[d][4 * rq + e] * inv));
            *(u16x4*)(op + 32 * d + 8 * rq) = o4;
        }
}

}  // namespace sm

using namespace sm;

extern "C" int sm_latent_attn_tiles(const void* q, const void* cache, const int32_t* block_tables, const int32_t* qstart,
                                    const int32_t* seq_pos0, void* o, float scale, int B, int max_q, int H, int R, int block_size,
                                    int max_blocks, int RV, int window, void* stream) {
    if (RV <= 0) RV = R;
    if (B < 0 || max_q < 0 || H < 1 || R < 1 || RV > R || window < 0 || block_size < 1 || max_blocks < 1 ||
        (B > 0 && max_q > 0 && (!q || !cache || !block_tables || !qstart || !seq_pos0 || !o))) {
        set_error("sm_latent_attn_tiles: bad argument");
        return SM_EINVAL;
    }
    if (R % 8 || RV % 4 || R > 256 || block_size % 64 || B > 65535) {
        set_error("sm_latent_attn_tiles: needs R %% 8 == 0, R <= 256, block_size %% 64 == 0, at most 65535 sequences");
        return SM_ESHAPE;
    }
    if (B == 0 || max_q == 0) return SM_OK;
    const int64_t tiles = ((int64_t)max_q * H + 127) / 128;
    dim3 grid((unsigned)tiles, (unsigned)B), block(256);
    const float c = scale * 1.4426950408889634f;
    hipStream_t s = as_stream(stream);
    const int nb = (R + 31) / 32, nbv = (RV + 31) / 32;
#define SM_TILES(NB_, NBV_)                                                                                               \
    hipLaunchKernelGGL((latent_attn_tiles_kernel<NB_, NBV_>), grid, block, 0, s, (const unsigned short*)q,                 \
                       (const unsigned short*)cache, block_tables, qstart, seq_pos0, (unsigned short*)o, c, H, R, block_size, \
                       max_blocks, RV, window)
    SM_BY_LATENT_SIZE(nb, nbv, SM_TILES);
#undef SM_TILES
    SM_CHECK_LAUNCH("sm_latent_attn_tiles");
    return SM_OK;
}
