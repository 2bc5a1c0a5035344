// The tile loop of paged key/value attention on the matrix cores (bf16 operands, f32 accumulation).
//
// A wave owns 32 query rows that read the same key/value head (the query heads of one group, token after token).  Both
// products are computed transposed, so that everything a softmax row needs sits in one lane pair:
//   S^T = K . Q^T    (A = key rows of a 64-key tile from LDS, B = Q^T kept in registers): lane l holds query (l & 31)
//                    and the keys (r & 3) + 8 (r >> 2) + 4 (l >> 5) of a 32-key half;
//   O^T += V^T . P^T (A = the value tile through the transposing LDS read, B = the lane's own probabilities): the
//                    accumulator keeps query (l & 31) per lane, so the online rescale is lane-local.
// Head sizes are padded to 32 NBK / 32 NBV columns of zeros; LDS rows are an odd number of 16-byte chunks apart.  The
// next tile's global loads are issued before the current tile's math and land in LDS after it.  A tile never straddles
// a cache block (block_size % 64 == 0); rows past the last needed key are read from that key's row and masked.
//
// Tiles are 64 keys from key 0, whatever the step brings, so the order of every sum depends on positions alone.  With a
// window the walk is over a list: the tiles that hold kept first tokens, then the tiles from the window's start; tiles
// between are skipped (every score in them is masked, and a masked score adds an exact zero).  With pooled blocks the
// list starts with tiles of 64 pooled entries (block means, read from the pooled caches row by row through the block
// table); an entry is masked for the rows whose window has not yet passed its block.
#pragma once
#include "hm_common.h"

namespace hm {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

constexpr int kTileKeys = 64;

template <int NB>
struct TileGeom {
    static constexpr int P = 32 * NB, CH = P / 8, RS = P * 2 + 16, LDS_BYTES = kTileKeys * RS;
};

// The list of tiles a group of rows walks.  keep_tiles tiles from key 0, then tiles from key win_lo (a multiple of 64,
// >= 64 keep_tiles) up to the causal end.
struct TileWalk {
    int pool_tiles, n_pool, keep_tiles, win_lo;
    // first key of token tile vt (vt >= pool_tiles); a pooled tile vt < pool_tiles starts at entry 64 vt
    __device__ __forceinline__ int key0(int vt) const {
        const int u = vt - pool_tiles;
        return u < keep_tiles ? u * kTileKeys : win_lo + (u - keep_tiles) * kTileKeys;
    }
    __device__ __forceinline__ int count(int n_keys) const {
        return pool_tiles + keep_tiles + (n_keys - win_lo + kTileKeys - 1) / kTileKeys;
    }
};

// min_pos / max_pos = the smallest / largest position among the rows that walk together
// chunk > 0: a row also sees nothing before the start of its own chunk of `chunk` positions
__device__ __forceinline__ TileWalk make_walk(int min_pos, int max_pos, int window, int keep_first, int pool, int chunk = 0) {
    TileWalk w;
    w.n_pool = pooled_seen(max_pos, window, pool);
    w.pool_tiles = (w.n_pool + kTileKeys - 1) / kTileKeys;
    int lo = window > 0 ? max(0, min_pos - window + 1) : 0;
    if (chunk > 0) lo = max(lo, min_pos / chunk * chunk);
    w.win_lo = lo / kTileKeys * kTileKeys;
    w.keep_tiles = window > 0 ? min((keep_first + kTileKeys - 1) / kTileKeys, w.win_lo / kTileKeys) : 0;
    return w;
}

// Walks tiles [vt_lo, vt_hi) of `walk` for the calling lane's query row at position row_pos; wave_min_pos = the smallest
// position of the wave's rows.  Every wave of the workgroup must call this with the same tiles.  On return oacc holds the
// unnormalised output (lane: query l & 31, columns 32 d + 8 (r >> 2) + 4 (l >> 5) + (r & 3)), m_run the row maximum of
// the raw scores (-inf if the row saw no key) and l_tot the sum of exp2((s - m_run) * c_log2) over the row.
// SIG: the weight of a visible key is sigmoid(score * scale + bias), bias_log2 = the row's bias times log2(e); the weights
// are not normalised, oacc is the output itself, m_run = 0 and l_tot = 1.
template <int NBK, int NBV, int WAVES, bool SIG = false>
__device__ __forceinline__ void kv_tile_loop(const unsigned short* __restrict__ qrow, const unsigned short* __restrict__ kc,
                                             const unsigned short* __restrict__ vc, const int32_t* __restrict__ table, int D, int V,
                                             int G, int g, int block_size, TileWalk walk, int vt_lo, int vt_hi, int n_keys,
                                             int row_pos, int wave_min_pos, int window, int keep_first, float c_log2,
                                             const unsigned short* __restrict__ kp, const unsigned short* __restrict__ vp,
                                             int pool, int pool_rows, unsigned char* lds_k, unsigned char* lds_v, f32x16 (&oacc)[NBV], float& m_run,
                                             float& l_tot, int chunk = 0, float bias_log2 = 0.f) {
    typedef TileGeom<NBK> GK;
    typedef TileGeom<NBV> GV;
    constexpr int NLK = GK::CH / WAVES, NLV = GV::CH / WAVES;      // 16-byte chunks a thread stages per tile
    const int tid = threadIdx.x, lane = tid & 63, l31 = lane & 31, hi = lane >> 5;

    bf16x8 qf[2 * NBK];                                    // Q^T as the B operand: k-step ks = columns 16 ks + 8 hi .. +8
#pragma unroll
    for (int ks = 0; ks < 2 * NBK; ++ks) {
        const int c0 = 16 * ks + 8 * hi;
        i32x4 v = {0, 0, 0, 0};
        if (c0 < D) v = *(const i32x4*)(qrow + c0);
        qf[ks] = __builtin_bit_cast(bf16x8, v);
    }

    i32x4 kreg[NLK], vreg[NLV];
    auto load_tile = [&](int vt) {
        if (vt < walk.pool_tiles) {                        // 64 pooled entries, each found through the block table
#pragma unroll
            for (int j = 0; j < NLK; ++j) {
                const int c = tid + 64 * WAVES * j;
                const int row = c / GK::CH, ch = c % GK::CH;
                const int e = min(vt * kTileKeys + row, walk.n_pool - 1);
                const size_t prow = (size_t)table[e / pool_rows] * pool_rows + e % pool_rows;
                i32x4 v = {0, 0, 0, 0};
                if (ch * 8 < D) v = *(const i32x4*)(kp + (prow * G + g) * D + ch * 8);
                kreg[j] = v;
            }
#pragma unroll
            for (int j = 0; j < NLV; ++j) {
                const int c = tid + 64 * WAVES * j;
                const int row = c / GV::CH, ch = c % GV::CH;
                const int e = min(vt * kTileKeys + row, walk.n_pool - 1);
                const size_t prow = (size_t)table[e / pool_rows] * pool_rows + e % pool_rows;
                i32x4 v = {0, 0, 0, 0};
                if (ch * 8 < V) v = *(const i32x4*)(vp + (prow * G + g) * V + ch * 8);
                vreg[j] = v;
            }
            return;
        }
        const int kt0 = walk.key0(vt);
        const size_t row0 = (size_t)table[kt0 / block_size] * block_size + (kt0 % block_size);
#pragma unroll
        for (int j = 0; j < NLK; ++j) {
            const int c = tid + 64 * WAVES * j;
            const int row = c / GK::CH, ch = c % GK::CH;
            const int key = min(kt0 + row, n_keys - 1) - kt0;
            i32x4 v = {0, 0, 0, 0};
            if (ch * 8 < D) v = *(const i32x4*)(kc + ((row0 + key) * G + g) * D + ch * 8);
            kreg[j] = v;
        }
#pragma unroll
        for (int j = 0; j < NLV; ++j) {
            const int c = tid + 64 * WAVES * j;
            const int row = c / GV::CH, ch = c % GV::CH;
            const int key = min(kt0 + row, n_keys - 1) - kt0;
            i32x4 v = {0, 0, 0, 0};
            if (ch * 8 < V) v = *(const i32x4*)(vc + ((row0 + key) * G + g) * V + ch * 8);
            vreg[j] = v;
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int j = 0; j < NLK; ++j) {
            const int c = tid + 64 * WAVES * j;
            *(i32x4*)(lds_k + (c / GK::CH) * GK::RS + (c % GK::CH) * 16) = kreg[j];
        }
#pragma unroll
        for (int j = 0; j < NLV; ++j) {
            const int c = tid + 64 * WAVES * j;
            *(i32x4*)(lds_v + (c / GV::CH) * GV::RS + (c % GV::CH) * 16) = vreg[j];
        }
    };

#pragma unroll
    for (int d = 0; d < NBV; ++d)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[d][r] = 0.f;
    m_run = -INFINITY;
    float l_run = 0.f;
    const int gq = (lane >> 4) & 1, ti = lane & 15, tq = ti >> 2, tp = ti & 3;      // transposed-read address pieces

    const int my_pool = pooled_seen(row_pos, window, pool);   // pooled entries this row sees
    const int chunk_lo = chunk > 0 ? row_pos / chunk * chunk : 0;
    load_tile(vt_lo);
    store_tile();
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < 2 * NBK; ++ks) asm volatile("" ::"v"(__builtin_bit_cast(i32x4, qf[ks])));   // loaded before the loop
    for (int vt = vt_lo; vt < vt_hi; ++vt) {
        const bool pooled = vt < walk.pool_tiles;
        const int kt0 = pooled ? vt * kTileKeys : walk.key0(vt);
        const bool more = vt + 1 < vt_hi;
        if (more) load_tile(vt + 1);

        f32x16 s[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int r = 0; r < 16; ++r) s[j][r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < 2 * NBK; ++ks) {
                const bf16x8 kf = *(const bf16x8*)(lds_k + (32 * j + l31) * GK::RS + (2 * ks + hi) * 16);
                s[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], s[j], 0, 0, 0);
            }
        }
        if (SIG) {                                           // the logit in log2 units, before the mask
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) s[j][r] = __builtin_fmaf(s[j][r], c_log2, bias_log2);
        }
        if (pooled) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int e = kt0 + 32 * j + (r & 3) + 8 * (r >> 2) + 4 * hi;
                    if (e >= my_pool) s[j][r] = -INFINITY;
                }
        } else if (window > 0 || chunk > 0 || kt0 + kTileKeys - 1 > wave_min_pos) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = kt0 + 32 * j + (r & 3) + 8 * (r >> 2) + 4 * hi;
                    const bool seen = key <= row_pos && key >= chunk_lo &&
                                      (window <= 0 || row_pos - key < window || key < keep_first);
                    if (!seen) s[j][r] = -INFINITY;
                }
        }
        bf16x8 pf[2][2];
        if (SIG) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int e = 0; e < 8; ++e)          // a masked logit is -inf: exp2(+inf) = inf and the weight is 0
                        pf[j][t][e] = (bf16_t)__builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-s[j][8 * t + e]));
        } else {
            float mx = s[0][0];
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[j][r]);
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run, mx);
            // a row may have seen nothing yet (its window starts in a later tile): no rescale, and every weight is zero
            const bool none = m_new == -INFINITY;
            const float alpha = none ? 1.f : __builtin_amdgcn_exp2f((m_run - m_new) * c_log2);
            const float mc = none ? 0.f : m_new * c_log2;
            float psum = 0.f;
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[j][8 * t + e], c_log2, -mc));
                        psum += p;
                        pf[j][t][e] = (bf16_t)p;
                    }
            l_run = l_run * alpha + psum;
            m_run = m_new;
            if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
                for (int d = 0; d < NBV; ++d)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[d][r] *= alpha;
            }
        }
#pragma unroll
        for (int d = 0; d < NBV; ++d)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const int r0 = 32 * j + 16 * t + 4 * hi;
                    const int c0 = 4 * d + 2 * gq;
                    const int off = (c0 + (tp >> 1)) * 16 + 8 * (tp & 1);
                    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (s16x4 __attribute__((address_space(3)))*)(lds_v + (r0 + tq) * GV::RS + off));
                    const s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (s16x4 __attribute__((address_space(3)))*)(lds_v + (r0 + 8 + tq) * GV::RS + off));
                    const s16x8 vv = {lo[0], lo[1], lo[2], lo[3], hi4[0], hi4[1], hi4[2], hi4[3]};
                    oacc[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vv), pf[j][t], oacc[d], 0, 0, 0);
                }
        __syncthreads();
        if (more) {
            store_tile();
            __syncthreads();
        }
    }
    l_tot = l_run + __shfl_xor(l_run, 32);
    if (SIG) { m_run = 0.f; l_tot = 1.f; }
}

}  // namespace hm
