// The tile loop of latent attention on the matrix cores (bf16 operands, f32 accumulation).
//
// The cached latents are keys AND values, so one LDS image of a 64-key tile feeds both products.  A wave owns 32
// query rows (a row = one head of one token, an "absorbed" query of R numbers); both products are computed
// transposed so that everything a softmax row needs sits in one lane pair:
//   S^T = C . Q^T    (A = tile rows from LDS, B = Q^T kept in registers): lane l holds query (l & 31) and the keys
//                    (r & 3) + 8 (r >> 2) + 4 (l >> 5) of a 32-key half;
//   O^T += C^T . P^T (A = the same tile through the transposing LDS read, B = the lane's own probabilities): the
//                    accumulator keeps query (l & 31) per lane, so the online rescale is lane-local.
// R is padded to RP = 32 NB columns of zeros (tile and queries), rows are 2 RP + 16 bytes apart in LDS (an odd
// number of 16-byte chunks: row reads and transposed reads spread over the banks).  The next tile's global loads
// are issued before the current tile's math and land in LDS after it.  A tile never straddles a cache block
// (block_size % 64 == 0), and rows past the last needed key are read from that key's row and masked.
#pragma once
#include "sm_common.h"

namespace sm {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

constexpr int kTileKeys = 64;

template <int NB>
struct TileGeom {
    static constexpr int RP = 32 * NB, CH = RP / 8, RS = RP * 2 + 16, LDS_BYTES = kTileKeys * RS;
};

// Walks keys [k_lo, k_hi) (k_lo % 64 == 0, k_lo < k_hi) for the calling lane's query row, whose last visible key is
// row_pos; wave_min_pos = the smallest row_pos of the wave (tiles wholly below it skip the mask).  Every wave of the
// workgroup must call this with the same key range.  On return oacc holds the unnormalised output (lane: query
// l & 31, columns 32 d + 8 (r >> 2) + 4 (l >> 5) + (r & 3)), m_run the row maximum of the raw scores and l_tot the
// sum of exp2((s - m_run) * c_log2) over the row.  Only the first 32 NBV columns of a cache row are values (NBV <= NB:
// the rest of the row is key only, e.g. a rotated part).  window > 0: a row sees only the keys > row_pos - window; a
// row whose window starts behind the range's first tiles has seen nothing there (its maximum stays -inf, its weights 0).
template <int NB, int NBV, int WAVES>
__device__ __forceinline__ void latent_tile_loop(const unsigned short* __restrict__ qrow, const unsigned short* __restrict__ cache,
                                                 const int32_t* __restrict__ table, int R, int block_size, int k_lo, int k_hi,
                                                 int row_pos, int wave_min_pos, float c_log2, int window, unsigned char* lds,
                                                 f32x16 (&oacc)[NBV], float& m_run, float& l_tot) {
    typedef TileGeom<NB> G;
    constexpr int NLD = G::CH / WAVES;                     // 16-byte chunks a thread stages per tile
    const int tid = threadIdx.x, lane = tid & 63, l31 = lane & 31, hi = lane >> 5;

    bf16x8 qf[2 * NB];                                     // Q^T as the B operand: k-step ks = columns 16 ks + 8 hi .. +8
#pragma unroll
    for (int ks = 0; ks < 2 * NB; ++ks) {
        const int c0 = 16 * ks + 8 * hi;
        i32x4 v = {0, 0, 0, 0};
        if (c0 < R) v = *(const i32x4*)(qrow + c0);
        qf[ks] = __builtin_bit_cast(bf16x8, v);
    }

    i32x4 creg[NLD];
    auto load_tile = [&](int kt0) {
        const size_t row0 = (size_t)table[kt0 / block_size] * block_size + (kt0 % block_size);
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
            const int c = tid + 64 * WAVES * j;
            const int row = c / G::CH, ch = c % G::CH;
            const int key = min(kt0 + row, k_hi - 1) - kt0;
            i32x4 v = {0, 0, 0, 0};
            if (ch * 8 < R) v = *(const i32x4*)(cache + (row0 + key) * R + ch * 8);
            creg[j] = v;
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
            const int c = tid + 64 * WAVES * j;
            *(i32x4*)(lds + (c / G::CH) * G::RS + (c % G::CH) * 16) = creg[j];
        }
    };

#pragma unroll
    for (int d = 0; d < NBV; ++d)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[d][r] = 0.f;
    m_run = -INFINITY;
    float l_run = 0.f;
    const int gq = (lane >> 4) & 1, ti = lane & 15, tq = ti >> 2, tp = ti & 3;      // transposed-read address pieces

    load_tile(k_lo);
    store_tile();
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < 2 * NB; ++ks) asm volatile("" ::"v"(__builtin_bit_cast(i32x4, qf[ks])));   // loaded before the loop
    for (int kt0 = k_lo; kt0 < k_hi; kt0 += kTileKeys) {
        const bool more = kt0 + kTileKeys < k_hi;
        if (more) load_tile(kt0 + kTileKeys);

        f32x16 s[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int r = 0; r < 16; ++r) s[j][r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < 2 * NB; ++ks) {
                const bf16x8 cf = *(const bf16x8*)(lds + (32 * j + l31) * G::RS + (2 * ks + hi) * 16);
                s[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cf, qf[ks], s[j], 0, 0, 0);
            }
        }
        if (window > 0 || kt0 + kTileKeys - 1 > wave_min_pos) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = kt0 + 32 * j + (r & 3) + 8 * (r >> 2) + 4 * hi;
                    if (key > row_pos || (window > 0 && row_pos - key >= window)) s[j][r] = -INFINITY;
                }
        }
        float mx = s[0][0];
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[j][r]);
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);
        // without a window the first key of the range is visible to every row; with one a row may have seen nothing yet
        const bool none = m_new == -INFINITY;
        const float alpha = none ? 1.f : __builtin_amdgcn_exp2f((m_run - m_new) * c_log2);
        const float mc = none ? 0.f : m_new * c_log2;
        float psum = 0.f;
        bf16x8 pf[2][2];
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
                        (s16x4 __attribute__((address_space(3)))*)(lds + (r0 + tq) * G::RS + off));
                    const s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (s16x4 __attribute__((address_space(3)))*)(lds + (r0 + 8 + tq) * G::RS + off));
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
}

}  // namespace sm

// run M(NB, NBV) with the padded key and value widths of a latent row: rows whose values are the whole row, and the
// common case of a rotated key part of up to 64 columns behind the values
#define SM_BY_LATENT_SIZE(nb, nbv, M)                                                         \
    do {                                                                                      \
        if (nbv == nb || nb - nbv > 2) {                                                      \
            if (nb <= 1) M(1, 1); else if (nb == 2) M(2, 2); else if (nb == 3) M(3, 3);       \
            else if (nb == 4) M(4, 4); else if (nb <= 6) M(6, 6); else M(8, 8);               \
        } else if (nb - nbv == 1) {                                                           \
            if (nb == 2) M(2, 1); else if (nb == 3) M(3, 2); else if (nb == 4) M(4, 3);       \
            else if (nb == 5) M(5, 4); else if (nb <= 7) M(7, 6); else M(8, 7);               \
        } else {                                                                              \
            if (nb == 3) M(3, 1); else if (nb == 4) M(4, 2); else if (nb <= 6) M(6, 4);       \
            else M(8, 6);                                                                     \
        }                                                                                     \
    } while (0)
