// Expert products for many tokens on the matrix cores (bf16): the (token, expert) pairs are grouped by expert into
// tiles of 32 rows (sm_moe_align), so that one workgroup multiplies 32 rows of one expert by 128 of its output
// columns; gate and up are produced together and leave as the clamped GLU, the down product leaves per pair and a
// last launch sums a token's pairs with their weights (and the shared expert) in a fixed order.
//
// A row of the result depends only on its own inputs: which other pairs share its tile does not change it, so the
// (arbitrary) order of pairs inside an expert's group leaves every value as it is.
//
// Operands go from global memory straight to the MFMA registers: both matrices are K-contiguous, a lane owns one row
// and 32 consecutive k of a 64-k step (four 16-byte loads, four MFMA steps; the k order inside a step is free as
// long as both operands agree).
#include "sm_common.h"

namespace sm {

constexpr int kRowsPerTile = 32;

__global__ __launch_bounds__(1024) void moe_align_kernel(const int32_t* __restrict__ idx, int P, int E, int max_tiles,
                                                         int32_t* __restrict__ row_pair, int32_t* __restrict__ tile_expert,
                                                         int32_t* __restrict__ pair_row) {
    extern __shared__ int sh[];                 // counts[E], offs[E], cursor[E]
    int* counts = sh;
    int* offs = sh + E;
    int* cursor = sh + 2 * E;
    for (int e = threadIdx.x; e < E; e += blockDim.x) { counts[e] = 0; cursor[e] = 0; }
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += blockDim.x) atomicAdd(&counts[idx[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int tiles = 0;
        for (int e = 0; e < E; ++e) {
            offs[e] = tiles * kRowsPerTile;
            const int n = (counts[e] + kRowsPerTile - 1) / kRowsPerTile;
            for (int i = 0; i < n; ++i) tile_expert[tiles + i] = e;
            tiles += n;
        }
        for (int i = tiles; i < max_tiles; ++i) tile_expert[i] = -1;
    }
    for (int r = threadIdx.x; r < max_tiles * kRowsPerTile; r += blockDim.x) row_pair[r] = -1;
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += blockDim.x) {
        const int e = idx[p];
        const int r = offs[e] + atomicAdd(&cursor[e], 1);
        row_pair[r] = p;
        pair_row[p] = r;
    }
}

__device__ __forceinline__ float glu_bf16(float g, float u, float limit, float alpha, int act) {
    // the products leave the matrix unit in bf16, as a GEMM's output would
    return gated_act((float)(bf16_t)g, (float)(bf16_t)u, limit, alpha, act);
}

__device__ __forceinline__ bf16x8 load8(const unsigned short* p, int k, int K) {
    i32x4 v = {0, 0, 0, 0};
    if (k + 8 <= K) v = *(const i32x4*)(p + k);
    return __builtin_bit_cast(bf16x8, v);
}

// GATE_UP: A = h rows gathered by token, B = the expert's gate and up rows, out = act [rows, N] (N = F, K = W)
// else:    A = act rows,                 B = the expert's down rows,       out = per-row products [rows, N] (N = W, K = F)
// MODE 0: the down product; 1: gate and up with the gated activation (act_kind: clamped GLU or silu(g) u); 2: the up product alone with a GELU (act_kind)
template <int MODE>
__global__ __launch_bounds__(256) void moe_grouped_kernel(const unsigned short* __restrict__ a, const unsigned short* __restrict__ w,
                                                          const int32_t* __restrict__ row_pair, const int32_t* __restrict__ tile_expert,
                                                          unsigned short* __restrict__ out, int top, int N, int K, float limit,
                                                          float alpha, int act_kind) {
    constexpr bool GATE_UP = MODE == 1, FROM_TOKENS = MODE != 0;
    const int tile = blockIdx.x;
    const int e = tile_expert[tile];
    if (e < 0) return;
    const int lane = threadIdx.x & 63, l31 = lane & 31, hi = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n0 = blockIdx.y * 128 + wave * 32;
    if (n0 >= N) return;
    const int row = tile * kRowsPerTile + l31;
    const int pair = row_pair[row];
    const unsigned short* ap = FROM_TOKENS ? a + (size_t)(pair < 0 ? 0 : pair / top) * K : a + (size_t)row * K;
    // weights in the tiled layout of sm_moe_tile_weights: block (expert, 32-row block, 64-k step) = 4 KB, chunk s of
    // lane L at 16 (64 s + L): a wave's load is one contiguous KB
    const int nb32 = (N + 31) / 32, ksteps = (K + 63) / 64;
    const unsigned short* bp = w + (((size_t)e * (GATE_UP ? 2 : 1) * nb32 + n0 / 32) * ksteps) * 2048 + 8 * lane;
    const unsigned short* bp2 = bp + (size_t)nb32 * ksteps * 2048;      // the up blocks follow the gate blocks
    f32x16 acc = {0}, acc2 = {0};
    // A ring of three 64-k steps in flight: with a handful of rows per expert (decode) a wave's eight MFMAs per step
    // hide nothing, so the weight stream has to be kept busy by outstanding loads (3 x 12 KB per wave).  Steps past K
    // load zeros (both operands), which leave the sums as they are.
    struct Stage { bf16x8 a[4], b[4], b2[4]; };
    auto request = [&](Stage& st, int k0) {
        const int kb = k0 + 32 * hi;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            st.a[s] = load8(ap, kb + 8 * s, K);
            // (steps past K: the ring runs up to two steps over; clamp to the last block and let A's zeros cancel it)
            const size_t boff = (size_t)min(k0 / 64, ksteps - 1) * 2048 + 512 * s;
            st.b[s] = *(const bf16x8*)(bp + boff);
            if (GATE_UP) st.b2[s] = *(const bf16x8*)(bp2 + boff);
        }
    };
    auto consume = [&](const Stage& st) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(st.a[s], st.b[s], acc, 0, 0, 0);
            if (GATE_UP) acc2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(st.a[s], st.b2[s], acc2, 0, 0, 0);
        }
    };
    Stage s0, s1, s2;
    request(s0, 0);
    request(s1, 64);
    request(s2, 128);
    for (int k0 = 0; k0 < K; k0 += 192) {
        consume(s0);
        request(s0, k0 + 192);
        consume(s1);
        request(s1, k0 + 256);
        consume(s2);
        request(s2, k0 + 320);
    }
    if (n0 + l31 >= N) return;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int orow = tile * kRowsPerTile + (r & 3) + 8 * (r >> 2) + 4 * hi;
        if (row_pair[orow] < 0) continue;
        const float v = GATE_UP ? glu_bf16(acc[r], acc2[r], limit, alpha, act_kind) : (MODE == 2 ? plain_act((float)(bf16_t)acc[r], act_kind) : acc[r]);
        out[(size_t)orow * N + n0 + l31] = __builtin_bit_cast(unsigned short, (bf16_t)v);
    }
}

__global__ void moe_combine_kernel(const unsigned short* __restrict__ prod, const int32_t* __restrict__ pair_row,
                                   const float* __restrict__ wts, const unsigned short* __restrict__ shared,
                                   unsigned short* __restrict__ y, int top, int W) {
    const size_t t = blockIdx.x;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        float tot = 0.f;
        for (int k = 0; k < top; ++k) {
            const size_t r = pair_row[t * top + k];
            tot += wts[t * top + k] * (float)__builtin_bit_cast(bf16_t, prod[r * W + c]);
        }
        if (shared) tot += (float)__builtin_bit_cast(bf16_t, shared[t * W + c]);
        y[t * W + c] = __builtin_bit_cast(unsigned short, (bf16_t)tot);
    }
}

}  // namespace sm

using namespace sm;

extern "C" int sm_moe_grouped_tiles(int64_t T, int top, int E) {
    if (T <= 0 || top <= 0 || E <= 0) return 0;
    return (int)((T * top + kRowsPerTile - 1) / kRowsPerTile + E);
}

extern "C" int sm_moe_grouped(const void* h, const int32_t* idx, const float* wts, const void* w_gu, const void* w_down,
                              const void* shared, float limit, float alpha, int act_kind, void* y, int64_t T, int top, int E, int W, int F,
                              int32_t* row_pair, int32_t* tile_expert, int32_t* pair_row, void* act, void* prod, void* stream) {
    if (T < 0 || top < 1 || E < 1 || W < 1 || F < 1 || act_kind < 0 || act_kind > SM_ACT_SILU_GLU ||
        (T > 0 && (!h || !idx || !wts || !w_gu || !w_down || !y || !row_pair || !tile_expert || !pair_row || !act || !prod))) {
        set_error("sm_moe_grouped: bad argument");
        return SM_EINVAL;
    }
    if (W % 8 || F % 8 || E > 4096 || T * top > (int64_t)1 << 30) {
        set_error("sm_moe_grouped: needs W %% 8 == 0, F %% 8 == 0, at most 4096 experts");
        return SM_ESHAPE;
    }
    if (T == 0) return SM_OK;
    const int tiles = sm_moe_grouped_tiles(T, top, E);
    hipStream_t s = as_stream(stream);
    hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), (size_t)3 * E * sizeof(int), s, idx, (int)(T * top), E, tiles, row_pair,
                       tile_expert, pair_row);
    SM_CHECK_LAUNCH("sm_moe_grouped (align)");
    if (act_kind == SM_ACT_CLAMPED_GLU || act_kind == SM_ACT_SILU_GLU)
        hipLaunchKernelGGL(moe_grouped_kernel<1>, dim3((unsigned)tiles, (unsigned)((F + 127) / 128)), dim3(256), 0, s,
                           (const unsigned short*)h, (const unsigned short*)w_gu, row_pair, tile_expert, (unsigned short*)act, top, F,
                           W, limit, alpha, act_kind);
    else
        hipLaunchKernelGGL(moe_grouped_kernel<2>, dim3((unsigned)tiles, (unsigned)((F + 127) / 128)), dim3(256), 0, s,
                           (const unsigned short*)h, (const unsigned short*)w_gu, row_pair, tile_expert, (unsigned short*)act, top, F,
                           W, limit, alpha, act_kind);
    SM_CHECK_LAUNCH("sm_moe_grouped (gate/up)");
    hipLaunchKernelGGL(moe_grouped_kernel<0>, dim3((unsigned)tiles, (unsigned)((W + 127) / 128)), dim3(256), 0, s,
                       (const unsigned short*)act, (const unsigned short*)w_down, row_pair, tile_expert, (unsigned short*)prod, top, W,
                       F, 0.f, 0.f, 0);
    SM_CHECK_LAUNCH("sm_moe_grouped (down)");
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)T), dim3(256), 0, s, (const unsigned short*)prod, pair_row, wts,
                       (const unsigned short*)shared, (unsigned short*)y, top, W);
    SM_CHECK_LAUNCH("sm_moe_grouped (combine)");
    return SM_OK;
}

// The grouping and the final sum on their own, for callers that run the expert products themselves (the engine gives
// large groups to the vendor GEMM, one call per expert on the rows sm_moe_align put together).
extern "C" int sm_moe_align(const int32_t* idx, int64_t T, int top, int E, int32_t* row_pair, int32_t* tile_expert,
                            int32_t* pair_row, void* stream) {
    if (T < 0 || top < 1 || E < 1 || E > 4096 || (T > 0 && (!idx || !row_pair || !tile_expert || !pair_row))) {
        set_error("sm_moe_align: bad argument");
        return SM_EINVAL;
    }
    if (T == 0) return SM_OK;
    hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), (size_t)3 * E * sizeof(int), as_stream(stream), idx, (int)(T * top), E,
                       sm_moe_grouped_tiles(T, top, E), row_pair, tile_expert, pair_row);
    SM_CHECK_LAUNCH("sm_moe_align");
    return SM_OK;
}

extern "C" int sm_moe_combine(const void* prod, const int32_t* pair_row, const float* wts, const void* shared, void* y, int64_t T,
                              int top, int W, void* stream) {
    if (T < 0 || top < 1 || W < 1 || (T > 0 && (!prod || !pair_row || !wts || !y))) {
        set_error("sm_moe_combine: bad argument");
        return SM_EINVAL;
    }
    if (T == 0) return SM_OK;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)T), dim3(256), 0, as_stream(stream), (const unsigned short*)prod, pair_row,
                       wts, (const unsigned short*)shared, (unsigned short*)y, top, W);
    SM_CHECK_LAUNCH("sm_moe_combine");
    return SM_OK;
}
