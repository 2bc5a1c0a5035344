// Expert products for large groups (prefill) on the matrix cores, bf16: tiles of 128 rows of one expert by 128 output
// columns.  The 128 x 64 activation block of a k-step is staged once in LDS and shared by the four waves (each wave
// owns 32 columns and all 128 rows: four row fragments reuse every weight fragment), the weights go from global
// memory straight to the MFMA registers (a lane owns one weight row and 32 consecutive k of the 64-k step).
// Against the 32-row form of sm_moe_grouped.hip this reads an expert's weights 4x less often and the activations
// once per workgroup instead of once per wave.
//
// Row r of a group is the same sum whatever else shares its tile, so both forms agree bit for bit on a row's
// products (same k order inside a 64-k step, same accumulation).
#include "sm_common.h"

namespace sm {

constexpr int kBigRows = 128;                 // rows per tile
constexpr int kAStride = 64 * 2 + 16;         // bytes between rows of the staged block (odd number of 16-byte chunks)

__global__ __launch_bounds__(1024) void moe_align128_kernel(const int32_t* __restrict__ idx, int P, int E, int max_tiles,
                                                            int32_t* __restrict__ row_pair, int32_t* __restrict__ tile_expert,
                                                            int32_t* __restrict__ pair_row) {
    extern __shared__ int sh[];                 // counts[E], offs[E], cursor[E]
    int* counts = sh;
    int* offs = sh + E;
    int* cursor = sh + 2 * E;
    for (int e = threadIdx.x; e < E; e += blockDim.x) { counts[e] = 0; cursor[e] = 0; }
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += blockDim.x) {
        const int e = idx[p];
        if (e >= 0 && e < E) atomicAdd(&counts[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int tiles = 0;
        for (int e = 0; e < E; ++e) {
            offs[e] = tiles * kBigRows;
            const int n = (counts[e] + kBigRows - 1) / kBigRows;
            for (int i = 0; i < n && tiles + i < max_tiles; ++i) tile_expert[tiles + i] = e;
            tiles += n;
        }
        for (int i = tiles; i < max_tiles; ++i) tile_expert[i] = -1;
    }
    for (int r = threadIdx.x; r < max_tiles * kBigRows; r += blockDim.x) row_pair[r] = -1;
    __syncthreads();
    for (int p = threadIdx.x; p < P; p += blockDim.x) {
        const int e = idx[p];
        if (e < 0 || e >= E) { pair_row[p] = 0; continue; }
        const int r = offs[e] + atomicAdd(&cursor[e], 1);
        if (r < max_tiles * kBigRows) row_pair[r] = p;
        pair_row[p] = min(r, max_tiles * kBigRows - 1);
    }
}

__device__ __forceinline__ float glu_bf16_big(float g, float u, float limit, float alpha, int act) {
    // the products leave the matrix unit in bf16, as a GEMM's output would
    return gated_act((float)(bf16_t)g, (float)(bf16_t)u, limit, alpha, act);
}

__device__ __forceinline__ i32x4 load16(const unsigned short* p, int k, int K) {
    i32x4 v = {0, 0, 0, 0};
    if (k + 8 <= K) v = *(const i32x4*)(p + k);
    return v;
}

// GATE_UP: A = h rows gathered by token, B = the expert's gate and up rows, out = act [rows, N] (N = F, K = W)
// else:    A = act rows,                 B = the expert's down rows,       out = per-row products [rows, N] (N = W, K = F)
// MODE 0: the down product; 1: gate and up with the gated activation (act_kind: clamped GLU or silu(g) u); 2: the up product alone with a GELU (act_kind)
template <int MODE>
__global__ __launch_bounds__(256) void moe_tiles128_kernel(const unsigned short* __restrict__ a, const unsigned short* __restrict__ w,
                                                           const int32_t* __restrict__ row_pair, const int32_t* __restrict__ tile_expert,
                                                           unsigned short* __restrict__ out, int top, int N, int K, float limit,
                                                           float alpha, int act_kind) {
    __shared__ __attribute__((aligned(16))) unsigned char a_lds[kBigRows * kAStride];
    constexpr bool GATE_UP = MODE == 1, FROM_TOKENS = MODE != 0;
    const int tile = blockIdx.x;
    const int e = tile_expert[tile];
    if (e < 0) return;                                        // (uniform over the workgroup)
    const int tid = threadIdx.x, lane = tid & 63, l31 = lane & 31, hi = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n0 = blockIdx.y * 128 + wave * 32;              // (n0 >= N: the wave still stages and keeps the barriers)
    // staging: thread -> row tid / 2, k half tid % 2 (32 consecutive k = 64 bytes)
    const int srow = tid >> 1, shalf = tid & 1;
    const int spair = row_pair[tile * kBigRows + srow];
    const unsigned short* ap = FROM_TOKENS ? a + (size_t)(spair < 0 ? 0 : spair / top) * K : a + ((size_t)tile * kBigRows + srow) * K;
    // weights in the tiled layout of sm_moe_tile_weights (see sm_moe_grouped.hip): a wave's load is one contiguous KB
    const int nb32 = (N + 31) / 32, ksteps = (K + 63) / 64;
    const unsigned short* bp = w + (((size_t)e * (GATE_UP ? 2 : 1) * nb32 + min(n0, N - 1) / 32) * ksteps) * 2048 + 8 * lane;
    const unsigned short* bp2 = bp + (size_t)nb32 * ksteps * 2048;      // the up blocks follow the gate blocks
    f32x16 acc[4], acc2[4];
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
        for (int r = 0; r < 16; ++r) { acc[m][r] = 0.f; acc2[m][r] = 0.f; }
    // software pipeline: the operands of step k+1 are requested before the MFMAs of step k
    i32x4 ar[4], bn[4], bn2[4];
    auto request = [&](int k0) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            ar[s] = load16(ap, k0 + 32 * shalf + 8 * s, K);
            const size_t boff = (size_t)(k0 / 64) * 2048 + 512 * s;
            bn[s] = *(const i32x4*)(bp + boff);
            if (GATE_UP) bn2[s] = *(const i32x4*)(bp2 + boff);
        }
    };
    request(0);
    for (int k0 = 0; k0 < K; k0 += 64) {
        i32x4 bf[4], bf2[4];
        __syncthreads();                                      // the previous step's reads of a_lds are done
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            *(i32x4*)(a_lds + srow * kAStride + 64 * shalf + 16 * s) = ar[s];
            bf[s] = bn[s];
            if (GATE_UP) bf2[s] = bn2[s];
        }
        __syncthreads();
        if (k0 + 64 < K) request(k0 + 64);
        if (n0 < N) {
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    const bf16x8 af = *(const bf16x8*)(a_lds + (32 * m + l31) * kAStride + 64 * hi + 16 * s);
                    acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, __builtin_bit_cast(bf16x8, bf[s]), acc[m], 0, 0, 0);
                    if (GATE_UP)
                        acc2[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, __builtin_bit_cast(bf16x8, bf2[s]), acc2[m], 0, 0, 0);
                }
        }
    }
    if (n0 + l31 >= N) return;
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int orow = tile * kBigRows + 32 * m + (r & 3) + 8 * (r >> 2) + 4 * hi;
            if (row_pair[orow] < 0) continue;
            const float v = GATE_UP ? glu_bf16_big(acc[m][r], acc2[m][r], limit, alpha, act_kind)
                                    : (MODE == 2 ? plain_act((float)(bf16_t)acc[m][r], act_kind) : acc[m][r]);
            out[(size_t)orow * N + n0 + l31] = __builtin_bit_cast(unsigned short, (bf16_t)v);
        }
}

}  // namespace sm

using namespace sm;

extern "C" int sm_moe_tiles128_count(int64_t T, int top, int E) {
    if (T <= 0 || top <= 0 || E <= 0) return 0;
    return (int)((T * top + kBigRows - 1) / kBigRows + E);
}

extern "C" int sm_moe_tiles128(const void* h, const int32_t* idx, const float* wts, const void* w_gu, const void* w_down,
                               const void* shared, float limit, float alpha, int act_kind, void* y, int64_t T, int top, int E, int W, int F,
                               int32_t* row_pair, int32_t* tile_expert, int32_t* pair_row, void* act, void* prod, void* stream) {
    if (T < 0 || top < 1 || E < 1 || W < 1 || F < 1 || act_kind < 0 || act_kind > SM_ACT_SILU_GLU ||
        (T > 0 && (!h || !idx || !wts || !w_gu || !w_down || !y || !row_pair || !tile_expert || !pair_row || !act || !prod))) {
        set_error("sm_moe_tiles128: bad argument");
        return SM_EINVAL;
    }
    if (W % 8 || F % 8 || E > 4096 || T * top > (int64_t)1 << 28) {
        set_error("sm_moe_tiles128: needs W %% 8 == 0, F %% 8 == 0, at most 4096 experts");
        return SM_ESHAPE;
    }
    if (T == 0) return SM_OK;
    const int tiles = sm_moe_tiles128_count(T, top, E);
    hipStream_t s = as_stream(stream);
    hipLaunchKernelGGL(moe_align128_kernel, dim3(1), dim3(1024), (size_t)3 * E * sizeof(int), s, idx, (int)(T * top), E, tiles, row_pair,
                       tile_expert, pair_row);
    SM_CHECK_LAUNCH("sm_moe_tiles128 (align)");
    if (act_kind == SM_ACT_CLAMPED_GLU || act_kind == SM_ACT_SILU_GLU)
        hipLaunchKernelGGL(moe_tiles128_kernel<1>, dim3((unsigned)tiles, (unsigned)((F + 127) / 128)), dim3(256), 0, s,
                           (const unsigned short*)h, (const unsigned short*)w_gu, row_pair, tile_expert, (unsigned short*)act, top, F,
                           W, limit, alpha, act_kind);
    else
        hipLaunchKernelGGL(moe_tiles128_kernel<2>, dim3((unsigned)tiles, (unsigned)((F + 127) / 128)), dim3(256), 0, s,
                           (const unsigned short*)h, (const unsigned short*)w_gu, row_pair, tile_expert, (unsigned short*)act, top, F,
                           W, limit, alpha, act_kind);
    SM_CHECK_LAUNCH("sm_moe_tiles128 (gate/up)");
    hipLaunchKernelGGL(moe_tiles128_kernel<0>, dim3((unsigned)tiles, (unsigned)((W + 127) / 128)), dim3(256), 0, s,
                       (const unsigned short*)act, (const unsigned short*)w_down, row_pair, tile_expert, (unsigned short*)prod, top, W,
                       F, 0.f, 0.f, 0);
    SM_CHECK_LAUNCH("sm_moe_tiles128 (down)");
    return sm_moe_combine(prod, pair_row, wts, shared, y, T, top, W, stream);
}
