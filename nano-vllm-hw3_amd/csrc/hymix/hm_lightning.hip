// Linear attention with a constant decay per head ("lightning" attention): per head a float32 state S [D, V],
//   S_t = decay_h S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,
// with q, k, v = silu of column slices of the mixer's merged product.  The recurrence is sequential over a portion's
// tokens and parallel over sequences, heads and value channels; the update of S is one multiply-add per element, so a
// token's step costs 2 D V multiply-adds and nothing waits for a sum.  State f32 [slots, H, D, V] is read at a portion's
// start (zero at position 0, whatever the slot holds) and left at its end.
#include "hm_common.h"

namespace hm {

__device__ __forceinline__ float lt_sum8(float v) {       // sum over 8 neighbouring lanes; every lane gets the total
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));  // row_half_mirror
    return v;
}

// z sigmoid(z) from the hardware's exponential and reciprocal (float32, a few units in the last place)
__device__ __forceinline__ float silu_f(float z) { return z * __builtin_amdgcn_rcpf(1.f + __expf(-z)); }

// One workgroup of 256 threads per (sequence, head, 32 CV value channels).  A thread keeps CV neighbouring columns of S
// (value channels) over DK / 8 key channels in registers: a column (DK >= D key channels) is spread over 8 neighbouring
// lanes, and S^T q is summed over those lanes with a butterfly, so the order of every sum is fixed by DK alone.  Every q
// and k value a thread reads from LDS meets CV columns (2 CV multiply-adds per value read).  q and k (DK floats each,
// zero beyond D) and the workgroup's value channels of CH tokens are staged in LDS at a time, activation applied on the
// way in; the next chunk is requested from global memory before the current chunk's tokens run and written to the other
// buffer after them (one barrier per chunk).  Beyond the portion's end a chunk is padded with the identity step
// (decay 1, k = 0).
template <typename T, int DK, int CH, int CV>
__global__ __launch_bounds__(256) void lightning_kernel(const T* __restrict__ proj, int64_t row_stride, int q_off, int k_off,
                                                        int v_off, const float* __restrict__ decay, float* __restrict__ state,
                                                        const int32_t* __restrict__ qstart, const int32_t* __restrict__ seq_pos0,
                                                        const int32_t* __restrict__ seq_slot, float* __restrict__ o, int H, int D,
                                                        int V) {
    constexpr int SL = 8, KS = DK / SL, COLS = 256 / SL * CV, TOK = 2 * DK + COLS, NR = (CH * TOK + 255) / 256;
    static_assert(KS % 4 == 0, "a lane's key channels are read four at a time");
    __shared__ __attribute__((aligned(16))) float buf[2][CH * TOK];
    const int b = blockIdx.x, hd = blockIdx.y;
    const int q0 = qstart[b], n = qstart[b + 1] - q0;
    if (n <= 0) return;
    const int tid = threadIdx.x, slice = tid % SL, col = tid / SL;
    const int j0 = blockIdx.z * COLS + col * CV;           // the thread's first value channel
    float* st = state + ((size_t)seq_slot[b] * H + hd) * (size_t)D * V;
    const float dec = decay[hd];
    const bool fresh = seq_pos0[b] == 0;
    float s[KS][CV];
#pragma unroll
    for (int ii = 0; ii < KS; ++ii) {
        const int i = slice * KS + ii;
#pragma unroll
        for (int c = 0; c < CV; ++c) s[ii][c] = (!fresh && j0 + c < V && i < D) ? st[(size_t)i * V + j0 + c] : 0.f;
    }
    // Which value of a chunk a thread fetches does not change from chunk to chunk: its column in the row and its token
    // inside the chunk are worked out once (column -1: padding).  The loaded values stay untouched in registers until they
    // are deposited (silu(0) = 0 keeps the padding zero): nothing waits for global memory before the current chunk's tokens
    // have run.
    int col_of[NR], tok_of[NR];
#pragma unroll
    for (int k = 0; k < NR; ++k) {
        const int e = tid + 256 * k;
        const int tc = e / TOK, rem = e - tc * TOK;
        int c = -1;
        if (e < CH * TOK) {
            if (rem < 2 * DK) {
                const int part = rem / DK, i = rem - part * DK;
                if (i < D) c = (part ? k_off : q_off) + hd * D + i;
            } else {
                const int jj = blockIdx.z * COLS + (rem - 2 * DK);
                if (jj < V) c = v_off + hd * V + jj;
            }
        }
        col_of[k] = c;
        tok_of[k] = tc;
    }
    T regs[NR];
    auto request = [&](int tok0) {
#pragma unroll
        for (int k = 0; k < NR; ++k) {
            const int tok = tok0 + tok_of[k];
            T val = from_f<T>(0.f);
            if (col_of[k] >= 0 && tok < n) val = proj[(size_t)(q0 + tok) * row_stride + col_of[k]];
            regs[k] = val;
        }
    };
    auto deposit = [&](int which) {
#pragma unroll
        for (int k = 0; k < NR; ++k) {
            const int e = tid + 256 * k;
            if (e < CH * TOK) buf[which][e] = silu_f(to_f(regs[k]));
        }
    };
    request(0);
    deposit(0);
    __syncthreads();
    int which = 0;
    for (int tok0 = 0; tok0 < n; tok0 += CH) {
        const bool more = tok0 + CH < n;
        if (more) request(tok0 + CH);
#pragma unroll
        for (int tc = 0; tc < CH; ++tc) {
            const float* p = buf[which] + tc * TOK;
            const float d = tok0 + tc < n ? dec : 1.f;
            float vj[CV], out[CV];
#pragma unroll
            for (int c = 0; c < CV; ++c) { vj[c] = p[2 * DK + col * CV + c]; out[c] = 0.f; }
#pragma unroll
            for (int m = 0; m < KS / 4; ++m) {             // 16-byte LDS reads: four key channels of k and of q at a time
                const float4 k4 = *(const float4*)(p + DK + slice * KS + 4 * m), q4 = *(const float4*)(p + slice * KS + 4 * m);
                const float kk[4] = {k4.x, k4.y, k4.z, k4.w}, qq[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int c = 0; c < CV; ++c) {
                        s[4 * m + e][c] = d * s[4 * m + e][c] + kk[e] * vj[c];
                        out[c] += s[4 * m + e][c] * qq[e];
                    }
            }
#pragma unroll
            for (int c = 0; c < CV; ++c) out[c] = lt_sum8(out[c]);
            if (slice == 0 && tok0 + tc < n) {
                float* orow = o + ((size_t)(q0 + tok0 + tc) * H + hd) * V;
#pragma unroll
                for (int c = 0; c < CV; ++c)
                    if (j0 + c < V) orow[j0 + c] = out[c];
            }
        }
        if (more) {
            deposit(which ^ 1);                // the other buffer was last read one chunk ago, before that chunk's barrier
            __syncthreads();
            which ^= 1;
        }
    }
#pragma unroll
    for (int ii = 0; ii < KS; ++ii) {
        const int i = slice * KS + ii;
#pragma unroll
        for (int c = 0; c < CV; ++c)
            if (j0 + c < V && i < D) st[(size_t)i * V + j0 + c] = s[ii][c];
    }
}

template <typename DT>
static void launch_lightning(const void* proj, int64_t row_stride, int q_off, int k_off, int v_off, const float* decay, float* state,
                             const int32_t* qstart, const int32_t* seq_pos0, const int32_t* seq_slot, float* o, int B, int H, int D,
                             int V, int max_q, hipStream_t s) {
    // columns per thread: more of them give every q and k value read from LDS more columns to meet, fewer give more
    // workgroups; as many as still leave two workgroups per compute unit.  (Every sum is the same whatever the choice.)
    auto groups = [&](int c) { return (int64_t)B * H * ((V + 32 * c - 1) / (32 * c)); };
    const int cv = (V >= 128 && groups(4) >= 512) ? 4 : ((V >= 64 && groups(2) >= 512) ? 2 : 1);
#define HM_LIGHT(DK, CH, CV)                                                                                                 \
    hipLaunchKernelGGL((lightning_kernel<DT, DK, CH, CV>), dim3((unsigned)B, (unsigned)H, (unsigned)((V + 32 * CV - 1) / (32 * CV))), \
                       dim3(256), 0, s, (const DT*)proj, row_stride, q_off, k_off, v_off, decay, state, qstart, seq_pos0, seq_slot, \
                       o, H, D, V)
#define HM_LIGHT_CV(DK, CH)                                                   \
    do {                                                                      \
        if (cv == 4) HM_LIGHT(DK, CH, 4); else if (cv == 2) HM_LIGHT(DK, CH, 2); else HM_LIGHT(DK, CH, 1); \
    } while (0)
    if (max_q <= 1) {                          // single tokens: one token staged, so that many small workgroups fit a CU
        if (D <= 32) HM_LIGHT_CV(32, 1);
        else if (D <= 64) HM_LIGHT_CV(64, 1);
        else if (D <= 128) HM_LIGHT_CV(128, 1);
        else if (cv == 1) HM_LIGHT(256, 1, 1);
        else HM_LIGHT(256, 1, 2);
    } else if (D <= 32) HM_LIGHT_CV(32, 8);
    else if (D <= 64) HM_LIGHT_CV(64, 8);
    else if (D <= 128) HM_LIGHT_CV(128, 8);
    else if (cv == 1) HM_LIGHT(256, 4, 1);
    else HM_LIGHT(256, 4, 2);
#undef HM_LIGHT_CV
#undef HM_LIGHT
}

}  // namespace hm

using namespace hm;

extern "C" int hm_lightning_recurrence(int dtype, const void* proj, int64_t row_stride, int q_off, int k_off, int v_off,
                                       const float* decay, float* state, const int32_t* qstart, const int32_t* seq_pos0,
                                       const int32_t* seq_slot, float* o, int B, int H, int D, int V, int max_q, void* stream) {
    if (B < 0 || H < 1 || D < 1 || V < 1 || q_off < 0 || k_off < 0 || v_off < 0 ||
        row_stride < (int64_t)q_off + (int64_t)H * D || row_stride < (int64_t)k_off + (int64_t)H * D ||
        row_stride < (int64_t)v_off + (int64_t)H * V ||
        (B > 0 && (!proj || !decay || !state || !qstart || !seq_pos0 || !seq_slot || !o))) {
        set_error("hm_lightning_recurrence: bad argument");
        return HM_EINVAL;
    }
    if (D > 256 || H > 65535 || V > 32 * 65535) { set_error("hm_lightning_recurrence: dim <= 256 and heads <= 65535"); return HM_ESHAPE; }
    if (B == 0) return HM_OK;
    HM_DISPATCH(dtype, "hm_lightning_recurrence",
                launch_lightning<DT>(proj, row_stride, q_off, k_off, v_off, decay, state, qstart, seq_pos0, seq_slot, o, B, H, D, V,
                                     max_q, as_stream(stream)));
    HM_CHECK_LAUNCH("hm_lightning_recurrence");
    return HM_OK;
}
