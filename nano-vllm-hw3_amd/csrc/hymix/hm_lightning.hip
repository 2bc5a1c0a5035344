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

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }

// One workgroup of 256 threads per (sequence, head, 32 value channels).  A column of S (one value channel, DK >= D key
// channels) is spread over 8 neighbouring lanes, DK / 8 channels each in registers; S^T q is summed over those lanes with
// a butterfly, so the order of every sum is fixed by DK alone.  q and k (DK floats each, zero beyond D) and the 32 value
// channels of CH tokens are staged in LDS at a time, activation applied on the way in; the next chunk is requested from
// global memory before the current chunk's tokens run and written to the other buffer after them (one barrier per chunk).
// Beyond the portion's end a chunk is padded with the identity step (decay 1, k = 0).
template <typename T, int DK, int CH>
__global__ __launch_bounds__(256) void lightning_kernel(const T* __restrict__ proj, int64_t row_stride, int q_off, int k_off,
                                                        int v_off, const float* __restrict__ decay, float* __restrict__ state,
                                                        const int32_t* __restrict__ qstart, const int32_t* __restrict__ seq_pos0,
                                                        const int32_t* __restrict__ seq_slot, float* __restrict__ o, int H, int D,
                                                        int V) {
    constexpr int SL = 8, KS = DK / SL, COLS = 256 / SL, TOK = 2 * DK + COLS, NR = (CH * TOK + 255) / 256;
    __shared__ __attribute__((aligned(16))) float buf[2][CH * TOK];
    const int b = blockIdx.x, hd = blockIdx.y;
    const int q0 = qstart[b], n = qstart[b + 1] - q0;
    if (n <= 0) return;
    const int tid = threadIdx.x, slice = tid % SL, col = tid / SL;
    const int j = blockIdx.z * COLS + col;
    const bool live = j < V;
    float* st = state + ((size_t)seq_slot[b] * H + hd) * (size_t)D * V;
    const float dec = decay[hd];
    const bool fresh = seq_pos0[b] == 0;
    float s[KS];
#pragma unroll
    for (int ii = 0; ii < KS; ++ii) {
        const int i = slice * KS + ii;
        s[ii] = (!fresh && live && i < D) ? st[(size_t)i * V + j] : 0.f;
    }
    float regs[NR];
    auto request = [&](int tok0) {
#pragma unroll
        for (int k = 0; k < NR; ++k) {
            const int e = tid + 256 * k;
            const int tc = e / TOK, rem = e - tc * TOK, tok = tok0 + tc;
            float val = 0.f;
            if (e < CH * TOK && tok < n) {
                const T* row = proj + (size_t)(q0 + tok) * row_stride;
                if (rem < 2 * DK) {
                    const int part = rem / DK, i = rem - part * DK;
                    if (i < D) val = silu_f(to_f(row[(part ? k_off : q_off) + hd * D + i]));
                } else {
                    const int jj = blockIdx.z * COLS + (rem - 2 * DK);
                    if (jj < V) val = silu_f(to_f(row[v_off + hd * V + jj]));
                }
            }
            regs[k] = val;
        }
    };
    auto deposit = [&](int which) {
#pragma unroll
        for (int k = 0; k < NR; ++k) {
            const int e = tid + 256 * k;
            if (e < CH * TOK) buf[which][e] = regs[k];
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
            const float vj = p[2 * DK + col];
            float out = 0.f;
#pragma unroll
            for (int ii = 0; ii < KS; ++ii) {
                s[ii] = d * s[ii] + p[DK + slice * KS + ii] * vj;
                out += s[ii] * p[slice * KS + ii];
            }
            out = lt_sum8(out);
            if (live && slice == 0 && tok0 + tc < n) o[((size_t)(q0 + tok0 + tc) * H + hd) * V + j] = out;
        }
        if (more) {
            deposit(which ^ 1);                // the other buffer was last read one chunk ago, before that chunk's barrier
            __syncthreads();
            which ^= 1;
        }
    }
    if (live) {
#pragma unroll
        for (int ii = 0; ii < KS; ++ii) {
            const int i = slice * KS + ii;
            if (i < D) st[(size_t)i * V + j] = s[ii];
        }
    }
}

template <typename DT>
static void launch_lightning(const void* proj, int64_t row_stride, int q_off, int k_off, int v_off, const float* decay, float* state,
                             const int32_t* qstart, const int32_t* seq_pos0, const int32_t* seq_slot, float* o, int B, int H, int D,
                             int V, int max_q, hipStream_t s) {
    dim3 grid((unsigned)B, (unsigned)H, (unsigned)((V + 31) / 32));
#define HM_LIGHT(DK, CH)                                                                                                     \
    hipLaunchKernelGGL((lightning_kernel<DT, DK, CH>), grid, dim3(256), 0, s, (const DT*)proj, row_stride, q_off, k_off, v_off, \
                       decay, state, qstart, seq_pos0, seq_slot, o, H, D, V)
    if (max_q <= 1) {                          // single tokens: one token staged, so that many small workgroups fit a CU
        if (D <= 32) HM_LIGHT(32, 1);
        else if (D <= 64) HM_LIGHT(64, 1);
        else if (D <= 128) HM_LIGHT(128, 1);
        else HM_LIGHT(256, 1);
    } else if (D <= 32) HM_LIGHT(32, 8);
    else if (D <= 64) HM_LIGHT(64, 8);
    else if (D <= 128) HM_LIGHT(128, 8);
    else HM_LIGHT(256, 4);
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
