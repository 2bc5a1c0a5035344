// Mixture of experts: the router (softmax or sigmoid scores, an optional correction that only steers the choice,
// group-limited top-k, weights renormalised or not) and the expert products
// in their memory-bound form, one (token, chosen expert) pair at a time.
#include "sm_common.h"

namespace sm {

constexpr int kMaxExperts = 1024, kMaxTop = 32;

constexpr int kRouteTokens = 8;      // tokens per workgroup: every router row read serves all of them

template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(const T* __restrict__ h, const float* __restrict__ router_w,
                                                        int32_t* __restrict__ idx, float* __restrict__ wts, int64_t T_all, int W,
                                                        int E, int top, int groups, int keep, int score,
                                                        const float* __restrict__ correction, int group_top, int renorm,
                                                        int staged, const float* __restrict__ bias) {
    extern __shared__ float z_all[];             // per token: E scores, then `groups` group scores; then the staged rows
    const int64_t t0 = (int64_t)blockIdx.x * kRouteTokens;
    const int nt = (int)min((int64_t)kRouteTokens, T_all - t0);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (staged) {
        // the workgroup's token rows (one contiguous piece of h) go to LDS once; every expert's row is then read once per
        // workgroup in 16-byte pieces and meets all the tokens there
        T* h_lds = (T*)(z_all + kRouteTokens * (E + groups));
        const T* src = h + (size_t)t0 * W;
        struct alignas(sizeof(T) * 4) Pack4 { T v[4]; };
        for (int i = threadIdx.x * 4; i < nt * W; i += 1024) *(Pack4*)(h_lds + i) = *(const Pack4*)(src + i);     // W % 4 == 0
        __syncthreads();
        for (int e = wave; e < E; e += 4) {
            const float* wr = router_w + (size_t)e * W;
            float d[kRouteTokens];
            for (int i = 0; i < kRouteTokens; ++i) d[i] = 0.f;
            for (int c = lane * 4; c < W; c += 256) {
                const float4 wv = *(const float4*)(wr + c);
#pragma unroll
                for (int i = 0; i < kRouteTokens; ++i)
                    if (i < nt) {
                        const Pack4 hv = *(const Pack4*)(h_lds + (size_t)i * W + c);
                        d[i] += to_f(hv.v[0]) * wv.x + to_f(hv.v[1]) * wv.y + to_f(hv.v[2]) * wv.z + to_f(hv.v[3]) * wv.w;
                    }
            }
            for (int i = 0; i < kRouteTokens; ++i) {
                const float sum = wave_sum(d[i]);
                if (lane == 0) z_all[i * (E + groups) + e] = sum;
            }
        }
    } else {
        for (int e = wave; e < E; e += 4) {
            const float* wr = router_w + (size_t)e * W;
            float d[kRouteTokens];
            for (int i = 0; i < kRouteTokens; ++i) d[i] = 0.f;
            for (int c = lane; c < W; c += 64) {
                const float wv = wr[c];
                for (int i = 0; i < kRouteTokens; ++i)
                    if (i < nt) d[i] += to_f(h[(size_t)(t0 + i) * W + c]) * wv;
            }
            for (int i = 0; i < kRouteTokens; ++i) {
                const float sum = wave_sum(d[i]);
                if (lane == 0) z_all[i * (E + groups) + e] = sum;
            }
        }
    }
    __syncthreads();
    if (threadIdx.x >= nt) return;
    // one thread finishes a token: E is small and the selections are sequential by nature
    const int64_t t = t0 + threadIdx.x;
    float* z = z_all + threadIdx.x * (E + groups);
    if (bias != nullptr)
        for (int e = 0; e < E; ++e) z[e] += bias[e];
    if (score == SM_ROUTE_SIGMOID) {
        for (int e = 0; e < E; ++e) z[e] = 1.f / (1.f + expf(-z[e]));
    } else {
        float mx = -INFINITY;
        for (int e = 0; e < E; ++e) mx = fmaxf(mx, z[e]);
        float sum = 0.f;
        for (int e = 0; e < E; ++e) { z[e] = expf(z[e] - mx); sum += z[e]; }
        const float inv = 1.f / sum;
        for (int e = 0; e < E; ++e) z[e] *= inv;
    }
    float* gs = z + E;
    if (correction != nullptr || group_top > 1) {
        // The general form: choice scores c = s + correction (they may be negative) decide, the weights are s.  A group
        // scores the sum of its `group_top` largest c; experts outside the best `keep` groups count as -inf.
        const int per = E / groups;
        bool ok_all = groups <= 1;
        if (!ok_all) {
            for (int g = 0; g < groups; ++g) {
                float tot = 0.f;
                int used[4] = {-1, -1, -1, -1};                 // group_top <= 4
                for (int k = 0; k < group_top && k < per; ++k) {
                    int best = -1;
                    float bv = -INFINITY;
                    for (int e = 0; e < per; ++e) {
                        bool taken = false;
                        for (int j = 0; j < k; ++j) taken |= used[j] == e;
                        const float c = z[g * per + e] + (correction ? correction[g * per + e] : 0.f);
                        if (!taken && (best < 0 || c > bv)) { bv = c; best = e; }
                    }
                    used[k] = best;
                    tot += bv;
                }
                gs[g] = tot;
            }
            // keep the best groups: a kept group's score becomes +inf, the others' -inf afterwards
            for (int k = 0; k < keep; ++k) {
                int best = -1;
                float bv = -INFINITY;
                for (int g = 0; g < groups; ++g)
                    if (gs[g] != INFINITY && (best < 0 || gs[g] > bv)) { bv = gs[g]; best = g; }
                if (best >= 0) gs[best] = INFINITY;
            }
        }
        int chosen[kMaxTop];
        float cw[kMaxTop], tot = 0.f;
        for (int k = 0; k < top; ++k) {
            int best = -1;
            float bv = -INFINITY;
            for (int e = 0; e < E; ++e) {
                if (!ok_all && gs[e / per] != INFINITY) continue;
                bool taken = false;
                for (int j = 0; j < k; ++j) taken |= chosen[j] == e;
                const float c = z[e] + (correction ? correction[e] : 0.f);
                if (!taken && (best < 0 || c > bv)) { bv = c; best = e; }
            }
            chosen[k] = best < 0 ? 0 : best;
            cw[k] = best < 0 ? 0.f : z[best];
            tot += cw[k];
        }
        const float rn = renorm ? 1.f / (tot + 1e-20f) : 1.f;
        for (int k = 0; k < top; ++k) {
            idx[(size_t)t * top + k] = chosen[k];
            wts[(size_t)t * top + k] = cw[k] * rn;
        }
        return;
    }
    if (groups > 1) {
        const int per = E / groups;
        for (int g = 0; g < groups; ++g) {
            float m = -1.f;
            for (int e = 0; e < per; ++e) m = fmaxf(m, z[g * per + e]);
            gs[g] = m;
        }
        // mark the best `keep` groups by negating the others' score; a dropped group's experts become ineligible
        for (int k = 0; k < keep; ++k) {
            int best = -1;
            float bv = -1.f;
            for (int g = 0; g < groups; ++g)
                if (gs[g] >= 0.f && gs[g] > bv) { bv = gs[g]; best = g; }
            if (best >= 0) gs[best] = -2.f;                     // -2 = kept
        }
    }
    int chosen[kMaxTop];
    float cw[kMaxTop];
    float tot = 0.f;
    for (int k = 0; k < top; ++k) {
        int best = -1;
        float bv = -1.f;
        for (int e = 0; e < E; ++e) {
            if (groups > 1 && gs[e / (E / groups)] != -2.f) continue;
            bool taken = false;
            for (int j = 0; j < k; ++j) taken |= chosen[j] == e;
            if (!taken && z[e] > bv) { bv = z[e]; best = e; }
        }
        chosen[k] = best < 0 ? 0 : best;
        cw[k] = best < 0 ? 0.f : bv;
        tot += cw[k];
    }
    const float rn = renorm ? 1.f / (tot + 1e-20f) : 1.f;
    for (int k = 0; k < top; ++k) {
        idx[(size_t)t * top + k] = chosen[k];
        wts[(size_t)t * top + k] = cw[k] * rn;
    }
}

// workgroup = one (token, expert) pair; every wave produces outputs f = wave, wave + 4, ...
template <typename T>
__global__ __launch_bounds__(256) void moe_pairs_gate_up_kernel(const T* __restrict__ h, const int32_t* __restrict__ idx,
                                                                const T* __restrict__ w_gu, float limit, float alpha,
                                                                T* __restrict__ act, int top, int W, int F, int act_kind) {
    extern __shared__ float h_lds[];
    const int64_t p = blockIdx.x, t = p / top;
    const int e = idx[p];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int c = threadIdx.x; c < W; c += 256) h_lds[c] = to_f(h[(size_t)t * W + c]);
    __syncthreads();
    if (!act_is_gated(act_kind)) {                   // one product per expert: w_gu is [E, F, W]
        const T* wu = w_gu + (size_t)e * F * W;
        for (int f = wave; f < F; f += 4) {
            const T* u_row = wu + (size_t)f * W;
            float u = 0.f;
            for (int c = lane; c < W; c += 64) u += h_lds[c] * to_f(u_row[c]);
            u = wave_sum(u);
            if (lane == 0) act[(size_t)p * F + f] = from_f<T>(plain_act(to_f(from_f<T>(u)), act_kind));
        }
        return;
    }
    const T* wg = w_gu + (size_t)e * 2 * F * W;
    for (int f = wave; f < F; f += 4) {
        const T* g_row = wg + (size_t)f * W;
        const T* u_row = wg + (size_t)(F + f) * W;
        float g = 0.f, u = 0.f;
        for (int c = lane; c < W; c += 64) {
            const float x = h_lds[c];
            g += x * to_f(g_row[c]);
            u += x * to_f(u_row[c]);
        }
        g = wave_sum(g);
        u = wave_sum(u);
        // the products leave the matrix unit in the storage type, as a GEMM's output would
        if (lane == 0) act[(size_t)p * F + f] = from_f<T>(gated_act(to_f(from_f<T>(g)), to_f(from_f<T>(u)), limit, alpha, act_kind));
    }
}

// workgroup = one token; every wave produces output columns w = wave, wave + 4, ...
template <typename T>
__global__ __launch_bounds__(256) void moe_pairs_down_kernel(const T* __restrict__ act, const int32_t* __restrict__ idx,
                                                             const float* __restrict__ wts, const T* __restrict__ w_down,
                                                             const T* __restrict__ shared, T* __restrict__ y, int top, int W, int F,
                                                             int staged) {
    extern __shared__ float a_lds[];             // top * F activations of the token's pairs (staged: they fit)
    const int64_t t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (staged) {
        for (int c = threadIdx.x; c < top * F; c += 256) a_lds[c] = to_f(act[(size_t)t * top * F + c]);
        __syncthreads();
    }
    const T* a_row = act + (size_t)t * top * F;
    for (int w = wave; w < W; w += 4) {
        float tot = 0.f;
        for (int k = 0; k < top; ++k) {
            const int e = idx[(size_t)t * top + k];
            const T* row = w_down + ((size_t)e * W + w) * F;
            float d = 0.f;
            if (staged) {
                for (int c = lane; c < F; c += 64) d += a_lds[k * F + c] * to_f(row[c]);
            } else {                                 // the same sum from global memory
                for (int c = lane; c < F; c += 64) d += to_f(a_row[k * F + c]) * to_f(row[c]);
            }
            d = wave_sum(d);
            tot += wts[(size_t)t * top + k] * to_f(from_f<T>(d));
        }
        if (lane == 0) {
            if (shared) tot += to_f(shared[(size_t)t * W + w]);
            y[(size_t)t * W + w] = from_f<T>(tot);
        }
    }
}

}  // namespace sm

using namespace sm;

extern "C" int sm_moe_route(int dtype, const void* h, const float* router_w, int32_t* idx, float* wts, int64_t T, int W, int E,
                            int top, int groups, int keep, int score, const float* correction, int group_top, int renorm,
                            const float* bias, void* stream) {
    if (T < 0 || W < 1 || E < 1 || top < 1 || (score != SM_ROUTE_SOFTMAX && score != SM_ROUTE_SIGMOID) || group_top < 1 ||
        group_top > 4 || (T > 0 && (!h || !router_w || !idx || !wts))) {
        set_error("sm_moe_route: bad argument");
        return SM_EINVAL;
    }
    if (groups < 1) groups = 1;
    if (E > kMaxExperts || top > kMaxTop || top > E || E % groups || keep < 1 || keep > groups || top > keep * (E / groups)) {
        set_error("sm_moe_route: unsupported routing shape (E=%d top=%d groups=%d keep=%d)", E, top, groups, keep);
        return SM_ESHAPE;
    }
    if (T == 0) return SM_OK;
    // the token rows of a workgroup are staged in LDS when they fit and the rows can be moved in pieces of four channels
    const size_t scores = (size_t)kRouteTokens * (E + groups) * 4;
    const size_t rows = (size_t)kRouteTokens * W * (dtype == SM_F32 ? 4 : 2);
    const int staged = W % 4 == 0 && scores % 16 == 0 && scores + rows <= 60 * 1024 && ((uintptr_t)h | (uintptr_t)router_w) % 16 == 0;
    SM_DISPATCH(dtype, "sm_moe_route",
                hipLaunchKernelGGL(moe_route_kernel<DT>, dim3((unsigned)((T + kRouteTokens - 1) / kRouteTokens)), dim3(256),
                                   scores + (staged ? rows : 0), as_stream(stream), (const DT*)h, router_w, idx, wts, T, W, E,
                                   top, groups, keep, score, correction, group_top, renorm, staged, bias));
    SM_CHECK_LAUNCH("sm_moe_route");
    return SM_OK;
}

extern "C" int sm_moe_pairs_gate_up(int dtype, const void* h, const int32_t* idx, const void* w_gu, float limit, float alpha,
                                    int act_kind, void* act, int64_t T, int top, int W, int F, void* stream) {
    if (T < 0 || top < 1 || W < 1 || F < 1 || act_kind < 0 || act_kind > SM_ACT_SILU_GLU || (T > 0 && (!h || !idx || !w_gu || !act))) {
        set_error("sm_moe_pairs_gate_up: bad argument");
        return SM_EINVAL;
    }
    if ((size_t)W * 4 > 60000) { set_error("sm_moe_pairs_gate_up: width too large"); return SM_ESHAPE; }
    if (T == 0) return SM_OK;
    SM_DISPATCH(dtype, "sm_moe_pairs_gate_up",
                hipLaunchKernelGGL(moe_pairs_gate_up_kernel<DT>, dim3((unsigned)(T * top)), dim3(256), (size_t)W * 4,
                                   as_stream(stream), (const DT*)h, idx, (const DT*)w_gu, limit, alpha, (DT*)act, top, W, F, act_kind));
    SM_CHECK_LAUNCH("sm_moe_pairs_gate_up");
    return SM_OK;
}

extern "C" int sm_moe_pairs_down(int dtype, const void* act, const int32_t* idx, const float* wts, const void* w_down,
                                 const void* shared, void* y, int64_t T, int top, int W, int F, void* stream) {
    if (T < 0 || top < 1 || W < 1 || F < 1 || (T > 0 && (!act || !idx || !wts || !w_down || !y))) {
        set_error("sm_moe_pairs_down: bad argument");
        return SM_EINVAL;
    }
    if (T == 0) return SM_OK;
    const int staged = (size_t)top * F * 4 <= 60000;            // a token's activations in LDS when they fit
    SM_DISPATCH(dtype, "sm_moe_pairs_down",
                hipLaunchKernelGGL(moe_pairs_down_kernel<DT>, dim3((unsigned)T), dim3(256), staged ? (size_t)top * F * 4 : 0,
                                   as_stream(stream), (const DT*)act, idx, wts, (const DT*)w_down, (const DT*)shared, (DT*)y, top, W,
                                   F, staged));
    SM_CHECK_LAUNCH("sm_moe_pairs_down");
    return SM_OK;
}
