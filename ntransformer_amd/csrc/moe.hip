// moe.hip -- the routing side of a mixture of experts: router scores and the choice (F32), the stable grouping of (token, slot) pairs by expert that
// the grouped product (dense.hip) consumes, the clipped gated activation between an expert's two products, and the weighted sum back into the
// residual stream.  The experts' products themselves are ntk_dense calls over the stacked expert matrices.
//
// A token's result never depends on the other tokens of the launch: the grouping only decides WHERE a pair's row sits, each row is computed on its
// own, and the sum over a token's slots runs in slot order.
#include "common.hip.h"
#include "../../include/ntk_layers.h"

namespace ntk {

constexpr int kMaxExperts = 256;

// one workgroup per token: its 16 waves share the experts (wave w: experts w, w + 16, ...), a lane requests its whole part of the router row before
// it uses any of it; thread 0 then does the softmax and the `top` picks over the scores in LDS
constexpr int kRouteThreads = 1024;
struct RouteForm { int score, groups, keep, group_top, renorm; float scale; };

// the largest of a wave's 4 x 64 values (lane l holds entries l, l + 64, l + 128, l + 192); equal values: the lower index
__device__ __forceinline__ void wave_argmax4(const float (&v)[4], int lane, float& bv, int& bi) {
    bv = v[0];
    bi = lane;
#pragma unroll
    for (int c = 1; c < 4; ++c)
        if (v[c] > bv) { bv = v[c]; bi = lane + 64 * c; }      // (equal values: the lower index stays)
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
}

__global__ __launch_bounds__(kRouteThreads) void moe_route_kernel(int* ids, float* wts, float* sgate, const float* h, int ldh, const float* wr, const float* wsg,
                                                                 int n, int E, int top, const RouteForm f) {
    __shared__ float z[kMaxExperts];
    extern __shared__ __attribute__((aligned(16))) float xs[];   // the token's row
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = kRouteThreads / 64;
    const long long t = blockIdx.x;
    const float* x = h + t * ldh;
    for (int k = threadIdx.x; k < n; k += kRouteThreads) xs[k] = x[k];
    __syncthreads();
    const bool vec = (n % 4 == 0) && !((uintptr_t)wr & 15) && !(wsg && ((uintptr_t)wsg & 15));
    for (int e = wave; e < E + (wsg ? 1 : 0); e += nw) {
        const float* w = e < E ? wr + (long long)e * n : wsg;
        float s = 0.0f;
        if (vec) {
#pragma unroll 4
            for (int k = lane * 4; k < n; k += 256) {
                const float4 a4 = *reinterpret_cast<const float4*>(w + k), x4 = *reinterpret_cast<const float4*>(xs + k);
                s = fmaf(a4.x, x4.x, s); s = fmaf(a4.y, x4.y, s); s = fmaf(a4.z, x4.z, s); s = fmaf(a4.w, x4.w, s);
            }
        } else {
            for (int k = lane; k < n; k += 64) s = fmaf(w[k], xs[k], s);
        }
        s = wave_sum(s);
        if (lane == 0) {
            if (e < E) z[e] = s;
            else if (sgate) sgate[t] = 1.0f / (1.0f + expf(-s));
        }
    }
    __syncthreads();
    if (wave != 0) return;
    // scores and the picks by one wave: lane l holds experts l, l + 64, l + 128, l + 192
    float v[4];
    float den = 1.0f;
    if (f.score == 0) {
        float m = -INFINITY;
#pragma unroll
        for (int c = 0; c < 4; ++c) { v[c] = lane + 64 * c < E ? z[lane + 64 * c] : -INFINITY; m = fmaxf(m, v[c]); }
        m = wave_max(m);
        den = 0.0f;
#pragma unroll
        for (int c = 0; c < 4; ++c) { v[c] = lane + 64 * c < E ? expf(v[c] - m) : -1.0f; den += fmaxf(v[c], 0.0f); }
        den = wave_sum(den);
    } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) v[c] = lane + 64 * c < E ? 1.0f / (1.0f + expf(-z[lane + 64 * c])) : -1.0f;
    }
    __shared__ int pick_id[kMaxExperts];
    __shared__ float pick_sc[kMaxExperts];
    if (f.groups > 1) {
        // group scores: lane l owns groups l, l + 64, ...: the sum of the group's `group_top` largest scores (scores are >= 0; taken ones are marked -1)
        __shared__ float sc[kMaxExperts];
        __shared__ unsigned char open_group[kMaxExperts];
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (lane + 64 * c < E) sc[lane + 64 * c] = v[c];
        __builtin_amdgcn_wave_barrier();
        const int per = E / f.groups;
        float gs[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int g = lane + 64 * c;
            gs[c] = -1.0f;
            if (g < f.groups) {
                float sum = 0.0f;
                int taken[8];
                const int nt = min(min(f.group_top, per), 8);
                for (int k = 0; k < nt; ++k) {
                    float best = -1.0f;
                    int bi = -1;
                    for (int e = g * per; e < (g + 1) * per; ++e) {
                        bool used = false;
                        for (int u = 0; u < k; ++u) used = used || taken[u] == e;
                        if (!used && sc[e] > best) { best = sc[e]; bi = e; }
                    }
                    taken[k] = bi;
                    sum += best;
                }
                gs[c] = sum;
            }
            if (g < kMaxExperts) open_group[g] = 0;
        }
        __builtin_amdgcn_wave_barrier();
        for (int k = 0; k < f.keep; ++k) {
            float bv;
            int bi;
            wave_argmax4(gs, lane, bv, bi);
            if (lane == 0) open_group[bi] = 1;
            if ((bi & 63) == lane) gs[bi >> 6] = -2.0f;
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (lane + 64 * c < E && !open_group[(lane + 64 * c) / per]) v[c] = -1.0f;
    }
    float chosen = 0.0f;
    for (int s = 0; s < top; ++s) {
        float bv;
        int bi;
        wave_argmax4(v, lane, bv, bi);
        const float sc1 = bv / den;
        chosen += sc1;
        if (lane == 0) { pick_id[s] = bi; pick_sc[s] = sc1; }
        if ((bi & 63) == lane) v[bi >> 6] = -2.0f;
    }
    const float mul = (f.renorm ? 1.0f / (chosen + 1e-20f) : 1.0f) * f.scale;
    for (int s = lane; s < top; s += 64) { ids[t * top + s] = pick_id[s]; wts[t * top + s] = pick_sc[s] * mul; }   // (same wave wrote them: in order)
}

// Stable counting sort of the pairs by expert, one workgroup of 1024: the pairs are cut into S = 1024 / E' contiguous segments (E' = E rounded up to a
// power of two), thread (segment, expert) counts its expert in its segment, one scan in (expert, segment) order gives every thread the place of its
// first row, and it walks its segment once more to place them.  The ids sit in LDS when they fit.
constexpr int kGroupThreads = 1024, kGroupLdsIds = 24 * 1024;
__global__ __launch_bounds__(kGroupThreads) void moe_group_kernel(int* offsets, int* order, int* where, const int* ids_g, int n_pairs, int E, int Ep) {
    __shared__ int cnt[kGroupThreads + 1];
    __shared__ int ids_s[kGroupLdsIds];
    const int* ids = ids_g;
    if (n_pairs <= kGroupLdsIds) {
        for (int i = threadIdx.x; i < n_pairs; i += kGroupThreads) ids_s[i] = ids_g[i];
        ids = ids_s;
    }
    const int S = kGroupThreads / Ep;
    const int e = threadIdx.x % Ep, seg = threadIdx.x / Ep;
    const int per = (n_pairs + S - 1) / S;
    const int i0 = min(seg * per, n_pairs), i1 = min(i0 + per, n_pairs);
    __syncthreads();
    int c = 0;
    if (e < E && seg < S)
        for (int i = i0; i < i1; ++i) c += ids[i] == e;
    // place of thread (e, seg) in (expert, segment) order
    const int slot = e * S + seg;
    cnt[slot] = e < E ? c : 0;             // Ep * S = 1024: every thread has a slot
    __syncthreads();
    {   // exclusive scan of the Ep * S (= 1024) counts: inside each wave by shuffles, the 16 wave totals by the first lanes
        __shared__ int wave_total[kGroupThreads / 64];
        const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
        const int mine = cnt[threadIdx.x];
        int inc = mine;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int up = __shfl_up(inc, o, 64);
            if (lane >= o) inc += up;
        }
        if (lane == 63) wave_total[wv] = inc;
        __syncthreads();
        int before = 0;
        for (int k = 0; k < wv; ++k) before += wave_total[k];
        cnt[threadIdx.x] = before + inc - mine;
        if (threadIdx.x == kGroupThreads - 1) cnt[kGroupThreads] = before + inc;
    }
    __syncthreads();
    if (threadIdx.x <= E) offsets[threadIdx.x] = threadIdx.x < E ? cnt[threadIdx.x * S] : cnt[kGroupThreads];
    if (e < E && seg < S) {
        int at = cnt[slot];
        for (int i = i0; i < i1; ++i)
            if (ids[i] == e) { order[at] = i; where[i] = at; ++at; }
    }
}

__global__ void clipped_glu_kernel(float* a, const float* gu, int ldgu, int ff, float limit, float alpha, float cubic, float up_offset) {
    const long long r = blockIdx.y;
    const int f = blockIdx.x * blockDim.x + threadIdx.x;
    if (f >= ff) return;
    const float g = fminf(gu[r * ldgu + f], limit);
    const float u = fminf(fmaxf(gu[r * ldgu + ff + f], -limit), limit);
    const float z = cubic != 0.0f ? fmaf(cubic * g * g, g, g) : g;
    a[r * ff + f] = g * (1.0f / (1.0f + expf(-alpha * z))) * (u + up_offset);
}

template <bool ADD>
__global__ void moe_combine_kernel(float* x, const float* mix, const float* d, const int* where, const float* wts, const float* shared, const float* sgate,
                                   int top, int n) {
    const long long t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float s = 0.0f;
    for (int k = 0; k < top; ++k) s = fmaf(wts[t * top + k], d[(long long)where[t * top + k] * n + i], s);
    if (shared) s = sgate ? fmaf(sgate[t], shared[t * n + i], s) : s + shared[t * n + i];
    if (mix) s += mix[t * n + i];
    if constexpr (ADD) x[t * n + i] += s; else x[t * n + i] = s;
}

}  // namespace ntk

using namespace ntk;

int ntk_moe_route(int* ids, float* wts, float* sgate, const float* h, int ldh, const float* w_router, const float* shared_gate_w, int T, int n, int E, int top,
                  void* stream) {
    const ntk_route_desc r{0, 1, 1, 1, 1, 1.0f};   // softmax scores, no groups, weights renormalised over the chosen
    return ntk_moe_route_ex(ids, wts, sgate, h, ldh, w_router, shared_gate_w, T, n, E, top, &r, stream);
}

int ntk_moe_route_ex(int* ids, float* wts, float* sgate, const float* h, int ldh, const float* w_router, const float* shared_gate_w, int T, int n, int E, int top,
                     const ntk_route_desc* r, void* stream) {
    if (!ids || !wts || !h || !w_router || !r) return NTK_E_NULL;
    if (T < 0 || n <= 0 || E <= 0 || E > kMaxExperts || top <= 0 || top > E || ldh < n) return NTK_E_SHAPE;
    if (r->score != 0 && r->score != 1) return NTK_E_SHAPE;
    const int groups = r->groups > 1 ? r->groups : 1;
    if (groups > 1 && (E % groups || r->keep < 1 || r->keep > groups || r->group_top < 1 || r->group_top > 8 || (long long)r->keep * (E / groups) < top)) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    if ((size_t)n * 4 > 128 * 1024) return NTK_E_SHAPE;
    const RouteForm f{r->score, groups, r->keep, r->group_top, r->renorm, r->scale};
    hipLaunchKernelGGL(moe_route_kernel, dim3(T), dim3(kRouteThreads), (size_t)n * 4, resolve_stream(stream), ids, wts, sgate, h, ldh, w_router, shared_gate_w, n, E, top, f);
    return last_launch_status();
}

int ntk_moe_group(int* offsets, int* order, int* where, const int* ids, int T, int top, int E, void* stream) {
    if (!offsets || !order || !where || !ids) return NTK_E_NULL;
    if (T < 0 || top <= 0 || E <= 0 || E >= 256) return NTK_E_SHAPE;
    int Ep = 1;
    while (Ep < E) Ep *= 2;
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(kGroupThreads), 0, resolve_stream(stream), offsets, order, where, ids, T * top, E, Ep);
    return last_launch_status();
}

int ntk_clipped_glu(float* a, const float* gu, int rows, int ff, float limit, float alpha, void* stream) {
    return ntk_glu(a, gu, rows, ff, limit, alpha, 1.0f, stream);
}

int ntk_glu(float* a, const float* gu, int rows, int ff, float limit, float alpha, float up_offset, void* stream) {
    if (!a || !gu) return NTK_E_NULL;
    if (rows < 0 || ff <= 0) return NTK_E_SHAPE;
    if (rows == 0) return NTK_OK;
    hipLaunchKernelGGL(clipped_glu_kernel, dim3((ff + 255) / 256, rows), dim3(256), 0, resolve_stream(stream), a, gu, 2 * ff, ff, limit, alpha, 0.0f, up_offset);
    return last_launch_status();
}

int ntk_glu_cubic(float* a, const float* gu, int ldgu, int rows, int ff, float limit, float alpha, float cubic, float up_offset, void* stream) {
    if (!a || !gu) return NTK_E_NULL;
    if (rows < 0 || ff <= 0 || ldgu < 2 * ff) return NTK_E_SHAPE;
    if (rows == 0) return NTK_OK;
    hipLaunchKernelGGL(clipped_glu_kernel, dim3((ff + 255) / 256, rows), dim3(256), 0, resolve_stream(stream), a, gu, ldgu, ff, limit, alpha, cubic, up_offset);
    return last_launch_status();
}

int ntk_moe_combine(float* x, const float* mix, const float* d, const int* where, const float* wts, const float* shared, const float* sgate, int T, int top,
                    int n, void* stream) {
    if (!x || !d || !where || !wts || (shared && !sgate)) return NTK_E_NULL;
    if (T < 0 || top <= 0 || n <= 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(moe_combine_kernel<true>, dim3((n + 255) / 256, T), dim3(256), 0, resolve_stream(stream), x, mix, d, where, wts, shared, sgate, top, n);
    return last_launch_status();
}

int ntk_moe_sum(float* out, const float* d, const int* where, const float* wts, const float* shared, const float* sgate, int T, int top, int n, void* stream) {
    if (!out || !d || !where || !wts) return NTK_E_NULL;
    if (T < 0 || top <= 0 || n <= 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(moe_combine_kernel<false>, dim3((n + 255) / 256, T), dim3(256), 0, resolve_stream(stream), out, (const float*)nullptr, d, where, wts, shared, sgate, top, n);
    return last_launch_status();
}
