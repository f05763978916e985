// gated_recurrence.hip -- linear attention whose state forgets per token, head and KEY CHANNEL, optionally with the delta rule's removal term:
//
//     S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T        o_t = S_t^T (q_scale q_t)        u_t = k_t / sqrt(sum k_t^2 + unit_eps)
//
// (the removal is taken from S_(t-1) as it was, not from the decayed state).  Without the removal term this is gated linear attention.  Everything behind the projections is F32.
//
// A column of the state never meets another column: u^T S, the update and S^T q are sums over key channels only.  So a lane owns RP rows of ONE value
// column, SPLIT lanes next to each other share a column (their partial sums meet in a DPP reduction, twice per token with the removal term, once without),
// and a wave walks the tokens in order without ever waiting for another wave: no barrier per token, the state stays in registers for the whole portion
// and crosses HBM once in and once out.  The four waves of a workgroup share one head, so the per-token vectors -- q, k, the decay formed from its raw
// projection, the removal rate times the unit key -- are staged for all of them in LDS, a batch of tokens at a time; the NEXT batch's raw values are
// requested into registers before the current batch is walked, so their latency hides behind the walk.
// The walk is the same whatever the portion: a sequence cut anywhere gives the same sums in the same order.
#include <algorithm>
#include "common.hip.h"
#include "../../include/ntk_layers.h"

namespace ntk {

struct RecArgs {
    float* out; int ldo;
    const float* q; int ldq;
    const float* k; int ldk;
    const float* v; int ldv;
    const float* wz; int ldw; const float* wb; int decay_form; float decay_param;
    const float* az; int lda; const float* ab; float unit_eps;
    float* state;
    int H, dn, dv;
    float q_scale;
    int pos0, T, TB;
};

constexpr int REC_PF = 8;        // staged (token, channel) entries a thread carries from one batch to the next: TB * SPLIT * RP <= 256 * REC_PF

__device__ __forceinline__ float decay_of(float z, int form, float param) {
    if (form == NTK_DECAY_SIGMOID_ROOT) {
        // sigmoid(z)^(1/param) = exp(-softplus(-z) / param), softplus(x) = max(x, 0) + log1p(exp(-|x|))
        const float sp = fmaxf(-z, 0.0f) + log1pf(expf(-fabsf(z)));
        return expf(-sp / param);
    }
    if (form == NTK_DECAY_EXP_SIGMOID) return expf(-param / (1.0f + expf(-z)));
    return z;
}

template <int SPLIT, int RP, bool DELTA>
__global__ __launch_bounds__(256) void gated_recurrence_kernel(const RecArgs a) {
    constexpr int CW = 64 / SPLIT, CB = 4 * CW;          // value columns per wave / per workgroup
    constexpr int RS = RP + 4;                           // LDS floats per lane group: the groups' 16-byte reads fall into different banks
    constexpr int DP = SPLIT * RP, DL = SPLIT * RS;      // key channels a workgroup covers (>= dn) / their LDS footprint
    constexpr int NV = DELTA ? 5 : 3;                    // staged vectors per token: q, k, w (, u, a * u)
    extern __shared__ __attribute__((aligned(16))) float lds[];
    float* Vec = lds;                                    // [TB][NV][DL]
    float* Vs = lds + (size_t)a.TB * NV * DL;            // [TB][CB]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int cl = lane / SPLIT, rg = lane % SPLIT;
    const int h = blockIdx.y, c0 = blockIdx.x * CB, c = c0 + wave * CW + cl;
    const bool col_ok = c < a.dv;
    // ---- the state slice: rows rg * RP + i of column c
    float S[RP];
    float* st = a.state + ((long long)h * a.dn) * a.dv + c;
#pragma unroll
    for (int i = 0; i < RP; ++i) {
        const int r = rg * RP + i;
        S[i] = (a.pos0 > 0 && col_ok && r < a.dn) ? st[(long long)r * a.dv] : 0.0f;
    }
    // ---- raw values of a batch into registers (requests only), and from registers through the activations into LDS
    float pq[REC_PF], pk[REC_PF], pw[REC_PF], pa[REC_PF], pv[2];
    auto request = [&](int t0, int nb) {
#pragma unroll
        for (int u = 0; u < REC_PF; ++u) {
            const int idx = threadIdx.x + 256 * u, tb = idx / DP, d = idx % DP;
            const bool ok = tb < nb && d < a.dn;
            const long long t = t0 + tb;
            pq[u] = ok ? a.q[t * a.ldq + (long long)h * a.dn + d] : 0.0f;
            pk[u] = ok ? a.k[t * a.ldk + (long long)h * a.dn + d] : 0.0f;
            pw[u] = ok ? a.wz[t * a.ldw + (long long)h * a.dn + d] + (a.wb ? a.wb[h * a.dn + d] : 0.0f) : 0.0f;
            if constexpr (DELTA) pa[u] = ok ? a.az[t * a.lda + (long long)h * a.dn + d] + (a.ab ? a.ab[h * a.dn + d] : 0.0f) : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int idx = threadIdx.x + 256 * u, tb = idx / CB, cc = idx % CB;
            pv[u] = (tb < nb && c0 + cc < a.dv) ? a.v[(long long)(t0 + tb) * a.ldv + (long long)h * a.dv + c0 + cc] : 0.0f;
        }
    };
    auto stage = [&](int nb) {
#pragma unroll
        for (int u = 0; u < REC_PF; ++u) {
            const int idx = threadIdx.x + 256 * u, tb = idx / DP, d = idx % DP;
            if (tb >= a.TB) continue;
            const bool ok = tb < nb && d < a.dn;
            float* dst = Vec + (size_t)tb * NV * DL + (d / RP) * RS + d % RP;
            dst[0] = pq[u] * a.q_scale;
            dst[DL] = pk[u];
            dst[2 * DL] = ok ? decay_of(pw[u], a.decay_form, a.decay_param) : 1.0f;
            if constexpr (DELTA) dst[4 * DL] = ok ? 1.0f / (1.0f + expf(-pa[u])) : 0.0f;     // the removal rate; times the unit key below
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int idx = threadIdx.x + 256 * u;
            if (idx < a.TB * CB) Vs[idx] = pv[u];
        }
        if constexpr (DELTA) {
            __syncthreads();
            for (int tb = wave; tb < nb; tb += 4) {      // a wave per token: the unit key (one sum over the head's channels, lanes in a fixed order)
                float* base = Vec + (size_t)tb * NV * DL;
                float ss = 0.0f;
                for (int d = lane; d < a.dn; d += 64) { const float kk = base[DL + (d / RP) * RS + d % RP]; ss = fmaf(kk, kk, ss); }
                const float inv = 1.0f / sqrtf(wave_sum(ss) + a.unit_eps);
                for (int d = lane; d < DP; d += 64) {
                    const int o = (d / RP) * RS + d % RP;
                    const float uu = base[DL + o] * inv;
                    base[3 * DL + o] = uu;
                    base[4 * DL + o] *= uu;
                }
            }
        }
    };
    request(0, min(a.TB, a.T));
    for (int t0 = 0; t0 < a.T; t0 += a.TB) {
        const int nb = min(a.TB, a.T - t0);
        __syncthreads();                                 // the previous batch has been walked by every wave
        stage(nb);
        __syncthreads();
        if (t0 + a.TB < a.T) request(t0 + a.TB, min(a.TB, a.T - t0 - a.TB));
        for (int tb = 0; tb < nb; ++tb) {
            const float* base = Vec + (size_t)tb * NV * DL + rg * RS;
            float qv[RP], kv[RP], wv[RP];
#pragma unroll
            for (int i = 0; i < RP; i += 4) {
                const float4 x = *reinterpret_cast<const float4*>(base + i), y = *reinterpret_cast<const float4*>(base + DL + i), z = *reinterpret_cast<const float4*>(base + 2 * DL + i);
                qv[i] = x.x; qv[i + 1] = x.y; qv[i + 2] = x.z; qv[i + 3] = x.w;
                kv[i] = y.x; kv[i + 1] = y.y; kv[i + 2] = y.z; kv[i + 3] = y.w;
                wv[i] = z.x; wv[i + 1] = z.y; wv[i + 2] = z.z; wv[i + 3] = z.w;
            }
            const float vv = Vs[tb * CB + wave * CW + cl];
            if constexpr (DELTA) {
                float uv[RP], av[RP];
#pragma unroll
                for (int i = 0; i < RP; i += 4) {
                    const float4 x = *reinterpret_cast<const float4*>(base + 3 * DL + i), y = *reinterpret_cast<const float4*>(base + 4 * DL + i);
                    uv[i] = x.x; uv[i + 1] = x.y; uv[i + 2] = x.z; uv[i + 3] = x.w;
                    av[i] = y.x; av[i + 1] = y.y; av[i + 2] = y.z; av[i + 3] = y.w;
                }
                float p = 0.0f;
#pragma unroll
                for (int i = 0; i < RP; ++i) p = fmaf(uv[i], S[i], p);
                const float us = group_sum<SPLIT>(p);    // u^T S(t-1) of this column
#pragma unroll
                for (int i = 0; i < RP; ++i) S[i] = fmaf(wv[i], S[i], fmaf(-av[i], us, kv[i] * vv));
            } else {
#pragma unroll
                for (int i = 0; i < RP; ++i) S[i] = fmaf(wv[i], S[i], kv[i] * vv);
            }
            float o = 0.0f;
#pragma unroll
            for (int i = 0; i < RP; ++i) o = fmaf(S[i], qv[i], o);
            o = group_sum<SPLIT>(o);
            if (rg == 0 && col_ok) a.out[(long long)(t0 + tb) * a.ldo + (long long)h * a.dv + c] = o;
        }
    }
#pragma unroll
    for (int i = 0; i < RP; ++i) {
        const int r = rg * RP + i;
        if (col_ok && r < a.dn) st[(long long)r * a.dv] = S[i];
    }
}

template <int SPLIT, int RP>
static int launch_rec(const RecArgs& a0, hipStream_t s) {
    RecArgs a = a0;
    constexpr int CB = 4 * (64 / SPLIT), DP = SPLIT * RP, DL = SPLIT * (RP + 4);
    const bool delta = a.az != nullptr;
    const int NV = delta ? 5 : 3;
    int tb = (256 * REC_PF) / DP;                        // what a thread's registers carry
    tb = std::min(tb, (2 * 256) / CB);                   // ... and of the values
    tb = std::min(tb, 16);
    tb = std::min(tb, (int)(40 * 1024 / ((NV * DL + CB) * sizeof(float))));   // a batch's LDS stays under 40 KB: several workgroups per CU
    tb = std::min(tb, std::max(a.T, 1));
    a.TB = std::max(tb, 1);
    const size_t lds = ((size_t)a.TB * NV * DL + (size_t)a.TB * CB) * sizeof(float);
    const dim3 grid((a.dv + CB - 1) / CB, a.H);
    if (delta) hipLaunchKernelGGL((gated_recurrence_kernel<SPLIT, RP, true>), grid, dim3(256), lds, s, a);
    else hipLaunchKernelGGL((gated_recurrence_kernel<SPLIT, RP, false>), grid, dim3(256), lds, s, a);
    return last_launch_status();
}

}  // namespace ntk

using namespace ntk;

int ntk_gated_recurrence(const ntk_gated_recurrence_desc* d, void* stream) {
    if (!d || !d->out || !d->q || !d->k || !d->v || !d->wz || !d->state) return NTK_E_NULL;
    if (d->T < 0 || d->H <= 0 || d->dn <= 0 || d->dv <= 0 || d->pos0 < 0 || d->dn > 1024) return NTK_E_SHAPE;
    if (d->decay_form != NTK_DECAY_GIVEN && d->decay_form != NTK_DECAY_SIGMOID_ROOT && d->decay_form != NTK_DECAY_EXP_SIGMOID) return NTK_E_SHAPE;
    if (d->decay_form == NTK_DECAY_SIGMOID_ROOT && !(d->decay_param > 0.0f)) return NTK_E_SHAPE;
    const int hd = d->H * d->dn;
    if (d->ldq < hd || d->ldk < hd || d->ldw < hd || (d->az && d->lda < hd) || d->ldv < d->H * d->dv || d->ldo < d->H * d->dv) return NTK_E_SHAPE;
    if (d->T == 0) return NTK_OK;
    RecArgs a{d->out, d->ldo, d->q, d->ldq, d->k, d->ldk, d->v, d->ldv, d->wz, d->ldw, d->wb, d->decay_form, d->decay_param, d->az, d->lda, d->ab, d->unit_eps,
              d->state, d->H, d->dn, d->dv, d->q_scale, d->pos0, d->T, 0};
    hipStream_t s = resolve_stream(stream);
    // Lanes per column: 32 (two columns per wave, 16 x the waves of the wide form) while the launch would otherwise leave most of the chip idle or the
    // head's channels would not fit 8 lanes; rows per lane: the smallest of 4 / 8 / 16 / 32 that covers the channels.
    const long long cols = (long long)d->H * d->dv;
    const bool narrow = d->dn > 8 * 32 || cols / 8 < 2048;
    if (narrow) {
        if (d->dn <= 32 * 4) return launch_rec<32, 4>(a, s);
        if (d->dn <= 32 * 8) return launch_rec<32, 8>(a, s);
        if (d->dn <= 32 * 16) return launch_rec<32, 16>(a, s);
        return launch_rec<32, 32>(a, s);
    }
    if (d->dn <= 8 * 4) return launch_rec<8, 4>(a, s);
    if (d->dn <= 8 * 8) return launch_rec<8, 8>(a, s);
    if (d->dn <= 8 * 16) return launch_rec<8, 16>(a, s);
    return launch_rec<8, 32>(a, s);
}
