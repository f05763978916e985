// gated_recurrence.hip -- linear attention whose state forgets per token, head and KEY CHANNEL, optionally with the delta rule's removal term:
//
//     S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T        o_t = S_t^T (q_scale q_t)        u_t = k_t / sqrt(sum k_t^2 + unit_eps)
//
// (the removal is taken from S_(t-1) as it was, not from the decayed state).  Without the removal term this is gated linear attention.  Everything behind the projections is F32.
//
// A column of the state never meets another column: u^T S, the update and S^T q are sums over key channels only.  So a lane owns RP rows of ONE value
// column, SPLIT lanes next to each other share a column (their partial sums meet in a DPP reduction, twice per token with the removal term, once without;
// only the first of the two lies on the chain from one token to the next),
// and a wave walks the tokens in order without ever waiting for another wave: no barrier per token, the state stays in registers for the whole portion
// and crosses HBM once in and once out.  The four waves of a workgroup share one head, so the per-token vectors -- q, k, the decay formed from its raw
// projection, the removal rate times the unit key -- are staged for all of them in LDS, a batch of tokens at a time; the NEXT batch's raw values are
// requested into registers before the current batch is walked, so their latency hides behind the walk.
// Portions of more than a few tokens run a pre-pass first (one wave per token and head, the whole chip at once) that leaves those vectors ready-made in a
// packed buffer [T][H][vectors][dn]: the walk's staging is then a copy, and what a head's workgroups would each have recomputed is computed once.
// Long portions are walked in SEGMENTS side by side (the chain from token to token is latency, and a wave that waits costs its neighbours nothing): every
// segment but the first starts from a zero state, and dn extra columns that start as the identity and take no k v^T ride along -- they hold P, the product
// of the segment's transitions M_t = diag(w_t) - (a_t u_t) u_t^T, and their outputs are P_t^T q_t.  Then x(g + 1) = P(g) x(g) + L(g) hands the true state
// from segment to segment (recurrence_chain_kernel, a few small products in turn) and out_t += x(g)^T (P_t^T q_t) settles what every token's output was
// still owed (recurrence_owed_kernel).  Only products of decays <= 1 appear, nothing is divided by a decay: no overflow whatever the decays are.
// Within a segment the walk is the same whatever the portion; where the segments' borders fall changes the order of the sums, i.e. rounding only.
//
// The delta rule with one gate per head is the same walk with other vectors: S' = w S, S = S' - a u (u^T S') + a k v^T with a scalar w and a per head is
// S = w S - (a u) ((w u)^T S) + k (a v)^T, so the pre-pass leaves (w u) where the walk takes the sum, (a u) where it removes, and a copy of the values
// times a.  Unit queries and keys, q / k heads shared by several state heads and the per-head decay forms are the pre-pass's too.
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
    float* packed;                   // [T][H][NV][dn] ready-made vectors (q * scale, k, w (, u, a * u)), or NULL: formed while staging
    // segments walked side by side (nseg > 1, packed only): segment g owns tokens [g * seg_len, (g + 1) * seg_len)
    int nseg, seg_len;
    float* rbuf;                     // [T][H][dn]: P_t^T q_t, P_t the product of the segment's transitions up to t
    float* pbuf;                     // [nseg][H][dn][dn]: the segment's whole transition
    float* lbuf;                     // [nseg][H][dn][dv]: the state the segment's own tokens leave (segment 0: from the sequence's state)
    float* sbuf;                     // [nseg][H][dn][dv]: the state at the segment's start
    // the per-head options (pre-pass only)
    int G, unit_q, unit_k, head_gates, write_gated;
    const float* decay_rates;
    float* vpacked;                  // [T][H][dv]: values times the removal rate (write_gated); the walk then reads these
    // a short causal convolution + silu on the raw q, k, v of ONE token inside the pre-pass (conv_w [2 G dn + H dv][taps], the carried inputs conv_state)
    const float* conv_w; float* conv_state; int conv_taps;
};

constexpr int kRecFewTokens = 8;  // up to this many tokens (decoding) the walk forms its vectors itself: one launch
// staged (token, channel) entries a thread carries from one batch to the next: TB * SPLIT * RP <= threads * rec_pf
constexpr int rec_pf(int waves) { return waves == 1 ? 16 : 8; }

__device__ __forceinline__ float decay_of(float z, int form, float param) {
    if (form == NTK_DECAY_SIGMOID_ROOT) {
        // sigmoid(z)^(1/param) = exp(-softplus(-z) / param), softplus(x) = max(x, 0) + log1p(exp(-|x|))
        const float sp = fmaxf(-z, 0.0f) + log1pf(expf(-fabsf(z)));
        return expf(-sp / param);
    }
    if (form == NTK_DECAY_EXP_SIGMOID) return expf(-param / (1.0f + expf(-z)));
    if (form == NTK_DECAY_EXP_SOFTPLUS) return expf(-param * (fmaxf(z, 0.0f) + log1pf(expf(-fabsf(z)))));
    return z;
}

// the per-token vectors of one (token, head), ready for the walk: one wave each
template <bool DELTA>
__global__ __launch_bounds__(64) void gated_recurrence_prepare_kernel(const RecArgs a) {
    constexpr int NV = DELTA ? 5 : 3;
    const int lane = threadIdx.x, h = blockIdx.x % a.H;
    const long long t = blockIdx.x / a.H;
    float* dst = a.packed + (t * a.H + h) * NV * a.dn;
    const long long oq = (long long)(a.G > 0 ? h / (a.H / a.G) : h) * a.dn;      // where this state head's q and k lie
    const long long oc = (long long)h * a.dn;                                     // ... and its per-channel gates
    float ss = 0.0f, sq = 0.0f;
    for (int d = lane; d < a.dn; d += 64) {
        const float kk = a.k[t * a.ldk + oq + d], qq = a.q[t * a.ldq + oq + d];
        ss = fmaf(kk, kk, ss);
        sq = fmaf(qq, qq, sq);
    }
    const float inv_k = 1.0f / sqrtf(wave_sum(ss) + a.unit_eps);      // (the same sum in the same lane order as the staging of the walk forms it)
    const float qmul = a.unit_q ? a.q_scale / sqrtf(wave_sum(sq) + a.unit_eps) : a.q_scale;
    const float kmul = a.unit_k ? inv_k : 1.0f;
    float wh = 1.0f, ah = 0.0f;                                        // one decay and one removal rate for the head
    if (a.head_gates) {
        wh = decay_of(a.wz[t * a.ldw + h] + (a.wb ? a.wb[h] : 0.0f), a.decay_form, a.decay_rates ? a.decay_rates[h] : a.decay_param);
        if constexpr (DELTA) ah = 1.0f / (1.0f + expf(-(a.az[t * a.lda + h] + (a.ab ? a.ab[h] : 0.0f))));
    }
    for (int d = lane; d < a.dn; d += 64) {
        const float kk = a.k[t * a.ldk + oq + d];
        const float w = a.head_gates ? wh : decay_of(a.wz[t * a.ldw + oc + d] + (a.wb ? a.wb[oc + d] : 0.0f), a.decay_form, a.decay_rates ? a.decay_rates[h] : a.decay_param);
        dst[d] = a.q[t * a.ldq + oq + d] * qmul;
        dst[a.dn + d] = kk * kmul;
        dst[2 * a.dn + d] = w;
        if constexpr (DELTA) {
            const float uu = kk * inv_k;
            const float aa = a.head_gates ? ah : 1.0f / (1.0f + expf(-(a.az[t * a.lda + oc + d] + (a.ab ? a.ab[oc + d] : 0.0f))));
            dst[3 * a.dn + d] = a.write_gated ? uu * w : uu;
            dst[4 * a.dn + d] = uu * aa;
        }
    }
    if constexpr (DELTA) {
        if (a.write_gated)
            for (int c = lane; c < a.dv; c += 64) a.vpacked[(t * a.H + h) * a.dv + c] = a.v[t * a.ldv + (long long)h * a.dv + c] * ah;
    }
}

// One token (decoding) whose q, k, v still have to pass their short convolutions: a workgroup per q / k head.  It convolves the head's q and k channels and the
// value channels of the state heads that share them (each channel's carried inputs are read, used and shifted by the one thread that owns the channel), then
// forms the same vectors as the kernel above, with the same sums in the same lane order.
constexpr int kStepConvTaps = 16;
struct ConvTaps {                                        // one channel's carried inputs, taps and present input, all requested before anything is stored
    float hist[kStepConvTaps - 1], w[kStepConvTaps], x;
    __device__ __forceinline__ void load(const float* cw, const float* state, int taps, int n, int c, float xin, int pos0) {
#pragma unroll
        for (int j = 0; j < kStepConvTaps - 1; ++j) hist[j] = (j < taps - 1 && pos0 - (taps - 1) + j >= 0) ? state[(long long)j * n + c] : 0.0f;
#pragma unroll
        for (int j = 0; j < kStepConvTaps; ++j) w[j] = j < taps ? cw[(long long)c * taps + j] : 0.0f;
        x = xin;
    }
    // the convolution and silu; the carried rows shift in place
    __device__ __forceinline__ float finish(float* state, int taps, int n, int c) const {
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < kStepConvTaps - 1; ++j)
            if (j < taps - 1) s = fmaf(w[j], hist[j], s);
#pragma unroll
        for (int j = 0; j < kStepConvTaps; ++j)
            if (j == taps - 1) s = fmaf(w[j], x, s);
#pragma unroll
        for (int j = 1; j < kStepConvTaps - 1; ++j)
            if (j < taps - 1) state[(long long)(j - 1) * n + c] = hist[j];
        if (taps > 1) state[(long long)(taps - 2) * n + c] = x;
        return s / (1.0f + expf(-s));
    }
};

template <bool DELTA>
__global__ __launch_bounds__(256) void gated_recurrence_prepare_step_kernel(const RecArgs a) {
    constexpr int NV = DELTA ? 5 : 3;
    extern __shared__ float cs[];                        // [dn] q, [dn] k after convolution and silu
    const int G = a.G > 0 ? a.G : a.H, R = a.H / G, g = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nch = 2 * G * a.dn + a.H * a.dv;           // convolved channels: q | k | v
    float* qs = cs;
    float* ks = cs + a.dn;
    // the gates of the wave's first state head: requested now, used after the convolutions
    float wz0 = 0.0f, az0 = 0.0f, rate0 = a.decay_param;
    if (a.head_gates && wave < R) {
        const int h = g * R + wave;
        wz0 = a.wz[h] + (a.wb ? a.wb[h] : 0.0f);
        if (a.decay_rates) rate0 = a.decay_rates[h];
        if constexpr (DELTA) az0 = a.az[h] + (a.ab ? a.ab[h] : 0.0f);
    }
    const int nqk = 2 * a.dn, nv = R * a.dv;
    for (int e = threadIdx.x; e < max(nqk, nv); e += 256) {
        // the head's q and k channels, and the value channels of the state heads that share them (times the head's removal rate): one round of requests for both
        ConvTaps A, B;
        const bool ha = e < nqk, hb = e < nv;
        const int which = e / a.dn, d = e % a.dn, cA = which * G * a.dn + g * a.dn + d;
        const int h = g * R + e / a.dv, c = e % a.dv, cB = 2 * G * a.dn + h * a.dv + c;
        float azv = 0.0f;
        if (ha) A.load(a.conv_w, a.conv_state, a.conv_taps, nch, cA, which ? a.k[(long long)g * a.dn + d] : a.q[(long long)g * a.dn + d], a.pos0);
        if (hb) {
            B.load(a.conv_w, a.conv_state, a.conv_taps, nch, cB, a.v[(long long)h * a.dv + c], a.pos0);
            if constexpr (DELTA) { if (a.write_gated) azv = a.az[h] + (a.ab ? a.ab[h] : 0.0f); }
        }
        if (ha) cs[e] = A.finish(a.conv_state, a.conv_taps, nch, cA);
        if (hb) {
            const float vv = B.finish(a.conv_state, a.conv_taps, nch, cB);
            a.vpacked[(long long)h * a.dv + c] = (DELTA && a.write_gated) ? vv * (1.0f / (1.0f + expf(-azv))) : vv;
        }
    }
    __syncthreads();
    float ss = 0.0f, sq = 0.0f;
    for (int d = lane; d < a.dn; d += 64) { ss = fmaf(ks[d], ks[d], ss); sq = fmaf(qs[d], qs[d], sq); }
    const float inv_k = 1.0f / sqrtf(wave_sum(ss) + a.unit_eps);
    const float qmul = a.unit_q ? a.q_scale / sqrtf(wave_sum(sq) + a.unit_eps) : a.q_scale;
    const float kmul = a.unit_k ? inv_k : 1.0f;
    for (int r = wave; r < R; r += 4) {                  // a wave per state head of the group
        const int h = g * R + r;
        float* dst = a.packed + (long long)h * NV * a.dn;
        const long long oc = (long long)h * a.dn;
        float wh = 1.0f, ah = 0.0f;
        if (a.head_gates) {
            const bool first = r == wave;
            wh = decay_of(first ? wz0 : a.wz[h] + (a.wb ? a.wb[h] : 0.0f), a.decay_form, first ? rate0 : a.decay_rates ? a.decay_rates[h] : a.decay_param);
            if constexpr (DELTA) ah = 1.0f / (1.0f + expf(-(first ? az0 : a.az[h] + (a.ab ? a.ab[h] : 0.0f))));
        }
        for (int d = lane; d < a.dn; d += 64) {
            const float kk = ks[d];
            const float w = a.head_gates ? wh : decay_of(a.wz[oc + d] + (a.wb ? a.wb[oc + d] : 0.0f), a.decay_form, a.decay_rates ? a.decay_rates[h] : a.decay_param);
            dst[d] = qs[d] * qmul;
            dst[a.dn + d] = kk * kmul;
            dst[2 * a.dn + d] = w;
            if constexpr (DELTA) {
                const float uu = kk * inv_k;
                const float aa = a.head_gates ? ah : 1.0f / (1.0f + expf(-(a.az[oc + d] + (a.ab ? a.ab[oc + d] : 0.0f))));
                dst[3 * a.dn + d] = a.write_gated ? uu * w : uu;
                dst[4 * a.dn + d] = uu * aa;
            }
        }
    }
}

template <int RP, bool DELTA>
struct TokVec {                      // one token's vectors as a lane needs them: its RP rows of q, k, w (, u, a * u) and its column's value
    float q[RP], k[RP], w[RP], u[DELTA ? RP : 1], a[DELTA ? RP : 1], v;
};

template <int SPLIT, int RP, bool DELTA, bool PACKED, int NW>
__global__ __launch_bounds__(64 * NW) void gated_recurrence_kernel(const RecArgs a) {
    constexpr int NT = 64 * NW, REC_PF = rec_pf(NW);
    constexpr int CW = 64 / SPLIT, CB = NW * CW;         // value columns per wave / per workgroup
    constexpr int RS = RP + 4;                           // LDS floats per lane group: the groups' 16-byte reads fall into different banks
    constexpr int DP = SPLIT * RP, DL = SPLIT * RS;      // key channels a workgroup covers (>= dn) / their LDS footprint
    constexpr int NV = DELTA ? 5 : 3;                    // staged vectors per token: q, k, w (, u, a * u)
    extern __shared__ __attribute__((aligned(16))) float lds[];
    float* Vec = lds;                                    // [TB][NV][DL]
    constexpr int EXTRA = RP <= 8 ? 2 : 0;               // token slots behind a batch (see the walk)
    float* Vs = lds + (size_t)(a.TB + EXTRA) * NV * DL;  // [TB + EXTRA][CB]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int cl = lane / SPLIT, rg = lane % SPLIT;
    const int h = blockIdx.y, c0 = blockIdx.x * CB, c = c0 + wave * CW + cl;
    // a segment of the portion; with several segments dn more columns ride along that start as the identity and receive no k v^T: they hold the product
    // of the segment's transitions, and their outputs are what the state at the segment's start still owes every token's output
    const int sg = blockIdx.z, tbase = sg * a.seg_len, T = min(a.T - tbase, a.seg_len);
    const int ncols = (DELTA && a.nseg > 1) ? a.dv + a.dn : a.dv;
    const bool col_ok = c < ncols, aug = c >= a.dv;
    // ---- the state slice: rows rg * RP + i of column c
    float S[RP];
    float* st = a.state + ((long long)h * a.dn) * a.dv + c;
#pragma unroll
    for (int i = 0; i < RP; ++i) {
        const int r = rg * RP + i;
        if (aug) S[i] = r == c - a.dv ? 1.0f : 0.0f;
        else S[i] = (sg == 0 && a.pos0 > 0 && col_ok && r < a.dn) ? st[(long long)r * a.dv] : 0.0f;
    }
    // ---- the two slots behind a full batch: a token that leaves the state as it is and asks for nothing
    for (int e = threadIdx.x; e < EXTRA * NV * DL; e += NT) Vec[(size_t)a.TB * NV * DL + e] = (e % (NV * DL)) / DL == 2 ? 1.0f : 0.0f;
    for (int e = threadIdx.x; e < EXTRA * CB; e += NT) Vs[a.TB * CB + e] = 0.0f;
    // ---- raw values of a batch into registers (requests only), and from registers through the activations into LDS
    float pq[REC_PF], pk[REC_PF], pw[REC_PF], pa[REC_PF], pu[REC_PF], pv[2];
    auto request = [&](int t0, int nb) {
#pragma unroll
        for (int u = 0; u < REC_PF; ++u) {
            const int idx = threadIdx.x + NT * u, tb = idx / DP, d = idx % DP;
            const bool ok = tb < nb && d < a.dn;
            const long long t = tbase + t0 + tb;
            if constexpr (PACKED) {
                const float* src = a.packed + ((t * a.H + h) * NV) * a.dn + d;
                pq[u] = ok ? src[0] : 0.0f;
                pk[u] = ok ? src[a.dn] : 0.0f;
                pw[u] = ok ? src[2 * a.dn] : 1.0f;
                if constexpr (DELTA) { pu[u] = ok ? src[3 * a.dn] : 0.0f; pa[u] = ok ? src[4 * a.dn] : 0.0f; }
                continue;
            }
            pq[u] = ok ? a.q[t * a.ldq + (long long)h * a.dn + d] : 0.0f;
            pk[u] = ok ? a.k[t * a.ldk + (long long)h * a.dn + d] : 0.0f;
            pw[u] = ok ? a.wz[t * a.ldw + (long long)h * a.dn + d] + (a.wb ? a.wb[h * a.dn + d] : 0.0f) : 0.0f;
            if constexpr (DELTA) pa[u] = ok ? a.az[t * a.lda + (long long)h * a.dn + d] + (a.ab ? a.ab[h * a.dn + d] : 0.0f) : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int idx = threadIdx.x + NT * u, tb = idx / CB, cc = idx % CB;
            pv[u] = (tb < nb && c0 + cc < a.dv) ? a.v[(long long)(tbase + t0 + tb) * a.ldv + (long long)h * a.dv + c0 + cc] : 0.0f;
        }
    };
    auto stage = [&](int nb) {
#pragma unroll
        for (int u = 0; u < REC_PF; ++u) {
            const int idx = threadIdx.x + NT * u, tb = idx / DP, d = idx % DP;
            if (tb >= a.TB) continue;
            const bool ok = tb < nb && d < a.dn;
            float* dst = Vec + (size_t)tb * NV * DL + (d / RP) * RS + d % RP;
            if constexpr (PACKED) {
                dst[0] = pq[u]; dst[DL] = pk[u]; dst[2 * DL] = pw[u];
                if constexpr (DELTA) { dst[3 * DL] = pu[u]; dst[4 * DL] = pa[u]; }
                continue;
            }
            dst[0] = pq[u] * a.q_scale;
            dst[DL] = pk[u];
            dst[2 * DL] = ok ? decay_of(pw[u], a.decay_form, a.decay_param) : 1.0f;
            if constexpr (DELTA) { dst[3 * DL] = 0.0f; dst[4 * DL] = ok ? 1.0f / (1.0f + expf(-pa[u])) : 0.0f; }   // the removal rate; times the unit key below
        }
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int idx = threadIdx.x + NT * u;
            if (idx < a.TB * CB) Vs[idx] = pv[u];
        }
        if constexpr (DELTA && !PACKED) {
            __syncthreads();
            for (int tb = wave; tb < nb; tb += NW) {     // a wave per token: the unit key (one sum over the head's channels, lanes in a fixed order)
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
    request(0, min(a.TB, T));
    for (int t0 = 0; t0 < T; t0 += a.TB) {
        const int nb = min(a.TB, T - t0);
        __syncthreads();                                 // the previous batch has been walked by every wave
        stage(nb);
        __syncthreads();
        if (t0 + a.TB < T) request(t0 + a.TB, min(a.TB, T - t0 - a.TB));
        // The walk.  A token's vectors leave LDS one token AHEAD of their use (a second register set while the rows per lane are few), so the only chain from
        // token to token is the state's own: u^T S, its reduction, the update.
        auto load_tok = [&](int tb, TokVec<RP, DELTA>& x) {
            const float* base = Vec + (size_t)tb * NV * DL + rg * RS;
#pragma unroll
            for (int i = 0; i < RP; i += 4) {
                const float4 q4 = *reinterpret_cast<const float4*>(base + i), k4 = *reinterpret_cast<const float4*>(base + DL + i), w4 = *reinterpret_cast<const float4*>(base + 2 * DL + i);
                x.q[i] = q4.x; x.q[i + 1] = q4.y; x.q[i + 2] = q4.z; x.q[i + 3] = q4.w;
                x.k[i] = k4.x; x.k[i + 1] = k4.y; x.k[i + 2] = k4.z; x.k[i + 3] = k4.w;
                x.w[i] = w4.x; x.w[i + 1] = w4.y; x.w[i + 2] = w4.z; x.w[i + 3] = w4.w;
                if constexpr (DELTA) {
                    const float4 u4 = *reinterpret_cast<const float4*>(base + 3 * DL + i), a4 = *reinterpret_cast<const float4*>(base + 4 * DL + i);
                    x.u[i] = u4.x; x.u[i + 1] = u4.y; x.u[i + 2] = u4.z; x.u[i + 3] = u4.w;
                    x.a[i] = a4.x; x.a[i + 1] = a4.y; x.a[i + 2] = a4.z; x.a[i + 3] = a4.w;
                }
            }
            x.v = Vs[tb * CB + wave * CW + cl];
        };
        // one token: the state's update, and the column's output as this lane's partial sum (the lanes' sums meet later, off the chain)
        auto step = [&](const TokVec<RP, DELTA>& x) -> float {
            if constexpr (DELTA) {
                float p0 = 0.0f, p1 = 0.0f;              // (two partial sums: half the chain; rows in a fixed order either way)
#pragma unroll
                for (int i = 0; i < RP; i += 2) { p0 = fmaf(x.u[i], S[i], p0); p1 = fmaf(x.u[i + 1], S[i + 1], p1); }
                const float us = group_sum<SPLIT>(p0 + p1);   // u^T S(t-1) of this column
#pragma unroll
                for (int i = 0; i < RP; ++i) S[i] = fmaf(x.w[i], S[i], fmaf(-x.a[i], us, x.k[i] * x.v));
            } else {
#pragma unroll
                for (int i = 0; i < RP; ++i) S[i] = fmaf(x.w[i], S[i], x.k[i] * x.v);
            }
            float o0 = 0.0f, o1 = 0.0f;
#pragma unroll
            for (int i = 0; i < RP; i += 2) { o0 = fmaf(S[i], x.q[i], o0); o1 = fmaf(S[i + 1], x.q[i + 1], o1); }
            return o0 + o1;
        };
        const long long ostep = aug ? (long long)a.H * a.dn : a.ldo;
        float* orow = aug ? a.rbuf + (long long)(tbase + t0) * ostep + (long long)h * a.dn + (c - a.dv) : a.out + (long long)(tbase + t0) * ostep + (long long)h * a.dv + c;
        if constexpr (RP <= 8) {
            // two tokens per pass of the loop, no branch inside: the slots behind a batch's last token hold a token that changes nothing (decay one, the rest zero),
            // so both register sets are always loaded and walked, and only the stores look at the token's number
            TokVec<RP, DELTA> x0, x1;
            load_tok(0, x0);
            for (int tb = 0; tb < nb; tb += 2) {
                load_tok(tb + 1, x1);
                const float oa = step(x0);
                load_tok(tb + 2, x0);
                const float ob = step(x1);
                const float ra = group_sum<SPLIT>(oa), rb = group_sum<SPLIT>(ob);
                if (rg == 0 && col_ok) {
                    orow[tb * ostep] = ra;
                    if (tb + 1 < nb) orow[(tb + 1) * ostep] = rb;
                }
            }
        } else {
            for (int tb = 0; tb < nb; ++tb) {
                TokVec<RP, DELTA> cur;
                load_tok(tb, cur);
                const float o = group_sum<SPLIT>(step(cur));
                if (rg == 0 && col_ok) orow[tb * ostep] = o;
            }
        }
    }
    // ---- what the walk leaves: the sequence's state, or with several segments the segment's own end state and its whole transition
    float* end = st;
    long long estep = a.dv;
    if (a.nseg > 1) {
        if (aug) { end = a.pbuf + (((long long)sg * a.H + h) * a.dn) * a.dn + (c - a.dv); estep = a.dn; }
        else end = a.lbuf + (((long long)sg * a.H + h) * a.dn) * a.dv + c;
    }
#pragma unroll
    for (int i = 0; i < RP; ++i) {
        const int r = rg * RP + i;
        if (col_ok && r < a.dn) end[r * estep] = S[i];
    }
}

// Without the removal term a segment's transition is diagonal: P_t = diag(B_t), B_t the running product of the segment's decays per channel.  A thread
// per (segment, head, channel) walks its tokens (sixteen tokens' loads in flight at a time): r_t = q_t * B_t, and the segment's whole product at the end.
__global__ __launch_bounds__(64) void recurrence_cumdecay_kernel(const RecArgs a) {
    const int d = blockIdx.x * 64 + threadIdx.x, h = blockIdx.y, g = blockIdx.z;
    if (d >= a.dn) return;
    const int t0 = g * a.seg_len, t1 = min(a.T, t0 + a.seg_len);
    float B = 1.0f;
    for (int t = t0; t < t1; t += 16) {
        float w[16], q[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const float* src = a.packed + (((long long)min(t + j, t1 - 1) * a.H + h) * 3) * a.dn + d;
            q[j] = src[0];
            w[j] = src[2 * a.dn];
        }
#pragma unroll
        for (int j = 0; j < 16; ++j)
            if (t + j < t1) { B *= w[j]; a.rbuf[((long long)(t + j) * a.H + h) * a.dn + d] = q[j] * B; }
    }
    a.pbuf[((long long)g * a.H + h) * a.dn + d] = B;
}

// The states at the segments' starts, one after the other: x(1) = what segment 0 left (it started from the sequence's state), x(g + 1) = P(g) x(g) + L(g).
// A workgroup owns 16 columns of one head: lane = (column, one of 4 row groups), wave = 4 more row groups, a thread the rows of its group (every 16th);
// x and the segment's P in LDS; the NEXT segment's P and L are requested into registers (PFN floats of P per thread) while the current product runs, so a
// step waits for its own arithmetic only.  DIAG: P is a vector (no removal term).
template <bool DIAG, int PFN>
__global__ __launch_bounds__(256) void recurrence_chain_kernel(const RecArgs a) {
    extern __shared__ __attribute__((aligned(16))) float cl_[];
    const int DS = ((a.dn + 3) & ~3) + 4;                // floats per row of P in LDS
    float* x0 = cl_;                                     // [dn][16]
    float* x1 = x0 + a.dn * 16;
    float* Pl = x1 + a.dn * 16;                          // [dn][DS]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, h = blockIdx.y;
    const int cc = lane & 15, rgrp = wave * 4 + (lane >> 4), c = blockIdx.x * 16 + cc;
    const bool ok = c < a.dv;
    const long long hs = (long long)a.dn * a.dv;
    for (int r = rgrp; r < a.dn; r += 16) x0[r * 16 + cc] = ok ? a.lbuf[(long long)h * hs + (long long)r * a.dv + c] : 0.0f;
    float pn[PFN], ln[8];
    auto request = [&](int g) {
        const float* P = a.pbuf + ((long long)g * a.H + h) * a.dn * a.dn;
        const float* L = a.lbuf + ((long long)g * a.H + h) * hs;
#pragma unroll
        for (int u = 0; u < PFN; ++u) { const int e = threadIdx.x + 256 * u; pn[u] = e < a.dn * a.dn ? P[e] : 0.0f; }
#pragma unroll
        for (int j = 0; j < 8; ++j) { const int r = rgrp + 16 * j; ln[j] = (ok && r < a.dn) ? L[(long long)r * a.dv + c] : 0.0f; }
    };
    if constexpr (!DIAG) { if (a.nseg > 1) request(1); }
    for (int g = 1; g < a.nseg; ++g) {
        const float* L = a.lbuf + ((long long)g * a.H + h) * hs;
        float* Sg = a.sbuf + ((long long)g * a.H + h) * hs;
        if constexpr (DIAG) {
            const float* Pd = a.pbuf + ((long long)g * a.H + h) * a.dn;
            for (int r = rgrp; r < a.dn; r += 16) {      // (a thread's own entries only: no barrier between the segments)
                const float cur = x0[r * 16 + cc];
                if (ok) Sg[(long long)r * a.dv + c] = cur;
                x0[r * 16 + cc] = fmaf(Pd[r], cur, ok ? L[(long long)r * a.dv + c] : 0.0f);
            }
        } else {
            __syncthreads();                             // the previous segment's readers of Pl and x1 are done
            float lv[8];
#pragma unroll
            for (int u = 0; u < PFN; ++u) { const int e = threadIdx.x + 256 * u; if (e < a.dn * a.dn) Pl[(e / a.dn) * DS + e % a.dn] = pn[u]; }
#pragma unroll
            for (int j = 0; j < 8; ++j) lv[j] = ln[j];
            if (g + 1 < a.nseg) request(g + 1);
            if (DS - 4 > a.dn)
                for (int r = threadIdx.x; r < a.dn; r += 256)
                    for (int k = a.dn; k < DS - 4; ++k) Pl[r * DS + k] = 0.0f;
            __syncthreads();
            float acc[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
            for (int k = 0; k < a.dn; k += 4) {          // (entries of P past dn are zero, x is read below dn only)
                const float xa = x0[k * 16 + cc], xb = k + 1 < a.dn ? x0[(k + 1) * 16 + cc] : 0.0f, xc = k + 2 < a.dn ? x0[(k + 2) * 16 + cc] : 0.0f,
                            xd = k + 3 < a.dn ? x0[(k + 3) * 16 + cc] : 0.0f;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int r = rgrp + 16 * j;
                    if (r < a.dn) {
                        const float4 p4 = *reinterpret_cast<const float4*>(Pl + r * DS + k);
                        acc[j] = fmaf(p4.x, xa, acc[j]); acc[j] = fmaf(p4.y, xb, acc[j]); acc[j] = fmaf(p4.z, xc, acc[j]); acc[j] = fmaf(p4.w, xd, acc[j]);
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int r = rgrp + 16 * j;
                if (r < a.dn) {
                    if (ok) Sg[(long long)r * a.dv + c] = x0[r * 16 + cc];
                    x1[r * 16 + cc] = acc[j] + lv[j];
                }
            }
            float* t = x0; x0 = x1; x1 = t;
        }
    }
    if constexpr (!DIAG) __syncthreads();
    for (int r = rgrp; r < a.dn; r += 16)
        if (ok) a.state[(long long)h * hs + (long long)r * a.dv + c] = x0[r * 16 + cc];
}

// out[t] += S(g)^T r[t] for the tokens of segments g >= 1: a workgroup owns 16 tokens of one head (r rows in LDS), lane = column, wave = 4 tokens
__global__ __launch_bounds__(256) void recurrence_owed_kernel(const RecArgs a) {
    extern __shared__ float rs[];                        // [16][dn]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, h = blockIdx.y;
    const int g = 1 + blockIdx.x / ((a.seg_len + 15) / 16), tile = blockIdx.x % ((a.seg_len + 15) / 16);
    const int t0 = g * a.seg_len + tile * 16, tend = min(a.T, (g + 1) * a.seg_len);
    if (t0 >= tend) return;                              // (uniform over the workgroup)
    for (int e = threadIdx.x; e < 16 * a.dn; e += 256) {
        const int t = t0 + e / a.dn;
        rs[e] = t < tend ? a.rbuf[((long long)t * a.H + h) * a.dn + e % a.dn] : 0.0f;
    }
    __syncthreads();
    const float* Sg = a.sbuf + ((long long)g * a.H + h) * a.dn * a.dv;
    const float* r4 = rs + wave * 4 * a.dn;
    for (int c = lane; c < a.dv; c += 64) {
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int k = 0; k < a.dn; ++k) {
            const float sv = Sg[(long long)k * a.dv + c];
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = fmaf(r4[j * a.dn + k], sv, acc[j]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int t = t0 + wave * 4 + j;
            if (t < tend) a.out[(long long)t * a.ldo + (long long)h * a.dv + c] += acc[j];
        }
    }
}

template <int SPLIT, int RP, int NW>
static int launch_rec_waves(const RecArgs& a0, hipStream_t s) {
    RecArgs a = a0;
    constexpr int CB = NW * (64 / SPLIT), DP = SPLIT * RP, DL = SPLIT * (RP + 4), NT = 64 * NW;
    const bool delta = a.az != nullptr;
    const int NV = delta ? 5 : 3, extra = RP <= 8 ? 2 : 0;
    int tb = (NT * rec_pf(NW)) / DP;                     // what a thread's registers carry
    tb = std::min(tb, (2 * NT) / CB);                    // ... and of the values
    tb = std::min(tb, 16);
    tb = std::min(tb, (int)(40 * 1024 / ((NV * DL + CB) * sizeof(float))) - extra);   // a batch's LDS stays under 40 KB: several workgroups per CU
    tb = std::min(tb, std::max(a.T, 1));
    a.TB = std::max(tb, 1);
    const size_t lds = (size_t)(a.TB + extra) * (NV * DL + CB) * sizeof(float);
    const int ncols = (delta && a.nseg > 1) ? a.dv + a.dn : a.dv;
    const dim3 grid((ncols + CB - 1) / CB, a.H, a.nseg);
    if (a.packed) {
        if (a.conv_w) {
            const dim3 pgrid(a.G > 0 ? a.G : a.H);
            if (delta) hipLaunchKernelGGL(gated_recurrence_prepare_step_kernel<true>, pgrid, dim3(256), (size_t)2 * a.dn * sizeof(float), s, a);
            else hipLaunchKernelGGL(gated_recurrence_prepare_step_kernel<false>, pgrid, dim3(256), (size_t)2 * a.dn * sizeof(float), s, a);
        } else if (delta) hipLaunchKernelGGL(gated_recurrence_prepare_kernel<true>, dim3(a.T * a.H), dim3(64), 0, s, a);
        else hipLaunchKernelGGL(gated_recurrence_prepare_kernel<false>, dim3(a.T * a.H), dim3(64), 0, s, a);
        const int st = last_launch_status();
        if (st != NTK_OK) return st;
        if (a.vpacked) { a.v = a.vpacked; a.ldv = a.H * a.dv; }
        if (delta) hipLaunchKernelGGL((gated_recurrence_kernel<SPLIT, RP, true, true, NW>), grid, dim3(NT), lds, s, a);
        else hipLaunchKernelGGL((gated_recurrence_kernel<SPLIT, RP, false, true, NW>), grid, dim3(NT), lds, s, a);
        if (a.nseg == 1) return last_launch_status();
        const dim3 cgrid((a.dv + 15) / 16, a.H);
        if (delta) {
            const size_t clds = ((size_t)2 * a.dn * 16 + (size_t)a.dn * (((a.dn + 3) & ~3) + 4)) * sizeof(float);
            static bool raised = false;   // (idempotent: a race sets the same attribute twice)
            if (!raised) {
                NTK_HIP_TRY(hipFuncSetAttribute((const void*)recurrence_chain_kernel<false, 64>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
                raised = true;
            }
            if (a.dn <= 64) hipLaunchKernelGGL((recurrence_chain_kernel<false, 16>), cgrid, dim3(256), clds, s, a);
            else hipLaunchKernelGGL((recurrence_chain_kernel<false, 64>), cgrid, dim3(256), clds, s, a);
        } else {
            hipLaunchKernelGGL(recurrence_cumdecay_kernel, dim3((a.dn + 63) / 64, a.H, a.nseg), dim3(64), 0, s, a);
            hipLaunchKernelGGL((recurrence_chain_kernel<true, 1>), cgrid, dim3(256), (size_t)2 * a.dn * 16 * sizeof(float), s, a);
        }
        const int tiles = (a.seg_len + 15) / 16;
        hipLaunchKernelGGL(recurrence_owed_kernel, dim3((a.nseg - 1) * tiles, a.H), dim3(256), (size_t)16 * a.dn * sizeof(float), s, a);
        return last_launch_status();
    }
    if (delta) hipLaunchKernelGGL((gated_recurrence_kernel<SPLIT, RP, true, false, NW>), grid, dim3(NT), lds, s, a);
    else hipLaunchKernelGGL((gated_recurrence_kernel<SPLIT, RP, false, false, NW>), grid, dim3(NT), lds, s, a);
    return last_launch_status();
}

// waves per workgroup: four share a head's staged vectors while that still leaves a workgroup per CU; fewer (down to one) where the columns are few, so
// that the walk -- one chain per column, nothing to gain from a second wave on the same column -- spreads over the chip
template <int SPLIT, int RP>
static int launch_rec(const RecArgs& a, hipStream_t s) {
    const long long col_groups = (long long)a.H * ((((a.az && a.nseg > 1) ? a.dv + a.dn : a.dv) + 64 / SPLIT - 1) / (64 / SPLIT)) * a.nseg;   // waves of the launch
    if (col_groups >= 4 * 256) return launch_rec_waves<SPLIT, RP, 4>(a, s);
    if (col_groups >= 2 * 256) return launch_rec_waves<SPLIT, RP, 2>(a, s);
    return launch_rec_waves<SPLIT, RP, 1>(a, s);
}

}  // namespace ntk

using namespace ntk;

// segments of a portion: at least kRecSegTokens tokens each, at most kRecMaxSegs; channels beyond 128 stay in one segment (the transition of a segment
// is a dn x dn matrix per head)
// ... and no more segments than fill the chip a few waves deep: beyond that the walk is bound by what it issues, not by its chain, and the extra columns
// and the settling launches only cost
constexpr int kRecSegTokens = 64, kRecMaxSegs = 16, kRecWaves = 2048;
static int rec_segments(int T, int H, int dn, int dv, bool removal) {
    if (dn > 128 || dv > 1024) return 1;
    const long long waves = ((long long)H * (dv + (removal ? dn : 0)) + 3) / 4;        // of one segment, 16 lanes per column
    const int by_chip = (int)std::max<long long>(1, kRecWaves / std::max<long long>(waves, 1));
    return std::max(1, std::min(std::min(kRecMaxSegs, by_chip), T / kRecSegTokens));
}

// any of the per-head options: the vectors are always formed by the pre-pass
static bool rec_needs_prepass(const ntk_gated_recurrence_desc* d) {
    return d->G > 0 || d->unit_q || d->unit_k || d->head_gates || d->write_gated || d->decay_rates || d->decay_form == NTK_DECAY_EXP_SOFTPLUS || d->conv_w;
}

static size_t rec_scratch(int T, int H, int dn, int dv, bool removal, bool always, bool values) {
    if (T <= kRecFewTokens && !always) return 0;
    size_t n = (size_t)T * H * (removal ? 5 : 3) * dn + (values ? (size_t)T * H * dv : 0);
    const int ns = rec_segments(T, H, dn, dv, removal);
    if (ns > 1) n += (size_t)T * H * dn + (size_t)ns * H * dn * dn + 2 * (size_t)ns * H * dn * dv;
    return n;
}

size_t ntk_gated_recurrence_scratch(int T, int H, int dn, int dv, int removal) { return rec_scratch(T, H, dn, dv, removal != 0, false, false); }

size_t ntk_gated_recurrence_scratch_ex(const ntk_gated_recurrence_desc* d) {
    if (!d || d->T <= 0 || d->H <= 0 || d->dn <= 0 || d->dv <= 0) return 0;
    return rec_scratch(d->T, d->H, d->dn, d->dv, d->az != nullptr, rec_needs_prepass(d), d->write_gated != 0 || d->conv_w != nullptr);
}

int ntk_gated_recurrence(const ntk_gated_recurrence_desc* d, void* stream) {
    if (!d || !d->out || !d->q || !d->k || !d->v || !d->wz || !d->state) return NTK_E_NULL;
    if (d->T < 0 || d->H <= 0 || d->dn <= 0 || d->dv <= 0 || d->pos0 < 0 || d->dn > 1024) return NTK_E_SHAPE;
    if (d->decay_form != NTK_DECAY_GIVEN && d->decay_form != NTK_DECAY_SIGMOID_ROOT && d->decay_form != NTK_DECAY_EXP_SIGMOID && d->decay_form != NTK_DECAY_EXP_SOFTPLUS)
        return NTK_E_SHAPE;
    if (d->decay_form == NTK_DECAY_SIGMOID_ROOT && !(d->decay_param > 0.0f)) return NTK_E_SHAPE;
    if (d->G < 0 || (d->G > 0 && d->H % d->G)) return NTK_E_SHAPE;
    if (d->write_gated && (!d->az || !d->head_gates)) return NTK_E_SHAPE;   // (the write is scaled by ONE rate per head)
    if (d->conv_w && (d->T != 1 || d->conv_taps < 1 || d->conv_taps > kStepConvTaps || (d->conv_taps > 1 && !d->conv_state))) return NTK_E_SHAPE;
    const int hd = d->H * d->dn, qd = (d->G > 0 ? d->G : d->H) * d->dn, gd = d->head_gates ? d->H : hd;
    if (d->ldq < qd || d->ldk < qd || d->ldw < gd || (d->az && d->lda < gd) || d->ldv < d->H * d->dv || d->ldo < d->H * d->dv) return NTK_E_SHAPE;
    if (d->T == 0) return NTK_OK;
    const bool always = rec_needs_prepass(d);
    if (always && !d->scratch) return NTK_E_NULL;
    RecArgs a{d->out, d->ldo, d->q, d->ldq, d->k, d->ldk, d->v, d->ldv, d->wz, d->ldw, d->wb, d->decay_form, d->decay_param, d->az, d->lda, d->ab, d->unit_eps,
              d->state, d->H, d->dn, d->dv, d->q_scale, d->pos0, d->T, 0, (d->T > kRecFewTokens || always) ? d->scratch : nullptr, 1, d->T, nullptr, nullptr, nullptr, nullptr,
              d->G, d->unit_q, d->unit_k, d->head_gates, d->write_gated, d->decay_rates, nullptr, d->conv_w, d->conv_state, d->conv_taps};
    if (a.packed) {
        float* next = a.packed + (size_t)d->T * d->H * (d->az ? 5 : 3) * d->dn;
        if (d->write_gated || d->conv_w) { a.vpacked = next; next += (size_t)d->T * d->H * d->dv; }
        a.nseg = rec_segments(d->T, d->H, d->dn, d->dv, d->az != nullptr);
        if (a.nseg > 1) {
            a.seg_len = (d->T + a.nseg - 1) / a.nseg;
            a.nseg = (d->T + a.seg_len - 1) / a.seg_len;
            a.rbuf = next;
            a.pbuf = a.rbuf + (size_t)d->T * d->H * d->dn;
            a.lbuf = a.pbuf + (size_t)a.nseg * d->H * d->dn * d->dn;
            a.sbuf = a.lbuf + (size_t)a.nseg * d->H * d->dn * d->dv;
        }
    }
    hipStream_t s = resolve_stream(stream);
    // 16 lanes share a column (their sums meet in DPP steps inside a 16-lane row, no trip through LDS on the chain from token to token); rows per lane: the
    // smallest of 4 / 8 / 16 / 32 that covers the head's channels; beyond 512 channels 32 lanes per column.
    if (d->dn <= 16 * 4) return launch_rec<16, 4>(a, s);
    if (d->dn <= 16 * 8) return launch_rec<16, 8>(a, s);
    if (d->dn <= 16 * 16) return launch_rec<16, 16>(a, s);
    if (d->dn <= 16 * 32) return launch_rec<16, 32>(a, s);
    return launch_rec<32, 32>(a, s);
}
