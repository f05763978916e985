// window_attention.hip -- grouped-query softmax attention over a cache of rotated keys and values: causal, optional sliding window, one or two score
// maps per head over the same values (two maps: the differential pair out = a_0 - lambda * a_1), optional unit norm of every head's output, optional
// learned bias by bucketed distance on the scaled score (a table of distances -> buckets, a table of buckets x heads), optional cap on the score
// (cap * tanh(score / cap)), optional sink (a key of score 0 without a value in every softmax), and instead of the sliding window a mask of chunks
// (a query sees the keys of its own chunk of `window` positions, counted from position 0, up to itself).
//
// Cache row of a position: [G][maps][dn] rotated keys | [G][dv] values, F32.  Scores, softmax, weights and sums are F32 on the vector units.
// A workgroup owns 16 (token, head) rows of ONE key/value head -- consecutive tokens times the heads that share it, so a key or value slab that was
// staged in LDS serves every query head of the group -- and walks the visible keys in chunks of 64: lane = key for the scores (key slabs of 64 entries
// in LDS), online softmax per row and map, lane = value column for the weighted sums (the value slab is loaded once for both maps).  When few rows
// face many keys (decoding), the chunks go round `splits` workgroups and a second launch merges their (max, sum, vector) states.
#include <algorithm>
#include "common.hip.h"
#include "../../include/ntk_layers.h"

namespace ntk {

// one workgroup per token: q rotated in place, k rotated into the cache row, v copied behind.  Angles in double (position times frequency), applied in F32.
// Optional: what the projections left to their consumer -- bias vectors on q, k and v, and a query temperature that grows with the position.
__global__ __launch_bounds__(256) void window_prepare_kernel(float* cache, int row, float* q, int ldq, const float* k, int ldk, const float* v, int ldv, int nq, int nk,
                                                             int dn, int nv, const double* freq, float mag, int dims, int pos0, const float* qb, const float* kb,
                                                             const float* vb, float temp_coef, double temp_every, int halves, const float* v_other, int ld_other,
                                                             float v_blend, float* v_keep, int ld_keep) {
    extern __shared__ float cs[];   // [dims / 2] cos, [dims / 2] sin
    const int t = blockIdx.x, pos = pos0 + t;
    const int half = dims / 2;
    if (qb || temp_coef != 0.0f) {     // (uniform over the launch) q = (q + bias) * temperature, ahead of the rotation: a thread rewrites its own entries
        float* qt0 = q + (long long)t * ldq;
        const float temp = temp_coef != 0.0f ? 1.0f + temp_coef * logf((float)floor((double)(pos + 1) / temp_every) + 1.0f) : 1.0f;
        for (int j = threadIdx.x; j < nq * dn; j += 256) qt0[j] = (qt0[j] + (qb ? qb[j] : 0.0f)) * temp;
        __syncthreads();
    }
    for (int i = threadIdx.x; i < half; i += 256) {
        const double a = (double)pos * freq[i];
        cs[i] = (float)(cos(a) * (double)mag);
        cs[half + i] = (float)(sin(a) * (double)mag);
    }
    __syncthreads();
    float* dst = cache + (long long)pos * row;
    float* qt = q + (long long)t * ldq;
    const float* kt = k + (long long)t * ldk;
    const float* vt = v + (long long)t * ldv;
    const int pair = halves ? half : 1, step = halves ? 1 : 2;   // pair i = entries (i * step, i * step + pair)
    for (int j = threadIdx.x; j < nq * half; j += 256) {       // nq = heads x maps vectors of dn
        float* p = qt + (j / half) * dn + step * (j % half);
        float ra, rb;
        rope_rotate(p[0], p[pair], cs[j % half], cs[half + j % half], ra, rb);
        p[0] = ra;
        p[pair] = rb;
    }
    for (int j = threadIdx.x; j < nk * half; j += 256) {
        const int o = (j / half) * dn + step * (j % half);
        float ra, rb;
        rope_rotate(kt[o] + (kb ? kb[o] : 0.0f), kt[o + pair] + (kb ? kb[o + pair] : 0.0f), cs[j % half], cs[half + j % half], ra, rb);
        dst[o] = ra;
        dst[o + pair] = rb;
    }
    const int rest = dn - dims;
    for (int j = threadIdx.x; j < nk * rest; j += 256) {
        const int o = (j / rest) * dn + dims + j % rest;
        dst[o] = kt[o] + (kb ? kb[o] : 0.0f);
    }
    for (int j = threadIdx.x; j < nv; j += 256) {
        float vv = vt[j] + (vb ? vb[j] : 0.0f);
        if (v_keep) v_keep[(long long)t * ld_keep + j] = vv;
        if (v_other) vv = fmaf(v_blend, v_other[(long long)t * ld_other + j], (1.0f - v_blend) * vv);
        dst[nk * dn + j] = vv;
    }
}

struct WinArgs {
    float* out; int ldo;
    const float* q; int ldq;
    const float* cache; int row;
    int H, G, dn, dv, pos0, T, window;
    float scale, lambda;
    int sub_norm; float eps, out_scale;
    int splits; float* scratch;       // splits > 1: states [T * H][splits][maps][2 + dv]
    const float* rel; const int* bucket_of; int n_dist;   // rel != NULL: rel[bucket_of[min(distance, n_dist - 1)] * H + head] joins the scaled score
    int chunks; float softcap; int sink;                  // chunks != 0: `window` is a chunk size
    const float* gate; int ldg;                           // gate != NULL: out[t][h][c] *= sigmoid(gate[t * ldg + h * dv + c])
};

// first key a query at position p sees
__device__ __forceinline__ int first_visible(int p, int window, int chunks) {
    if (window <= 0) return 0;
    return chunks ? (p / window) * window : max(0, p - window + 1);
}

constexpr int WROWS = 16, WQPW = 4, WKCH = 64, WSLAB = 64, WMAXC = 8;   // dv <= WMAXC * WSLAB

// the differential pair, the unit norm and the scale on a row whose lanes hold columns c * 64 + lane
template <int M>
__device__ __forceinline__ void finish_row(float (&a)[M][WMAXC], int lane, int dv, float lambda, int sub_norm, float eps, float out_scale, float* o, const float* gate) {
    float r[WMAXC];
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < WMAXC; ++c) {
        float x = a[0][c];
        if constexpr (M == 2) x = x - lambda * a[1][c];
        if (c * WSLAB + lane >= dv) x = 0.0f;
        r[c] = x;
        ss = fmaf(x, x, ss);
    }
    float mul = out_scale;
    if (sub_norm) mul = out_scale / sqrtf(wave_sum(ss) / (float)dv + eps);
#pragma unroll
    for (int c = 0; c < WMAXC; ++c)
        if (c * WSLAB + lane < dv) o[c * WSLAB + lane] = gate ? r[c] * mul / (1.0f + expf(-gate[c * WSLAB + lane])) : r[c] * mul;
}

template <int M>
__global__ __launch_bounds__(256) void window_attention_kernel(const WinArgs a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int DNP = (a.dn + 3) & ~3;
    float* Qs = lds;                               // [WROWS][M][DNP]
    float* Sl = Qs + WROWS * M * DNP;              // [WKCH][WSLAB + 1] key slab / [WKCH][WSLAB] value slab
    float* Ps = Sl + WKCH * (WSLAB + 1);           // [M][WROWS][WKCH]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = blockIdx.y, R = a.H / a.G, n_rows = a.T * R;
    const int row0 = blockIdx.x * WROWS;
    const int last = min(row0 + WROWS, n_rows) - 1;
    const int pmin = a.pos0 + row0 / R, pmax = a.pos0 + last / R;
    const int jlo = first_visible(pmin, a.window, a.chunks);
    const int jhi = pmax;   // inclusive
    // queries into LDS
    for (int e0 = threadIdx.x; e0 < WROWS * M * DNP; e0 += 256 * 4) {     // (four of a thread's entries asked for before the first is stored)
        float qv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int e = e0 + 256 * u, i = e / (M * DNP), md = e % (M * DNP), m = md / DNP, d = md % DNP;
            const int rho = row0 + i;
            qv[u] = (e < WROWS * M * DNP && rho < n_rows && d < a.dn) ? a.q[(long long)(rho / R) * a.ldq + ((long long)(g * R + rho % R) * M + m) * a.dn + d] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (e0 + 256 * u < WROWS * M * DNP) Qs[e0 + 256 * u] = qv[u];
    }
    float mx[M][WQPW], l[M][WQPW], acc[M][WQPW][WMAXC];
    int rpos[WQPW], rhead[WQPW];
#pragma unroll
    for (int i = 0; i < WQPW; ++i) {
        const int rho = row0 + wave * WQPW + i;
        rpos[i] = rho < n_rows ? a.pos0 + rho / R : -1;
        rhead[i] = g * R + rho % R;
        // the sink is a key of score 0 without a value: the running maximum and sum start from it (in the first part only when the keys are split)
        const bool sunk = a.sink && (a.splits <= 1 || blockIdx.z == 0);
#pragma unroll
        for (int m = 0; m < M; ++m) {
            mx[m][i] = sunk ? 0.0f : -INFINITY; l[m][i] = sunk ? 1.0f : 0.0f;
#pragma unroll
            for (int c = 0; c < WMAXC; ++c) acc[m][i][c] = 0.0f;
        }
    }
    const int vbase = a.G * M * a.dn + g * a.dv;
    int chunk = 0;
    for (int j0 = jlo; j0 <= jhi; j0 += WKCH, ++chunk) {
        if (a.splits > 1 && chunk % a.splits != (int)blockIdx.z) continue;     // (uniform over the workgroup)
        const int nk = min(WKCH, jhi + 1 - j0);
        const int j = j0 + lane;
#pragma unroll
        for (int m = 0; m < M; ++m) {
            float s[WQPW];
#pragma unroll
            for (int i = 0; i < WQPW; ++i) s[i] = 0.0f;
            // ---- scores of map m: slabs of WSLAB key entries
            for (int d0 = 0; d0 < a.dn; d0 += WSLAB) {
                const int nd = min(WSLAB, a.dn - d0);
                __syncthreads();
                {   // thread -> (key wave + 4 u, entry lane): the sixteen requests of a thread in flight before the first is stored
                    const float* src = a.cache + (long long)j0 * a.row + (g * M + m) * a.dn + d0 + lane;
                    float v[16];
#pragma unroll
                    for (int u = 0; u < 16; ++u) {
                        const int k = wave + 4 * u;
                        v[u] = (k < nk && lane < nd) ? src[(long long)k * a.row] : 0.0f;
                    }
#pragma unroll
                    for (int u = 0; u < 16; ++u) Sl[(wave + 4 * u) * (WSLAB + 1) + lane] = v[u];
                }
                __syncthreads();
                const float* kr = Sl + lane * (WSLAB + 1);
                for (int d = 0; d < nd; d += 4) {      // (entries past nd are zero in the slab, past dn in the queries)
                    const float k0 = kr[d], k1 = kr[d + 1], k2 = kr[d + 2], k3 = kr[d + 3];
#pragma unroll
                    for (int i = 0; i < WQPW; ++i) {
                        const float4 q4 = *reinterpret_cast<const float4*>(Qs + ((wave * WQPW + i) * M + m) * DNP + d0 + d);
                        s[i] = fmaf(q4.x, k0, s[i]); s[i] = fmaf(q4.y, k1, s[i]); s[i] = fmaf(q4.z, k2, s[i]); s[i] = fmaf(q4.w, k3, s[i]);
                    }
                }
            }
            // ---- online softmax of map m, weights to LDS
#pragma unroll
            for (int i = 0; i < WQPW; ++i) {
                const bool vis = lane < nk && rpos[i] >= 0 && j <= rpos[i] && j >= first_visible(rpos[i], a.window, a.chunks);
                float sv = vis ? s[i] * a.scale : -INFINITY;
                if (a.rel && vis) sv += a.rel[(long long)a.bucket_of[min(rpos[i] - j, a.n_dist - 1)] * a.H + rhead[i]];
                if (a.softcap > 0.0f && vis) sv = a.softcap * tanhf(sv / a.softcap);
                const float mn = fmaxf(mx[m][i], wave_max(sv));
                const float ms = mn == -INFINITY ? 0.0f : mn;
                const float p = vis ? expf(sv - ms) : 0.0f;
                const float corr = mx[m][i] == -INFINITY ? 0.0f : expf(mx[m][i] - ms);
                l[m][i] = l[m][i] * corr + wave_sum(p);
                mx[m][i] = mn;
#pragma unroll
                for (int c = 0; c < WMAXC; ++c) acc[m][i][c] *= corr;
                Ps[(m * WROWS + wave * WQPW + i) * WKCH + lane] = p;
            }
        }
        // ---- weighted sums: slabs of WSLAB value columns, lane = column, one slab for all maps
#pragma unroll
        for (int c = 0; c < WMAXC; ++c) {
            const int v0 = c * WSLAB;
            if (v0 < a.dv) {
                const int nvv = min(WSLAB, a.dv - v0);
                __syncthreads();
                {
                    const float* src = a.cache + (long long)j0 * a.row + vbase + v0 + lane;
                    float v[16];
#pragma unroll
                    for (int u = 0; u < 16; ++u) {
                        const int k = wave + 4 * u;
                        v[u] = (k < nk && lane < nvv) ? src[(long long)k * a.row] : 0.0f;
                    }
#pragma unroll
                    for (int u = 0; u < 16; ++u) Sl[(wave + 4 * u) * WSLAB + lane] = v[u];
                }
                __syncthreads();
                for (int k = 0; k < nk; k += 4) {      // (weights and value rows past nk are zero)
                    const float x0 = Sl[k * WSLAB + lane], x1 = Sl[(k + 1) * WSLAB + lane], x2 = Sl[(k + 2) * WSLAB + lane], x3 = Sl[(k + 3) * WSLAB + lane];
#pragma unroll
                    for (int m = 0; m < M; ++m)
#pragma unroll
                        for (int i = 0; i < WQPW; ++i) {
                            const float4 p4 = *reinterpret_cast<const float4*>(Ps + (m * WROWS + wave * WQPW + i) * WKCH + k);
                            acc[m][i][c] = fmaf(p4.x, x0, acc[m][i][c]); acc[m][i][c] = fmaf(p4.y, x1, acc[m][i][c]);
                            acc[m][i][c] = fmaf(p4.z, x2, acc[m][i][c]); acc[m][i][c] = fmaf(p4.w, x3, acc[m][i][c]);
                        }
                }
            }
        }
    }
    // ---- results
#pragma unroll
    for (int i = 0; i < WQPW; ++i) {
        const int rho = row0 + wave * WQPW + i;
        if (rho >= n_rows) continue;
        const int t = rho / R, h = g * R + rho % R;
        if (a.splits > 1) {
#pragma unroll
            for (int m = 0; m < M; ++m) {
                float* st = a.scratch + ((((long long)t * a.H + h) * a.splits + blockIdx.z) * M + m) * (2 + a.dv);
                if (lane == 0) { st[0] = mx[m][i]; st[1] = l[m][i]; }
#pragma unroll
                for (int c = 0; c < WMAXC; ++c)
                    if (c * WSLAB + lane < a.dv) st[2 + c * WSLAB + lane] = acc[m][i][c];
            }
            continue;
        }
        float r[M][WMAXC];
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const float inv = l[m][i] > 0.0f ? 1.0f / l[m][i] : 0.0f;
#pragma unroll
            for (int c = 0; c < WMAXC; ++c) r[m][c] = acc[m][i][c] * inv;
        }
        finish_row<M>(r, lane, a.dv, a.lambda, a.sub_norm, a.eps, a.out_scale, a.out + (long long)t * a.ldo + (long long)h * a.dv,
                      a.gate ? a.gate + (long long)t * a.ldg + (long long)h * a.dv : nullptr);
    }
}

// merge of the partial states of one (token, head) row, one wave per row: lane = part for the weights exp(max_s - max) and the sum (splits <= 64), then
// lane = column for the weighted vectors, the parts in order with their loads independent of each other
template <int M>
__global__ __launch_bounds__(64) void window_attention_merge_kernel(const WinArgs a) {
    const int lane = threadIdx.x, row = blockIdx.x;       // row = t * H + h
    float r[M][WMAXC];
#pragma unroll
    for (int m = 0; m < M; ++m) {
        const float* st = a.scratch + ((long long)row * a.splits * M + m) * (2 + a.dv);
        const long long step = (long long)M * (2 + a.dv);
        const float ms = lane < a.splits ? st[lane * step] : -INFINITY;
        const float ls = lane < a.splits ? st[lane * step + 1] : 0.0f;
        const float mm = wave_max(ms);
        const float w = ms == -INFINITY ? 0.0f : expf(ms - mm);
        const float L = wave_sum(w * ls);
#pragma unroll
        for (int c = 0; c < WMAXC; ++c) r[m][c] = 0.0f;
        const int nc = (a.dv + WSLAB - 1) / WSLAB;
        for (int s0 = 0; s0 < a.splits; s0 += 8) {       // eight parts' loads in flight before the first is used
            for (int c = 0; c < nc; ++c) {
                float x[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) x[u] = (s0 + u < a.splits && c * WSLAB + lane < a.dv) ? st[(s0 + u) * step + 2 + c * WSLAB + lane] : 0.0f;
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const float ws = __shfl(w, (s0 + u) & 63, 64);
#pragma unroll
                    for (int cc = 0; cc < WMAXC; ++cc)
                        if (cc == c) r[m][cc] = fmaf(ws, x[u], r[m][cc]);
                }
            }
        }
        const float inv = L > 0.0f ? 1.0f / L : 0.0f;
#pragma unroll
        for (int c = 0; c < WMAXC; ++c) r[m][c] *= inv;
    }
    finish_row<M>(r, lane, a.dv, a.lambda, a.sub_norm, a.eps, a.out_scale, a.out + (long long)(row / a.H) * a.ldo + (long long)(row % a.H) * a.dv,
                  a.gate ? a.gate + (long long)(row / a.H) * a.ldg + (long long)(row % a.H) * a.dv : nullptr);
}

// parts the key chunks of a row tile go round: only when few tiles face many chunks
static int window_splits(int T, int H, int G, int nkeys) {
    const int tiles = ((T * (H / G) + WROWS - 1) / WROWS) * G;
    const int chunks = (nkeys + WKCH - 1) / WKCH + 1;
    if (tiles >= 128 || chunks < 4) return 1;
    int s = 256 / tiles;
    if (s > chunks) s = chunks;
    if (s > 64) s = 64;
    return s < 2 ? 1 : s;
}
static int window_keys(int pos0, int T, int window, int chunks) {
    const int all = pos0 + T;
    if (chunks && window > 0) return all - (pos0 / window) * window;     // from the start of the first token's chunk
    return window > 0 && window + T - 1 < all ? window + T - 1 : all;
}

}  // namespace ntk

using namespace ntk;

int ntk_window_prepare(float* cache, int row, float* q, int ldq, const float* k, int ldk, const float* v, int ldv, int H, int G, int maps, int dn, int dv,
                       const ntk_rotary* rot, int pos0, int T, void* stream) {
    return ntk_window_prepare_biased(cache, row, q, ldq, k, ldk, v, ldv, H, G, maps, dn, dv, rot, nullptr, nullptr, nullptr, 0.0f, 1.0, pos0, T, stream);
}

int ntk_window_prepare_biased(float* cache, int row, float* q, int ldq, const float* k, int ldk, const float* v, int ldv, int H, int G, int maps, int dn, int dv,
                              const ntk_rotary* rot, const float* qb, const float* kb, const float* vb, float temp_coef, double temp_every, int pos0, int T,
                              void* stream) {
    ntk_window_prepare_desc d{};
    d.cache = cache; d.row = row; d.q = q; d.ldq = ldq; d.k = k; d.ldk = ldk; d.v = v; d.ldv = ldv; d.H = H; d.G = G; d.maps = maps; d.dn = dn; d.dv = dv; d.rot = rot;
    d.qb = qb; d.kb = kb; d.vb = vb; d.temp_coef = temp_coef; d.temp_every = temp_every; d.pos0 = pos0; d.T = T;
    return ntk_window_prepare_ex(&d, stream);
}

int ntk_window_prepare_ex(const ntk_window_prepare_desc* d, void* stream) {
    if (!d || !d->cache || !d->q || !d->k || !d->v || !d->rot || (d->rot->dims > 0 && !d->rot->freq)) return NTK_E_NULL;
    const ntk_rotary* rot = d->rot;
    if (d->temp_coef != 0.0f && !(d->temp_every > 0.0)) return NTK_E_SHAPE;
    if (d->T < 0 || d->H <= 0 || d->G <= 0 || d->H % d->G || d->maps < 1 || d->dn <= 0 || d->dv <= 0 || d->pos0 < 0) return NTK_E_SHAPE;
    if (rot->dims < 0 || (rot->dims & 1) || rot->dims > d->dn || (rot->layout != NTK_ROT_NEIGHBOURS && rot->layout != NTK_ROT_HALVES)) return NTK_E_SHAPE;
    if (d->row < d->G * (d->maps * d->dn + d->dv) || d->ldq < d->H * d->maps * d->dn || d->ldk < d->G * d->maps * d->dn || d->ldv < d->G * d->dv) return NTK_E_SHAPE;
    if ((d->v_other && d->ld_other < d->G * d->dv) || (d->v_keep && d->ld_keep < d->G * d->dv)) return NTK_E_SHAPE;
    if (d->T == 0) return NTK_OK;
    hipLaunchKernelGGL(window_prepare_kernel, dim3(d->T), dim3(256), (size_t)(rot->dims + 2) * sizeof(float), resolve_stream(stream), d->cache, d->row, d->q, d->ldq,
                       d->k, d->ldk, d->v, d->ldv, d->H * d->maps, d->G * d->maps, d->dn, d->G * d->dv, rot->freq, rot->mag, rot->dims, d->pos0, d->qb, d->kb, d->vb,
                       d->temp_coef, d->temp_every, rot->layout == NTK_ROT_HALVES ? 1 : 0, d->v_other, d->ld_other, d->v_blend, d->v_keep, d->ld_keep);
    return last_launch_status();
}

size_t ntk_window_attention_scratch(int T, int H, int maps, int dv, int nkeys) {
    // rows x splits <= 16 x 256: a launch is only split while it has fewer than 128 row tiles, into at most 256 / tiles (and 64) parts
    const size_t states = std::min<size_t>((size_t)T * H * 64, 4096);
    return nkeys > 0 ? states * maps * (2 + dv) : 0;
}

int ntk_window_attention(const ntk_window_attention_desc* d, void* stream) {
    if (!d || !d->out || !d->q || !d->cache) return NTK_E_NULL;
    if (d->T < 0 || d->H <= 0 || d->G <= 0 || d->H % d->G || d->dn <= 0 || d->dv <= 0 || d->pos0 < 0) return NTK_E_SHAPE;
    if (d->maps != 1 && d->maps != 2) return NTK_E_SHAPE;
    if (d->dv > WMAXC * WSLAB) return NTK_E_SHAPE;
    if (d->row < d->G * (d->maps * d->dn + d->dv) || d->ldq < d->H * d->maps * d->dn || d->ldo < d->H * d->dv) return NTK_E_SHAPE;
    if (d->T == 0) return NTK_OK;
    WinArgs a{};
    a.out = d->out; a.ldo = d->ldo; a.q = d->q; a.ldq = d->ldq; a.cache = d->cache; a.row = d->row; a.H = d->H; a.G = d->G; a.dn = d->dn; a.dv = d->dv;
    a.pos0 = d->pos0; a.T = d->T; a.window = d->window; a.scale = d->scale; a.lambda = d->lambda; a.sub_norm = d->sub_norm; a.eps = d->eps; a.out_scale = d->out_scale;
    if ((d->mask_mode != NTK_MASK_SLIDING && d->mask_mode != NTK_MASK_CHUNKS) || d->softcap < 0.0f) return NTK_E_SHAPE;
    a.chunks = d->mask_mode == NTK_MASK_CHUNKS; a.softcap = d->softcap; a.sink = d->sink;
    if (d->gate && d->ldg < d->H * d->dv) return NTK_E_SHAPE;
    a.gate = d->gate; a.ldg = d->ldg;
    a.splits = d->scratch ? window_splits(d->T, d->H, d->G, window_keys(d->pos0, d->T, d->window, a.chunks)) : 1;
    a.scratch = d->scratch;
    a.rel = d->rel; a.bucket_of = d->bucket_of; a.n_dist = d->n_dist;
    if (a.rel && (!a.bucket_of || a.n_dist <= 0)) return NTK_E_NULL;
    const int DNP = (d->dn + 3) & ~3;
    const size_t lds = ((size_t)WROWS * d->maps * DNP + WKCH * (WSLAB + 1) + (size_t)d->maps * WROWS * WKCH) * sizeof(float);
    if (lds > 150 * 1024) return NTK_E_SHAPE;
    hipStream_t s = resolve_stream(stream);
    const dim3 grid((d->T * (d->H / d->G) + WROWS - 1) / WROWS, d->G, a.splits);
    if (lds > 48 * 1024) {
        static bool raised = false;   // (idempotent: a race sets the same attribute twice)
        if (!raised) {
            NTK_HIP_TRY(hipFuncSetAttribute((const void*)window_attention_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024));
            NTK_HIP_TRY(hipFuncSetAttribute((const void*)window_attention_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024));
            raised = true;
        }
    }
    if (d->maps == 1) hipLaunchKernelGGL(window_attention_kernel<1>, grid, dim3(256), lds, s, a);
    else hipLaunchKernelGGL(window_attention_kernel<2>, grid, dim3(256), lds, s, a);
    int st = last_launch_status();
    if (st != NTK_OK || a.splits == 1) return st;
    if (d->maps == 1) hipLaunchKernelGGL(window_attention_merge_kernel<1>, dim3(d->T * d->H), dim3(64), 0, s, a);
    else hipLaunchKernelGGL(window_attention_merge_kernel<2>, dim3(d->T * d->H), dim3(64), 0, s, a);
    return last_launch_status();
}
