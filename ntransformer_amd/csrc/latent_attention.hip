// latent_attention.hip -- attention over a cache of one normed latent and one rotated key part per position.
//
// What is cached per position and layer run is [latent c (kv_rank) | rotated key part (rot_dim)], F32.  Two ways to the same sums:
//   * expanded (prompt portions): the caller up-projects the cached latents of the visible range into per-head keys and values (two products over
//     the cache rows) and the kernel runs ordinary multi-head attention on them, reading the shared rotated part from the cache rows;
//   * shared (few query tokens, decoding): the query's unrotated part is folded through the key up-projection first (ntk_latent_fold_query), so every
//     head scores against the cache rows themselves, [c | rotated] . [folded q | rotated q]; the weighted sum is taken over c and the value
//     up-projection is applied once afterwards (ntk_latent_unfold_value).  Nothing per head is ever materialised for the cached positions.
// Expanded: a workgroup owns 16 tokens of one head and walks the visible keys in chunks of 64 -- lane = key for the scores (key slabs of 64 entries in
// LDS), online softmax per row in F32, lane = value column for the weighted sum.  Shared: a workgroup owns 16 (token, head) rows and whole tiles of 32
// cache rows; the tiles go round up to 128 workgroups and a second launch merges their (max, sum, vector) states.
#include "common.hip.h"
#include "../../include/ntk_layers.h"

namespace ntk {

// ------------------------------------------------------------------------------------------------------------------- cache rows and rotation
// one workgroup per token: latent / rms * w and the rotated key part into the cache row, the rotated part of every query head in place.
// Angles in double (position times frequency, then cos / sin), applied in F32.
__global__ __launch_bounds__(256) void latent_prepare_kernel(float* cache, int row, const float* kv, int ldkv, const float* norm_w, float eps, int R, int dr,
                                                             float* q, int ldq, int H, int qd, const double* freq, float mag, int dims, int pos0, int halves) {
    __shared__ float red[16];
    extern __shared__ float cs[];   // [dims / 2] cos, [dims / 2] sin
    const int t = blockIdx.x, pos = pos0 + t;
    const float* src = kv + (long long)t * ldkv;
    float* dst = cache + (long long)pos * row;
    const int half = dims / 2;   // dims <= dr: what lies behind the rotated entries passes unchanged
    for (int i = threadIdx.x; i < half; i += 256) {
        const double a = (double)pos * freq[i];
        cs[i] = (float)(cos(a) * (double)mag);
        cs[half + i] = (float)(sin(a) * (double)mag);
    }
    float ss = 0.0f;
    for (int i = threadIdx.x; i < R; i += 256) ss = fmaf(src[i], src[i], ss);
    ss = block_sum(ss, red);   // (its barriers also publish cs)
    const float inv = 1.0f / sqrtf(ss / (float)R + eps);
    for (int i = threadIdx.x; i < R; i += 256) dst[i] = src[i] * inv * norm_w[i];
    const int pair = halves ? half : 1, step = halves ? 1 : 2;   // pair i = entries (i * step, i * step + pair)
    for (int i = threadIdx.x; i < half; i += 256) {
        float ra, rb;
        rope_rotate(src[R + step * i], src[R + step * i + pair], cs[i], cs[half + i], ra, rb);
        dst[R + step * i] = ra;
        dst[R + step * i + pair] = rb;
    }
    for (int i = dims + threadIdx.x; i < dr; i += 256) dst[R + i] = src[R + i];
    if (q) {
        float* qt = q + (long long)t * ldq;
        for (int j = threadIdx.x; j < H * half; j += 256) {
            const int h = j / half, i = j % half;
            float* p = qt + h * qd + (qd - dr) + step * i;
            float ra, rb;
            rope_rotate(p[0], p[pair], cs[i], cs[half + i], ra, rb);
            p[0] = ra;
            p[pair] = rb;
        }
    }
}

// ------------------------------------------------------------------------------------------------------------------- the attention kernel
struct AttnArgs {
    float* out; int ldo;              // per token
    const float* q; int ldq;          // per token; head h at h * DK
    const float* kA; long long ldA; int nA; int hA;   // first part of a key: kA + (j - keyA0) * ldA + h * hA, nA entries
    const float* kB; long long ldB; int nB;           // second part: kB + j * ldB, nB entries (the rotated part inside the cache row)
    const float* v; long long ldV; int nV; int hV;    // value: v + (j - keyA0) * ldV + h * hV
    int keyA0;
    int H, pos0, T, window;
    float scale;
};

constexpr int QROWS = 16, QPW = 4, KCH = 64, SLAB = 64;

__global__ __launch_bounds__(256) void latent_attention_kernel(const AttnArgs a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int DK = a.nA + a.nB;
    const int DKP = (DK + 3) & ~3;
    float* Qs = lds;                               // [QROWS][DKP]
    float* Sl = Qs + QROWS * DKP;                  // [KCH][SLAB + 1] key slab / [KCH][SLAB] value slab
    float* Ps = Sl + KCH * (SLAB + 1);             // [QROWS][KCH]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // rows of this workgroup
    const int head = blockIdx.y, n_rows_total = a.T;   // rows = the tokens of this portion, for one head
    const int row0 = blockIdx.x * QROWS;
    auto row_token = [&](int i) { return row0 + i; };
    auto row_head = [&](int) { return head; };
    const int last_row = min(row0 + QROWS, n_rows_total) - 1;
    const int pmin = a.pos0 + row0;
    const int pmax = a.pos0 + last_row;
    const int jlo = a.window > 0 ? max(0, pmin - a.window + 1) : 0;
    const int jhi = pmax;   // inclusive
    // queries into LDS
    for (int d = threadIdx.x; d < DKP; d += 256) {
        float qv[QROWS];
#pragma unroll
        for (int i = 0; i < QROWS; ++i) qv[i] = (row0 + i < n_rows_total && d < DK) ? a.q[(long long)row_token(i) * a.ldq + (long long)row_head(i) * DK + d] : 0.0f;
#pragma unroll
        for (int i = 0; i < QROWS; ++i) Qs[i * DKP + d] = qv[i];
    }
    float m[QPW], l[QPW], acc[QPW][8];
    int rpos[QPW];
#pragma unroll
    for (int i = 0; i < QPW; ++i) {
        m[i] = -INFINITY; l[i] = 0.0f;
        const int ri = wave * QPW + i;
        rpos[i] = row0 + ri < n_rows_total ? a.pos0 + row_token(ri) : -1;
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[i][c] = 0.0f;
    }
    const int hk = head;
    for (int j0 = jlo; j0 <= jhi; j0 += KCH) {
        const int nk = min(KCH, jhi + 1 - j0);
        float s[QPW];
#pragma unroll
        for (int i = 0; i < QPW; ++i) s[i] = 0.0f;
        // ---- scores: slabs of SLAB key entries
        for (int d0 = 0; d0 < DK; d0 += SLAB) {
            const int nd = min(SLAB, DK - d0);
            __syncthreads();
            {   // thread -> (key wave + 4 u, entry lane): the sixteen requests of a thread in flight before the first is stored
                const int d = lane, dd = d0 + d;
                const bool first = dd < a.nA;
                const float* src = first ? a.kA + (long long)(j0 - a.keyA0) * a.ldA + (long long)hk * a.hA + dd : a.kB + (long long)j0 * a.ldB + (dd - a.nA);
                const long long ld = first ? a.ldA : a.ldB;
                float v[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    const int k = wave + 4 * u;
                    v[u] = (k < nk && d < nd) ? src[k * ld] : 0.0f;
                }
#pragma unroll
                for (int u = 0; u < 16; ++u) Sl[(wave + 4 * u) * (SLAB + 1) + d] = v[u];
            }
            __syncthreads();
            const float* kr = Sl + lane * (SLAB + 1);
            for (int d = 0; d < nd; d += 4) {      // (entries past nd are zero in the slab, past DK in the queries)
                const float k0 = kr[d], k1 = kr[d + 1], k2 = kr[d + 2], k3 = kr[d + 3];
#pragma unroll
                for (int i = 0; i < QPW; ++i) {
                    const float4 q4 = *reinterpret_cast<const float4*>(Qs + (wave * QPW + i) * DKP + d0 + d);
                    s[i] = fmaf(q4.x, k0, s[i]); s[i] = fmaf(q4.y, k1, s[i]); s[i] = fmaf(q4.z, k2, s[i]); s[i] = fmaf(q4.w, k3, s[i]);
                }
            }
        }
        // ---- online softmax, weights to LDS
        const int j = j0 + lane;
#pragma unroll
        for (int i = 0; i < QPW; ++i) {
            const bool vis = lane < nk && rpos[i] >= 0 && j <= rpos[i] && (a.window <= 0 || rpos[i] - j < a.window);
            const float sv = vis ? s[i] * a.scale : -INFINITY;
            const float mn = fmaxf(m[i], wave_max(sv));
            const float ms = mn == -INFINITY ? 0.0f : mn;
            const float p = vis ? expf(sv - ms) : 0.0f;
            const float corr = m[i] == -INFINITY ? 0.0f : expf(m[i] - ms);
            l[i] = l[i] * corr + wave_sum(p);
            m[i] = mn;
#pragma unroll
            for (int c = 0; c < 8; ++c) acc[i][c] *= corr;
            Ps[(wave * QPW + i) * KCH + lane] = p;
        }
        // ---- weighted sum: slabs of SLAB value columns, lane = column
        const int hv = head;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const int v0 = c * SLAB;
            if (v0 < a.nV) {
                const int nvv = min(SLAB, a.nV - v0);
                __syncthreads();
                {
                    const float* src = a.v + (long long)(j0 - a.keyA0) * a.ldV + (long long)hv * a.hV + v0 + lane;
                    float v[16];
#pragma unroll
                    for (int u = 0; u < 16; ++u) {
                        const int k = wave + 4 * u;
                        v[u] = (k < nk && lane < nvv) ? src[k * a.ldV] : 0.0f;
                    }
#pragma unroll
                    for (int u = 0; u < 16; ++u) Sl[(wave + 4 * u) * SLAB + lane] = v[u];
                }
                __syncthreads();
                for (int k = 0; k < nk; k += 4) {      // (weights and value rows past nk are zero)
                    const float x0 = Sl[k * SLAB + lane], x1 = Sl[(k + 1) * SLAB + lane], x2 = Sl[(k + 2) * SLAB + lane], x3 = Sl[(k + 3) * SLAB + lane];
#pragma unroll
                    for (int i = 0; i < QPW; ++i) {
                        const float4 p4 = *reinterpret_cast<const float4*>(Ps + (wave * QPW + i) * KCH + k);
                        acc[i][c] = fmaf(p4.x, x0, acc[i][c]); acc[i][c] = fmaf(p4.y, x1, acc[i][c]);
                        acc[i][c] = fmaf(p4.z, x2, acc[i][c]); acc[i][c] = fmaf(p4.w, x3, acc[i][c]);
                    }
                }
            }
        }
    }
    // ---- results
#pragma unroll
    for (int i = 0; i < QPW; ++i) {
        const int ri = wave * QPW + i;
        if (row0 + ri >= n_rows_total) continue;
        const int t = row_token(ri), h = row_head(ri);
        const float inv = l[i] > 0.0f ? 1.0f / l[i] : 0.0f;
        float* o = a.out + (long long)t * a.ldo + (long long)h * a.nV;
#pragma unroll
        for (int c = 0; c < 8; ++c)
            if (c * SLAB + lane < a.nV) o[c * SLAB + lane] = acc[i][c] * inv;
    }
}

// ------------------------------------------------------------------------------------------------------------------- the shared form (decoding)
// Keys and values are the cache rows themselves, so a workgroup loads a tile of KB = 32 rows [latent | rotated] ONCE (all requests in flight together) and
// uses it for every (token, head) row of its tile of 16: thread (key, row pair) forms two scores over the whole row, sixteen threads run the online softmax
// of their row, then thread r sums the weighted latents column r of all 16 rows.  The tiles of 32 keys go round `splits` workgroups; each leaves one
// (max, sum, vector) state per row and latent_attention_merge_kernel adds them.
constexpr int KB = 32, SROWS = 16;
struct SharedArgs {
    const float* q; int ldq;          // [T][H][R + dr], ldq floats between tokens
    const float* cache; int row;      // cache rows
    int R, dr, H, pos0, T, window, splits;
    float scale;
    float* scratch;                   // [rows][splits][2 + R]
};

__global__ __launch_bounds__(256) void latent_attention_shared_kernel(const SharedArgs a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int DK = a.R + a.dr;
    const int DKP = ((DK + 3) & ~3) + 4;           // rows 16-byte aligned, 4 banks apart
    float* Ks = lds;                               // [KB][DKP]
    float* Qs = Ks + KB * DKP;                     // [SROWS][DKP]
    float* Ps = Qs + SROWS * DKP;                  // [SROWS][KB]
    float* ms = Ps + SROWS * KB;                   // [SROWS] running max
    float* ls = ms + SROWS;                        // [SROWS] running sum
    float* cr = ls + SROWS;                        // [SROWS] correction of this tile
    const int tid = threadIdx.x;
    const int n_rows = a.T * a.H, row0 = blockIdx.x * SROWS;
    const int last_row = min(row0 + SROWS, n_rows) - 1;
    const int pmin = a.pos0 + row0 / a.H, pmax = a.pos0 + last_row / a.H;
    const int jlo = a.window > 0 ? max(0, pmin - a.window + 1) : 0, jhi = pmax;
    for (int d = tid; d < DKP; d += 256) {          // the 16 query rows: all requests of a pass in flight before the first is stored
        float qv[SROWS];
#pragma unroll
        for (int i = 0; i < SROWS; ++i) {
            const int r = row0 + i;
            qv[i] = (r < n_rows && d < DK) ? a.q[(long long)(r / a.H) * a.ldq + (long long)(r % a.H) * DK + d] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < SROWS; ++i) Qs[i * DKP + d] = qv[i];
    }
    if (tid < SROWS) { ms[tid] = -INFINITY; ls[tid] = 0.0f; }
    const int lane = tid & 63, wave = tid >> 6;
    const int key = tid % KB, rg = tid / KB;       // scores: rows 2 rg, 2 rg + 1
    const int rpos0 = row0 + 2 * rg < n_rows ? a.pos0 + (row0 + 2 * rg) / a.H : -1;
    const int rpos1 = row0 + 2 * rg + 1 < n_rows ? a.pos0 + (row0 + 2 * rg + 1) / a.H : -1;
    constexpr int RC = 2;                          // latent columns per thread: R <= 512
    float acc[RC][SROWS];
#pragma unroll
    for (int c = 0; c < RC; ++c)
#pragma unroll
        for (int i = 0; i < SROWS; ++i) acc[c][i] = 0.0f;
    const bool vec4 = (DK % 4 == 0) && (a.row % 4 == 0) && !((uintptr_t)a.cache & 15);
    int tile = 0;
    for (int j0 = jlo; j0 <= jhi; j0 += KB, ++tile) {
        if (tile % a.splits != (int)blockIdx.y) continue;
        const int nk = min(KB, jhi + 1 - j0);
        __syncthreads();                           // the previous tile is used up (and Qs / ms are written)
        if (vec4) {                                // 16 bytes per request, eight requests of a thread in flight before the first is stored
            const int q4 = DK / 4, total = KB * q4, dk = 256 / q4, dc = 256 % q4;
            int k = tid / q4, c = tid % q4;
            for (int base = tid; base < total; base += 256 * 8) {
                float4 v[8];
                int at[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    at[u] = k * DKP + 4 * c;
                    v[u] = float4{0.f, 0.f, 0.f, 0.f};
                    if (base + 256 * u < total && k < nk) v[u] = *reinterpret_cast<const float4*>(a.cache + (long long)(j0 + k) * a.row + 4 * c);
                    c += dc; k += dk;
                    if (c >= q4) { c -= q4; ++k; }
                }
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (base + 256 * u < total) *reinterpret_cast<float4*>(Ks + at[u]) = v[u];
            }
        } else {
            for (int k = wave; k < KB; k += 4)
                for (int d = lane; d < DKP; d += 64) Ks[k * DKP + d] = (k < nk && d < DK) ? a.cache[(long long)(j0 + k) * a.row + d] : 0.0f;
        }
        __syncthreads();
        // ---- scores
        float s0 = 0.0f, s1 = 0.0f;
        const float* kr = Ks + key * DKP;
        const float* qa = Qs + (2 * rg) * DKP;
        const float* qb = qa + DKP;
        for (int d = 0; d < DK; d += 4) {          // (entries past DK are zero on both sides)
            const float4 kv = *reinterpret_cast<const float4*>(kr + d), xa = *reinterpret_cast<const float4*>(qa + d), xb = *reinterpret_cast<const float4*>(qb + d);
            s0 = fmaf(xa.x, kv.x, s0); s0 = fmaf(xa.y, kv.y, s0); s0 = fmaf(xa.z, kv.z, s0); s0 = fmaf(xa.w, kv.w, s0);
            s1 = fmaf(xb.x, kv.x, s1); s1 = fmaf(xb.y, kv.y, s1); s1 = fmaf(xb.z, kv.z, s1); s1 = fmaf(xb.w, kv.w, s1);
        }
        const int j = j0 + key;
        const bool v0 = key < nk && rpos0 >= 0 && j <= rpos0 && (a.window <= 0 || rpos0 - j < a.window);
        const bool v1 = key < nk && rpos1 >= 0 && j <= rpos1 && (a.window <= 0 || rpos1 - j < a.window);
        Ps[(2 * rg) * KB + key] = v0 ? s0 * a.scale : -INFINITY;
        Ps[(2 * rg + 1) * KB + key] = v1 ? s1 * a.scale : -INFINITY;
        __syncthreads();
        // ---- online softmax: 16 lanes per row, two keys each
        {
            const int row = tid >> 4, sub = tid & 15;
            float* p = Ps + row * KB;
            const float a0 = p[sub], a1 = p[sub + 16];
            float mc = fmaxf(a0, a1);
#pragma unroll
            for (int o = 8; o >= 1; o >>= 1) mc = fmaxf(mc, __shfl_xor(mc, o, 16));
            const float mo = ms[row];
            const float mn = fmaxf(mo, mc), msafe = mn == -INFINITY ? 0.0f : mn;
            const float e0 = a0 == -INFINITY ? 0.0f : expf(a0 - msafe), e1 = a1 == -INFINITY ? 0.0f : expf(a1 - msafe);
            float sum = e0 + e1;
#pragma unroll
            for (int o = 8; o >= 1; o >>= 1) sum += __shfl_xor(sum, o, 16);
            p[sub] = e0;
            p[sub + 16] = e1;
            __syncthreads();                       // every lane has read ms[row]
            if (sub == 0) {
                const float corr = mo == -INFINITY ? 0.0f : expf(mo - msafe);
                ls[row] = ls[row] * corr + sum;
                ms[row] = mn;
                cr[row] = corr;
            }
        }
        __syncthreads();
        // ---- weighted latents: thread -> column tid (+ 256)
#pragma unroll
        for (int c = 0; c < RC; ++c) {
            const int r = tid + 256 * c;
            if (r < a.R) {
#pragma unroll
                for (int i = 0; i < SROWS; ++i) acc[c][i] *= cr[i];
                for (int k = 0; k < KB; k += 4) {
                    const float x0 = Ks[(k + 0) * DKP + r], x1 = Ks[(k + 1) * DKP + r], x2 = Ks[(k + 2) * DKP + r], x3 = Ks[(k + 3) * DKP + r];
#pragma unroll
                    for (int i = 0; i < SROWS; ++i) {
                        const float4 p4 = *reinterpret_cast<const float4*>(Ps + i * KB + k);
                        acc[c][i] = fmaf(p4.x, x0, acc[c][i]); acc[c][i] = fmaf(p4.y, x1, acc[c][i]);
                        acc[c][i] = fmaf(p4.z, x2, acc[c][i]); acc[c][i] = fmaf(p4.w, x3, acc[c][i]);
                    }
                }
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < SROWS; ++i) {              // (unrolled: the sums stay in registers)
        if (row0 + i < n_rows) {
            float* st = a.scratch + ((long long)(row0 + i) * a.splits + blockIdx.y) * (2 + a.R);
            if (tid == 0) { st[0] = ms[i]; st[1] = ls[i]; }
#pragma unroll
            for (int c = 0; c < RC; ++c)
                if (tid + 256 * c < a.R) st[2 + tid + 256 * c] = acc[c][i];
        }
    }
}

// merge of the partial states of one (token, head) row: weights of the states first, then every thread sums its columns over the states
__global__ __launch_bounds__(256) void latent_attention_merge_kernel(float* out, int ldo, const float* scratch, int splits, int nV, int H) {
    __shared__ float wt[256];
    __shared__ float red[16];
    const int r = blockIdx.x;   // r = t * H + h
    const float* st = scratch + (long long)r * splits * (2 + nV);
    float mx = -INFINITY;
    for (int s = threadIdx.x; s < splits; s += 256) mx = fmaxf(mx, st[(long long)s * (2 + nV)]);
    mx = block_max(mx, red);
    float den = 0.0f;
    for (int s = threadIdx.x; s < splits; s += 256) {
        const float m = st[(long long)s * (2 + nV)];
        const float w = m == -INFINITY ? 0.0f : expf(m - mx);
        wt[s] = w;
        den += w * st[(long long)s * (2 + nV) + 1];
    }
    den = block_sum(den, red);   // (its barriers publish wt)
    const float inv = den > 0.0f ? 1.0f / den : 0.0f;
    float* o = out + (long long)(r / H) * ldo + (long long)(r % H) * nV;
    for (int v = threadIdx.x; v < nV; v += 256) {
        float s2 = 0.0f;
        int s = 0;
        for (; s + 8 <= splits; s += 8) {          // eight states requested together, added in order
            float x[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) x[u] = st[(long long)(s + u) * (2 + nV) + 2 + v];
#pragma unroll
            for (int u = 0; u < 8; ++u) s2 = fmaf(x[u], wt[s + u], s2);
        }
        for (; s < splits; ++s) s2 = fmaf(st[(long long)s * (2 + nV) + 2 + v], wt[s], s2);
        o[v] = s2 * inv;
    }
}

// ------------------------------------------------------------------------------------------------------------------- fold / unfold
// qf[t][h][r] = sum_d q[t][h][d] W_uk[h * dn + d][r]; rotated part copied behind.  grid (R / 64, H, T): 64 columns per workgroup, the d range in
// four parts (one per wave), added through LDS in wave order
template <typename WT>
__global__ __launch_bounds__(256) void latent_fold_query_kernel(float* qf, const float* q, int ldq, const WT* w, int H, int dn, int dr, int R) {
    extern __shared__ float qs[];      // [dn + dr] then [4][64] partial sums
    float* part = qs + dn + dr;
    const int h = blockIdx.y, t = blockIdx.z;
    const float* qh = q + (long long)t * ldq + (long long)h * (dn + dr);
    float* o = qf + ((long long)t * H + h) * (R + dr);
    for (int d = threadIdx.x; d < dn + dr; d += 256) qs[d] = qh[d];
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = blockIdx.x * 64 + lane;
    const int per = (dn + 3) / 4, d0 = wave * per, d1 = min(d0 + per, dn);
    const WT* wh = w + (long long)h * dn * R;
    float s = 0.0f;
    if (r < R) {
#pragma unroll 8
        for (int d = d0; d < d1; ++d) {
            float wv;
            if constexpr (sizeof(WT) == 2) wv = __uint_as_float((uint32_t)wh[(long long)d * R + r] << 16); else wv = wh[(long long)d * R + r];
            s = fmaf(qs[d], wv, s);
        }
    }
    part[wave * 64 + lane] = s;
    __syncthreads();
    if (wave == 0 && r < R) o[r] = ((part[lane] + part[64 + lane]) + part[128 + lane]) + part[192 + lane];
    if (blockIdx.x == 0)
        for (int d = threadIdx.x; d < dr; d += 256) o[R + d] = qs[dn + d];
}

// out[t][h * dv + v] = W_uv[h * dv + v][:] . lat[t][h][:] (* sigmoid(gate));  grid (dv / 16, H, T): a wave owns 4 outputs and walks their rows together
template <typename WT>
__global__ __launch_bounds__(256) void latent_unfold_value_kernel(float* out, int ldo, const float* lat, const WT* w, const float* gate, int ldg, int H, int dv,
                                                                 int R, int head_gate) {
    extern __shared__ float ls[];
    const int h = blockIdx.y, t = blockIdx.z;
    const float* lh = lat + ((long long)t * H + h) * R;
    for (int r = threadIdx.x; r < R; r += 256) ls[r] = lh[r];
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int v0 = blockIdx.x * 16 + wave * 4;
    if (v0 >= dv) return;
    const WT* wr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) wr[i] = w + ((long long)h * dv + min(v0 + i, dv - 1)) * R;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    for (int r = lane; r < R; r += 64) {
        float wv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if constexpr (sizeof(WT) == 2) wv[i] = __uint_as_float((uint32_t)wr[i][r] << 16); else wv[i] = wr[i][r];
        }
        const float x = ls[r];
#pragma unroll
        for (int i = 0; i < 4; ++i) s[i] = fmaf(wv[i], x, s[i]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float tsum = wave_sum_lane63(s[i]);
        if (lane == 63 && v0 + i < dv) {
            if (gate) tsum *= 1.0f / (1.0f + expf(-gate[(long long)t * ldg + (head_gate ? h : h * dv + v0 + i)]));
            out[(long long)t * ldo + h * dv + v0 + i] = tsum;
        }
    }
}

static int shared_splits(int nkeys) {       // workgroups per row tile: one per tile of KB keys, at most 128
    const int tiles = (nkeys + KB - 1) / KB + 1;     // (+ 1: a tile's first key is the window's, not a multiple of KB)
    return tiles < 1 ? 1 : tiles > 128 ? 128 : tiles;
}

}  // namespace ntk

using namespace ntk;

int ntk_latent_prepare(float* cache, int row, const float* kv, int ldkv, const float* norm_w, float eps, int kv_rank, int rot_dim, float* q, int ldq, int H, int qd,
                       const ntk_rotary* rot, int pos0, int T, void* stream) {
    if (!cache || !kv || !norm_w || !rot || !rot->freq) return NTK_E_NULL;
    if (T < 0 || kv_rank <= 0 || rot_dim < 0 || rot->dims < 0 || (rot->dims & 1) || rot->dims > rot_dim || row < kv_rank + rot_dim || ldkv < kv_rank + rot_dim || pos0 < 0) return NTK_E_SHAPE;
    if (q && (H <= 0 || qd < rot_dim || ldq < H * qd)) return NTK_E_SHAPE;
    if (rot->layout != NTK_ROT_NEIGHBOURS && rot->layout != NTK_ROT_HALVES) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(latent_prepare_kernel, dim3(T), dim3(256), (size_t)(rot_dim + 2) * sizeof(float), resolve_stream(stream), cache, row, kv, ldkv, norm_w,
                       eps, kv_rank, rot_dim, q, ldq, H, qd, rot->freq, rot->mag, rot->dims, pos0, rot->layout == NTK_ROT_HALVES ? 1 : 0);
    return last_launch_status();
}

size_t ntk_latent_attention_scratch(int T, int H, int vdim_or_rank, int nkeys) {
    return (size_t)T * H * shared_splits(nkeys) * (2 + vdim_or_rank);
}

int ntk_latent_attention(float* out, int ldo, const float* q, int ldq, const float* K, int ldk, const float* V, int ldv, const float* cache, int row,
                         int kv_rank, int rot_dim, int H, int dn, int dv, int shared, int pos0, int T, int key0, int window, float scale, float* scratch,
                         void* stream) {
    if (!out || !q || !cache) return NTK_E_NULL;
    if (!shared && (!K || !V)) return NTK_E_NULL;
    if (T < 0 || H <= 0 || kv_rank <= 0 || rot_dim < 0 || pos0 < 0 || key0 < 0 || row < kv_rank + rot_dim) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipStream_t s = resolve_stream(stream);
    if (shared) {
        if (!scratch) return NTK_E_NULL;
        if (kv_rank > 512) return NTK_E_SHAPE;
        SharedArgs sa{};
        sa.q = q; sa.ldq = ldq; sa.cache = cache; sa.row = row; sa.R = kv_rank; sa.dr = rot_dim; sa.H = H; sa.pos0 = pos0; sa.T = T; sa.window = window;
        sa.scale = scale; sa.scratch = scratch;
        const int nkeys = window > 0 ? (window + T - 1 < pos0 + T ? window + T - 1 : pos0 + T) : pos0 + T;
        sa.splits = shared_splits(nkeys);
        const int rows = T * H, DKP = ((kv_rank + rot_dim + 3) & ~3) + 4;
        const size_t lds = ((size_t)(KB + SROWS) * DKP + SROWS * KB + 3 * SROWS) * sizeof(float);
        if (lds > 156 * 1024) return NTK_E_SHAPE;
        static bool raised_s = false;   // (idempotent: a race sets the same attribute twice)
        if (!raised_s) { NTK_HIP_TRY(hipFuncSetAttribute((const void*)latent_attention_shared_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024)); raised_s = true; }
        hipLaunchKernelGGL(latent_attention_shared_kernel, dim3((rows + SROWS - 1) / SROWS, sa.splits), dim3(256), lds, s, sa);
        int st = last_launch_status();
        if (st != NTK_OK) return st;
        hipLaunchKernelGGL(latent_attention_merge_kernel, dim3(rows), dim3(256), 0, s, out, ldo, (const float*)scratch, sa.splits, kv_rank, H);
        return last_launch_status();
    }
    if (dn <= 0 || dv <= 0) return NTK_E_SHAPE;
    AttnArgs a{};
    a.out = out; a.ldo = ldo; a.q = q; a.ldq = ldq;
    a.kB = cache + kv_rank; a.ldB = row; a.nB = rot_dim;
    a.H = H; a.pos0 = pos0; a.T = T; a.window = window; a.scale = scale;
    a.kA = K; a.ldA = ldk; a.nA = dn; a.hA = dn;
    a.v = V; a.ldV = ldv; a.nV = dv; a.hV = dv;
    a.keyA0 = key0;
    const int rows = T;
    if (a.nV > 8 * SLAB) return NTK_E_SHAPE;
    const int DKP = (a.nA + a.nB + 3) & ~3;
    const size_t lds = ((size_t)QROWS * DKP + KCH * (SLAB + 1) + QROWS * KCH) * sizeof(float);
    if (lds > 150 * 1024) return NTK_E_SHAPE;
    const dim3 grid((rows + QROWS - 1) / QROWS, H, 1);
    if (lds > 48 * 1024) {
        static bool raised = false;   // (idempotent: a race sets the same attribute twice)
        if (!raised) { NTK_HIP_TRY(hipFuncSetAttribute((const void*)latent_attention_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024)); raised = true; }
    }
    hipLaunchKernelGGL(latent_attention_kernel, grid, dim3(256), lds, s, a);
    return last_launch_status();
}

int ntk_latent_fold_query(float* qf, const float* q, int ldq, const void* w_uk, int wdtype, int T, int H, int dn, int dr, int R, void* stream) {
    if (!qf || !q || !w_uk) return NTK_E_NULL;
    if (T < 0 || H <= 0 || dn <= 0 || dr < 0 || R <= 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    const size_t lds = (size_t)(dn + dr + 256) * sizeof(float);
    const dim3 grid((R + 63) / 64, H, T);
    if (wdtype == NTK_DT_BF16) hipLaunchKernelGGL(latent_fold_query_kernel<uint16_t>, grid, dim3(256), lds, resolve_stream(stream), qf, q, ldq, (const uint16_t*)w_uk, H, dn, dr, R);
    else if (wdtype == NTK_DT_F32) hipLaunchKernelGGL(latent_fold_query_kernel<float>, grid, dim3(256), lds, resolve_stream(stream), qf, q, ldq, (const float*)w_uk, H, dn, dr, R);
    else return NTK_E_DTYPE;
    return last_launch_status();
}

int ntk_latent_unfold_value(float* out, int ldo, const float* lat, const void* w_uv, int wdtype, const float* gate, int ldg, int T, int H, int dv, int R,
                            void* stream) {
    return ntk_latent_unfold_value_ex(out, ldo, lat, w_uv, wdtype, gate, ldg, 0, T, H, dv, R, stream);
}

int ntk_latent_unfold_value_ex(float* out, int ldo, const float* lat, const void* w_uv, int wdtype, const float* gate, int ldg, int head_gate, int T, int H, int dv,
                               int R, void* stream) {
    if (!out || !lat || !w_uv) return NTK_E_NULL;
    if (T < 0 || H <= 0 || dv <= 0 || R <= 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    const size_t lds = (size_t)R * sizeof(float);
    const dim3 grid((dv + 15) / 16, H, T);
    if (wdtype == NTK_DT_BF16) hipLaunchKernelGGL(latent_unfold_value_kernel<uint16_t>, grid, dim3(256), lds, resolve_stream(stream), out, ldo, lat, (const uint16_t*)w_uv, gate, ldg, H, dv, R, head_gate);
    else if (wdtype == NTK_DT_F32) hipLaunchKernelGGL(latent_unfold_value_kernel<float>, grid, dim3(256), lds, resolve_stream(stream), out, ldo, lat, (const float*)w_uv, gate, ldg, H, dv, R, head_gate);
    else return NTK_E_DTYPE;
    return last_launch_status();
}
