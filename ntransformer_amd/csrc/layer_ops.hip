// layer_ops.hip -- the small F32 operators around the products of the layer-list families: dense embedding rows, RMS norms whose weight is stored
// plain or around zero (two outputs from one pass over x: the two norms of a parallel layer read the same residual row), layer norms with weight and
// bias (also added onto the stream), the short causal convolution that is added to a sublayer's input (with its carried inputs), the polynomial
// activation with unit-norm terms, the gated RMS norm, row concatenation, sigmoid gates, the residual sum.  Everything is F32; one workgroup per row
// where a row is reduced.
#include "common.hip.h"
#include "../../include/ntk_layers.h"

namespace ntk {

template <typename TT>
__global__ __launch_bounds__(256) void embed_dense_kernel(float* out, const TT* table, const int* tokens, int vocab, int width, float scale) {
    const int t = blockIdx.x, tok = tokens[t];
    float* o = out + (long long)t * width;
    const bool ok = tok >= 0 && tok < vocab;
    const TT* row = table + (long long)(ok ? tok : 0) * width;
    for (int i = threadIdx.x; i < width; i += 256) {
        float v = 0.0f;
        if (ok) {
            if constexpr (sizeof(TT) == 2) v = __uint_as_float((uint32_t)row[i] << 16); else v = row[i];
        }
        o[i] = v * scale;
    }
}

__global__ __launch_bounds__(256) void rmsnorm_offset_kernel(float* y1, const float* w1, float* y2, const float* w2, int ldy, const float* x, int ldx, int n,
                                                             float eps, float offset) {
    __shared__ float red[16];
    const float* xr = x + (long long)blockIdx.x * ldx;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < n; i += 256) ss = fmaf(xr[i], xr[i], ss);
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    float* o1 = y1 + (long long)blockIdx.x * ldy;
    float* o2 = y2 ? y2 + (long long)blockIdx.x * ldy : nullptr;
    for (int i = threadIdx.x; i < n; i += 256) {
        const float u = xr[i] * inv;
        o1[i] = u * (offset + w1[i]);
        if (o2) o2[i] = u * (offset + w2[i]);
    }
}

__global__ void concat_rows_kernel(float* out, const float* a, const float* b, int n) {
    const long long t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= 2 * n) return;
    out[t * 2 * n + i] = i < n ? a[t * n + i] : b[t * n + (i - n)];
}

__global__ void sigmoid_gate_kernel(float* y, int ldy, const float* g, int ldg, int n) {
    const long long t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    y[t * ldy + i] *= 1.0f / (1.0f + expf(-g[t * ldg + i]));
}

__global__ void rows_copy_kernel(float* dst, const float* src, long long n) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

__global__ void residual_add_kernel(float* x, const float* a, const float* b, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float s = a[i];
    if (b) s += b[i];
    x[i] += s;
}

__global__ void scale_kernel(float* x, long long n, float s) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] *= s;
}

// mean first, then the mean of the squared deviations, then the outputs.  A thread keeps its first LN_KEEP entries (i = tid + 256 k) in registers -- rows up to
// 4096 wide are read once --; what lies beyond is read again (it sits in the cache).  Returns through (mean, inv); `emit(i, normed value)` writes.
// Workgroups of NT threads: 256 where a launch has many rows, 1024 where it has few (decoding: a row's entries are then spread over four times the threads,
// whose loads are in flight together -- a thread's own entries follow each other through load, use and store).
template <int NT, typename Emit>
__device__ __forceinline__ void layernorm_row(const float* xr, const float* w, const float* b, int n, float eps, float* red, Emit emit) {
    constexpr int KEEP = 4096 / NT;
    float v[KEEP], wv[KEEP], bv[KEEP];
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
        const int i = threadIdx.x + NT * k;
        v[k] = i < n ? xr[i] : 0.0f;
        wv[k] = i < n ? w[i] : 0.0f;
        bv[k] = i < n && b ? b[i] : 0.0f;
        s += v[k];
    }
    for (int i = threadIdx.x + NT * KEEP; i < n; i += NT) s += xr[i];
    const float mean = block_sum(s, red) / (float)n;
    float q = 0.0f;
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
        const float d = v[k] - mean;
        if ((int)threadIdx.x + NT * k < n) q = fmaf(d, d, q);
    }
    for (int i = threadIdx.x + NT * KEEP; i < n; i += NT) { const float d = xr[i] - mean; q = fmaf(d, d, q); }
    const float inv = 1.0f / sqrtf(block_sum(q, red) / (float)n + eps);
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
        const int i = threadIdx.x + NT * k;
        if (i < n) emit(i, (v[k] - mean) * inv * wv[k] + bv[k]);
    }
    for (int i = threadIdx.x + NT * KEEP; i < n; i += NT) emit(i, (xr[i] - mean) * inv * w[i] + (b ? b[i] : 0.0f));
}

template <int NT>
__global__ __launch_bounds__(NT) void layernorm_kernel(float* y, int ldy, const float* x, int ldx, const float* w, const float* b, int n, float eps, int accumulate) {
    __shared__ float red[16];
    float* yr = y + (long long)blockIdx.x * ldy;
    if (accumulate) layernorm_row<NT>(x + (long long)blockIdx.x * ldx, w, b, n, eps, red, [&](int i, float o) { yr[i] += o; });
    else layernorm_row<NT>(x + (long long)blockIdx.x * ldx, w, b, n, eps, red, [&](int i, float o) { yr[i] = o; });
}

// rows 0 .. taps-2: the carried inputs (zeros before the sequence's start); rows taps-1 ..: the layer norm of the portion's tokens.  With add_y the stream row
// first takes the sublayer output that is still owed to it, x[t] += layer norm of add_y[t] (weights add_w / add_b): the norm after one sublayer and the norm
// before the next in one pass over the row (a thread reads back only what it wrote itself).
__global__ __launch_bounds__(256) void layernorm_history_kernel(float* hist, float* x, int ldx, const float* w, const float* b, const float* state, int taps,
                                                                int pos0, int n, float eps, const float* add_y, int ldy, const float* add_w, const float* add_b) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    float* o = hist + (long long)r * n;
    if (r < taps - 1) {
        const bool before = pos0 - (taps - 1) + r < 0;
        for (int i = threadIdx.x; i < n; i += 256) o[i] = before ? 0.0f : state[(long long)r * n + i];
        return;
    }
    float* xr = x + (long long)(r - (taps - 1)) * ldx;
    if (add_y) layernorm_row<256>(add_y + (long long)(r - (taps - 1)) * ldy, add_w, add_b, n, eps, red, [&](int i, float v) { xr[i] += v; });
    layernorm_row<256>(xr, w, b, n, eps, red, [&](int i, float v) { o[i] = v; });
}

// one token (decoding), one workgroup: the owed sublayer output onto the stream, the norm, the convolution over the carried inputs and their shift -- every
// channel's history belongs to the thread that owns the channel.  Same sums in the same order as the two launches of a longer portion.
constexpr int kStepThreads = 1024;
__global__ __launch_bounds__(kStepThreads) void sandwich_step_kernel(float* out, float* x, const float* w, const float* b, const float* canon, float* state, int taps, int pos0,
                                                            int n, float eps, const float* add_y, const float* add_w, const float* add_b) {
    __shared__ float red[16];
    if (add_y) layernorm_row<kStepThreads>(add_y, add_w, add_b, n, eps, red, [&](int i, float v) { x[i] += v; });
    layernorm_row<kStepThreads>(x, w, b, n, eps, red, [&](int i, float h) {
        const float* cw = canon + (long long)i * taps;
        float s = 0.0f;
        for (int j = 0; j < taps - 1; ++j) {
            const float hj = pos0 - (taps - 1) + j >= 0 ? state[(long long)j * n + i] : 0.0f;
            s = fmaf(cw[j], hj, s);
            if (j > 0) state[(long long)(j - 1) * n + i] = hj;
        }
        s = fmaf(cw[taps - 1], h, s);
        if (taps > 1) state[(long long)(taps - 2) * n + i] = h;
        out[i] = h + s;
    });
}

// blocks y < T: out[y] = hist[taps-1+y] + sum_j w[:, j] * hist[y+j] (j ascending); blocks y >= T: the carried rows for the next portion
__global__ void causal_conv_mix_kernel(float* out, int ldo, const float* hist, const float* w, float* state, int taps, int T, int n) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, y = blockIdx.y;
    if (c >= n) return;
    if (y >= T) { state[(long long)(y - T) * n + c] = hist[(long long)y * n + c]; return; }
    float s = 0.0f;
    for (int j = 0; j < taps; ++j) s = fmaf(w[(long long)c * taps + j], hist[(long long)(y + j) * n + c], s);
    out[(long long)y * ldo + c] = hist[(long long)(y + taps - 1) * n + c] + s;
}

__global__ __launch_bounds__(1024) void polynorm_kernel(float* y, int ldy, const float* z, int ldz, const float* coef, int n, float eps) {
    __shared__ float red[16];
    const float* zr = z + (long long)blockIdx.x * ldz;
    float s2 = 0.0f, s4 = 0.0f, s6 = 0.0f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = zr[i], v2 = v * v, v3 = v2 * v;
        s2 += v2; s4 = fmaf(v2, v2, s4); s6 = fmaf(v3, v3, s6);
    }
    s2 = block_sum(s2, red); s4 = block_sum(s4, red); s6 = block_sum(s6, red);
    const float i1 = coef[0] / sqrtf(s2 / (float)n + eps), i2 = coef[1] / sqrtf(s4 / (float)n + eps), i3 = coef[2] / sqrtf(s6 / (float)n + eps), e = coef[3];
    float* o = y + (long long)blockIdx.x * ldy;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = zr[i], v2 = v * v, v3 = v2 * v;
        o[i] = i1 * v + i2 * v2 + i3 * v3 + e;
    }
}

__global__ __launch_bounds__(1024) void gated_rmsnorm_kernel(float* y, int ldy, const float* x, int ldx, const float* w, const float* g, int ldg, int n, float eps) {
    __shared__ float red[16];
    const float* xr = x + (long long)blockIdx.x * ldx;
    float ss = 0.0f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) ss = fmaf(xr[i], xr[i], ss);
    const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)n + eps);
    float* o = y + (long long)blockIdx.x * ldy;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = xr[i] * inv * w[i];
        if (g) v *= 1.0f / (1.0f + expf(-g[(long long)blockIdx.x * ldg + i]));
        o[i] = v;
    }
}

constexpr int kFewRows = 32;   // up to this many rows a row kernel runs workgroups of 1024 threads

}  // namespace ntk

using namespace ntk;

int ntk_embed_dense(float* out, const void* table, int tdtype, const int* tokens, int T, int vocab, int width, void* stream) {
    return ntk_embed_dense_scaled(out, table, tdtype, tokens, T, vocab, width, 1.0f, stream);
}

int ntk_embed_dense_scaled(float* out, const void* table, int tdtype, const int* tokens, int T, int vocab, int width, float scale, void* stream) {
    if (!out || !table || !tokens) return NTK_E_NULL;
    if (T < 0 || vocab <= 0 || width <= 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    if (tdtype == NTK_DT_BF16) hipLaunchKernelGGL(embed_dense_kernel<uint16_t>, dim3(T), dim3(256), 0, resolve_stream(stream), out, (const uint16_t*)table, tokens, vocab, width, scale);
    else if (tdtype == NTK_DT_F32) hipLaunchKernelGGL(embed_dense_kernel<float>, dim3(T), dim3(256), 0, resolve_stream(stream), out, (const float*)table, tokens, vocab, width, scale);
    else return NTK_E_DTYPE;
    return last_launch_status();
}

int ntk_rmsnorm_offset(float* y1, const float* w1, float* y2, const float* w2, int ldy, const float* x, int ldx, int T, int n, float eps, float offset,
                       void* stream) {
    if (!y1 || !w1 || !x || (y2 && !w2)) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldy < n || ldx < n) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(rmsnorm_offset_kernel, dim3(T), dim3(256), 0, resolve_stream(stream), y1, w1, y2, w2, ldy, x, ldx, n, eps, offset);
    return last_launch_status();
}

int ntk_concat_rows(float* out, const float* a, const float* b, int T, int n, void* stream) {
    if (!out || !a || !b) return NTK_E_NULL;
    if (T < 0 || n <= 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(concat_rows_kernel, dim3((2 * n + 255) / 256, T), dim3(256), 0, resolve_stream(stream), out, a, b, n);
    return last_launch_status();
}

int ntk_sigmoid_gate(float* y, int ldy, const float* g, int ldg, int T, int n, void* stream) {
    if (!y || !g) return NTK_E_NULL;
    if (T < 0 || n <= 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(sigmoid_gate_kernel, dim3((n + 255) / 256, T), dim3(256), 0, resolve_stream(stream), y, ldy, g, ldg, n);
    return last_launch_status();
}

int ntk_rows_copy(float* dst, const float* src, long long n, void* stream) {
    if (!dst || !src) return NTK_E_NULL;
    if (n < 0 || n > (1ll << 38)) return NTK_E_SHAPE;
    if (n == 0) return NTK_OK;
    hipLaunchKernelGGL(rows_copy_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, resolve_stream(stream), dst, src, n);
    return last_launch_status();
}

int ntk_residual_add(float* x, const float* a, const float* b, int n, void* stream) {
    if (!x || !a) return NTK_E_NULL;
    if (n < 0) return NTK_E_SHAPE;
    if (n == 0) return NTK_OK;
    hipLaunchKernelGGL(residual_add_kernel, dim3((n + 255) / 256), dim3(256), 0, resolve_stream(stream), x, a, b, n);
    return last_launch_status();
}

int ntk_scale(float* x, long long n, float s, void* stream) {
    if (!x) return NTK_E_NULL;
    if (n < 0 || n > (1ll << 38)) return NTK_E_SHAPE;
    if (n == 0) return NTK_OK;
    hipLaunchKernelGGL(scale_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, resolve_stream(stream), x, n, s);
    return last_launch_status();
}

int ntk_layernorm(float* y, int ldy, const float* x, int ldx, const float* w, const float* b, int T, int n, float eps, int accumulate, void* stream) {
    if (!y || !x || !w) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldy < n || ldx < n) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    if (T <= kFewRows) hipLaunchKernelGGL(layernorm_kernel<1024>, dim3(T), dim3(1024), 0, resolve_stream(stream), y, ldy, x, ldx, w, b, n, eps, accumulate);
    else hipLaunchKernelGGL(layernorm_kernel<256>, dim3(T), dim3(256), 0, resolve_stream(stream), y, ldy, x, ldx, w, b, n, eps, accumulate);
    return last_launch_status();
}

int ntk_layernorm_history(float* hist, const float* x, int ldx, const float* w, const float* b, const float* state, int taps, int pos0, int T, int n, float eps,
                          void* stream) {
    if (!hist || !x || !w || (taps > 1 && !state)) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldx < n || taps < 1 || pos0 < 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(layernorm_history_kernel, dim3(T + taps - 1), dim3(256), 0, resolve_stream(stream), hist, const_cast<float*>(x), ldx, w, b, state, taps, pos0, n,
                       eps, (const float*)nullptr, 0, (const float*)nullptr, (const float*)nullptr);
    return last_launch_status();
}

int ntk_sandwich_norm_conv(float* out, int ldo, float* x, int ldx, const float* add_y, int ldy, const float* add_w, const float* add_b, const float* w, const float* b,
                           const float* canon, float* state, float* hist, int taps, int pos0, int T, int n, float eps, void* stream) {
    if (!out || !x || !w || !canon || (taps > 1 && !state) || (add_y && !add_w)) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldx < n || ldo < n || (add_y && ldy < n) || taps < 1 || pos0 < 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipStream_t s = resolve_stream(stream);
    if (T == 1) {
        hipLaunchKernelGGL(sandwich_step_kernel, dim3(1), dim3(kStepThreads), 0, s, out, x, w, b, canon, state, taps, pos0, n, eps, add_y, add_w, add_b);
        return last_launch_status();
    }
    if (!hist) return NTK_E_NULL;
    hipLaunchKernelGGL(layernorm_history_kernel, dim3(T + taps - 1), dim3(256), 0, s, hist, x, ldx, w, b, (const float*)state, taps, pos0, n, eps, add_y, ldy, add_w, add_b);
    const int st = last_launch_status();
    if (st != NTK_OK) return st;
    return ntk_causal_conv_mix(out, ldo, hist, canon, state, taps, T, n, stream);
}

int ntk_causal_conv_mix(float* out, int ldo, const float* hist, const float* w, float* state, int taps, int T, int n, void* stream) {
    if (!out || !hist || !w || (taps > 1 && !state)) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldo < n || taps < 1) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(causal_conv_mix_kernel, dim3((n + 255) / 256, T + taps - 1), dim3(256), 0, resolve_stream(stream), out, ldo, hist, w, state, taps, T, n);
    return last_launch_status();
}

int ntk_polynorm(float* y, int ldy, const float* z, int ldz, const float* coef, int T, int n, float eps, void* stream) {
    if (!y || !z || !coef) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldy < n || ldz < n) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(polynorm_kernel, dim3(T), dim3(T <= kFewRows ? 1024 : 256), 0, resolve_stream(stream), y, ldy, z, ldz, coef, n, eps);
    return last_launch_status();
}

int ntk_gated_rmsnorm(float* y, int ldy, const float* x, int ldx, const float* w, const float* g, int ldg, int T, int n, float eps, void* stream) {
    if (!y || !x || !w) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldy < n || ldx < n || (g && ldg < n)) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(gated_rmsnorm_kernel, dim3(T), dim3(T <= kFewRows ? 1024 : 256), 0, resolve_stream(stream), y, ldy, x, ldx, w, g, ldg, n, eps);
    return last_launch_status();
}

// ---------------------------------------------------------------------------------------------------------------- layers with gated residuals
// The dynamic-tanh norm is element by element (no row sums), so it rides in whatever launch produces its input: the embedding (token row + position row),
// and the seam between sublayers (gated residual sum, the average over the layer results so far, the next norm).
namespace ntk {

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }

__global__ void dyt_kernel(float* y, int ldy, const float* x, int ldx, const float* w, const float* b, float alpha, int n) {
    const long long t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    y[t * ldy + i] = fmaf(tanhf(alpha * x[t * ldx + i]), w[i], b ? b[i] : 0.0f);
}

template <typename TT>
__global__ void embed_positions_kernel(float* out, float* copy, const TT* table, const TT* pos_table, const int* tokens, int vocab, int width, int pos0, int n_pos,
                                       const float* w, const float* b, float alpha) {
    const long long t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= width) return;
    const int tok = tokens[t];
    const long long p = pos0 + t;
    float e = 0.0f, pv = 0.0f;
    if (tok >= 0 && tok < vocab) {
        if constexpr (sizeof(TT) == 2) e = __uint_as_float((uint32_t)table[(long long)tok * width + i] << 16); else e = table[(long long)tok * width + i];
    }
    if (p < n_pos) {
        if constexpr (sizeof(TT) == 2) pv = __uint_as_float((uint32_t)pos_table[p * width + i] << 16); else pv = pos_table[p * width + i];
    }
    float v = e + pv;
    if (w) v = fmaf(tanhf(alpha * v), w[i], b ? b[i] : 0.0f);
    out[t * width + i] = v;
    if (copy) copy[t * width + i] = v;
}

__global__ void sigmoid_gate_scaled_kernel(float* y, int ldy, const float* g, int ldg, const float* gb, float scale, int n) {
    const long long t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    y[t * ldy + i] = y[t * ldy + i] * sigmoidf_(g[t * ldg + i] + (gb ? gb[i] : 0.0f)) * scale;
}

__global__ void tanh_rows_kernel(float* x, int ldx, int n) {
    const long long t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[t * ldx + i] = tanhf(x[t * ldx + i]);
}

// one wave per (token, head): the head's dv values in registers (dv <= 64 * 16), mean of squares over the wave, weight, gate
constexpr int HRN_MAXC = 16;
__global__ __launch_bounds__(64) void head_rmsnorm_gate_kernel(float* y, int ldy, const float* x, int ldx, const float* w, int w_head_stride, const float* g, int ldg,
                                                               int act, float scale, int H, int dv, float eps) {
    const int lane = threadIdx.x, h = blockIdx.x % H;
    const long long t = blockIdx.x / H;
    const float* xr = x + t * ldx + (long long)h * dv;
    float v[HRN_MAXC];
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < HRN_MAXC; ++c) {
        v[c] = c * 64 + lane < dv ? xr[c * 64 + lane] : 0.0f;
        ss = fmaf(v[c], v[c], ss);
    }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)dv + eps);
#pragma unroll
    for (int c = 0; c < HRN_MAXC; ++c) {
        const int i = c * 64 + lane;
        if (i >= dv) continue;
        float r = v[c] * inv * w[(long long)h * w_head_stride + i];
        if (act) {
            const float gg = g[t * ldg + (long long)h * dv + i];
            r *= act == 1 ? sigmoidf_(gg) : gg * sigmoidf_(gg);
        }
        y[t * ldy + (long long)h * dv + i] = r * scale;
    }
}

struct SeamArgs {
    float* x; int ldx;
    const float* y; int ldy; const float* yb;
    const float* g; int ldg; const float* gb;
    float* hist; long long hist_stride; int n_hist; const float* coef;
    float* h; int ldh; const float* nw; const float* nb; float alpha;
    int n;
};
__global__ void gated_seam_kernel(const SeamArgs a) {
    const long long t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= a.n) return;
    float r = a.x[t * a.ldx + i];
    if (a.y) {
        const float yy = a.y[t * a.ldy + i] + (a.yb ? a.yb[i] : 0.0f);
        r = fmaf(yy, sigmoidf_(a.g[t * a.ldg + i] + (a.gb ? a.gb[i] : 0.0f)), r);
    }
    if (a.n_hist > 0) {
        float s = 0.0f;
        for (int j = 0; j + 1 < a.n_hist; ++j) s = fmaf(a.coef[j], a.hist[j * a.hist_stride + t * a.n + i], s);
        a.hist[(a.n_hist - 1) * a.hist_stride + t * a.n + i] = r;
        r = fmaf(a.coef[a.n_hist - 1], r, s);
    }
    a.x[t * a.ldx + i] = r;
    if (a.h) a.h[t * a.ldh + i] = fmaf(tanhf(a.alpha * r), a.nw[i], a.nb ? a.nb[i] : 0.0f);
}

}  // namespace ntk

int ntk_dyt(float* y, int ldy, const float* x, int ldx, const float* w, const float* b, float alpha, int T, int n, void* stream) {
    if (!y || !x || !w) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldy < n || ldx < n) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(ntk::dyt_kernel, dim3((n + 255) / 256, T), dim3(256), 0, resolve_stream(stream), y, ldy, x, ldx, w, b, alpha, n);
    return last_launch_status();
}

int ntk_embed_positions(float* out, float* copy, const void* table, const void* pos_table, int tdtype, const int* tokens, int T, int vocab, int width, int pos0,
                        int n_pos, const float* w, const float* b, float alpha, void* stream) {
    if (!out || !table || !pos_table || !tokens) return NTK_E_NULL;
    if (tdtype != NTK_DT_BF16 && tdtype != NTK_DT_F32) return NTK_E_DTYPE;
    if (T < 0 || vocab <= 0 || width <= 0 || pos0 < 0 || n_pos < 0) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    const dim3 grid((width + 255) / 256, T);
    if (tdtype == NTK_DT_BF16)
        hipLaunchKernelGGL(ntk::embed_positions_kernel<uint16_t>, grid, dim3(256), 0, resolve_stream(stream), out, copy, (const uint16_t*)table, (const uint16_t*)pos_table,
                           tokens, vocab, width, pos0, n_pos, w, b, alpha);
    else
        hipLaunchKernelGGL(ntk::embed_positions_kernel<float>, grid, dim3(256), 0, resolve_stream(stream), out, copy, (const float*)table, (const float*)pos_table, tokens,
                           vocab, width, pos0, n_pos, w, b, alpha);
    return last_launch_status();
}

int ntk_sigmoid_gate_scaled(float* y, int ldy, const float* g, int ldg, const float* gb, float scale, int T, int n, void* stream) {
    if (!y || !g) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldy < n || ldg < n) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(ntk::sigmoid_gate_scaled_kernel, dim3((n + 255) / 256, T), dim3(256), 0, resolve_stream(stream), y, ldy, g, ldg, gb, scale, n);
    return last_launch_status();
}

int ntk_tanh_rows(float* x, int ldx, int T, int n, void* stream) {
    if (!x) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldx < n) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(ntk::tanh_rows_kernel, dim3((n + 255) / 256, T), dim3(256), 0, resolve_stream(stream), x, ldx, n);
    return last_launch_status();
}

int ntk_head_rmsnorm_gate(float* y, int ldy, const float* x, int ldx, const float* w, int w_head_stride, const float* g, int ldg, int act, float scale, int T, int H,
                          int dv, float eps, void* stream) {
    if (!y || !x || !w || (act && !g)) return NTK_E_NULL;
    if (T < 0 || H <= 0 || dv <= 0 || dv > 64 * ntk::HRN_MAXC || act < 0 || act > 2 || ldy < H * dv || ldx < H * dv || (act && ldg < H * dv)) return NTK_E_SHAPE;
    if (w_head_stride != 0 && w_head_stride != dv) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(ntk::head_rmsnorm_gate_kernel, dim3(T * H), dim3(64), 0, resolve_stream(stream), y, ldy, x, ldx, w, w_head_stride, g, ldg, act, scale, H, dv, eps);
    return last_launch_status();
}

int ntk_gated_seam(const ntk_gated_seam_desc* d, void* stream) {
    if (!d || !d->x || (d->y && !d->g) || (d->n_hist > 0 && (!d->hist || !d->coef)) || (d->h && !d->nw)) return NTK_E_NULL;
    if (d->T < 0 || d->n <= 0 || d->ldx < d->n || (d->y && (d->ldy < d->n || d->ldg < d->n)) || (d->h && d->ldh < d->n) || d->n_hist < 0) return NTK_E_SHAPE;
    if (d->n_hist > 0 && d->hist_stride < (long long)d->T * d->n) return NTK_E_SHAPE;
    if (d->T == 0) return NTK_OK;
    ntk::SeamArgs a{d->x, d->ldx, d->y, d->ldy, d->yb, d->g, d->ldg, d->gb, d->hist, d->hist_stride, d->n_hist, d->coef, d->h, d->ldh, d->nw, d->nb, d->alpha, d->n};
    hipLaunchKernelGGL(ntk::gated_seam_kernel, dim3((d->n + 255) / 256, d->T), dim3(256), 0, resolve_stream(stream), a);
    return last_launch_status();
}

// ---------------------------------------------------------------------------------------------------------------- layers with scaled, RMS-normed sublayer results
// The seam between two sublayers: the result the stream is still owed joins it (RMS norm, weight, a fixed factor), and the norm in front of the next sublayer
// reads the row the same launch has just written (a thread reads back only what it wrote itself).  The short convolution of a recurrent mixer's projections
// carries its last inputs from portion to portion; one token is one launch (a channel's history belongs to the thread that owns the channel).
namespace ntk {

template <int NT>
__global__ __launch_bounds__(NT) void rms_seam_kernel(float* h, int ldh, float* x, int ldx, const float* add_y, int ldy, const float* add_w, float mult, const float* w,
                                                      int n, float eps) {
    __shared__ float red[16];
    constexpr int KEEP = 4096 / NT;              // a thread's first entries stay in registers: rows up to 4096 wide cross memory once
    float* xr = x + (long long)blockIdx.x * ldx;
    float v[KEEP];
    if (add_y) {
        const float* yr = add_y + (long long)blockIdx.x * ldy;
        float ss = 0.0f;
#pragma unroll
        for (int k = 0; k < KEEP; ++k) {
            const int i = threadIdx.x + NT * k;
            v[k] = i < n ? yr[i] : 0.0f;
            ss = fmaf(v[k], v[k], ss);
        }
        for (int i = threadIdx.x + NT * KEEP; i < n; i += NT) ss = fmaf(yr[i], yr[i], ss);
        const float inv = mult / sqrtf(block_sum(ss, red) / (float)n + eps);
#pragma unroll
        for (int k = 0; k < KEEP; ++k) {
            const int i = threadIdx.x + NT * k;
            if (i < n) { v[k] = fmaf(v[k] * inv, add_w[i], xr[i]); xr[i] = v[k]; }
        }
        for (int i = threadIdx.x + NT * KEEP; i < n; i += NT) xr[i] = fmaf(yr[i] * inv, add_w[i], xr[i]);
    } else {
#pragma unroll
        for (int k = 0; k < KEEP; ++k) {
            const int i = threadIdx.x + NT * k;
            v[k] = i < n ? xr[i] : 0.0f;
        }
    }
    if (!h) return;                              // (uniform over the launch)
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < KEEP; ++k)
        if ((int)threadIdx.x + NT * k < n) ss = fmaf(v[k], v[k], ss);
    for (int i = threadIdx.x + NT * KEEP; i < n; i += NT) ss = fmaf(xr[i], xr[i], ss);
    const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)n + eps);
    float* hr = h + (long long)blockIdx.x * ldh;
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
        const int i = threadIdx.x + NT * k;
        if (i < n) hr[i] = v[k] * inv * w[i];
    }
    for (int i = threadIdx.x + NT * KEEP; i < n; i += NT) hr[i] = xr[i] * inv * w[i];
}

constexpr int kConvMaxTaps = 16;
__device__ __forceinline__ float conv_act(float s, int act) { return act == 1 ? s / (1.0f + expf(-s)) : s; }

// the input `back` rows before row t of the portion: the portion's own row, a carried one, or zero before the sequence's start
__device__ __forceinline__ float conv_input(const float* x, int ldx, const float* state, int taps, int pos0, int n, int c, int idx) {
    if (idx >= 0) return x[(long long)idx * ldx + c];
    if (pos0 + idx < 0) return 0.0f;
    return state[(long long)(taps - 1 + idx) * n + c];   // carried row taps - 1 + idx: the row that lay idx before this portion
}

// blocks y < T: the outputs; one more launch shifts the carried rows (they are read here)
__global__ void causal_conv_act_kernel(float* y, int ldy, const float* x, int ldx, const float* w, const float* state, int taps, int act, int pos0, int n) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, t = blockIdx.y;
    if (c >= n) return;
    float s = 0.0f;
    for (int j = 0; j < taps; ++j) s = fmaf(w[(long long)c * taps + j], conv_input(x, ldx, state, taps, pos0, n, c, t - (taps - 1) + j), s);
    y[(long long)t * ldy + c] = conv_act(s, act);
}

// the carried rows after the portion: a thread owns a channel, reads its taps - 1 new rows (some of them old carried rows when the portion is shorter) and
// then writes them.  T == 1 with an output: the whole operator for one token in this one launch.
__global__ void causal_conv_carry_kernel(float* y, const float* x, int ldx, const float* w, float* state, int taps, int act, int pos0, int T, int n) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= n) return;
    float keep[kConvMaxTaps];
#pragma unroll
    for (int r = 0; r < kConvMaxTaps; ++r)
        if (r < taps) keep[r] = conv_input(x, ldx, state, taps, pos0, n, c, T - taps + r);      // rows T - taps .. T - 1 (the first only for the output)
    if (y) {
        float s = 0.0f;
#pragma unroll
        for (int r = 0; r < kConvMaxTaps; ++r)
            if (r < taps) s = fmaf(w[(long long)c * taps + r], keep[r], s);
        y[c] = conv_act(s, act);
    }
#pragma unroll
    for (int r = 1; r < kConvMaxTaps; ++r)
        if (r < taps) state[(long long)(r - 1) * n + c] = keep[r];
}

__global__ void softcap_rows_kernel(float* x, int ldx, float cap, int n) {
    const long long t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[t * ldx + i] = cap * tanhf(x[t * ldx + i] / cap);
}

__global__ void head_gate_kernel(float* y, int ldy, const float* g, int ldg, int H, int dv) {
    const long long t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= H * dv) return;
    y[t * ldy + i] *= sigmoidf_(g[t * ldg + i / dv]);
}

}  // namespace ntk

int ntk_rms_seam(float* h, int ldh, float* x, int ldx, const float* add_y, int ldy, const float* add_w, float mult, const float* w, int T, int n, float eps,
                 void* stream) {
    if (!x || (add_y && !add_w) || (h && !w)) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldx < n || (h && ldh < n) || (add_y && ldy < n)) return NTK_E_SHAPE;
    if (T == 0 || (!add_y && !h)) return NTK_OK;
    if (T <= kFewRows) hipLaunchKernelGGL(ntk::rms_seam_kernel<1024>, dim3(T), dim3(1024), 0, resolve_stream(stream), h, ldh, x, ldx, add_y, ldy, add_w, mult, w, n, eps);
    else hipLaunchKernelGGL(ntk::rms_seam_kernel<256>, dim3(T), dim3(256), 0, resolve_stream(stream), h, ldh, x, ldx, add_y, ldy, add_w, mult, w, n, eps);
    return last_launch_status();
}

int ntk_causal_conv_act(float* y, int ldy, const float* x, int ldx, const float* w, float* state, int taps, int act, int pos0, int T, int n, void* stream) {
    if (!y || !x || !w || (taps > 1 && !state)) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldy < n || ldx < n || taps < 1 || taps > ntk::kConvMaxTaps || pos0 < 0 || act < 0 || act > 1) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipStream_t s = resolve_stream(stream);
    if (T == 1) {
        hipLaunchKernelGGL(ntk::causal_conv_carry_kernel, dim3((n + 255) / 256), dim3(256), 0, s, y, x, ldx, w, state, taps, act, pos0, T, n);
        return last_launch_status();
    }
    hipLaunchKernelGGL(ntk::causal_conv_act_kernel, dim3((n + 255) / 256, T), dim3(256), 0, s, y, ldy, x, ldx, w, (const float*)state, taps, act, pos0, n);
    const int st = last_launch_status();
    if (st != NTK_OK || taps == 1) return st;
    hipLaunchKernelGGL(ntk::causal_conv_carry_kernel, dim3((n + 255) / 256), dim3(256), 0, s, (float*)nullptr, x, ldx, w, state, taps, act, pos0, T, n);
    return last_launch_status();
}

int ntk_softcap_rows(float* x, int ldx, float cap, int T, int n, void* stream) {
    if (!x) return NTK_E_NULL;
    if (T < 0 || n <= 0 || ldx < n || !(cap > 0.0f)) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(ntk::softcap_rows_kernel, dim3((n + 255) / 256, T), dim3(256), 0, resolve_stream(stream), x, ldx, cap, n);
    return last_launch_status();
}

int ntk_head_gate(float* y, int ldy, const float* g, int ldg, int T, int H, int dv, void* stream) {
    if (!y || !g) return NTK_E_NULL;
    if (T < 0 || H <= 0 || dv <= 0 || ldy < H * dv || ldg < H) return NTK_E_SHAPE;
    if (T == 0) return NTK_OK;
    hipLaunchKernelGGL(ntk::head_gate_kernel, dim3((H * dv + 255) / 256, T), dim3(256), 0, resolve_stream(stream), y, ldy, g, ldg, H, dv);
    return last_launch_status();
}
