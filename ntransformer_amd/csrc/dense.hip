// dense.hip -- products with dense weight matrices (bfloat16 or float32, row-major [out][in]) for the layer-list model families.
//
// One entry point (ntk_dense) and three kernel forms behind it:
//   * dense_mfma_kernel   bf16 weights, more than kGemvRows rows: 128 x 128 / 64 x 128 / 64 x 64 output tiles on v_mfma_f32_16x16x32_bf16; the F32 activations are rounded
//                         to bfloat16 (nearest even) on their way into LDS, sums stay F32 in the accumulators;
//   * dense_fma_kernel    float32 weights, more than kGemvRows rows: the same tiling with plain F32 FMAs, k ascending (true 32-bit);
//   * dense_gemv_kernel   up to kGemvRows rows (decoding): every wave streams a few weight rows at once, 16 bytes per lane and row, the activation
//                         row sits in LDS; bf16 weights are widened exactly and multiplied in F32.
// Rows can be grouped (a mixture of experts: sorted rows of group g take matrix g) and gathered (row r reads activation row rows[r] / row_div).
// Group sizes live on the device, so the grid covers the worst case and workgroups outside their group's range leave at once.
#include "common.hip.h"
#include "../../include/ntk_layers.h"

namespace ntk {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uintx4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint16_t f2bf(float f) {   // round to nearest even; NaN stays NaN
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float bf2f(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }

struct DenseArgs {
    float* Y; int ldy;
    const float* X; int ldx;
    const void* W; long long wstride;
    const int* offsets;
    const int* rows; int row_div;
    int T, N, K, accumulate, G, vec;
    int glu_ff; float glu_limit, glu_alpha, glu_up_offset, glu_cubic;   // few-row form only: outputs f < glu_ff = gated unit of rows f (gate) and glu_ff + f (up)
    const float* norm_w; float norm_eps, norm_offset;   // few-row form only: the activation row is RMS-normed with weight (offset + norm_w) first
};

__device__ __forceinline__ bool group_range(const DenseArgs& a, int g, int& r0, int& r1) {
    if (a.offsets) { r0 = a.offsets[g]; r1 = a.offsets[g + 1]; } else { r0 = 0; r1 = a.T; }
    return r1 > r0;
}

// ---------------------------------------------------------------------------------------------------------------- bf16, matrix cores
// A workgroup of four waves (2 x 2) owns a TM x TN tile of Y; a wave owns (TM / 2) x (TN / 2) of it as 16 x 16 accumulator tiles.  K goes by in chunks
// of 32: the NEXT chunk's operands are requested into registers before the current one is multiplied out of LDS (global latency behind the MFMAs),
// activations are rounded to bfloat16 (nearest even, the hardware conversion) on their way into LDS.
constexpr int BK = 32, LDSK = BK + 8;   // LDS rows of 40 bf16 = 80 bytes: 16-byte aligned operand reads, rows 20 banks apart
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    const bf16x2_t v = __builtin_convertvector(floatx2_t{a, b}, bf16x2_t);
    uint32_t u;
    __builtin_memcpy(&u, &v, 4);
    return u;
}

template <int TM, int TN, bool VEC>
__global__ __launch_bounds__(256) void dense_mfma_kernel(const DenseArgs a) {
    constexpr int PX = TM / 64, PW = TN / 64;        // loader passes of 64 rows
    constexpr int MI = TM / 32, NJ = TN / 32;        // 16 x 16 tiles per wave
    int r0, r1;
    if (!group_range(a, blockIdx.z, r0, r1)) return;
    const int row_base = r0 + blockIdx.y * TM;
    if (row_base >= r1) return;
    const int n_base = blockIdx.x * TN;
    const uint16_t* W = (const uint16_t*)a.W + (long long)blockIdx.z * a.wstride;
    __shared__ __attribute__((aligned(16))) uint16_t Xs[TM][LDSK];
    __shared__ __attribute__((aligned(16))) uint16_t Ws[TN][LDSK];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave & 1, wn = wave >> 1;
    // loader: thread -> (row tid / 4 + 64 * pass, eight k from (tid & 3) * 8)
    const int lr = tid >> 2, lk = (tid & 3) * 8;
    const float* xrow[PX];
    const uint16_t* wrow[PW];
#pragma unroll
    for (int p = 0; p < PX; ++p) {
        const int xr = row_base + lr + 64 * p;
        xrow[p] = xr < r1 ? a.X + (long long)(a.rows ? a.rows[xr] / a.row_div : xr) * a.ldx : nullptr;
    }
#pragma unroll
    for (int p = 0; p < PW; ++p) {
        const int wr = n_base + lr + 64 * p;
        wrow[p] = wr < a.N ? W + (long long)wr * a.K : nullptr;
    }
    floatx4_t acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) acc[i][j] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    uintx4_t xreg[PX], wreg[PW];
    auto fetch = [&](int k0) {
        const int k = k0 + lk;
#pragma unroll
        for (int p = 0; p < PX; ++p) {
            xreg[p] = uintx4_t{0u, 0u, 0u, 0u};
            if (xrow[p]) {
                if (VEC) {
                    if (k < a.K) {
                        const float4 v0 = *reinterpret_cast<const float4*>(xrow[p] + k), v1 = *reinterpret_cast<const float4*>(xrow[p] + k + 4);
                        xreg[p] = uintx4_t{pack_bf16(v0.x, v0.y), pack_bf16(v0.z, v0.w), pack_bf16(v1.x, v1.y), pack_bf16(v1.z, v1.w)};
                    }
                } else {
                    float v[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[j] = k + j < a.K ? xrow[p][k + j] : 0.0f;
                    xreg[p] = uintx4_t{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7])};
                }
            }
        }
#pragma unroll
        for (int p = 0; p < PW; ++p) {
            wreg[p] = uintx4_t{0u, 0u, 0u, 0u};
            if (wrow[p]) {
                if (VEC) {
                    if (k < a.K) wreg[p] = *reinterpret_cast<const uintx4_t*>(wrow[p] + k);
                } else {
                    uint32_t v[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[j] = k + j < a.K ? (uint32_t)wrow[p][k + j] : 0u;
                    wreg[p] = uintx4_t{v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16)};
                }
            }
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < a.K; k0 += BK) {
        __syncthreads();   // the previous chunk's operand reads are done
#pragma unroll
        for (int p = 0; p < PX; ++p) *reinterpret_cast<uintx4_t*>(&Xs[lr + 64 * p][lk]) = xreg[p];
#pragma unroll
        for (int p = 0; p < PW; ++p) *reinterpret_cast<uintx4_t*>(&Ws[lr + 64 * p][lk]) = wreg[p];
        __syncthreads();
        if (k0 + BK < a.K) fetch(k0 + BK);
        bf16x8_t af[MI], bfr[NJ];
#pragma unroll
        for (int i = 0; i < MI; ++i) af[i] = *reinterpret_cast<const bf16x8_t*>(&Xs[wm * (TM / 2) + i * 16 + (lane & 15)][(lane >> 4) * 8]);
#pragma unroll
        for (int j = 0; j < NJ; ++j) bfr[j] = *reinterpret_cast<const bf16x8_t*>(&Ws[wn * (TN / 2) + j * 16 + (lane & 15)][(lane >> 4) * 8]);
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
    // accumulator lane map: row 4 * (lane / 16) + r, column lane % 16
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = row_base + wm * (TM / 2) + i * 16 + (lane >> 4) * 4 + r, col = n_base + wn * (TN / 2) + j * 16 + (lane & 15);
                if (row < r1 && col < a.N) {
                    float* y = a.Y + (long long)row * a.ldy + col;
                    *y = a.accumulate ? *y + acc[i][j][r] : acc[i][j][r];
                }
            }
}

// ---------------------------------------------------------------------------------------------------------------- float32, vector FMA
constexpr int FK = 16, TM = 64, TN = 64;
__global__ __launch_bounds__(256) void dense_fma_kernel(const DenseArgs a) {
    int r0, r1;
    if (!group_range(a, blockIdx.z, r0, r1)) return;
    const int row_base = r0 + blockIdx.y * TM;
    if (row_base >= r1) return;
    const int n_base = blockIdx.x * TN;
    const float* W = (const float*)a.W + (long long)blockIdx.z * a.wstride;
    __shared__ __attribute__((aligned(16))) float Xs[FK][TM + 4];
    __shared__ __attribute__((aligned(16))) float Ws[FK][TN + 4];
    const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
    const int lr = tid >> 2, lk = (tid & 3) * 4;
    const int xr = row_base + lr;
    const bool x_ok = xr < r1;
    const float* xrow = nullptr;
    if (x_ok) xrow = a.X + (long long)(a.rows ? a.rows[xr] / a.row_div : xr) * a.ldx;
    const int wr = n_base + lr;
    const bool w_ok = wr < a.N;
    const float* wrow = W + (long long)wr * a.K;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < a.K; k0 += FK) {
        float xv[4], wv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + lk + j;
            xv[j] = (x_ok && k < a.K) ? xrow[k] : 0.0f;
            wv[j] = (w_ok && k < a.K) ? wrow[k] : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j) { Xs[lk + j][lr] = xv[j]; Ws[lk + j][lr] = wv[j]; }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < FK; ++k) {
            const float4 xa = *reinterpret_cast<const float4*>(&Xs[k][ty * 4]);
            const float4 wa = *reinterpret_cast<const float4*>(&Ws[k][tx * 4]);
            const float xs[4] = {xa.x, xa.y, xa.z, xa.w}, ws[4] = {wa.x, wa.y, wa.z, wa.w};
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(xs[i], ws[j], acc[i][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = row_base + ty * 4 + i, col = n_base + tx * 4 + j;
            if (row < r1 && col < a.N) {
                float* y = a.Y + (long long)row * a.ldy + col;
                *y = a.accumulate ? *y + acc[i][j] : acc[i][j];
            }
        }
}

// ---------------------------------------------------------------------------------------------------------------- few rows: waves stream weight rows
// One workgroup per (group of 4 * RW outputs, activation row): the activation row sits in LDS, each wave owns RW consecutive weight rows and walks
// them together -- per step a lane requests 16 bytes of each of its RW rows before it uses any (RW loads in flight per lane), reads its 8 activations
// once and feeds RW sums; one DPP reduction per row at the end.  RW is picked so that the launch still has a few workgroups per CU.
constexpr int kGemvRows = 8;       // up to this many rows take this form
template <typename WT, int RW, bool GLU>
__global__ __launch_bounds__(256) void dense_gemv_kernel(const DenseArgs a) {
    extern __shared__ __attribute__((aligned(16))) float xs[];   // the activation row
    const int r = blockIdx.y;
    int g = 0;
    if (a.offsets) {
        if (r >= a.offsets[a.G]) return;
        while (r >= a.offsets[g + 1]) ++g;
    }
    const float* xrow = a.X + (long long)(a.rows ? a.rows[r] / a.row_div : r) * a.ldx;
    float ss = 0.0f;
    for (int k = threadIdx.x; k < a.K; k += 256) { const float v = xrow[k]; xs[k] = v; ss = fmaf(v, v, ss); }
    if (a.norm_w) {                                         // (uniform over the launch)
        __shared__ float red[16];
        ss = block_sum(ss, red);
        const float inv = 1.0f / sqrtf(ss / (float)a.K + a.norm_eps);
        for (int k = threadIdx.x; k < a.K; k += 256) xs[k] = xs[k] * inv * (a.norm_offset + a.norm_w[k]);   // (each thread rewrites what it wrote)
    }
    __syncthreads();
    const WT* W = (const WT*)a.W + (long long)g * a.wstride;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // GLU: the wave's RW rows are RW / 2 (gate, up) pairs of RW / 2 consecutive outputs
    constexpr int OUT = GLU ? RW / 2 : RW;
    const int n_out = GLU ? a.glu_ff : a.N;
    const int n0 = (blockIdx.x * 4 + wave) * OUT;
    if (n0 >= n_out) return;                                // uniform per wave
    const WT* w[RW];
#pragma unroll
    for (int i = 0; i < RW; ++i) {                          // rows past the end re-read the last one and are not stored
        const int row = GLU ? (i < OUT ? min(n0 + i, n_out - 1) : a.glu_ff + min(n0 + i - OUT, n_out - 1)) : min(n0 + i, n_out - 1);
        w[i] = W + (long long)row * a.K;
    }
    float s[RW];
#pragma unroll
    for (int i = 0; i < RW; ++i) s[i] = 0.0f;
    if (a.vec) {
#pragma unroll 2
        for (int k = lane * 8; k < a.K; k += 64 * 8) {
            float wv[RW][8];
            if constexpr (sizeof(WT) == 2) {
                uintx4_t u[RW];
#pragma unroll
                for (int i = 0; i < RW; ++i) u[i] = __builtin_nontemporal_load(reinterpret_cast<const uintx4_t*>(w[i] + k));
#pragma unroll
                for (int i = 0; i < RW; ++i) {
                    const uint32_t uu[4] = {u[i].x, u[i].y, u[i].z, u[i].w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) { wv[i][2 * j] = __uint_as_float(uu[j] << 16); wv[i][2 * j + 1] = __uint_as_float(uu[j] & 0xffff0000u); }
                }
            } else {
                float4 u0[RW], u1[RW];
#pragma unroll
                for (int i = 0; i < RW; ++i) { u0[i] = *reinterpret_cast<const float4*>(w[i] + k); u1[i] = *reinterpret_cast<const float4*>(w[i] + k + 4); }
#pragma unroll
                for (int i = 0; i < RW; ++i) {
                    wv[i][0] = u0[i].x; wv[i][1] = u0[i].y; wv[i][2] = u0[i].z; wv[i][3] = u0[i].w;
                    wv[i][4] = u1[i].x; wv[i][5] = u1[i].y; wv[i][6] = u1[i].z; wv[i][7] = u1[i].w;
                }
            }
            const float4 x0 = *reinterpret_cast<const float4*>(xs + k), x1 = *reinterpret_cast<const float4*>(xs + k + 4);
            const float xv[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
            for (int i = 0; i < RW; ++i)
#pragma unroll
                for (int j = 0; j < 8; ++j) s[i] = fmaf(wv[i][j], xv[j], s[i]);
        }
    } else {
        for (int k = lane; k < a.K; k += 64) {
            const float xv = xs[k];
#pragma unroll
            for (int i = 0; i < RW; ++i) {
                float wv;
                if constexpr (sizeof(WT) == 2) wv = bf2f(((const uint16_t*)w[i])[k]); else wv = ((const float*)w[i])[k];
                s[i] = fmaf(wv, xv, s[i]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < RW; ++i) s[i] = wave_sum_lane63(s[i]);
#pragma unroll
    for (int i = 0; i < OUT; ++i) {
        if (lane == 63 && n0 + i < n_out) {
            float t = s[i];
            if constexpr (GLU) {
                const float gg = fminf(s[i], a.glu_limit), uu = fminf(fmaxf(s[i + OUT], -a.glu_limit), a.glu_limit);
                const float zz = a.glu_cubic != 0.0f ? fmaf(a.glu_cubic * gg * gg, gg, gg) : gg;
                t = gg * (1.0f / (1.0f + expf(-a.glu_alpha * zz))) * (uu + a.glu_up_offset);
            }
            float* y = a.Y + (long long)r * a.ldy + n0 + i;
            *y = a.accumulate ? *y + t : t;
        }
    }
}

template <typename WT>
static void launch_gemv(const DenseArgs& a, int rows, hipStream_t s) {
    const size_t lds = ((size_t)a.K * 4 + 15) & ~(size_t)15;
    // Rows per wave, measured over layer-like shapes (2048 .. 64000 outputs of 768 .. 4096 inputs, 1 .. 6 activation rows): two rows per wave are
    // the best or within noise everywhere from 4096 outputs x rows on (a 64000 x 4096 head: 84 us against 98 with one or eight), one below; launches
    // under ~20 MB sit at 4 - 6 us whatever the choice.  The GLU form keeps pairs: 4 pairs per wave for the large expert launches.
    const long long work = (long long)a.N * rows;
    int rw = work >= 4096 ? 2 : 1;
    if (const int force = NTK_TUNE_ENV_INT("NTK_DENSE_GEMV_RW", 0)) rw = force;   // (tuning builds only)
    if (a.glu_ff > 0) {
        const int out = work >= 4 * 8 * 512 ? 4 : work >= 4 * 4 * 512 ? 2 : 1;   // (gate, up) pairs per wave
        const dim3 grid((a.glu_ff + 4 * out - 1) / (4 * out), rows, 1);
        if (out == 4) hipLaunchKernelGGL((dense_gemv_kernel<WT, 8, true>), grid, dim3(256), lds, s, a);
        else if (out == 2) hipLaunchKernelGGL((dense_gemv_kernel<WT, 4, true>), grid, dim3(256), lds, s, a);
        else hipLaunchKernelGGL((dense_gemv_kernel<WT, 2, true>), grid, dim3(256), lds, s, a);
        return;
    }
    const dim3 grid((a.N + 4 * rw - 1) / (4 * rw), rows, 1);
    if (rw == 8) hipLaunchKernelGGL((dense_gemv_kernel<WT, 8, false>), grid, dim3(256), lds, s, a);
    else if (rw == 4) hipLaunchKernelGGL((dense_gemv_kernel<WT, 4, false>), grid, dim3(256), lds, s, a);
    else if (rw == 2) hipLaunchKernelGGL((dense_gemv_kernel<WT, 2, false>), grid, dim3(256), lds, s, a);
    else hipLaunchKernelGGL((dense_gemv_kernel<WT, 1, false>), grid, dim3(256), lds, s, a);
}

}  // namespace ntk

using namespace ntk;

int ntk_dense(const ntk_dense_desc* d, void* stream) {
    if (!d || !d->Y || !d->X || !d->W) return NTK_E_NULL;
    if (d->wdtype != NTK_DT_BF16 && d->wdtype != NTK_DT_F32) return NTK_E_DTYPE;
    if (d->T < 0 || d->N <= 0 || d->K <= 0 || d->ldx < d->K || d->ldy < (d->glu_ff > 0 ? d->glu_ff : d->N)) return NTK_E_SHAPE;
    if (d->offsets && d->G <= 0) return NTK_E_SHAPE;
    if (d->rows && d->row_div <= 0) return NTK_E_SHAPE;
    if (d->glu_ff > 0 && (d->T > kGemvRows || d->N != 2 * d->glu_ff || d->accumulate)) return NTK_E_SHAPE;
    if (d->norm_w && d->T > kGemvRows) return NTK_E_SHAPE;
    if (d->T == 0) return NTK_OK;
    const int G = d->offsets ? d->G : 1;
    DenseArgs a{d->Y, d->ldy, d->X, d->ldx, d->W, d->wstride, d->offsets, d->rows, d->rows ? d->row_div : 1, d->T, d->N, d->K, d->accumulate, G, 0, 0, 0.0f, 0.0f, 0.0f, 0.0f, nullptr, 0.0f, 0.0f};
    hipStream_t s = resolve_stream(stream);
    if (d->T <= kGemvRows) {
        if ((size_t)d->K * 4 > 160 * 1024 - 1024) return NTK_E_SHAPE;
        a.glu_ff = d->glu_ff; a.glu_limit = d->glu_limit; a.glu_alpha = d->glu_alpha; a.glu_up_offset = d->glu_up_offset; a.glu_cubic = d->glu_cubic;
        a.norm_w = d->norm_w; a.norm_eps = d->norm_eps; a.norm_offset = d->norm_offset;
        a.vec = (d->K % 8 == 0) && !((uintptr_t)d->W & 15) && !((d->wstride * (d->wdtype == NTK_DT_BF16 ? 2 : 4)) & 15);
        if (d->wdtype == NTK_DT_BF16) launch_gemv<uint16_t>(a, d->T, s);
        else launch_gemv<float>(a, d->T, s);
        return last_launch_status();
    }
    if (d->wdtype == NTK_DT_BF16) {
        const bool vec = (d->K % 8 == 0) && (d->ldx % 4 == 0) && !((uintptr_t)d->X & 15) && !((uintptr_t)d->W & 15) && (d->wstride % 8 == 0);
        // 128 x 128 tiles where a group has the rows and the launch still fills the chip; 64-row tiles for short groups (experts, short portions)
        const int rows_per_group = d->T / G;
        const bool big = rows_per_group >= 192 && d->N >= 128 && (long long)((d->T + 127) / 128) * ((d->N + 127) / 128) >= 224;
        if (big) {
            const dim3 grid((d->N + 127) / 128, (d->T + 127) / 128, G);
            if (vec) hipLaunchKernelGGL((dense_mfma_kernel<128, 128, true>), grid, dim3(256), 0, s, a);
            else hipLaunchKernelGGL((dense_mfma_kernel<128, 128, false>), grid, dim3(256), 0, s, a);
        } else if (d->N >= 128) {
            const dim3 grid((d->N + 127) / 128, (d->T + 63) / 64, G);
            if (vec) hipLaunchKernelGGL((dense_mfma_kernel<64, 128, true>), grid, dim3(256), 0, s, a);
            else hipLaunchKernelGGL((dense_mfma_kernel<64, 128, false>), grid, dim3(256), 0, s, a);
        } else {
            const dim3 grid((d->N + 63) / 64, (d->T + 63) / 64, G);
            if (vec) hipLaunchKernelGGL((dense_mfma_kernel<64, 64, true>), grid, dim3(256), 0, s, a);
            else hipLaunchKernelGGL((dense_mfma_kernel<64, 64, false>), grid, dim3(256), 0, s, a);
        }
    } else {
        const dim3 grid((d->N + TN - 1) / TN, (d->T + TM - 1) / TM, G);
        hipLaunchKernelGGL(dense_fma_kernel, grid, dim3(256), 0, s, a);
    }
    return last_launch_status();
}

int ntk_dense_few_rows(void) { return kGemvRows; }

int ntk_dense_linear(float* Y, int ldy, const float* X, int ldx, const void* W, int wdtype, int T, int N, int K, int accumulate, void* stream) {
    ntk_dense_desc d{};
    d.Y = Y; d.ldy = ldy; d.X = X; d.ldx = ldx; d.W = W; d.wstride = 0; d.wdtype = wdtype; d.offsets = nullptr; d.G = 1; d.rows = nullptr; d.row_div = 1;
    d.T = T; d.N = N; d.K = K; d.accumulate = accumulate;
    return ntk_dense(&d, stream);
}
