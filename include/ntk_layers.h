/* include/ntk_layers.h -- operators of the layer-list model families (csrc/dense.hip, csrc/latent_attention.hip, csrc/window_attention.hip,
 * csrc/lightning_attention.hip, csrc/gated_recurrence.hip, csrc/moe.hip, csrc/layer_ops.hip): dense bfloat16 / float32 weights, F32 activations and residual stream.
 *
 * Same conventions as ntk.h: plain pointers and sizes, stream ordered, no allocation, NTK_OK or a negative NTK_E_* code.  Nothing here knows a
 * model: every size and constant is a parameter.  Two precisions of one operator set:
 *   weights NTK_DT_BF16 : matrix products on the bf16 matrix cores (activations rounded to bfloat16 at the product's input, F32 accumulation);
 *   weights NTK_DT_F32  : every product in true F32 (FMA on the vector units).
 * Norms, rotary angles, attention scores and weights, routers and the residual sum are F32 in both.
 */
#ifndef NTK_LAYERS_H
#define NTK_LAYERS_H

#include "ntk.h"

#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif
#ifdef __cplusplus
extern "C" {
#endif

/* Y[r][0..N) (+)= X[src(r)][0..K) . W_g[N][K]^T for every row r of every group g.
 *   W        : G matrices [N][K], `wstride` elements apart, dtype NTK_DT_BF16 or NTK_DT_F32
 *   offsets  : device int [G + 1], rows [offsets[g], offsets[g+1]) belong to group g; NULL: one group of T rows
 *   rows     : device int [T], src(r) = rows[r] / row_div; NULL: src(r) = r
 *   T        : number of rows (all groups together); Y rows are `ldy` floats apart, X rows `ldx`
 *   accumulate != 0 : Y += instead of Y =
 * A row's result depends on that row alone (not on T, the group sizes or the row's place) up to the kernel form picked by T. */
typedef struct ntk_dense_desc {
    float* Y; int ldy;
    const float* X; int ldx;
    const void* W; long long wstride; int wdtype;
    const int* offsets; int G;
    const int* rows; int row_div;
    int T, N, K;
    int accumulate;
    /* glu_ff > 0 (only with T <= ntk_dense_few_rows(), N == 2 * glu_ff, no accumulate): W holds glu_ff gate rows then glu_ff up rows and
     * Y[r][f] = g' * sigmoid(glu_alpha * g') * (u' + glu_up_offset), g' = min(gate, glu_limit), u' = clamp(up, -glu_limit, glu_limit) -- the product and ntk_clipped_glu in one launch */
    int glu_ff; float glu_limit, glu_alpha;
    /* norm_w != NULL (only with T <= ntk_dense_few_rows()): every activation row is first divided by sqrt(mean(x^2) + norm_eps) and multiplied by
     * (norm_offset + norm_w[k]), norm_w F32 [K] -- ntk_rmsnorm_offset and the product in one launch */
    const float* norm_w; float norm_eps, norm_offset;
    /* what is added to the (clamped) up value inside the gated activation: 1 for the clipped form above, 0 for a plain gated unit
     * (g * sigmoid(alpha * g) * u; glu_limit = INFINITY switches the clamps off: silu(g) * u with alpha 1) */
    float glu_up_offset;
    /* a cubic term inside the gate's sigmoid: act(g') = g' * sigmoid(glu_alpha * (g' + glu_cubic * g'^3)).  0: none.  alpha = 2 sqrt(2 / pi) and
     * cubic = 0.044715 give the tanh form of gelu, 0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3))), since 0.5 (1 + tanh y) = sigmoid(2 y) */
    float glu_cubic;
} ntk_dense_desc;
int ntk_dense_few_rows(void);   /* up to this many rows a product takes the row-streaming form */
int ntk_dense(const ntk_dense_desc* d, void* stream);
/* the plain case: Y[T][N] = X[T][K] . W[N][K]^T */
int ntk_dense_linear(float* Y, int ldy, const float* X, int ldx, const void* W, int wdtype, int T, int N, int K, int accumulate, void* stream);

/* ---- layer_ops.hip ---------------------------------------------------------------------------------------------------------------- */
/* out[t][:] = table[tokens[t]][:] (table NTK_DT_BF16 or NTK_DT_F32 [vocab][width]); a token outside [0, vocab) gives a row of zeros */
int ntk_embed_dense(float* out, const void* table, int tdtype, const int* tokens, int T, int vocab, int width, void* stream);
/* y[t][:] = x[t][:] / sqrt(mean(x[t]^2) + eps) * (offset + w[:]) for up to two (w, y) pairs sharing x (w F32 [n]; y2 / w2 may be NULL).
 * offset 1: the weight is stored around zero; offset 0: plain.  x rows ldx floats apart, y rows ldy. */
int ntk_rmsnorm_offset(float* y1, const float* w1, float* y2, const float* w2, int ldy, const float* x, int ldx, int T, int n, float eps, float offset,
                       void* stream);
/* out[t] = [a[t] ; b[t]] (two rows of n floats side by side) */
int ntk_concat_rows(float* out, const float* a, const float* b, int T, int n, void* stream);
/* y[i] *= 1 / (1 + exp(-g[i])) over T rows of n (y rows ldy apart, g rows ldg) */
int ntk_sigmoid_gate(float* y, int ldy, const float* g, int ldg, int T, int n, void* stream);
/* dst[0..n) = src[0..n) */
int ntk_rows_copy(float* dst, const float* src, long long n, void* stream);
/* x[i] += a[i] (+ b[i] if b) */
int ntk_residual_add(float* x, const float* a, const float* b, int n, void* stream);

/* out[t][:] = table[tokens[t]][:] * scale */
int ntk_embed_dense_scaled(float* out, const void* table, int tdtype, const int* tokens, int T, int vocab, int width, float scale, void* stream);
/* x[i] *= s */
int ntk_scale(float* x, long long n, float s, void* stream);
/* Layer norm with weight and bias: y[t][:] (+)= (x[t] - mean) / sqrt(var + eps) * w + b, var = mean of the squared deviations (two passes).
 * b may be NULL (no bias); accumulate != 0 adds onto y (the residual sum of a layer whose sublayer output is normed before it is added). */
int ntk_layernorm(float* y, int ldy, const float* x, int ldx, const float* w, const float* b, int T, int n, float eps, int accumulate, void* stream);
/* The input side of a causal convolution over time that is ADDED to its input (out = h + conv(h)), h = layer norm of x:
 * ntk_layernorm_history fills hist [(taps - 1) + T][n]: rows 0 .. taps-2 = the last taps-1 inputs h of the sequence before this portion (from
 * `state` [taps - 1][n]; zeros where the position lies before the sequence's start, i.e. pos0 - (taps-1) + k < 0), rows taps-1 .. = layer norm of x[t].
 * ntk_causal_conv_mix then gives out[t][c] = hist[taps-1+t][c] + sum_j w[c][j] * hist[t+j][c] (w F32 [n][taps], tap taps-1 is the present token)
 * and leaves the portion's last taps-1 rows of hist in `state` for the next portion.  taps >= 1 (taps 1: no state is read or written). */
int ntk_layernorm_history(float* hist, const float* x, int ldx, const float* w, const float* b, const float* state, int taps, int pos0, int T, int n, float eps,
                          void* stream);
int ntk_causal_conv_mix(float* out, int ldo, const float* hist, const float* w, float* state, int taps, int T, int n, void* stream);
/* The whole seam between two sublayers of a layer whose sublayer outputs are normed before they join the stream, in one call:
 *   x[t] += layer norm of add_y[t] with (add_w, add_b)     -- the output still owed to the stream; add_y == NULL: nothing is owed
 *   h[t]  = layer norm of x[t] with (w, b);  out[t] = h[t] + conv(h)[t] as above, `state` carried on.
 * One token runs as ONE launch (the history of a channel belongs to the thread that owns it); more tokens as ntk_layernorm_history's kernel with the owed
 * output folded in, then ntk_causal_conv_mix (hist: [(taps - 1) + T][n] floats of work space, unused for T == 1).  Same sums in the same order either way. */
int ntk_sandwich_norm_conv(float* out, int ldo, float* x, int ldx, const float* add_y, int ldy, const float* add_w, const float* add_b, const float* w, const float* b,
                           const float* canon, float* state, float* hist, int taps, int pos0, int T, int n, float eps, void* stream);
/* y[t][i] = a N(z)_i + b N(z^2)_i + c N(z^3)_i + e with (a, b, c, e) = coef[0..3] (device F32), powers element by element and
 * N(u) = u / sqrt(mean(u^2) + eps) over the row of n values */
int ntk_polynorm(float* y, int ldy, const float* z, int ldz, const float* coef, int T, int n, float eps, void* stream);
/* y[t][i] = x[t][i] / sqrt(mean(x[t]^2) + eps) * w[i] * sigmoid(g[t][i]) (the norm runs over the whole row of n values; g rows ldg apart, g may be NULL) */
int ntk_gated_rmsnorm(float* y, int ldy, const float* x, int ldx, const float* w, const float* g, int ldg, int T, int n, float eps, void* stream);

/* Dynamic-tanh norm (no mean, no variance): y[t][i] = tanh(alpha * x[t][i]) * w[i] + b[i], alpha one number per norm; b may be NULL */
int ntk_dyt(float* y, int ldy, const float* x, int ldx, const float* w, const float* b, float alpha, int T, int n, void* stream);
/* out[t][:] = table[tokens[t]][:] + pos_table[pos0 + t][:] (both NTK_DT_BF16 or both NTK_DT_F32, the sum in F32; a learned vector per position, n_pos rows),
 * then, if w: the dynamic-tanh norm above with (w, b, alpha).  copy (may be NULL) receives the same rows. */
int ntk_embed_positions(float* out, float* copy, const void* table, const void* pos_table, int tdtype, const int* tokens, int T, int vocab, int width, int pos0,
                        int n_pos, const float* w, const float* b, float alpha, void* stream);
/* y[t][i] = y[t][i] * sigmoid(g[t][i] + (gb ? gb[i] : 0)) * scale */
int ntk_sigmoid_gate_scaled(float* y, int ldy, const float* g, int ldg, const float* gb, float scale, int T, int n, void* stream);
/* x[t][i] = tanh(x[t][i]) over T rows of n */
int ntk_tanh_rows(float* x, int ldx, int T, int n, void* stream);
/* Per head: y[t][h][c] = x[t][h][c] / sqrt(mean_c(x[t][h]^2) + eps) * w[h * w_head_stride + c] * act(g[t][h][c]) * scale, the mean over the head's dv values.
 * w_head_stride 0: one weight vector [dv] shared by the heads; dv: a weight per head and column.  act 0: no gate (g unused), 1: sigmoid, 2: silu. */
int ntk_head_rmsnorm_gate(float* y, int ldy, const float* x, int ldx, const float* w, int w_head_stride, const float* g, int ldg, int act, float scale, int T, int H,
                          int dv, float eps, void* stream);
/* The seam of a layer whose sublayer results join the stream through a gate and whose layer results are averaged over depth, in one launch:
 *   r[t]  = x[t] + (y[t] + yb) * sigmoid(g[t] + gb)                (yb, gb: bias vectors [n], may be NULL)
 *   n_hist == 0:  x[t] = r[t]
 *   n_hist  > 0:  hist[n_hist - 1][t] = r[t];  x[t] = sum_{j < n_hist} coef[j] * hist[j][t]   (j ascending, F32; hist entries hist_stride floats apart, rows of n;
 *                 coef device F32 [n_hist])
 *   h != NULL:    h[t] = tanh(alpha * x[t]) * nw + nb               (the dynamic-tanh norm in front of the next sublayer)                              */
typedef struct ntk_gated_seam_desc {
    float* x; int ldx;
    const float* y; int ldy; const float* yb;
    const float* g; int ldg; const float* gb;
    float* hist; long long hist_stride; int n_hist; const float* coef;
    float* h; int ldh; const float* nw; const float* nb; float alpha;
    int T, n;
} ntk_gated_seam_desc;
int ntk_gated_seam(const ntk_gated_seam_desc* d, void* stream);

/* The seam of a layer whose sublayer results are RMS-normed and scaled before they join the stream, in one launch per row:
 *   x[t] += mult * add_y[t] / sqrt(mean(add_y[t]^2) + eps) * add_w      (add_y may be NULL: nothing is owed)
 *   h[t]  = x[t] / sqrt(mean(x[t]^2) + eps) * w                          (h may be NULL: no norm follows)
 * Plain weights (nothing is added to them). */
int ntk_rms_seam(float* h, int ldh, float* x, int ldx, const float* add_y, int ldy, const float* add_w, float mult, const float* w, int T, int n, float eps,
                 void* stream);
/* A short causal convolution over time on every channel, then an activation: y[t][c] = act(sum_j w[c][j] * in(t - (taps - 1) + j)[c]), w F32 [n][taps] (tap
 * taps - 1 weighs the present token), in(.) = x rows of this portion, the carried inputs `state` [taps - 1][n] for the rows before it, zeros before the
 * sequence's start (position pos0 + index < 0).  The portion's last taps - 1 inputs are left in `state`.  act 0: none, 1: silu.  y must not overlap x.
 * 1 <= taps <= 16 (taps 1: no state is read or written). */
int ntk_causal_conv_act(float* y, int ldy, const float* x, int ldx, const float* w, float* state, int taps, int act, int pos0, int T, int n, void* stream);
/* x[t][i] = cap * tanh(x[t][i] / cap) over T rows of n */
int ntk_softcap_rows(float* x, int ldx, float cap, int T, int n, void* stream);
/* y[t][h][0..dv) *= sigmoid(g[t][h]): one gate per token and head (g rows ldg floats apart) */
int ntk_head_gate(float* y, int ldy, const float* g, int ldg, int T, int H, int dv, void* stream);

/* ---- latent_attention.hip ---------------------------------------------------------------------------------------------------------
 * Attention whose keys and values are up-projections of one cached latent per position plus one rotated key part shared by the heads.
 * The cache of a layer run holds rows of `row` = kv_rank + rot_dim floats: [latent (normed) | rotated key part].                       */
typedef struct ntk_rotary {       /* angle of pair i at position p: p * freq[i]; cos and sin times mag */
    const double* freq;           /* device F64 [dims / 2] (after any frequency scaling): angles are formed in double, applied in F32 */
    float mag;
    int dims;                     /* rotated entries at the head of the vector */
    int layout;                   /* NTK_ROT_NEIGHBOURS (0): entries (2i, 2i+1) form pair i; NTK_ROT_HALVES (1): entries (i, i + dims/2) do */
} ntk_rotary;
#define NTK_ROT_NEIGHBOURS 0
#define NTK_ROT_HALVES 1
/* For T tokens at positions pos0 ...: kv [T][ldkv] = [kv_rank raw latent | rot_dim raw key part] -> cache rows pos0 .. pos0+T-1:
 * latent / rms * norm_w, key part rotated (its first rot->dims entries, paired by rot->layout; the rest copied).  q [T][H][qd], ldq floats between tokens: the rot_dim entries at the
 * end of every head rotated in place the same way. */
int ntk_latent_prepare(float* cache, int row, const float* kv, int ldkv, const float* norm_w, float eps, int kv_rank, int rot_dim, float* q, int ldq, int H, int qd,
                       const ntk_rotary* rot, int pos0, int T, void* stream);
/* Softmax attention of query rows over cached positions.  Two forms of one kernel:
 *  expanded (shared == 0): K [nkeys][H][dn] and V [nkeys][H][dv] hold the up-projected keys / values of positions key0 .. key0+nkeys-1
 *           (ldk / ldv floats between positions), q [T][H][dn+dr]; the rotated part of the score reads the cache rows (offset kv_rank).
 *  shared   (shared != 0): q [T][H][R+dr] = [query folded through the key up-projection | rotated part]; keys AND values are the cache rows
 *           themselves (K = [latent | rotated], V = latent): out [T][H][R].  K / V arguments are unused.
 * Query t (position pos0 + t) sees position j iff j <= pos0 + t and (window <= 0 or pos0 + t - j < window).  scale multiplies the whole score.
 * out rows [T][H][dv] (expanded) / [T][H][R] (shared), ldo floats between tokens.  scratch: F32 [>= ntk_latent_attention_scratch(...)] . */
size_t ntk_latent_attention_scratch(int T, int H, int vdim_or_rank, int nkeys);
int ntk_latent_attention(float* out, int ldo, const float* q, int ldq, const float* K, int ldk, const float* V, int ldv, const float* cache, int row,
                         int kv_rank, int rot_dim, int H, int dn, int dv, int shared, int pos0, int T, int key0, int window, float scale, float* scratch,
                         void* stream);
/* fold the unrotated query part through the key up-projection: qf[t][h][0..R) = sum_d q[t][h][d] * W_uk[h*dn + d][0..R), and copy the rotated part behind it
 * (qf [T][H][R+dr]; q rows ldq floats apart); W_uk NTK_DT_BF16 / F32 [H*dn][R] */
int ntk_latent_fold_query(float* qf, const float* q, int ldq, const void* w_uk, int wdtype, int T, int H, int dn, int dr, int R, void* stream);
/* out[t][h*dv + v] = sum_r W_uv[h*dv + v][r] * lat[t][h][r]  (the value up-projection applied after the weighted sum), times sigmoid(gate[t][h*dv+v]) if gate */
int ntk_latent_unfold_value(float* out, int ldo, const float* lat, const void* w_uv, int wdtype, const float* gate, int ldg, int T, int H, int dv, int R,
                            void* stream);
/* ... head_gate != 0: the gate is one number per token and head, gate[t][h] (ldg >= H) */
int ntk_latent_unfold_value_ex(float* out, int ldo, const float* lat, const void* w_uv, int wdtype, const float* gate, int ldg, int head_gate, int T, int H, int dv,
                               int R, void* stream);

/* ---- window_attention.hip ---------------------------------------------------------------------------------------------------------
 * Grouped-query softmax attention over a cache of rotated keys and values, causal with an optional sliding window, with `maps` (1 or 2) score maps per
 * head that share the values.  Cache row of a position: [G][maps][dn] rotated keys | [G][dv] values (row >= G * (maps * dn + dv) floats).
 * Query head h uses key/value head h / (H / G); q [T][H][maps][dn].
 * ntk_window_prepare rotates q in place and k into the cache rows pos0 .. pos0+T-1 (the first rot->dims entries of every map of every head, paired by
 * rot->layout; the rest unchanged) and copies v behind the keys. */
int ntk_window_prepare(float* cache, int row, float* q, int ldq, const float* k, int ldk, const float* v, int ldv, int H, int G, int maps, int dn, int dv,
                       const ntk_rotary* rot, int pos0, int T, void* stream);
/* The same with what a projection leaves to its consumer: q = (q + qb) * (1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)) at position p before the
 * rotation (a query temperature that grows with the position; temp_coef 0: none), k + kb and v + vb into the cache rows.  qb [H*maps*dn], kb [G*maps*dn],
 * vb [G*dv] device F32, each may be NULL.  rot->dims may be 0 (no rotation). */
int ntk_window_prepare_biased(float* cache, int row, float* q, int ldq, const float* k, int ldk, const float* v, int ldv, int H, int G, int maps, int dn, int dv,
                              const ntk_rotary* rot, const float* qb, const float* kb, const float* vb, float temp_coef, double temp_every, int pos0, int T,
                              void* stream);
/* The general form.  Besides the above: values blended with another layer's values of the same tokens on their way into the cache rows,
 * v <- (1 - v_blend) * v + v_blend * v_other[t] (v_other [T][G*dv], ld_other floats between tokens; NULL: no blending), and the values as the projection
 * left them (+ vb) copied to v_keep [T][G*dv] (ld_keep; NULL: not kept) for a later layer to blend with. */
typedef struct ntk_window_prepare_desc {
    float* cache; int row;
    float* q; int ldq; const float* k; int ldk; const float* v; int ldv;
    int H, G, maps, dn, dv;
    const ntk_rotary* rot;
    const float* qb; const float* kb; const float* vb;
    float temp_coef; double temp_every;
    const float* v_other; int ld_other; float v_blend;
    float* v_keep; int ld_keep;
    int pos0, T;
} ntk_window_prepare_desc;
int ntk_window_prepare_ex(const ntk_window_prepare_desc* d, void* stream);
/* a_m = softmax_j(scale * q_m . k_m[j]) V over the visible j (j <= p, and p - j < window if window > 0), per map m.
 * maps == 1: out = a_0.  maps == 2: out = a_0 - lambda * a_1 (a differential pair).  sub_norm != 0: out is then divided by sqrt(mean(out^2) + eps) over
 * the head's dv values.  out_scale multiplies the result.  out [T][H][dv], ldo floats between tokens.
 * Long key ranges of few query rows are cut into `splits` parts that a second launch merges: scratch F32 [>= ntk_window_attention_scratch(...)] (may be NULL when that is 0). */
typedef struct ntk_window_attention_desc {
    float* out; int ldo;
    const float* q; int ldq;
    const float* cache; int row;
    int H, G, maps, dn, dv;
    int pos0, T, window;
    float scale, lambda;
    int sub_norm; float eps, out_scale;
    float* scratch;
    /* a learned bias by distance, added to the scaled score (not scaled itself): rel[bucket_of[min(p - j, n_dist - 1)] * H + h].
     * rel device F32 [buckets][H], bucket_of device int [n_dist].  rel == NULL: none. */
    const float* rel; const int* bucket_of; int n_dist;
    /* mask_mode NTK_MASK_CHUNKS: `window` is a chunk size -- j is visible iff j <= p and floor(j / window) == floor(p / window), chunks counted from
     * position 0 (NTK_MASK_SLIDING, 0: the sliding window above).
     * softcap > 0: the scaled (and biased) score s becomes softcap * tanh(s / softcap).
     * sink != 0: one more term exp(0) in the softmax's denominator (a key of score 0 that carries no value): p_j = exp(s_j) / (1 + sum exp(s)). */
    int mask_mode; float softcap; int sink;
    /* gate != NULL: the result (after the pair, the unit norm and out_scale) times sigmoid(gate[t][h][c]), gate rows ldg floats apart: an elementwise output gate
     * inside the launch that writes the result */
    const float* gate; int ldg;
} ntk_window_attention_desc;
#define NTK_MASK_SLIDING 0
#define NTK_MASK_CHUNKS 1
size_t ntk_window_attention_scratch(int T, int H, int maps, int dv, int nkeys);
int ntk_window_attention(const ntk_window_attention_desc* d, void* stream);

/* ---- lightning_attention.hip -------------------------------------------------------------------------------------------------------
 * Linear attention with a per-head decay: S_t = decay_h S_(t-1) + k_t v_t^T (S [dn][dv] per head, F32), o_t = S_t^T q_t, with q, k, v = act(raw)
 * (act = silu when silu != 0) applied on the way in.  Portions are walked in chunks (scores inside a chunk, the state between chunks), all in F32.
 * q [T][H][dn], k [T][H][dn], v [T][H][dv] with ldq / ldk / ldv floats between tokens; log_decay device F32 [H] = ln(decay_h) (-inf for 0);
 * state [H][dn][dv]: read unless pos0 == 0 (a sequence starts from zeros), written at the end.  out [T][H][dv].  dn <= 256.
 * scratch: F32 [>= ntk_lightning_attention_scratch(...)] lets the chunks of a long portion run side by side (three launches); NULL: one workgroup per
 * (head, 64 value columns) walks them in turn.  Up to 8 tokens (decoding) take a form of their own that keeps the state in registers. */
size_t ntk_lightning_attention_scratch(int T, int H, int dn, int dv);
int ntk_lightning_attention(float* out, int ldo, const float* q, int ldq, const float* k, int ldk, const float* v, int ldv, const float* log_decay, float* state,
                            int H, int dn, int dv, int silu, int pos0, int T, float* scratch, void* stream);

/* ---- gated_recurrence.hip -----------------------------------------------------------------------------------------------------------
 * Linear attention whose state forgets per token, head and KEY CHANNEL, optionally with the delta rule's removal term (taken from S_(t-1) as it was):
 *     S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T,      o_t = S_t^T (q_scale * q_t),      u_t = k_t / sqrt(sum(k_t^2) + unit_eps)
 * S [dn][dv] per head, F32; everything after the projections is F32.  q, k, wz [T][H][dn], v [T][H][dv] (ld* floats between tokens).
 * The decay comes from the raw projection wz (+ wb [H*dn], may be NULL) by `decay_form`:
 *     NTK_DECAY_SIGMOID_ROOT   w = sigmoid(z)^(1 / decay_param)            (formed as exp(log sigmoid(z) / param))
 *     NTK_DECAY_EXP_SIGMOID    w = exp(-decay_param * sigmoid(z))
 *     NTK_DECAY_GIVEN          w = z
 * az (may be NULL: no removal term -- gated linear attention): a = sigmoid(az + ab), [T][H][dn] (+ ab [H*dn], may be NULL).
 * state [H][dn][dv]: read unless pos0 == 0 (a sequence starts from zeros), written at the end.  out [T][H][dv].  dn <= 1024.
 * A lane owns a few state rows of one column and walks its tokens in order.  Without scratch a portion cut anywhere gives the same sums in the same order;
 * with it, where a long portion's segments end changes rounding only. */
#define NTK_DECAY_GIVEN 0
#define NTK_DECAY_SIGMOID_ROOT 1
#define NTK_DECAY_EXP_SIGMOID 2
#define NTK_DECAY_EXP_SOFTPLUS 3
typedef struct ntk_gated_recurrence_desc {
    float* out; int ldo;
    const float* q; int ldq;
    const float* k; int ldk;
    const float* v; int ldv;
    const float* wz; int ldw; const float* wb; int decay_form; float decay_param;
    const float* az; int lda; const float* ab; float unit_eps;
    float* state;
    int H, dn, dv;
    float q_scale;
    int pos0, T;
    float* scratch;   /* F32 [>= ntk_gated_recurrence_scratch(T, H, dn, dv, az != NULL)]: portions of more than a few tokens form their per-token vectors in a launch
                         of their own, once per head instead of once per workgroup, and long portions are walked in segments side by side (their states and
                         what the outputs are still owed are settled by two more launches); NULL: always inside the walk, tokens strictly in turn */
    /* ---- the delta rule with one gate per head (all zero / NULL: the forms above) ----
     * G > 0: q and k have G heads [T][G][dn] and state head h reads head h / (H / G) of them (H % G == 0).
     * unit_q / unit_k != 0: q (before q_scale) / the written key k are divided by sqrt(sum x^2 + unit_eps) over the head's dn entries.
     * head_gates != 0: wz and az hold ONE number per token and head ([T][H], ldw / lda >= H; wb, ab [H]): a decay and a removal rate for all channels.
     * decay_form NTK_DECAY_EXP_SOFTPLUS: w = exp(-rate * softplus(z)), rate = decay_rates[h] (device F32 [H]) or decay_param where that is NULL.
     * write_gated != 0 (needs az and head_gates): the delta rule proper -- the removal is taken from the DECAYED state and the write is scaled by the removal rate:
     *     S' = diag(w_t) S_(t-1),   S_t = S' - a_t u_t (u_t^T S') + a_t k_t v_t^T
     * Any of these makes every portion form its vectors in a launch of its own: scratch must hold ntk_gated_recurrence_scratch_ex(d) floats. */
    int G, unit_q, unit_k, head_gates, write_gated;
    const float* decay_rates;
    /* conv_w != NULL (T == 1 only: a decoded token): q, k, v are RAW projections that first pass the short causal convolution + silu of ntk_causal_conv_act inside
     * the pre-pass's launch -- conv_w F32 [2 G dn + H dv][conv_taps] and the carried inputs conv_state [conv_taps - 1][2 G dn + H dv], channels in the order q | k | v. */
    const float* conv_w; float* conv_state; int conv_taps;
} ntk_gated_recurrence_desc;
size_t ntk_gated_recurrence_scratch(int T, int H, int dn, int dv, int removal);
size_t ntk_gated_recurrence_scratch_ex(const ntk_gated_recurrence_desc* d);   /* from d's T, H, dn, dv, az and the per-head options */
int ntk_gated_recurrence(const ntk_gated_recurrence_desc* d, void* stream);

/* ---- moe.hip ---------------------------------------------------------------------------------------------------------------------- */
/* Router of a mixture of experts, one launch: z = W_r h (F32 weights [E][n]), s = softmax(z); the `top` largest (ties: the lower index), weights
 * s / (sum of the chosen + 1e-20) -> ids [T][top], wts [T][top].  shared_gate_w (F32 [n], may be NULL) -> sgate[t] = sigmoid(w . h[t]).  E <= 256. */
int ntk_moe_route(int* ids, float* wts, float* sgate, const float* h, int ldh, const float* w_router, const float* shared_gate_w, int T, int n, int E, int top,
                  void* stream);
/* The general router.  score 0: s = softmax(z), 1: s = sigmoid(z).  groups > 1: the experts form `groups` equal groups of neighbours, a group's
 * score is the sum of its `group_top` largest s, and only experts of the `keep` best groups can be chosen (ties: the lower index).  The `top` largest
 * allowed s are chosen; weights = s (renorm != 0: divided by the sum of the chosen + 1e-20) * scale. */
typedef struct ntk_route_desc {
    int score;
    int groups, keep, group_top;
    int renorm;
    float scale;
} ntk_route_desc;
int ntk_moe_route_ex(int* ids, float* wts, float* sgate, const float* h, int ldh, const float* w_router, const float* shared_gate_w, int T, int n, int E, int top,
                     const ntk_route_desc* r, void* stream);
/* Stable grouping of the T*top (token, slot) pairs by expert: offsets [E+1], order [T*top] (pair index t*top+slot of every sorted row),
 * where [T*top] (sorted row of every pair). */
int ntk_moe_group(int* offsets, int* order, int* where, const int* ids, int T, int top, int E, void* stream);
/* a[r][f] = g' * sigmoid(alpha * g') * (u' + 1), g' = min(gu[r][f], limit), u' = clamp(gu[r][ff + f], -limit, limit); gu rows of 2*ff, a rows of ff */
int ntk_clipped_glu(float* a, const float* gu, int rows, int ff, float limit, float alpha, void* stream);
/* the general gated unit: a[r][f] = g' * sigmoid(alpha * g') * (u' + up_offset) with the clamps of ntk_clipped_glu (limit = INFINITY: none) */
int ntk_glu(float* a, const float* gu, int rows, int ff, float limit, float alpha, float up_offset, void* stream);
/* ... with a cubic term inside the sigmoid, g' * sigmoid(alpha * (g' + cubic * g'^3)) * (u' + up_offset) (the tanh form of gelu: see ntk_dense_desc), and gu rows
 * ldgu floats apart (gate values at [0, ff), up values at [ff, 2 ff)) */
int ntk_glu_cubic(float* a, const float* gu, int ldgu, int rows, int ff, float limit, float alpha, float cubic, float up_offset, void* stream);
/* out[t][:] = sum_s wts[t][s] * d[where[t*top+s]][:] + (sgate ? sgate[t] : 1) * shared[t][:] (if shared): the experts' sum on its own, for layers that norm it before
 * it joins the stream */
int ntk_moe_sum(float* out, const float* d, const int* where, const float* wts, const float* shared, const float* sgate, int T, int top, int n, void* stream);
/* x[t][:] += mix[t][:] (if mix) + sum_s wts[t][s] * d[where[t*top+s]][:] + sgate[t] * shared[t][:] (if shared) -- slots in order, one rounding sequence per token */
int ntk_moe_combine(float* x, const float* mix, const float* d, const int* where, const float* wts, const float* shared, const float* sgate, int T, int top,
                    int n, void* stream);

#ifdef __cplusplus
}
#endif
#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#endif /* NTK_LAYERS_H */
