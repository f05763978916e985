// engine/layer_stack.h -- model families described by a LIST of layers in config.json (type of mixer, its sizes, its feed-forward), with dense
// bfloat16 weights in a safetensors file: a residual stream in F32, an optional repeated span of layers (each pass with its own cache and state), and an
// output norm + head.  A family fixes the FORM of a layer (StackForm):
//   parallel     x += mixer(norm1 x) + ff(norm2 x), RMS norms whose weight is stored around zero; the repeated span is entered through a projection
//                of [stream ; embedding]                                                                                   -- "Fabolorn"
//   sequential   x += norm1b(mixer(conv(norm1 x))), then x += norm2b(ff(conv(norm2 x))): layer norms with weight and bias before and after every
//                sublayer, a short causal convolution added to every sublayer's input (its last inputs are part of a sequence's state), scaled
//                embedding and logits                                                                                       -- "Nizorax"
//   gated        pre-norm, x += gate * mixer(norm1 x), then x += gate * ff(norm2 x): dynamic-tanh norms (element by element, no row sums), every sublayer's
//                result multiplied by sigmoid(W h + b) of the sublayer's input before it joins the stream, the stream that goes on after a layer a
//                learned weighted sum of ALL layer results so far (and the embedding), a learned vector per position added to the embedding, scaled
//                logits                                                                                                     -- "Tubazen"
//   scaled       x += m * norm1b(mixer(norm1 x)), then x += m * norm2b(ff(norm2 x)): RMS norms with a plain weight before and after every sublayer, one
//                fixed factor m on everything that joins the stream, scaled embedding, the embedding table as the head, capped logits
//                                                                                                                           -- "Fifotar"
//
// Mechanisms are parsed into parameter structs and run by the operators of include/ntk_layers.h, so another family can list them in another order
// or with other constants:
//   mixers        "latent_attention" (query through a normed latent, causal, optional frequency-scaled rotation) and "latent_attention_2" (query from
//                 one matrix, sliding window): one LatentMixer each -- which of the options a layer has is read from its config keys;
//                 "attention": grouped-query attention over rotated keys with a sliding window, as a differential pair of score maps when the
//                 config gives 'diff' (WindowMixer); "lightning": linear attention with a per-head decay and a recurrent state (LightningMixer);
//                 "gla": gated linear attention -- a recurrent state that forgets per token and key channel (decay from a low-rank projection), unit norm
//                 per head, silu gate (GlaMixer); "parallel": two mixers over the same input whose results are added with fixed weights -- grouped-query
//                 softmax attention with projection biases, a query temperature growing with the position and a learned bias by bucketed distance
//                 (BiasedAttention), beside a delta-rule recurrence with per-channel decay and removal rate (DeltaMixer);
//                 in the scaled form "attention" is grouped-query attention without positions over CHUNKS of the sequence, with capped scores, a sink
//                 in the softmax, values blended with those of the first such layer and an elementwise output gate (the same WindowMixer and kernels with
//                 other parameters), "latent_attention" pairs rotated entries half against half and gates per head, and "delta" is the delta rule with
//                 one decay and one write strength per head over unit queries and keys that went through a short convolution (GatedDeltaMixer);
//   feed-forward  kind "moe": routed gated experts + an optional shared expert (MoeFeedForward: softmax or sigmoid scores, optional expert groups,
//                 clipped or plain gated units); kind "dense": up, polynomial activation with unit-norm terms, down (DenseFeedForward), or in the
//                 gated form a gated unit with the tanh form of gelu (GatedFeedForward), in the scaled form the clipped gated unit of the experts as one
//                 dense unit (GatedExperts with one member).
// What a sequence holds per layer run: cache rows per position (attention kinds), a recurrent state (lightning, gla, delta rules), the convolutions' last inputs.
#pragma once
#include <string>
#include <vector>
#include "safetensors.h"
#include "sequence_model.h"
#include "../../../include/ntk_layers.h"

namespace nt {

struct DenseW {                 // a matrix (or a stack of equal matrices) in the model's product dtype, row-major [out][in]
    void* ptr = nullptr;
    int dtype = 0;
    int64_t out_f = 0, in_f = 0;
    int count = 1;
    long long stride() const { return (long long)out_f * in_f; }
};

struct LatentMixer {
    int heads = 0, dim = 0, rot_dim = 0, vdim = 0, kv_rank = 0, q_rank = 0;   // q_rank 0: the query comes from one matrix
    int window = 0;                                                             // 0: causal over everything
    float scale = 1.0f;
    int rot_dims = 0;
    float rot_mag = 1.0f;
    int rot_layout = NTK_ROT_NEIGHBOURS;
    bool head_gate = false;           // the output gate is one number per head (else one per head and value entry)
    double* rot_freq = nullptr;       // device [rot_dims / 2]
    DenseW in;                        // rows [query or query latent | kv_rank + rot_dim | gate] of one product over the normed input
    int q_off = 0, kv_off = 0, g_off = 0;
    DenseW uq, uk, uv, o;
    float* q_norm = nullptr;          // F32 [q_rank]
    float* kv_norm = nullptr;         // F32 [kv_rank]
    int qd() const { return dim + rot_dim; }
    int row() const { return kv_rank + rot_dim; }
};

struct WindowMixer {                  // grouped-query attention, sliding window, one score map per head or a differential pair
    int heads = 0, kv_heads = 0, dim = 0, vdim = 0, maps = 1;
    int window = 0;                   // 0: causal over everything
    float scale = 1.0f;
    float diff = 0.0f, lambda = 0.0f; // maps == 2: out = (a_0 - lambda a_1) / rms * (1 - diff)
    int rot_dims = 0;
    double* rot_freq = nullptr;       // device [rot_dims / 2]
    int mask_mode = NTK_MASK_SLIDING; // what `window` means: a sliding window or chunks of the sequence
    float softcap = 0.0f;             // > 0: scores pass cap * tanh(. / cap)
    bool sink = false;                // one more exp(0) in every softmax's denominator
    bool gated = false;               // elementwise sigmoid gate on the joined heads (its rows sit behind v in `in`)
    bool v_mix = false, v_source = false;   // values blended with those of the first such layer (v_source: this IS that layer, it only keeps them)
    float v_blend = 0.0f;
    DenseW in;                        // rows [q | k | v (| gate)] of one product over the mixer's input
    int k_off = 0, v_off = 0, g_off = 0;
    DenseW o;
    int row() const { return kv_heads * (maps * dim + vdim); }
};

struct GatedDeltaMixer {              // S' = w S, S = S' + k (beta (v - S'^T k))^T with one decay w = exp(-rate softplus(W_a h + bias)) and one beta = sigmoid(W_b h) per head
    int heads = 0, kv_heads = 0, dim = 0, vdim = 0, taps = 1;
    DenseW in;                        // rows [q | k | v | gate | beta | decay] of one product; q and k have kv_heads heads
    int k_off = 0, v_off = 0, g_off = 0, b_off = 0, a_off = 0;
    float* conv = nullptr;            // F32 [channels()][taps]: the short convolutions of q, k and v, one below the other
    float *rates = nullptr, *dt_bias = nullptr;   // F32 [heads]: exp(A_log) and the bias inside the softplus
    float* norm = nullptr;            // F32 [vdim], shared by the heads
    DenseW o;
    int channels() const { return 2 * kv_heads * dim + heads * vdim; }
    size_t recurrent_floats() const { return (size_t)heads * dim * vdim; }
    size_t state_floats() const { return recurrent_floats() + (size_t)(taps - 1) * channels(); }   // [S | the convolutions' last inputs]
};

struct LightningMixer {               // linear attention with a per-head decay; q, k, v through silu, gated RMS norm over the joined heads
    int heads = 0, dim = 0, vdim = 0;
    float* log_decay = nullptr;       // device F32 [heads]
    DenseW in;                        // rows [q | k | v | gate]
    int k_off = 0, v_off = 0, g_off = 0;
    float* norm = nullptr;            // F32 [heads * vdim]
    DenseW o;
    size_t state_floats() const { return (size_t)heads * dim * vdim; }
};

struct GlaMixer {                     // gated linear attention: S = diag(alpha_t) S + k v^T, alpha = sigmoid(W_a2 W_a1 h + b)^(1 / tau) per key channel
    int heads = 0, dim = 0, vdim = 0, rank = 0;
    float tau = 1.0f;
    DenseW in;                        // rows [q | k | v | gate | a1 | residual gate]
    int k_off = 0, v_off = 0, g_off = 0, a_off = 0, rg_off = 0;
    DenseW a2;                        // [heads * dim][rank]
    float* a2_b = nullptr;            // F32 [heads * dim]
    float* norm = nullptr;            // F32 [vdim], shared by the heads
    DenseW o;
    size_t state_floats() const { return (size_t)heads * dim * vdim; }
};

struct BiasedAttention {              // grouped-query softmax attention, causal, no rotation: biases on q / k / v / o, query temperature, bias by bucketed distance
    int heads = 0, kv_heads = 0, dim = 0, vdim = 0, buckets = 0;
    float scale = 1.0f, temp_coef = 0.0f;
    double temp_every = 1.0, bias_max = 1.0;
    float *q_b = nullptr, *k_b = nullptr, *v_b = nullptr;
    float* rel = nullptr;             // F32 [buckets][heads]
    int* bucket_of = nullptr;         // device int [slot capacity]: bucket of every distance
    int q_off = 0, k_off = 0, v_off = 0, g_off = 0;
    int row() const { return kv_heads * (dim + vdim); }
};

struct DeltaMixer {                   // S = diag(w) S - (a u)(u^T S) + k v^T, w = exp(-e^(-1/2) sigmoid(W_w2 tanh(W_w1 h) + w0)), a = sigmoid(W_a h + b), u the unit key
    int heads = 0, dim = 0, rank = 0;
    int r_off = 0, k_off = 0, v_off = 0, g_off = 0, a_off = 0, w1_off = 0;
    DenseW w2;                        // [heads * dim][rank]
    float *w0 = nullptr, *a_b = nullptr, *norm = nullptr;   // F32 [heads * dim] each
    size_t state_floats() const { return (size_t)heads * dim * dim; }
};

struct ParallelMixer {                // left_scale * attention + right_scale * delta rule, both over the same input
    BiasedAttention left;
    DeltaMixer right;
    float left_scale = 1.0f, right_scale = 1.0f;
    DenseW in;                        // rows [left q | k | v | gate | right r | k | v | gate | a | w1 | residual gate] of one product
    int rg_off = 0;
    DenseW o;                         // [width][left heads * vdim + right heads * dim]: both output projections side by side
    float* o_b = nullptr;             // F32 [width]: left_scale * the left output bias
};

struct GatedFeedForward {             // down(gelu_tanh(gate h) * (up h)), its result gated like the mixer's
    int ff = 0;
    DenseW in;                        // rows [gate | up | residual gate]
    DenseW down;
};

struct GatedExperts {                 // `count` experts of the same shape, stacked: gate rows then up rows, and the down matrices
    int ff = 0;
    float limit = 0.0f;               // clamp of the gate (from above) and the up value (both sides); INFINITY: none
    DenseW gate_up, down;
};

struct MoeFeedForward {
    int experts = 0, top = 0;
    ntk_route_desc route{};           // score function, expert groups, renormalisation, scale of the weights
    float glu_alpha = 1.0f, glu_up_offset = 0.0f;   // act(g) = g * sigmoid(alpha g), multiplied by (up + offset)
    float* router = nullptr;          // F32 [experts][width]
    GatedExperts routed;
    bool has_shared = false;
    GatedExperts shared;
    float* shared_gate = nullptr;     // F32 [width]; none: the shared expert is added as it is
};

struct DenseFeedForward {             // down(act(up h)), act = a N(z) + b N(z^2) + c N(z^3) + e
    int ff = 0;
    DenseW up, down;
    float* act = nullptr;             // F32 [4]
};

struct NormW { float* w = nullptr; float* b = nullptr; float alpha = 0.0f; };   // b: layer norm with bias (sequential form) / dynamic tanh with its alpha (gated form); none: RMS norm, weight around zero

enum MixerKind { kMixLatent = 0, kMixWindow = 1, kMixLightning = 2, kMixGla = 3, kMixParallel = 4, kMixGatedDelta = 5 };
enum MlpKind { kMlpNone = 0, kMlpMoe = 1, kMlpDense = 2, kMlpClipped = 3 };

struct StackLayer {
    std::string type;
    int mixer = kMixLatent;
    NormW norm1, norm2, norm1b, norm2b;     // (1b, 2b: the norms after a sublayer, sequential form)
    float* canon1 = nullptr;                // F32 [width][taps]: the convolution on the mixer's input
    float* canon2 = nullptr;                // ... on the feed-forward's input
    LatentMixer mix;
    WindowMixer att;
    LightningMixer lin;
    GlaMixer gla;
    ParallelMixer par;
    GatedDeltaMixer gdl;
    GatedExperts cff;                       // scaled form: one dense clipped gated unit
    GatedFeedForward gff;
    float *rg1_b = nullptr, *rg2_b = nullptr;   // gated form: biases of the residual gates, F32 [width]
    float* depth = nullptr;                 // gated form: weights of the layer results so far (embedding first), device F32 [layer + 2]
    int mlp_kind = kMlpNone;
    bool has_mlp = false;
    MoeFeedForward mlp;
    DenseFeedForward ffn;
    int cache_row() const { return mixer == kMixLatent ? mix.row() : mixer == kMixWindow ? att.row() : mixer == kMixParallel ? par.left.row() : 0; }
    size_t state_floats() const {
        return mixer == kMixLightning ? lin.state_floats() : mixer == kMixGla ? gla.state_floats() : mixer == kMixParallel ? par.right.state_floats() :
               mixer == kMixGatedDelta ? gdl.state_floats() : 0;
    }
};

// what a family fixes about its layers (everything else is read from config.json)
struct StackForm {
    bool sequential = false;          // see the head of this file
    bool gated = false;               // ...
    bool scaled = false;              // ... (none of the three: the parallel form)
    // the scaled form's mechanisms: what its design fixes about them
    bool mask_chunks = false;         // an attention layer's mask.size is a chunk size (else a sliding window)
    bool attention_sink = false;      // its softmax has a sink
    bool attention_gate = false;      // ... and an elementwise output gate
    bool rot_halves = false;          // rotated entries are paired half against half (else neighbours)
    bool latent_head_gate = false;    // latent attention's output gate is one number per head
    bool loop_projection = true;      // the repeated span is entered through 'loop.in' over [stream ; embedding]
    int router_score = 0;             // 0 softmax, 1 sigmoid
    bool router_renorm = true;
    bool clipped_glu = true;          // experts: clipped gated unit with slope kGluAlpha and up + 1; else silu(gate) * up
    bool shared_gate = true;          // the shared expert sits behind a per-token sigmoid gate
    int group_top = 2;                // a group's score: the sum of this many of its largest scores
};

class LayerStackModel : public SequenceModel {
public:
    explicit LayerStackModel(const StackForm& form) : form_(form) {}
    ~LayerStackModel() override;
    int load(const std::string& dir, const SeqLoadOptions& opt) override;
    const SeqModelInfo& info() const override { return info_; }
    const std::string& error() const override { return err_; }
    uint64_t weight_bytes() const override { return weight_bytes_; }
    int acquire_slot() override;
    int release_slot(int slot) override;
    int slot_length(int slot) const override { return slots_.length(slot); }
    int truncate_slot(int slot, int length) override;
    float* forward(int slot, const int* tokens, int n, const int* want, int n_want) override;
    int copy_logits(float* host, int rows) override;
    int set_capture(bool on) override { capture_ = on; return 0; }
    int copy_capture(float* host) override;
    int sync() override;
    void* stream() const override { return stream_; }
    static constexpr int kSharedRows = 8;     // up to this many tokens per portion take the decode form of the mixer (and the GEMV form of the products)

private:
    struct Run { int layer; bool enters; float* cache; float* state; float* conv; };   // per slot: cache rows, recurrent state, [2][taps - 1][width] last inputs
    int fail(int st, const std::string& why) { err_ = why; return st; }
    int parse(const ModelFolder& f);
    int parse_mixer(const Json& L, const std::string& type, LatentMixer& m);
    int parse_window(const Json& L, WindowMixer& m);
    int parse_lightning(const Json& L, LightningMixer& m);
    int parse_gla(const Json& L, GlaMixer& m);
    int parse_parallel(const Json& L, ParallelMixer& m);
    int upload_gated_mixer(const ModelFolder& f, const std::string& p, int i, StackLayer& L);
    int upload_hstack(const ModelFolder& f, const std::vector<std::string>& names, DenseW& out);
    int read_scalar(const ModelFolder& f, const std::string& name, float* out);
    int run_gla(const StackLayer& L, float* state, int T, int pos0);
    int run_parallel(const StackLayer& L, float* cache, float* state, int T, int pos0);
    int run_gated_ff(const StackLayer& L, int T);
    int parse_gated_delta(const Json& L, GatedDeltaMixer& m);
    int run_gated_delta(const StackLayer& L, float* state, int T, int pos0);
    int run_clipped_ff(const StackLayer& L, int T);
    int rms_seam(const NormW& nw, float* out, int T);
    int scaled_layer(const Run& run, const StackLayer& L, int slot, int T, int pos0);
    int gated_layer(size_t r, const StackLayer& L, int slot, int T, int pos0);
    int parse_mlp(const Json& ml, const std::string& where, StackLayer& S);
    int upload_norm(const ModelFolder& f, const std::string& name, NormW& out);
    int upload_mixer(const ModelFolder& f, const std::string& p, int i, StackLayer& L);
    int upload_mlp(const ModelFolder& f, const std::string& p, int i, StackLayer& L);
    int upload_layer(const ModelFolder& f, int i, StackLayer& L);
    int upload_vector(const ModelFolder& f, const std::string& name, int64_t n, float** out);
    int upload_matrix(const ModelFolder& f, const std::vector<std::string>& names, int64_t in_f, DenseW& out, int count = 1);
    int alloc_buffers();
    void* dev_alloc(size_t bytes);
    int portion(int slot, const int* tokens_dev, int T, int pos0, const int* want_dev, int n_want, float* logits_out);
    int run_mixer(const StackLayer& L, float* cache, int T, int pos0, bool normed_input = false);
    int run_window(const StackLayer& L, float* cache, int T, int pos0);
    int run_lightning(const StackLayer& L, float* state, int T, int pos0);
    int run_moe(const StackLayer& L, int T, bool into_stream);
    int run_dense_ff(const StackLayer& L, int T);
    int run_experts(float glu_alpha, float glu_up_offset, const GatedExperts& ex, const float* h, float* gu, float* act, float* out, int rows, const int* offsets, const int* order, int top);
    int norm_conv(const NormW& nw, const float* canon, float* conv_state, float* out, int T, int pos0);
    int settle(int T);
    int sequential_layer(const Run& run, const StackLayer& L, int slot, int T, int pos0);
    int parallel_layer(const Run& run, const StackLayer& L, int slot, int T, int pos0);

    struct Owed { const float* y = nullptr; NormW nb; };   // sequential form: a sublayer's output that its norm has yet to add to the stream
    Owed owed_;
    StackForm form_;
    SeqModelInfo info_;
    std::string err_;
    SeqLoadOptions opt_;
    int wdtype_ = NTK_DT_BF16;
    float eps_ = 1e-6f;
    int taps_ = 1;                    // the input convolutions' taps (sequential form)
    float embed_scale_ = 1.0f, logit_scale_ = 1.0f;
    float residual_mult_ = 1.0f, logit_softcap_ = 0.0f;   // scaled form
    float norm_offset_ = 1.0f;        // what is added to an RMS norm's stored weight: 1 where weights are stored around zero, 0 where plain
    bool has_state_ = false;          // some layer carries a recurrent state or convolution inputs: a slot can only be cut back to its start
    std::vector<StackLayer> layers_;
    std::vector<Run> runs_;
    bool has_loop_ = false;
    DenseW embed_, head_, loop_in_, pos_;   // pos_: a learned vector per position (gated form)
    NormW embed_norm_;
    int n_positions_ = 0;             // rows of the position table
    NormW final_norm_;
    uint64_t weight_bytes_ = 0;
    std::vector<void*> allocs_;
    SlotTable slots_;
    void* stream_ = nullptr;
    int chunk_ = 0;                   // tokens per internal portion
    // maxima over the layers (buffer sizes)
    int max_ffn_ = 0, max_in_ = 0, max_qrank_ = 0, max_hqd_ = 0, max_hdv_ = 0, max_hdn_ = 0, max_fold_ = 0, max_hr_ = 0, max_top_ = 0, max_e_ = 0, max_ff2_ = 0, max_sff2_ = 0;
    // activations
    float *x_ = nullptr, *x0_ = nullptr, *cat_ = nullptr, *h1_ = nullptr, *h2_ = nullptr, *a_ = nullptr, *cq_ = nullptr, *q_ = nullptr, *qf_ = nullptr, *lat_ = nullptr,
          *att_ = nullptr, *kx_ = nullptr, *vx_ = nullptr, *mix_ = nullptr, *wts_ = nullptr, *sg_ = nullptr, *gu_ = nullptr, *act_ = nullptr, *dn_ = nullptr,
          *sgu_ = nullptr, *sact_ = nullptr, *sdn_ = nullptr, *scratch_ = nullptr, *xw_ = nullptr, *hn_ = nullptr, *hist_ = nullptr, *ff_ = nullptr, *zf_ = nullptr, *wscratch_ = nullptr, *lscratch_ = nullptr,
          *results_ = nullptr, *zq_ = nullptr, *gu2_ = nullptr, *rscratch_ = nullptr, *cv_ = nullptr, *vfirst_ = nullptr;   // gated form: the layer results of the pass [runs + 1][chunk][width], decay pre-activations, [gate | up | residual gate]
    int max_rec_ = 0, max_gu2_ = 0, max_conv_ = 0, max_gv_ = 0;   // (scaled form: convolution channels, key heads x value size of the blending attention layers)
    int *ids_ = nullptr, *offsets_ = nullptr, *order_ = nullptr, *where_ = nullptr, *tokens_dev_ = nullptr, *want_dev_ = nullptr;
    int* h_stage_ = nullptr;          // pinned: tokens and wanted places of the pass being launched
    float* logits_ = nullptr;
    size_t logits_rows_ = 0;
    int last_rows_ = 0;
    bool capture_ = false;
    float* capture_buf_ = nullptr;
    size_t capture_floats_ = 0;
    int capture_T_ = 0;
};

}  // namespace nt
