// engine/layer_stack.cpp -- see layer_stack.h
#include "layer_stack.h"

#include <algorithm>
#include <cmath>
#include <cstring>

namespace nt {

#define LS_TRY(expr)                          \
    do {                                      \
        const int st__ = (expr);              \
        if (st__ != NTK_OK) return st__;      \
    } while (0)

static constexpr float kGluAlpha = 1.702f;   // the slope of the clipped gated unit's activation
static StackForm parallel_form() { return StackForm{}; }
static StackForm sequential_form() {
    StackForm f;
    f.sequential = true; f.loop_projection = false; f.router_score = 1; f.router_renorm = false; f.clipped_glu = false; f.shared_gate = false; f.group_top = 2;
    return f;
}
static StackForm gated_form() {
    StackForm f;
    f.gated = true; f.loop_projection = false;
    return f;
}
static StackForm scaled_form() {
    StackForm f;
    f.scaled = true; f.loop_projection = false;
    f.mask_chunks = true; f.attention_sink = true; f.attention_gate = true; f.rot_halves = true; f.latent_head_gate = true;
    return f;
}
// what the gated form's mechanisms fix
static constexpr float kGeluAlpha = 1.5957691216057308f;   // 2 sqrt(2 / pi): 0.5 (1 + tanh y) = sigmoid(2 y)
static constexpr float kGeluCubic = 0.044715f;
static constexpr float kDeltaDecayRate = 0.6065306597126334f;   // exp(-1/2): w = exp(-rate * sigmoid(.))
static constexpr float kUnitKeyEps = 1e-6f;
static FamilyRegistrar reg_fifotar("Fifotar", [] { return std::unique_ptr<SequenceModel>(new LayerStackModel(scaled_form())); });
static FamilyRegistrar reg_tubazen("Tubazen", [] { return std::unique_ptr<SequenceModel>(new LayerStackModel(gated_form())); });
static FamilyRegistrar reg_fabolorn("Fabolorn", [] { return std::unique_ptr<SequenceModel>(new LayerStackModel(parallel_form())); });
static FamilyRegistrar reg_nizorax("Nizorax", [] { return std::unique_ptr<SequenceModel>(new LayerStackModel(sequential_form())); });

LayerStackModel::~LayerStackModel() {
    if (stream_) ntk_stream_synchronize(stream_);
    for (void* p : allocs_) nt_hip_free(p);
    if (logits_) nt_hip_free(logits_);
    if (capture_buf_) nt_hip_free(capture_buf_);
    if (h_stage_) nt_hip_free_host(h_stage_);
}

void* LayerStackModel::dev_alloc(size_t bytes) {
    void* p = nt_hip_malloc(bytes ? bytes : 16);
    if (p) allocs_.push_back(p);
    return p;
}

// ------------------------------------------------------------------------------------------------------------------------ configuration
static bool need_int(const Json& o, const char* key, int& out, std::string& err, const std::string& where) {
    if (!o.at(key).is_number()) { err = where + ": '" + key + "' is missing"; return false; }
    out = (int)o.at(key).integer();
    if (out <= 0) { err = where + ": '" + key + "' must be positive"; return false; }
    return true;
}

int LayerStackModel::parse_mixer(const Json& L, const std::string& type, LatentMixer& m) {
    const Json& mx = L.at("mixer");
    const std::string where = "mixer '" + type + "'";
    if (!mx.is_object()) return fail(NTK_E_FORMAT, where + ": no 'mixer' object");
    if (!need_int(mx, "heads", m.heads, err_, where) || !need_int(mx, "dim", m.dim, err_, where) || !need_int(mx, "rot_dim", m.rot_dim, err_, where) ||
        !need_int(mx, "vdim", m.vdim, err_, where) || !need_int(mx, "kv_rank", m.kv_rank, err_, where))
        return NTK_E_FORMAT;
    if (type == "latent_attention") {
        if (!need_int(mx, "q_rank", m.q_rank, err_, where)) return NTK_E_FORMAT;
    } else {
        m.q_rank = 0;
    }
    if (!mx.at("scale").is_number()) return fail(NTK_E_FORMAT, where + ": 'scale' is missing");
    m.scale = (float)mx.at("scale").number();
    m.window = 0;
    if (mx.has("mask")) {
        if (!need_int(mx.at("mask"), "size", m.window, err_, where + " mask")) return NTK_E_FORMAT;
    } else if (type == "latent_attention_2") {
        return fail(NTK_E_FORMAT, where + ": 'mask' is missing");
    }
    const Json& rot = mx.at("rot");
    if (!rot.is_object() || !rot.at("base").is_number()) return fail(NTK_E_FORMAT, where + ": 'rot' is missing");
    m.rot_dims = rot.has("dims") ? (int)rot.at("dims").integer() : m.rot_dim;
    if (m.rot_dims < 0 || (m.rot_dims & 1) || m.rot_dims > m.rot_dim) return fail(NTK_E_FORMAT, where + ": rot.dims must be even and at most rot_dim");
    const double base = rot.at("base").number();
    const int half = m.rot_dims / 2;
    std::vector<double> f((size_t)std::max(half, 1));
    for (int i = 0; i < half; ++i) f[(size_t)i] = std::pow(base, -2.0 * i / m.rot_dims);
    m.rot_mag = 1.0f;
    if (rot.has("scaling")) {
        const Json& sc = rot.at("scaling");
        const double factor = sc.at("factor").number(1.0), orig = sc.at("original").number(1.0), fast = sc.at("fast").number(1.0), slow = sc.at("slow").number(1.0);
        auto where_dim = [&](double turns) { return m.rot_dims * std::log(orig / (2.0 * M_PI * turns)) / (2.0 * std::log(base)); };
        const double lo = std::max(std::floor(where_dim(fast)), 0.0), hi = std::min(std::ceil(where_dim(slow)), (double)m.rot_dims - 1.0);
        for (int i = 0; i < half; ++i) {
            const double ramp = std::min(std::max((i - lo) / std::max(hi - lo, 0.001), 0.0), 1.0);
            f[(size_t)i] = f[(size_t)i] / factor * ramp + f[(size_t)i] * (1.0 - ramp);
        }
        m.rot_mag = (float)(0.1 * std::log(factor) + 1.0);
    }
    m.rot_layout = form_.rot_halves ? NTK_ROT_HALVES : NTK_ROT_NEIGHBOURS;
    m.head_gate = form_.latent_head_gate;
    m.rot_freq = (double*)dev_alloc(f.size() * sizeof(double));
    if (!m.rot_freq) return fail(NTK_E_NOMEM, "out of device memory");
    nt_hip_memcpy_h2d(m.rot_freq, f.data(), f.size() * sizeof(double));
    return NTK_OK;
}

// rotary frequencies base^(-2i/dims), optionally rescaled by wavelength: kept below original/high, divided by factor above original/low, blended between
static std::vector<double> wavelength_scaled_frequencies(const Json& rot, int dims) {
    const double base = rot.at("base").number(10000.0);
    const int half = dims / 2;
    std::vector<double> f((size_t)std::max(half, 1));
    for (int i = 0; i < half; ++i) f[(size_t)i] = std::pow(base, -2.0 * i / dims);
    if (rot.has("scaling")) {
        const Json& sc = rot.at("scaling");
        const double factor = sc.at("factor").number(1.0), orig = sc.at("original").number(1.0), low = sc.at("low").number(1.0), high = sc.at("high").number(1.0);
        for (int i = 0; i < half; ++i) {
            const double fr = f[(size_t)i], wl = 2.0 * M_PI / fr;
            if (wl < orig / high) continue;
            if (wl > orig / low) { f[(size_t)i] = fr / factor; continue; }
            const double sm = (orig / wl - low) / (high - low);
            f[(size_t)i] = (1.0 - sm) * fr / factor + sm * fr;
        }
    }
    return f;
}

int LayerStackModel::parse_window(const Json& L, WindowMixer& m) {
    const Json& mx = L.at("mixer");
    const std::string where = "mixer 'attention'";
    if (!mx.is_object()) return fail(NTK_E_FORMAT, where + ": no 'mixer' object");
    if (!need_int(mx, "heads", m.heads, err_, where) || !need_int(mx, "dim", m.dim, err_, where) || !need_int(mx, "vdim", m.vdim, err_, where)) return NTK_E_FORMAT;
    m.kv_heads = m.heads;
    if (mx.has("kv_heads") && !need_int(mx, "kv_heads", m.kv_heads, err_, where)) return NTK_E_FORMAT;
    if (m.heads % m.kv_heads) return fail(NTK_E_FORMAT, where + ": heads must be a multiple of kv_heads");
    if (!mx.at("scale").is_number()) return fail(NTK_E_FORMAT, where + ": 'scale' is missing");
    m.scale = (float)mx.at("scale").number();
    m.maps = mx.has("diff") ? 2 : 1;
    m.diff = (float)mx.at("diff").number(0.0);
    m.window = 0;
    if (mx.has("mask") && !need_int(mx.at("mask"), "size", m.window, err_, where + " mask")) return NTK_E_FORMAT;
    m.mask_mode = form_.mask_chunks ? NTK_MASK_CHUNKS : NTK_MASK_SLIDING;
    m.sink = form_.attention_sink;
    m.gated = form_.attention_gate;
    m.softcap = (float)mx.at("softcap").number(0.0);
    if (m.softcap < 0.0f) return fail(NTK_E_FORMAT, where + ": 'softcap' must be positive");
    m.v_mix = form_.scaled && mx.at("v_mix").truth();
    m.rot_dims = 0;
    std::vector<double> f(1, 0.0);
    if (mx.has("rot")) {
        const Json& rot = mx.at("rot");
        m.rot_dims = rot.has("dims") ? (int)rot.at("dims").integer() : m.dim;
        if (m.rot_dims < 0 || (m.rot_dims & 1) || m.rot_dims > m.dim) return fail(NTK_E_FORMAT, where + ": rot.dims must be even and at most dim");
        f = wavelength_scaled_frequencies(rot, m.rot_dims);
    }
    m.rot_freq = (double*)dev_alloc(f.size() * sizeof(double));
    if (!m.rot_freq) return fail(NTK_E_NOMEM, "out of device memory");
    nt_hip_memcpy_h2d(m.rot_freq, f.data(), f.size() * sizeof(double));
    return NTK_OK;
}

int LayerStackModel::parse_lightning(const Json& L, LightningMixer& m) {
    const Json& mx = L.at("mixer");
    const std::string where = "mixer 'lightning'";
    if (!mx.is_object()) return fail(NTK_E_FORMAT, where + ": no 'mixer' object");
    if (!need_int(mx, "heads", m.heads, err_, where) || !need_int(mx, "dim", m.dim, err_, where) || !need_int(mx, "vdim", m.vdim, err_, where)) return NTK_E_FORMAT;
    if (m.dim > 256) return fail(NTK_E_SHAPE, where + ": dim up to 256 is supported");
    const Json& dc = mx.at("decay");
    std::vector<float> ld((size_t)m.heads);
    for (int h = 0; h < m.heads; ++h) {
        double d;
        if (dc.is_number()) d = dc.number();
        else if (dc.is_array() && (int)dc.arr.size() == m.heads && dc.arr[(size_t)h].is_number()) d = dc.arr[(size_t)h].number();
        else return fail(NTK_E_FORMAT, where + ": 'decay' must be a number or one number per head");
        if (d < 0.0 || d > 1.0) return fail(NTK_E_FORMAT, where + ": a decay lies in [0, 1]");
        ld[(size_t)h] = d > 0.0 ? (float)std::log(d) : -INFINITY;
    }
    m.log_decay = (float*)dev_alloc(ld.size() * sizeof(float));
    if (!m.log_decay) return fail(NTK_E_NOMEM, "out of device memory");
    nt_hip_memcpy_h2d(m.log_decay, ld.data(), ld.size() * sizeof(float));
    return NTK_OK;
}

int LayerStackModel::parse_gla(const Json& L, GlaMixer& m) {
    const Json& mx = L.at("mixer");
    const std::string where = "mixer 'gla'";
    if (!mx.is_object()) return fail(NTK_E_FORMAT, where + ": no 'mixer' object");
    if (!need_int(mx, "heads", m.heads, err_, where) || !need_int(mx, "dim", m.dim, err_, where) || !need_int(mx, "vdim", m.vdim, err_, where)) return NTK_E_FORMAT;
    if (!mx.at("tau").is_number() || !(mx.at("tau").number() > 0.0)) return fail(NTK_E_FORMAT, where + ": 'tau' must be a positive number");
    m.tau = (float)mx.at("tau").number();
    if (m.dim > 1024 || m.vdim > 1024) return fail(NTK_E_SHAPE, where + ": dim and vdim up to 1024 are supported");
    return NTK_OK;
}

int LayerStackModel::parse_gated_delta(const Json& L, GatedDeltaMixer& m) {
    const Json& mx = L.at("mixer");
    const std::string where = "mixer 'delta'";
    if (!mx.is_object()) return fail(NTK_E_FORMAT, where + ": no 'mixer' object");
    if (!need_int(mx, "heads", m.heads, err_, where) || !need_int(mx, "dim", m.dim, err_, where) || !need_int(mx, "vdim", m.vdim, err_, where)) return NTK_E_FORMAT;
    m.kv_heads = m.heads;
    if (mx.has("kv_heads") && !need_int(mx, "kv_heads", m.kv_heads, err_, where)) return NTK_E_FORMAT;
    if (m.heads % m.kv_heads) return fail(NTK_E_FORMAT, where + ": heads must be a multiple of kv_heads");
    m.taps = 1;
    if (mx.has("conv") && !need_int(mx, "conv", m.taps, err_, where)) return NTK_E_FORMAT;
    if (m.taps > 16) return fail(NTK_E_SHAPE, where + ": convolutions of up to 16 taps are supported");
    if (m.dim > 1024 || m.vdim > 1024) return fail(NTK_E_SHAPE, where + ": dim and vdim up to 1024 are supported");
    return NTK_OK;
}

int LayerStackModel::parse_parallel(const Json& L, ParallelMixer& m) {
    const Json& mx = L.at("mixer");
    const std::string where = "mixer 'parallel'";
    if (!mx.is_object() || !mx.at("left").is_object() || !mx.at("right").is_object()) return fail(NTK_E_FORMAT, where + ": 'mixer' needs 'left' and 'right'");
    const Json& l = mx.at("left");
    const Json& r = mx.at("right");
    BiasedAttention& a = m.left;
    if (!need_int(l, "heads", a.heads, err_, where + " left") || !need_int(l, "dim", a.dim, err_, where + " left") || !need_int(l, "vdim", a.vdim, err_, where + " left")) return NTK_E_FORMAT;
    a.kv_heads = a.heads;
    if (l.has("kv_heads") && !need_int(l, "kv_heads", a.kv_heads, err_, where + " left")) return NTK_E_FORMAT;
    if (a.heads % a.kv_heads) return fail(NTK_E_FORMAT, where + ": heads must be a multiple of kv_heads");
    if (!l.at("scale").is_number()) return fail(NTK_E_FORMAT, where + ": 'scale' is missing");
    a.scale = (float)l.at("scale").number();
    if (!l.at("bias_max").is_number() || !(l.at("bias_max").number() > 0.0)) return fail(NTK_E_FORMAT, where + ": 'bias_max' is missing");
    a.bias_max = l.at("bias_max").number();
    a.temp_coef = 0.0f; a.temp_every = 1.0;
    if (l.has("q_temp")) {
        a.temp_coef = (float)l.at("q_temp").at("coef").number(0.0);
        a.temp_every = l.at("q_temp").at("every").number(1.0);
        if (!(a.temp_every > 0.0)) return fail(NTK_E_FORMAT, where + ": q_temp.every must be positive");
    }
    if (a.vdim > 512) return fail(NTK_E_SHAPE, where + ": vdim up to 512 is supported");
    if (!need_int(r, "heads", m.right.heads, err_, where + " right") || !need_int(r, "dim", m.right.dim, err_, where + " right")) return NTK_E_FORMAT;
    if (m.right.dim > 1024) return fail(NTK_E_SHAPE, where + ": dim up to 1024 is supported");
    m.left_scale = (float)mx.at("left_scale").number(1.0);
    m.right_scale = (float)mx.at("right_scale").number(1.0);
    return NTK_OK;
}

int LayerStackModel::parse_mlp(const Json& ml, const std::string& where, StackLayer& S) {
    const std::string kind = ml.at("kind").is_string() ? ml.at("kind").str : "moe";
    if (kind == "dense" && form_.scaled) {
        S.mlp_kind = kMlpClipped;
        if (!need_int(ml, "ff", S.cff.ff, err_, where)) return NTK_E_FORMAT;
        S.cff.limit = ml.at("limit").is_number() ? (float)ml.at("limit").number() : INFINITY;
        if (!(S.cff.limit > 0.0f)) return fail(NTK_E_FORMAT, where + ": 'limit' must be positive");
        return NTK_OK;
    }
    if (kind == "dense") {
        S.mlp_kind = kMlpDense;
        if (!need_int(ml, "ff", form_.gated ? S.gff.ff : S.ffn.ff, err_, where)) return NTK_E_FORMAT;
        return NTK_OK;
    }
    if (form_.gated || form_.scaled) return fail(NTK_E_FORMAT, where + ": this family has the dense feed-forward only");
    if (kind != "moe") return fail(NTK_E_FORMAT, where + ": unknown kind '" + kind + "'");
    S.mlp_kind = kMlpMoe;
    MoeFeedForward& M = S.mlp;
    const Json& rt = ml.at("router");
    if (!need_int(rt, "experts", M.experts, err_, where) || !need_int(rt, "top", M.top, err_, where) || !need_int(ml.at("expert"), "ff", M.routed.ff, err_, where))
        return NTK_E_FORMAT;
    if (M.top > M.experts || M.experts > 255) return fail(NTK_E_FORMAT, where + ": top <= experts <= 255 is required");
    M.route.score = form_.router_score;
    M.route.renorm = form_.router_renorm ? 1 : 0;
    M.route.scale = (float)rt.at("scale").number(1.0);
    M.route.groups = 1; M.route.keep = 1; M.route.group_top = form_.group_top;
    if (rt.has("groups")) {
        if (!need_int(rt.at("groups"), "count", M.route.groups, err_, where + " groups") || !need_int(rt.at("groups"), "keep", M.route.keep, err_, where + " groups")) return NTK_E_FORMAT;
        if (M.experts % M.route.groups || M.route.keep > M.route.groups || (long long)M.route.keep * (M.experts / M.route.groups) < M.top)
            return fail(NTK_E_FORMAT, where + ": groups must divide the experts and the kept groups must hold 'top' experts");
    }
    if (form_.clipped_glu) { M.glu_alpha = kGluAlpha; M.glu_up_offset = 1.0f; M.routed.limit = (float)ml.at("expert").at("limit").number(); }
    else { M.glu_alpha = 1.0f; M.glu_up_offset = 0.0f; M.routed.limit = INFINITY; }
    M.has_shared = ml.has("shared");
    if (M.has_shared) {
        if (!need_int(ml.at("shared"), "ff", M.shared.ff, err_, where + " shared")) return NTK_E_FORMAT;
        M.shared.limit = form_.clipped_glu ? (float)ml.at("shared").at("limit").number() : INFINITY;
    }
    return NTK_OK;
}

int LayerStackModel::parse(const ModelFolder& f) {
    const Json& c = f.config();
    info_.architecture = c.at("architecture").str;
    if (!need_int(c, "vocab", info_.vocab, err_, "config") || !need_int(c, "width", info_.width, err_, "config")) return NTK_E_FORMAT;
    eps_ = (float)c.at("norm").at("eps").number(1e-6);
    if (form_.sequential) {
        taps_ = (int)c.at("canon").at("taps").integer(1);
        if (taps_ < 1 || taps_ > 64) return fail(NTK_E_FORMAT, "config: canon.taps must lie in 1 .. 64");
        embed_scale_ = (float)c.at("embedding").at("scale").number(1.0);
        logit_scale_ = (float)c.at("logit_scale").number(1.0);
        has_state_ = taps_ > 1;
    }
    if (form_.gated) {
        logit_scale_ = (float)c.at("logit_scale").number(1.0);
        has_state_ = true;
    }
    if (form_.scaled) {
        embed_scale_ = (float)c.at("embedding").at("scale").number(1.0);
        residual_mult_ = (float)c.at("residual_mult").number(1.0);
        logit_softcap_ = (float)c.at("logit_softcap").number(0.0);
        if (logit_softcap_ < 0.0f) return fail(NTK_E_FORMAT, "config: logit_softcap must be positive");
        norm_offset_ = 0.0f;
    }
    if (c.at("bos").is_number()) info_.bos = (int)c.at("bos").integer();
    if (c.at("eos").is_number()) info_.eos = (int)c.at("eos").integer();
    const Json& ls = c.at("layers");
    if (!ls.is_array() || ls.arr.empty()) return fail(NTK_E_FORMAT, "config: 'layers' is missing");
    layers_.resize(ls.arr.size());
    for (size_t i = 0; i < ls.arr.size(); ++i) {
        const Json& L = ls.arr[i];
        StackLayer& S = layers_[i];
        S.type = L.at("type").str;
        // which mixers a form lists: the parallel form's layers read two norms of one input, so its mixers are the latent kinds it was built around
        if (form_.scaled && S.type == "attention") { S.mixer = kMixWindow; LS_TRY(parse_window(L, S.att)); }
        else if (form_.scaled && S.type == "latent_attention") { S.mixer = kMixLatent; LS_TRY(parse_mixer(L, S.type, S.mix)); }
        else if (form_.scaled && S.type == "delta") { S.mixer = kMixGatedDelta; LS_TRY(parse_gated_delta(L, S.gdl)); has_state_ = true; }
        else if (form_.scaled) return fail(NTK_E_FORMAT, "layer " + std::to_string(i) + ": unknown mixer type '" + S.type + "'");
        else if (form_.gated && S.type == "gla") { S.mixer = kMixGla; LS_TRY(parse_gla(L, S.gla)); }
        else if (form_.gated && S.type == "parallel") { S.mixer = kMixParallel; LS_TRY(parse_parallel(L, S.par)); }
        else if (form_.gated) return fail(NTK_E_FORMAT, "layer " + std::to_string(i) + ": unknown mixer type '" + S.type + "'");
        else if (!form_.sequential && (S.type == "latent_attention" || S.type == "latent_attention_2")) { S.mixer = kMixLatent; LS_TRY(parse_mixer(L, S.type, S.mix)); }
        else if (form_.sequential && S.type == "attention") { S.mixer = kMixWindow; LS_TRY(parse_window(L, S.att)); }
        else if (form_.sequential && S.type == "lightning") { S.mixer = kMixLightning; LS_TRY(parse_lightning(L, S.lin)); has_state_ = true; }
        else return fail(NTK_E_FORMAT, "layer " + std::to_string(i) + ": unknown mixer type '" + S.type + "'");
        S.has_mlp = L.has("mlp") && !L.at("mlp").is_null();
        if (S.has_mlp) LS_TRY(parse_mlp(L.at("mlp"), "layer " + std::to_string(i) + " mlp", S));
        if (!form_.sequential && !form_.gated && !form_.scaled && S.mlp_kind == kMlpDense) return fail(NTK_E_FORMAT, "layer " + std::to_string(i) + ": this family has no dense feed-forward");
    }
    // the order of layer runs
    const int n = (int)layers_.size();
    runs_.clear();
    has_loop_ = c.has("loop") && !form_.gated && !form_.scaled;   // (the gated form's depth weights are per layer: it has no repeated span; the scaled form lists none)
    if (form_.scaled) {   // values are blended with those of the FIRST blending attention layer, which therefore only keeps its own
        const WindowMixer* first = nullptr;
        for (auto& S : layers_) {
            if (S.mixer != kMixWindow || !S.att.v_mix) continue;
            if (!first) { S.att.v_source = true; first = &S.att; continue; }
            if (S.att.kv_heads != first->kv_heads || S.att.vdim != first->vdim) return fail(NTK_E_FORMAT, "config: attention layers that blend their values must have the same kv_heads and vdim");
        }
    }
    if (has_loop_) {
        const Json& lp = c.at("loop");
        const int a = (int)lp.at("start").integer(), b = (int)lp.at("stop").integer(), times = (int)lp.at("times").integer(1);
        if (a < 0 || b <= a || b > n || times < 1) return fail(NTK_E_FORMAT, "config: loop needs 0 <= start < stop <= layers and times >= 1");
        for (int i = 0; i < a; ++i) runs_.push_back({i, false, nullptr, nullptr, nullptr});
        for (int t = 0; t < times; ++t)
            for (int i = a; i < b; ++i) runs_.push_back({i, form_.loop_projection && i == a, nullptr, nullptr, nullptr});
        for (int i = b; i < n; ++i) runs_.push_back({i, false, nullptr, nullptr, nullptr});
    } else {
        for (int i = 0; i < n; ++i) runs_.push_back({i, false, nullptr, nullptr, nullptr});
    }
    info_.n_layers = n;
    info_.n_layer_runs = (int)runs_.size();
    return NTK_OK;
}

// ------------------------------------------------------------------------------------------------------------------------ weights
static inline float bf16_to_f32(uint16_t b) { uint32_t u = (uint32_t)b << 16; float f; memcpy(&f, &u, 4); return f; }
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u; memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static bool tensor_to_f32(const StTensor& t, float* dst) {
    const int64_t n = t.numel();
    if (t.dtype == "BF16") { const uint16_t* s = (const uint16_t*)t.data; for (int64_t i = 0; i < n; ++i) dst[i] = bf16_to_f32(s[i]); return true; }
    if (t.dtype == "F32") { memcpy(dst, t.data, (size_t)n * 4); return true; }
    return false;
}

int LayerStackModel::upload_vector(const ModelFolder& f, const std::string& name, int64_t n, float** out) {
    const StTensor* t = f.tensor(name);
    if (!t) return fail(NTK_E_FORMAT, "tensor '" + name + "' is missing");
    if (t->numel() != n) return fail(NTK_E_SHAPE, "tensor '" + name + "' has " + std::to_string(t->numel()) + " elements, expected " + std::to_string(n));
    std::vector<float> h((size_t)n);
    if (!tensor_to_f32(*t, h.data())) return fail(NTK_E_DTYPE, "tensor '" + name + "': dtype " + t->dtype + " is not supported");
    *out = (float*)dev_alloc((size_t)n * 4);
    if (!*out) return fail(NTK_E_NOMEM, "out of device memory");
    nt_hip_memcpy_h2d(*out, h.data(), (size_t)n * 4);
    weight_bytes_ += t->nbytes;
    return NTK_OK;
}

// `names` one below the other as ONE matrix (count == 1), or `count` groups of names.size() / count tensors: a stack of equal matrices
int LayerStackModel::upload_matrix(const ModelFolder& f, const std::vector<std::string>& names, int64_t in_f, DenseW& out, int count) {
    int64_t rows = 0;
    for (const auto& nm : names) {
        const StTensor* t = f.tensor(nm);
        if (!t) return fail(NTK_E_FORMAT, "tensor '" + nm + "' is missing");
        if (t->shape.size() != 2 || t->shape[1] != in_f) return fail(NTK_E_SHAPE, "tensor '" + nm + "': expected [*, " + std::to_string(in_f) + "]");
        rows += t->shape[0];
    }
    if (rows % count) return fail(NTK_E_SHAPE, "stacked tensors of unequal shape around '" + names[0] + "'");
    const size_t es = wdtype_ == NTK_DT_BF16 ? 2 : 4;
    std::vector<uint8_t> h((size_t)rows * in_f * es);
    size_t at = 0;
    for (const auto& nm : names) {
        const StTensor* t = f.tensor(nm);
        const int64_t n = t->numel();
        if (wdtype_ == NTK_DT_BF16) {
            uint16_t* d = (uint16_t*)(h.data() + at);
            if (t->dtype == "BF16") memcpy(d, t->data, (size_t)n * 2);
            else if (t->dtype == "F32") { const float* s = (const float*)t->data; for (int64_t i = 0; i < n; ++i) d[i] = f32_to_bf16(s[i]); }
            else return fail(NTK_E_DTYPE, "tensor '" + nm + "': dtype " + t->dtype + " is not supported");
        } else {
            if (!tensor_to_f32(*t, (float*)(h.data() + at))) return fail(NTK_E_DTYPE, "tensor '" + nm + "': dtype " + t->dtype + " is not supported");
        }
        at += (size_t)n * es;
        weight_bytes_ += t->nbytes;
    }
    out.ptr = dev_alloc(h.size() + 256);
    if (!out.ptr) return fail(NTK_E_NOMEM, "out of device memory");
    nt_hip_memcpy_h2d(out.ptr, h.data(), h.size());
    out.dtype = wdtype_;
    out.in_f = in_f;
    out.out_f = rows / count;
    out.count = count;
    return NTK_OK;
}

int LayerStackModel::read_scalar(const ModelFolder& f, const std::string& name, float* out) {
    const StTensor* t = f.tensor(name);
    if (!t) return fail(NTK_E_FORMAT, "tensor '" + name + "' is missing");
    if (t->numel() != 1) return fail(NTK_E_SHAPE, "tensor '" + name + "' is not one number");
    if (!tensor_to_f32(*t, out)) return fail(NTK_E_DTYPE, "tensor '" + name + "': dtype " + t->dtype + " is not supported");
    weight_bytes_ += t->nbytes;
    return NTK_OK;
}

// matrices with the same number of rows side by side: row r of the result = [row r of the first | row r of the second | ...]
int LayerStackModel::upload_hstack(const ModelFolder& f, const std::vector<std::string>& names, DenseW& out) {
    int64_t rows = -1, cols = 0;
    for (const auto& nm : names) {
        const StTensor* t = f.tensor(nm);
        if (!t) return fail(NTK_E_FORMAT, "tensor '" + nm + "' is missing");
        if (t->shape.size() != 2 || (rows >= 0 && t->shape[0] != rows)) return fail(NTK_E_SHAPE, "tensor '" + nm + "': expected a matrix with the rows of its neighbours");
        rows = t->shape[0];
        cols += t->shape[1];
    }
    const size_t es = wdtype_ == NTK_DT_BF16 ? 2 : 4;
    std::vector<uint8_t> h((size_t)rows * cols * es);
    int64_t c0 = 0;
    for (const auto& nm : names) {
        const StTensor* t = f.tensor(nm);
        const int64_t n = t->shape[1];
        std::vector<float> tmp((size_t)t->numel());
        if (!tensor_to_f32(*t, tmp.data())) return fail(NTK_E_DTYPE, "tensor '" + nm + "': dtype " + t->dtype + " is not supported");
        for (int64_t r = 0; r < rows; ++r)
            for (int64_t c = 0; c < n; ++c) {
                const float v = tmp[(size_t)(r * n + c)];
                if (wdtype_ == NTK_DT_BF16) ((uint16_t*)h.data())[r * cols + c0 + c] = f32_to_bf16(v);   // (exact for values that were bfloat16)
                else ((float*)h.data())[r * cols + c0 + c] = v;
            }
        c0 += n;
        weight_bytes_ += t->nbytes;
    }
    out.ptr = dev_alloc(h.size() + 256);
    if (!out.ptr) return fail(NTK_E_NOMEM, "out of device memory");
    nt_hip_memcpy_h2d(out.ptr, h.data(), h.size());
    out.dtype = wdtype_; out.in_f = cols; out.out_f = rows; out.count = 1;
    return NTK_OK;
}

int LayerStackModel::upload_norm(const ModelFolder& f, const std::string& name, NormW& out) {
    LS_TRY(upload_vector(f, name, info_.width, &out.w));
    if (form_.sequential || form_.gated) LS_TRY(upload_vector(f, name + ".b", info_.width, &out.b));
    if (form_.gated) LS_TRY(read_scalar(f, name + ".alpha", &out.alpha));
    return NTK_OK;
}

// bucket of a distance n >= 0 for a table of B rows reaching out to distance D: the first B/2 distances have a row each, the rest share the other
// rows on a logarithmic scale, everything from D on the last row.  Formed in F32 like every position quantity.
static int distance_bucket(int n, int B, double D) {
    const int half = B / 2;
    if (n < half) return n;
    const float num = std::log((float)n / (float)half), den = (float)std::log(D / (double)half);
    const float v = num / den * (float)(B - half);
    const long long b = (long long)half + (long long)std::floor(v);
    return (int)std::min<long long>((long long)B - 1, std::max<long long>(b, 0));
}

int LayerStackModel::upload_gated_mixer(const ModelFolder& f, const std::string& p, int i, StackLayer& L) {
    const int W = info_.width;
    const std::string li = "layer " + std::to_string(i);
    auto rows_of = [&](const std::string& nm) -> int64_t { const StTensor* t = f.tensor(nm); return t && t->shape.size() == 2 ? t->shape[0] : -1; };
    if (L.mixer == kMixGla) {
        GlaMixer& m = L.gla;
        const int hq = m.heads * m.dim, hv = m.heads * m.vdim;
        const int64_t rank = rows_of(p + "mix.a1");
        if (rank <= 0) return fail(NTK_E_FORMAT, "tensor '" + p + "mix.a1' is missing");
        m.rank = (int)rank;
        LS_TRY(upload_matrix(f, {p + "mix.q", p + "mix.k", p + "mix.v", p + "mix.g", p + "mix.a1", p + "rg1"}, W, m.in));
        m.k_off = hq; m.v_off = 2 * hq; m.g_off = 2 * hq + hv; m.a_off = 2 * hq + 2 * hv; m.rg_off = m.a_off + m.rank;
        if (rows_of(p + "mix.q") != hq || rows_of(p + "mix.k") != hq || rows_of(p + "mix.v") != hv || rows_of(p + "mix.g") != hv || rows_of(p + "rg1") != W)
            return fail(NTK_E_SHAPE, li + ": the mixer's input projections do not have the configured sizes");
        LS_TRY(upload_matrix(f, {p + "mix.a2"}, m.rank, m.a2));
        if (m.a2.out_f != hq) return fail(NTK_E_SHAPE, "tensor '" + p + "mix.a2' does not have heads * dim rows");
        LS_TRY(upload_vector(f, p + "mix.a2.b", hq, &m.a2_b));
        LS_TRY(upload_vector(f, p + "mix.norm", m.vdim, &m.norm));
        LS_TRY(upload_matrix(f, {p + "mix.o"}, hv, m.o));
        if (m.o.out_f != W) return fail(NTK_E_SHAPE, "tensor '" + p + "mix.o' does not have 'width' rows");
        return NTK_OK;
    }
    ParallelMixer& m = L.par;
    BiasedAttention& a = m.left;
    DeltaMixer& d = m.right;
    const std::string l = p + "mix.left.", r = p + "mix.right.";
    const int hq = a.heads * a.dim, gk = a.kv_heads * a.dim, gv = a.kv_heads * a.vdim, hv = a.heads * a.vdim, hd = d.heads * d.dim;
    const int64_t rank = rows_of(r + "w1");
    if (rank <= 0) return fail(NTK_E_FORMAT, "tensor '" + r + "w1' is missing");
    d.rank = (int)rank;
    LS_TRY(upload_matrix(f, {l + "q", l + "k", l + "v", l + "g", r + "r", r + "k", r + "v", r + "g", r + "a", r + "w1", p + "rg1"}, W, m.in));
    a.q_off = 0; a.k_off = hq; a.v_off = hq + gk; a.g_off = hq + gk + gv;
    d.r_off = a.g_off + hv; d.k_off = d.r_off + hd; d.v_off = d.k_off + hd; d.g_off = d.v_off + hd; d.a_off = d.g_off + hd; d.w1_off = d.a_off + hd;
    m.rg_off = d.w1_off + d.rank;
    if (rows_of(l + "q") != hq || rows_of(l + "k") != gk || rows_of(l + "v") != gv || rows_of(l + "g") != hv || rows_of(r + "r") != hd || rows_of(r + "k") != hd ||
        rows_of(r + "v") != hd || rows_of(r + "g") != hd || rows_of(r + "a") != hd || rows_of(p + "rg1") != W)
        return fail(NTK_E_SHAPE, li + ": the mixer's input projections do not have the configured sizes");
    LS_TRY(upload_vector(f, l + "q.b", hq, &a.q_b));
    LS_TRY(upload_vector(f, l + "k.b", gk, &a.k_b));
    LS_TRY(upload_vector(f, l + "v.b", gv, &a.v_b));
    const StTensor* rel = f.tensor(l + "rel");
    if (!rel || rel->shape.size() != 2 || rel->shape[1] != a.heads || rel->shape[0] < 2) return fail(NTK_E_SHAPE, "tensor '" + l + "rel' is not [buckets >= 2, heads]");
    a.buckets = (int)rel->shape[0];
    if (!(a.bias_max > a.buckets / 2)) return fail(NTK_E_FORMAT, li + ": bias_max must lie beyond the table's first half");
    LS_TRY(upload_vector(f, l + "rel", (int64_t)a.buckets * a.heads, &a.rel));
    {
        std::vector<int> b((size_t)opt_.max_context);
        for (int n = 0; n < opt_.max_context; ++n) b[(size_t)n] = distance_bucket(n, a.buckets, a.bias_max);
        a.bucket_of = (int*)dev_alloc(b.size() * sizeof(int));
        if (!a.bucket_of) return fail(NTK_E_NOMEM, "out of device memory");
        nt_hip_memcpy_h2d(a.bucket_of, b.data(), b.size() * sizeof(int));
    }
    LS_TRY(upload_matrix(f, {r + "w2"}, d.rank, d.w2));
    if (d.w2.out_f != hd) return fail(NTK_E_SHAPE, "tensor '" + r + "w2' does not have heads * dim rows");
    LS_TRY(upload_vector(f, r + "w0", hd, &d.w0));
    LS_TRY(upload_vector(f, r + "a.b", hd, &d.a_b));
    LS_TRY(upload_vector(f, r + "norm", hd, &d.norm));
    LS_TRY(upload_hstack(f, {l + "o", r + "o"}, m.o));
    if (m.o.out_f != W || m.o.in_f != hv + hd) return fail(NTK_E_SHAPE, li + ": the output projections do not have the configured sizes");
    LS_TRY(upload_vector(f, l + "o.b", W, &m.o_b));
    if (ntk_scale(m.o_b, W, m.left_scale, stream_) != NTK_OK) return fail(NTK_E_LAUNCH, "scaling the output bias failed");
    return NTK_OK;
}

int LayerStackModel::upload_mixer(const ModelFolder& f, const std::string& p, int i, StackLayer& L) {
    const int W = info_.width;
    const std::string li = "layer " + std::to_string(i);
    if (L.mixer == kMixWindow) {
        WindowMixer& m = L.att;
        if (m.gated) LS_TRY(upload_matrix(f, {p + "mix.q", p + "mix.k", p + "mix.v", p + "mix.g"}, W, m.in));
        else LS_TRY(upload_matrix(f, {p + "mix.q", p + "mix.k", p + "mix.v"}, W, m.in));
        m.k_off = m.heads * m.maps * m.dim;
        m.v_off = m.k_off + m.kv_heads * m.maps * m.dim;
        m.g_off = m.v_off + m.kv_heads * m.vdim;
        const StTensor* tk = f.tensor(p + "mix.k");
        if (!tk || tk->shape[0] != m.v_off - m.k_off) return fail(NTK_E_SHAPE, "tensor '" + p + "mix.k' does not have kv_heads * maps * dim rows");
        if (m.v_mix && !m.v_source) LS_TRY(read_scalar(f, p + "mix.vmix", &m.v_blend));
        if (m.in.out_f != m.g_off + (m.gated ? m.heads * m.vdim : 0)) return fail(NTK_E_SHAPE, li + ": the mixer's input projections do not have the configured sizes");
        const StTensor* tq = f.tensor(p + "mix.q");
        if (!tq || tq->shape[0] != m.k_off) return fail(NTK_E_SHAPE, "tensor '" + p + "mix.q' does not have heads * maps * dim rows");
        LS_TRY(upload_matrix(f, {p + "mix.o"}, (int64_t)m.heads * m.vdim, m.o));
        if (m.o.out_f != W) return fail(NTK_E_SHAPE, "tensor '" + p + "mix.o' does not have 'width' rows");
        m.lambda = 0.0f;
        if (m.maps == 2) {
            // lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, one number for the layer, in F32
            float dots[2];
            for (int k = 0; k < 2; ++k) {
                const StTensor* a = f.tensor(p + "mix.lq" + std::to_string(k + 1));
                const StTensor* b = f.tensor(p + "mix.lk" + std::to_string(k + 1));
                if (!a || !b) return fail(NTK_E_FORMAT, "tensor '" + p + "mix.lq" + std::to_string(k + 1) + "' or its 'lk' is missing");
                if (a->numel() != m.dim || b->numel() != m.dim) return fail(NTK_E_SHAPE, li + ": the lambda vectors must have 'dim' entries");
                std::vector<float> va((size_t)m.dim), vb((size_t)m.dim);
                if (!tensor_to_f32(*a, va.data()) || !tensor_to_f32(*b, vb.data())) return fail(NTK_E_DTYPE, li + ": lambda vectors of an unsupported dtype");
                float sdot = 0.0f;
                for (int d = 0; d < m.dim; ++d) sdot = std::fma(va[(size_t)d], vb[(size_t)d], sdot);
                dots[k] = sdot;
                weight_bytes_ += a->nbytes + b->nbytes;
            }
            m.lambda = std::exp(dots[0]) - std::exp(dots[1]) + m.diff;
        }
        return NTK_OK;
    }
    if (L.mixer == kMixLightning) {
        LightningMixer& m = L.lin;
        const int hq = m.heads * m.dim, hv = m.heads * m.vdim;
        LS_TRY(upload_matrix(f, {p + "mix.q", p + "mix.k", p + "mix.v", p + "mix.g"}, W, m.in));
        m.k_off = hq; m.v_off = 2 * hq; m.g_off = 2 * hq + hv;
        const StTensor* tq = f.tensor(p + "mix.q");
        const StTensor* tk = f.tensor(p + "mix.k");
        if (m.in.out_f != m.g_off + hv || !tq || !tk || tq->shape[0] != hq || tk->shape[0] != hq) return fail(NTK_E_SHAPE, li + ": the mixer's input projections do not have the configured sizes");
        LS_TRY(upload_vector(f, p + "mix.norm", hv, &m.norm));
        LS_TRY(upload_matrix(f, {p + "mix.o"}, hv, m.o));
        if (m.o.out_f != W) return fail(NTK_E_SHAPE, "tensor '" + p + "mix.o' does not have 'width' rows");
        return NTK_OK;
    }
    if (L.mixer == kMixGatedDelta) {
        GatedDeltaMixer& m = L.gdl;
        const int gq = m.kv_heads * m.dim, hv = m.heads * m.vdim, nc = m.channels();
        LS_TRY(upload_matrix(f, {p + "mix.q", p + "mix.k", p + "mix.v", p + "mix.g", p + "mix.b", p + "mix.a"}, W, m.in));
        m.k_off = gq; m.v_off = 2 * gq; m.g_off = nc; m.b_off = nc + hv; m.a_off = m.b_off + m.heads;
        auto rows_of = [&](const std::string& nm) -> int64_t { const StTensor* t = f.tensor(nm); return t && t->shape.size() == 2 ? t->shape[0] : -1; };
        if (rows_of(p + "mix.q") != gq || rows_of(p + "mix.k") != gq || rows_of(p + "mix.v") != hv || rows_of(p + "mix.g") != hv || rows_of(p + "mix.b") != m.heads ||
            rows_of(p + "mix.a") != m.heads)
            return fail(NTK_E_SHAPE, li + ": the mixer's input projections do not have the configured sizes");
        // the three convolutions one below the other, like their channels in the product's result
        std::vector<float> cw((size_t)nc * m.taps);
        size_t at = 0;
        for (const char* nm : {"mix.q.conv", "mix.k.conv", "mix.v.conv"}) {
            const StTensor* t = f.tensor(p + nm);
            if (!t) return fail(NTK_E_FORMAT, "tensor '" + p + nm + "' is missing");
            if (t->shape.size() != 2 || t->shape[1] != m.taps || at + (size_t)t->numel() > cw.size()) return fail(NTK_E_SHAPE, "tensor '" + p + nm + "' is not [channels, conv]");
            if (!tensor_to_f32(*t, cw.data() + at)) return fail(NTK_E_DTYPE, "tensor '" + p + nm + "': dtype " + t->dtype + " is not supported");
            at += (size_t)t->numel();
            weight_bytes_ += t->nbytes;
        }
        if (at != cw.size()) return fail(NTK_E_SHAPE, li + ": the convolutions do not cover the channels of q, k and v");
        m.conv = (float*)dev_alloc(cw.size() * sizeof(float));
        if (!m.conv) return fail(NTK_E_NOMEM, "out of device memory");
        nt_hip_memcpy_h2d(m.conv, cw.data(), cw.size() * sizeof(float));
        // rate = exp(A_log), in F32
        const StTensor* al = f.tensor(p + "mix.A_log");
        if (!al || al->numel() != m.heads) return fail(NTK_E_SHAPE, "tensor '" + p + "mix.A_log' does not have one entry per head");
        std::vector<float> rate((size_t)m.heads);
        if (!tensor_to_f32(*al, rate.data())) return fail(NTK_E_DTYPE, "tensor '" + p + "mix.A_log': dtype " + al->dtype + " is not supported");
        for (auto& r : rate) r = std::exp(r);
        weight_bytes_ += al->nbytes;
        m.rates = (float*)dev_alloc(rate.size() * sizeof(float));
        if (!m.rates) return fail(NTK_E_NOMEM, "out of device memory");
        nt_hip_memcpy_h2d(m.rates, rate.data(), rate.size() * sizeof(float));
        LS_TRY(upload_vector(f, p + "mix.dt_bias", m.heads, &m.dt_bias));
        LS_TRY(upload_vector(f, p + "mix.norm", m.vdim, &m.norm));
        LS_TRY(upload_matrix(f, {p + "mix.o"}, hv, m.o));
        if (m.o.out_f != W) return fail(NTK_E_SHAPE, "tensor '" + p + "mix.o' does not have 'width' rows");
        return NTK_OK;
    }
    LatentMixer& m = L.mix;
    const int hq = m.heads * m.qd(), hv = m.heads * m.vdim;
    const std::string first = m.q_rank ? p + "mix.dq" : p + "mix.q";
    LS_TRY(upload_matrix(f, {first, p + "mix.dkv", p + "mix.g"}, W, m.in));
    m.q_off = 0;
    m.kv_off = m.q_rank ? m.q_rank : hq;
    m.g_off = m.kv_off + m.row();
    if (m.in.out_f != m.g_off + (m.head_gate ? m.heads : hv)) return fail(NTK_E_SHAPE, li + ": the mixer's input projections do not have the configured sizes");
    if (m.q_rank) {
        LS_TRY(upload_vector(f, p + "mix.dq.norm", m.q_rank, &m.q_norm));
        LS_TRY(upload_matrix(f, {p + "mix.uq"}, m.q_rank, m.uq));
        if (m.uq.out_f != hq) return fail(NTK_E_SHAPE, "tensor '" + p + "mix.uq' does not have heads * (dim + rot_dim) rows");
    }
    LS_TRY(upload_vector(f, p + "mix.dkv.norm", m.kv_rank, &m.kv_norm));
    LS_TRY(upload_matrix(f, {p + "mix.uk"}, m.kv_rank, m.uk));
    LS_TRY(upload_matrix(f, {p + "mix.uv"}, m.kv_rank, m.uv));
    LS_TRY(upload_matrix(f, {p + "mix.o"}, hv, m.o));
    if (m.uk.out_f != m.heads * m.dim || m.uv.out_f != hv || m.o.out_f != W) return fail(NTK_E_SHAPE, li + ": up-projections do not have the configured sizes");
    return NTK_OK;
}

int LayerStackModel::upload_mlp(const ModelFolder& f, const std::string& p, int i, StackLayer& L) {
    const int W = info_.width;
    const std::string li = "layer " + std::to_string(i);
    if (L.mlp_kind == kMlpClipped) {
        GatedExperts& D = L.cff;
        LS_TRY(upload_matrix(f, {p + "mlp.gate", p + "mlp.up"}, W, D.gate_up));
        LS_TRY(upload_matrix(f, {p + "mlp.down"}, D.ff, D.down));
        const StTensor* tg = f.tensor(p + "mlp.gate");
        if (D.gate_up.out_f != 2 * D.ff || !tg || tg->shape[0] != D.ff || D.down.out_f != W) return fail(NTK_E_SHAPE, li + ": feed-forward matrices do not have the configured sizes");
        return NTK_OK;
    }
    if (L.mlp_kind == kMlpDense) {
        DenseFeedForward& D = L.ffn;
        LS_TRY(upload_matrix(f, {p + "mlp.up"}, W, D.up));
        LS_TRY(upload_matrix(f, {p + "mlp.down"}, D.ff, D.down));
        if (D.up.out_f != D.ff || D.down.out_f != W) return fail(NTK_E_SHAPE, li + ": feed-forward matrices do not have the configured sizes");
        return upload_vector(f, p + "mlp.act", 4, &D.act);
    }
    MoeFeedForward& M = L.mlp;
    LS_TRY(upload_vector(f, p + "mlp.router", (int64_t)M.experts * W, &M.router));
    std::vector<std::string> gu, dn;
    for (int e = 0; e < M.experts; ++e) {
        const std::string q = p + "mlp.e" + std::to_string(e) + ".";
        gu.push_back(q + "gate"); gu.push_back(q + "up"); dn.push_back(q + "down");
    }
    LS_TRY(upload_matrix(f, gu, W, M.routed.gate_up, M.experts));
    LS_TRY(upload_matrix(f, dn, M.routed.ff, M.routed.down, M.experts));
    if (M.routed.gate_up.out_f != 2 * M.routed.ff || M.routed.down.out_f != W) return fail(NTK_E_SHAPE, li + ": expert matrices do not have the configured sizes");
    if (M.has_shared) {
        LS_TRY(upload_matrix(f, {p + "mlp.shared.gate", p + "mlp.shared.up"}, W, M.shared.gate_up));
        LS_TRY(upload_matrix(f, {p + "mlp.shared.down"}, M.shared.ff, M.shared.down));
        if (M.shared.gate_up.out_f != 2 * M.shared.ff || M.shared.down.out_f != W) return fail(NTK_E_SHAPE, li + ": shared expert matrices do not have the configured sizes");
        if (form_.shared_gate) LS_TRY(upload_vector(f, p + "mlp.shared.sg", W, &M.shared_gate));
    }
    return NTK_OK;
}

int LayerStackModel::upload_layer(const ModelFolder& f, int i, StackLayer& L) {
    const std::string p = "l" + std::to_string(i) + ".";
    const int W = info_.width;
    if (form_.gated) {
        LS_TRY(upload_norm(f, p + "norm1", L.norm1));
        LS_TRY(upload_gated_mixer(f, p, i, L));
        LS_TRY(upload_vector(f, p + "rg1.b", W, &L.rg1_b));
        if (L.has_mlp) {
            GatedFeedForward& G = L.gff;
            LS_TRY(upload_norm(f, p + "norm2", L.norm2));
            LS_TRY(upload_matrix(f, {p + "mlp.gate", p + "mlp.up", p + "rg2"}, W, G.in));
            LS_TRY(upload_matrix(f, {p + "mlp.down"}, G.ff, G.down));
            if (G.in.out_f != 2 * G.ff + W || G.down.out_f != W) return fail(NTK_E_SHAPE, "layer " + std::to_string(i) + ": feed-forward matrices do not have the configured sizes");
            LS_TRY(upload_vector(f, p + "rg2.b", W, &L.rg2_b));
        }
        return upload_vector(f, p + "dwa", i + 2, &L.depth);
    }
    LS_TRY(upload_norm(f, p + "norm1", L.norm1));
    if (form_.sequential) {
        LS_TRY(upload_norm(f, p + "norm1b", L.norm1b));
        LS_TRY(upload_vector(f, p + "canon1", (int64_t)W * taps_, &L.canon1));
    }
    if (form_.scaled) LS_TRY(upload_norm(f, p + "norm1b", L.norm1b));
    LS_TRY(upload_mixer(f, p, i, L));
    if (L.has_mlp) {
        LS_TRY(upload_norm(f, p + "norm2", L.norm2));
        if (form_.scaled) LS_TRY(upload_norm(f, p + "norm2b", L.norm2b));
        if (form_.sequential) {
            LS_TRY(upload_norm(f, p + "norm2b", L.norm2b));
            LS_TRY(upload_vector(f, p + "canon2", (int64_t)W * taps_, &L.canon2));
        }
        LS_TRY(upload_mlp(f, p, i, L));
    }
    return NTK_OK;
}

int LayerStackModel::load(const std::string& dir, const SeqLoadOptions& opt) {
    opt_ = opt;
    if (opt_.max_context < 1 || opt_.slots < 1) return fail(NTK_E_SHAPE, "max_context and slots must be positive");
    wdtype_ = opt.float32 ? NTK_DT_F32 : NTK_DT_BF16;
    if (ntk_device_count() <= 0) return fail(NTK_E_NODEVICE, "no GPU");
    stream_ = ntk_stream(0);
    if (!stream_) return fail(NTK_E_NODEVICE, "the HIP runtime did not start");
    ModelFolder f;
    const int st = f.open(dir);
    if (st != NTK_OK) return fail(st, f.error());
    LS_TRY(parse(f));
    const int W = info_.width;
    LS_TRY(upload_matrix(f, {"embed"}, W, embed_));
    if (form_.scaled) head_ = embed_;   // the embedding table itself (without the embedding's scale) is the head
    else LS_TRY(upload_matrix(f, {"head"}, W, head_));
    if (embed_.out_f != info_.vocab || head_.out_f != info_.vocab) return fail(NTK_E_SHAPE, "embed / head do not have 'vocab' rows");
    LS_TRY(upload_norm(f, "final.norm", final_norm_));
    if (form_.gated) {
        const StTensor* pt = f.tensor("pos");
        if (!pt || pt->shape.size() != 2 || pt->shape[1] != W) return fail(NTK_E_SHAPE, "tensor 'pos' is not [positions, width]");
        LS_TRY(upload_matrix(f, {"pos"}, W, pos_));
        n_positions_ = (int)pos_.out_f;
        opt_.max_context = std::min(opt_.max_context, n_positions_);   // a slot holds no more positions than the table has vectors
        LS_TRY(upload_norm(f, "embed.norm", embed_norm_));
    }
    if (final_norm_.b && logit_scale_ != 1.0f) {   // logits = head (norm x) * scale = head (norm x with weight and bias times scale): no launch of its own per step
        if (ntk_scale(final_norm_.w, W, logit_scale_, stream_) != NTK_OK || ntk_scale(final_norm_.b, W, logit_scale_, stream_) != NTK_OK) return fail(NTK_E_LAUNCH, "scaling the output norm failed");
        logit_scale_ = 1.0f;
    }
    if (has_loop_ && form_.loop_projection) {
        LS_TRY(upload_matrix(f, {"loop.in"}, 2 * W, loop_in_));
        if (loop_in_.out_f != W) return fail(NTK_E_SHAPE, "tensor 'loop.in' is not [width, 2 width]");
    }
    for (size_t i = 0; i < layers_.size(); ++i) LS_TRY(upload_layer(f, (int)i, layers_[i]));
    info_.max_context = opt_.max_context;
    slots_.reset(opt_.slots, opt_.max_context);
    return alloc_buffers();
}

int LayerStackModel::alloc_buffers() {
    const int W = info_.width;
    chunk_ = std::min(opt_.max_context, 1024);
    size_t sc = 0, wsc = 0, lsc = 0, rsc = 0;
    for (const auto& L : layers_) {
        if (L.mixer == kMixLatent) {
            const LatentMixer& m = L.mix;
            max_in_ = std::max<int>(max_in_, (int)m.in.out_f);
            max_qrank_ = std::max(max_qrank_, m.q_rank);
            max_hqd_ = std::max(max_hqd_, m.heads * m.qd());
            max_hdv_ = std::max(max_hdv_, m.heads * m.vdim);
            max_hdn_ = std::max(max_hdn_, m.heads * m.dim);
            max_fold_ = std::max(max_fold_, m.heads * m.row());
            max_hr_ = std::max(max_hr_, m.heads * m.kv_rank);
            if (m.kv_rank > 512 || m.vdim > 512) return fail(NTK_E_SHAPE, "kv_rank and vdim up to 512 are supported");
            sc = std::max(sc, ntk_latent_attention_scratch(kSharedRows, m.heads, m.kv_rank, opt_.max_context));
        } else if (L.mixer == kMixGatedDelta) {
            const GatedDeltaMixer& m = L.gdl;
            max_in_ = std::max<int>(max_in_, (int)m.in.out_f);
            max_hdv_ = std::max(max_hdv_, m.heads * m.vdim);
            max_conv_ = std::max(max_conv_, m.channels());
            static const float removal = 0.0f;         // (the size only asks whether there is a removal term)
            ntk_gated_recurrence_desc d{};
            d.T = chunk_; d.H = m.heads; d.dn = m.dim; d.dv = m.vdim; d.az = &removal; d.head_gates = 1; d.write_gated = 1;
            rsc = std::max(rsc, ntk_gated_recurrence_scratch_ex(&d));
        } else if (L.mixer == kMixWindow) {
            const WindowMixer& m = L.att;
            max_in_ = std::max<int>(max_in_, (int)m.in.out_f);
            max_hdv_ = std::max(max_hdv_, m.heads * m.vdim);
            if (m.vdim > 512) return fail(NTK_E_SHAPE, "vdim up to 512 is supported");
            if (m.v_mix) max_gv_ = std::max(max_gv_, m.kv_heads * m.vdim);
            wsc = std::max(wsc, ntk_window_attention_scratch(chunk_, m.heads, m.maps, m.vdim, opt_.max_context));
        } else if (L.mixer == kMixLightning) {
            const LightningMixer& m = L.lin;
            max_in_ = std::max<int>(max_in_, (int)m.in.out_f);
            max_hdv_ = std::max(max_hdv_, m.heads * m.vdim);
            lsc = std::max(lsc, ntk_lightning_attention_scratch(chunk_, m.heads, m.dim, m.vdim));
        } else if (L.mixer == kMixGla) {
            const GlaMixer& m = L.gla;
            max_in_ = std::max<int>(max_in_, (int)m.in.out_f);
            max_hdv_ = std::max(max_hdv_, m.heads * m.vdim);
            max_rec_ = std::max(max_rec_, m.heads * m.dim);
            rsc = std::max(rsc, ntk_gated_recurrence_scratch(chunk_, m.heads, m.dim, m.vdim, 0));
        } else {
            const ParallelMixer& m = L.par;
            max_in_ = std::max<int>(max_in_, (int)m.in.out_f);
            max_hdv_ = std::max<int>(max_hdv_, (int)m.o.in_f);
            max_rec_ = std::max(max_rec_, m.right.heads * m.right.dim);
            rsc = std::max(rsc, ntk_gated_recurrence_scratch(chunk_, m.right.heads, m.right.dim, m.right.dim, 1));
            wsc = std::max(wsc, ntk_window_attention_scratch(chunk_, m.left.heads, 1, m.left.vdim, opt_.max_context));
        }
        if (form_.gated && L.has_mlp) max_gu2_ = std::max<int>(max_gu2_, (int)L.gff.in.out_f), max_ffn_ = std::max(max_ffn_, L.gff.ff);
        if (L.mlp_kind == kMlpMoe) {
            max_top_ = std::max(max_top_, L.mlp.top);
            max_e_ = std::max(max_e_, L.mlp.experts);
            max_ff2_ = std::max(max_ff2_, 2 * L.mlp.routed.ff);
            if (L.mlp.has_shared) max_sff2_ = std::max(max_sff2_, 2 * L.mlp.shared.ff);
        } else if (L.mlp_kind == kMlpDense && !form_.gated) {
            max_ffn_ = std::max(max_ffn_, L.ffn.ff);
        } else if (L.mlp_kind == kMlpClipped) {
            max_ffn_ = std::max(max_ffn_, L.cff.ff);
        }
    }
    const size_t C = (size_t)chunk_, ctx = (size_t)opt_.max_context;
    auto fl = [&](float** p, size_t n) { *p = (float*)dev_alloc(std::max<size_t>(n, 1) * sizeof(float)); return *p != nullptr; };
    auto in = [&](int** p, size_t n) { *p = (int*)dev_alloc(n * sizeof(int)); return *p != nullptr; };
    bool ok = fl(&x_, C * W) && fl(&x0_, C * W) && fl(&h1_, C * W) && fl(&h2_, C * W) && fl(&a_, C * max_in_) && fl(&att_, C * max_hdv_) && fl(&mix_, C * W) &&
              fl(&xw_, C * W) && fl(&hn_, C * W) && in(&tokens_dev_, 2 * C);
    if (max_hqd_ > 0)      // latent mixers: query latents, folded queries, the up-projected keys and values of the visible range
        ok = ok && fl(&cat_, C * 2 * W) && fl(&cq_, C * std::max(max_qrank_, 1)) && fl(&q_, C * max_hqd_) && fl(&qf_, (size_t)kSharedRows * max_fold_) &&
             fl(&lat_, (size_t)kSharedRows * max_hr_) && fl(&kx_, ctx * max_hdn_) && fl(&vx_, ctx * max_hdv_) && fl(&scratch_, sc);
    if (form_.sequential) ok = ok && fl(&hist_, (C + (size_t)taps_ - 1) * W) && fl(&ff_, C * W) && fl(&zf_, C * max_ffn_) && fl(&wscratch_, wsc) && fl(&lscratch_, lsc);
    if (form_.gated)
        ok = ok && fl(&ff_, C * W) && fl(&zf_, C * max_ffn_) && fl(&wscratch_, wsc) && fl(&results_, (runs_.size() + 1) * C * W) && fl(&zq_, C * std::max(max_rec_, 1)) && fl(&rscratch_, rsc) &&
             fl(&gu2_, C * std::max(max_gu2_, 1));
    if (form_.scaled)
        ok = ok && fl(&ff_, C * W) && fl(&zf_, C * std::max(max_ffn_, 1)) && fl(&gu2_, C * 2 * std::max(max_ffn_, 1)) && fl(&wscratch_, wsc) && fl(&rscratch_, rsc) &&
             fl(&cv_, C * std::max(max_conv_, 1)) && fl(&vfirst_, C * std::max(max_gv_, 1));
    want_dev_ = tokens_dev_ ? tokens_dev_ + C : nullptr;   // one staging area: [tokens of a pass | wanted places], filled by ONE stream-ordered copy from pinned memory
    h_stage_ = (int*)nt_hip_malloc_host(2 * C * sizeof(int));
    ok = ok && h_stage_ != nullptr;
    if (max_top_ > 0) {
        const size_t P = C * max_top_;
        ok = ok && in(&ids_, P) && fl(&wts_, P) && fl(&sg_, C) && in(&offsets_, (size_t)max_e_ + 1) && in(&order_, P) && in(&where_, P) && fl(&gu_, P * max_ff2_) &&
             fl(&act_, P * (max_ff2_ / 2)) && fl(&dn_, P * W);
        if (max_sff2_ > 0) ok = ok && fl(&sgu_, C * max_sff2_) && fl(&sact_, C * (max_sff2_ / 2)) && fl(&sdn_, C * W);
    }
    if (!ok) return fail(NTK_E_NOMEM, "out of device memory (activation buffers)");
    // what every slot holds per layer run: cache rows per position, the recurrent state, the convolutions' last inputs (mixer's, then feed-forward's)
    for (auto& r : runs_) {
        const StackLayer& L = layers_[(size_t)r.layer];
        const size_t row = (size_t)L.cache_row();
        if (row) {
            r.cache = (float*)dev_alloc((size_t)opt_.slots * ctx * row * sizeof(float));
            if (!r.cache) return fail(NTK_E_NOMEM, "out of device memory (cache)");
        }
        if (L.state_floats()) {
            r.state = (float*)dev_alloc((size_t)opt_.slots * L.state_floats() * sizeof(float));
            if (!r.state) return fail(NTK_E_NOMEM, "out of device memory (state)");
        }
        if (form_.sequential && taps_ > 1) {
            r.conv = (float*)dev_alloc((size_t)opt_.slots * 2 * (taps_ - 1) * W * sizeof(float));
            if (!r.conv) return fail(NTK_E_NOMEM, "out of device memory (state)");
        }
    }
    return NTK_OK;
}

// ------------------------------------------------------------------------------------------------------------------------ slots
int LayerStackModel::acquire_slot() { const int s = slots_.acquire(); return s < 0 ? NTK_E_NOMEM : s; }
int LayerStackModel::release_slot(int slot) { return slots_.release(slot) ? NTK_OK : NTK_E_SHAPE; }
int LayerStackModel::truncate_slot(int slot, int length) {
    if (!slots_.live(slot) || length < 0 || length > slots_.length(slot)) return NTK_E_SHAPE;
    // a recurrent state or a convolution's last inputs cannot be rolled back: such a sequence restarts (position 0 reads no state) or stays
    if (has_state_ && length != 0 && length != slots_.length(slot)) return fail(NTK_E_SHAPE, "truncate: a model with recurrent state can only be cut back to its start");
    slots_.set_length(slot, length);
    return NTK_OK;
}

// ------------------------------------------------------------------------------------------------------------------------ the step
int LayerStackModel::run_mixer(const StackLayer& L, float* cache, int T, int pos0, bool normed_input) {
    const LatentMixer& m = L.mix;
    const int W = info_.width, H = m.heads, qd = m.qd(), row = m.row(), hv = H * m.vdim, na = (int)m.in.out_f;
    // one product for [query (latent) | latent + key part | gate]; decoding: the layer's first norm and the query latent's norm run inside the products
    // (normed_input: h1_ holds the normed stream already -- the seam in front of the mixer wrote it)
    const bool few = T <= ntk_dense_few_rows();
    ntk_dense_desc d{};
    d.Y = a_; d.ldy = na; d.X = few && !normed_input ? x_ : h1_; d.ldx = W; d.W = m.in.ptr; d.wdtype = m.in.dtype; d.G = 1; d.row_div = 1; d.T = T; d.N = na; d.K = W;
    if (few && !normed_input) { d.norm_w = L.norm1.w; d.norm_eps = eps_; d.norm_offset = norm_offset_; }
    LS_TRY(ntk_dense(&d, stream_));
    float* q = a_;
    int ldq = na;
    if (m.q_rank) {
        d.Y = q_; d.ldy = H * qd; d.X = few ? a_ : cq_; d.ldx = few ? na : m.q_rank; d.W = m.uq.ptr; d.wdtype = m.uq.dtype; d.N = H * qd; d.K = m.q_rank;
        if (few) { d.norm_w = m.q_norm; d.norm_offset = 0.0f; }
        else LS_TRY(ntk_rmsnorm_offset(cq_, m.q_norm, nullptr, nullptr, m.q_rank, a_, na, T, m.q_rank, eps_, 0.0f, stream_));
        LS_TRY(ntk_dense(&d, stream_));
        q = q_;
        ldq = H * qd;
    }
    ntk_rotary rot{m.rot_freq, m.rot_mag, m.rot_dims, m.rot_layout};
    LS_TRY(ntk_latent_prepare(cache, row, a_ + m.kv_off, na, m.kv_norm, eps_, m.kv_rank, m.rot_dim, q, ldq, H, qd, &rot, pos0, T, stream_));
    if (T <= kSharedRows) {
        LS_TRY(ntk_latent_fold_query(qf_, q, ldq, m.uk.ptr, m.uk.dtype, T, H, m.dim, m.rot_dim, m.kv_rank, stream_));
        LS_TRY(ntk_latent_attention(lat_, H * m.kv_rank, qf_, H * row, nullptr, 0, nullptr, 0, cache, row, m.kv_rank, m.rot_dim, H, m.dim, m.vdim, 1, pos0, T, 0,
                                    m.window, m.scale, scratch_, stream_));
        LS_TRY(ntk_latent_unfold_value_ex(att_, hv, lat_, m.uv.ptr, m.uv.dtype, a_ + m.g_off, na, m.head_gate ? 1 : 0, T, H, m.vdim, m.kv_rank, stream_));
    } else {
        const int key0 = m.window > 0 ? std::max(0, pos0 - m.window + 1) : 0;
        const int nkeys = pos0 + T - key0;
        LS_TRY(ntk_dense_linear(kx_, H * m.dim, cache + (size_t)key0 * row, row, m.uk.ptr, m.uk.dtype, nkeys, H * m.dim, m.kv_rank, 0, stream_));
        LS_TRY(ntk_dense_linear(vx_, hv, cache + (size_t)key0 * row, row, m.uv.ptr, m.uv.dtype, nkeys, hv, m.kv_rank, 0, stream_));
        LS_TRY(ntk_latent_attention(att_, hv, q, ldq, kx_, H * m.dim, vx_, hv, cache, row, m.kv_rank, m.rot_dim, H, m.dim, m.vdim, 0, pos0, T, key0, m.window, m.scale,
                                    nullptr, stream_));
        if (m.head_gate) LS_TRY(ntk_head_gate(att_, hv, a_ + m.g_off, na, T, H, m.vdim, stream_));
        else LS_TRY(ntk_sigmoid_gate(att_, hv, a_ + m.g_off, na, T, hv, stream_));
    }
    return ntk_dense_linear(mix_, W, att_, hv, m.o.ptr, m.o.dtype, T, W, hv, 0, stream_);
}

// the window mixer: one product for [q | k | v], rotation and cache rows, attention over the window, output projection -> mix_
int LayerStackModel::run_window(const StackLayer& L, float* cache, int T, int pos0) {
    const WindowMixer& m = L.att;
    const int W = info_.width, na = (int)m.in.out_f, hv = m.heads * m.vdim;
    LS_TRY(ntk_dense_linear(a_, na, h1_, W, m.in.ptr, m.in.dtype, T, na, W, 0, stream_));
    ntk_rotary rot{m.rot_freq, 1.0f, m.rot_dims, form_.rot_halves ? NTK_ROT_HALVES : NTK_ROT_NEIGHBOURS};
    ntk_window_prepare_desc pd{};
    pd.cache = cache; pd.row = m.row(); pd.q = a_; pd.ldq = na; pd.k = a_ + m.k_off; pd.ldk = na; pd.v = a_ + m.v_off; pd.ldv = na;
    pd.H = m.heads; pd.G = m.kv_heads; pd.maps = m.maps; pd.dn = m.dim; pd.dv = m.vdim; pd.rot = &rot; pd.temp_every = 1.0; pd.pos0 = pos0; pd.T = T;
    if (m.v_mix && m.v_source) { pd.v_keep = vfirst_; pd.ld_keep = m.kv_heads * m.vdim; }                 // the first blending layer keeps its values of this pass's tokens
    else if (m.v_mix) { pd.v_other = vfirst_; pd.ld_other = m.kv_heads * m.vdim; pd.v_blend = m.v_blend; }    // the later ones blend with them
    LS_TRY(ntk_window_prepare_ex(&pd, stream_));
    ntk_window_attention_desc d{};
    d.out = att_; d.ldo = hv; d.q = a_; d.ldq = na; d.cache = cache; d.row = m.row(); d.H = m.heads; d.G = m.kv_heads; d.maps = m.maps; d.dn = m.dim; d.dv = m.vdim;
    d.pos0 = pos0; d.T = T; d.window = m.window; d.scale = m.scale; d.lambda = m.lambda;
    d.sub_norm = m.maps == 2 ? 1 : 0; d.eps = eps_; d.out_scale = m.maps == 2 ? 1.0f - m.diff : 1.0f;
    d.scratch = wscratch_;
    d.mask_mode = m.mask_mode; d.softcap = m.softcap; d.sink = m.sink ? 1 : 0;
    if (m.gated) { d.gate = a_ + m.g_off; d.ldg = na; }     // the elementwise gate rides in the launch that writes the heads' results
    LS_TRY(ntk_window_attention(&d, stream_));
    return ntk_dense_linear(mix_, W, att_, hv, m.o.ptr, m.o.dtype, T, W, hv, 0, stream_);
}

// the lightning mixer: one product for [q | k | v | gate], the recurrence (silu on the way in), gated RMS norm over the joined heads, output projection -> mix_
int LayerStackModel::run_lightning(const StackLayer& L, float* state, int T, int pos0) {
    const LightningMixer& m = L.lin;
    const int W = info_.width, na = (int)m.in.out_f, hv = m.heads * m.vdim;
    LS_TRY(ntk_dense_linear(a_, na, h1_, W, m.in.ptr, m.in.dtype, T, na, W, 0, stream_));
    LS_TRY(ntk_lightning_attention(att_, hv, a_, na, a_ + m.k_off, na, a_ + m.v_off, na, m.log_decay, state, m.heads, m.dim, m.vdim, 1, pos0, T, lscratch_, stream_));
    LS_TRY(ntk_gated_rmsnorm(att_, hv, att_, hv, m.norm, a_ + m.g_off, na, T, hv, eps_, stream_));
    return ntk_dense_linear(mix_, W, att_, hv, m.o.ptr, m.o.dtype, T, W, hv, 0, stream_);
}

int LayerStackModel::run_experts(float glu_alpha, float glu_up_offset, const GatedExperts& ex, const float* h, float* gu, float* act, float* out, int rows, const int* offsets, const int* order, int top) {
    const int W = info_.width;
    ntk_dense_desc d{};
    d.Y = gu; d.ldy = 2 * ex.ff; d.X = h; d.ldx = W; d.W = ex.gate_up.ptr; d.wstride = ex.gate_up.stride(); d.wdtype = ex.gate_up.dtype;
    d.offsets = offsets; d.G = ex.gate_up.count; d.rows = order; d.row_div = top; d.T = rows; d.N = 2 * ex.ff; d.K = W; d.accumulate = 0;
    if (rows <= ntk_dense_few_rows()) {   // decoding: the activation inside the product's launch
        d.Y = act; d.ldy = ex.ff; d.glu_ff = ex.ff; d.glu_limit = ex.limit; d.glu_alpha = glu_alpha; d.glu_up_offset = glu_up_offset;
        LS_TRY(ntk_dense(&d, stream_));
        d.glu_ff = 0;
    } else {
        LS_TRY(ntk_dense(&d, stream_));
        LS_TRY(ntk_glu(act, gu, rows, ex.ff, ex.limit, glu_alpha, glu_up_offset, stream_));
    }
    d.Y = out; d.ldy = W; d.X = act; d.ldx = ex.ff; d.W = ex.down.ptr; d.wstride = ex.down.stride(); d.wdtype = ex.down.dtype;
    d.rows = nullptr; d.row_div = 1; d.N = W; d.K = ex.ff;
    return ntk_dense(&d, stream_);
}

// router, grouping, the experts' products; then either straight into the stream together with the mixer's output (parallel form) or as a sum of its own
// in ff_ (sequential form: it is normed before it joins the stream)
int LayerStackModel::run_moe(const StackLayer& L, int T, bool into_stream) {
    const MoeFeedForward& M = L.mlp;
    const int W = info_.width;
    float* sgate = M.has_shared && M.shared_gate ? sg_ : nullptr;
    LS_TRY(ntk_moe_route_ex(ids_, wts_, sgate, h2_, W, M.router, sgate ? M.shared_gate : nullptr, T, W, M.experts, M.top, &M.route, stream_));
    LS_TRY(ntk_moe_group(offsets_, order_, where_, ids_, T, M.top, M.experts, stream_));
    LS_TRY(run_experts(M.glu_alpha, M.glu_up_offset, M.routed, h2_, gu_, act_, dn_, T * M.top, offsets_, order_, M.top));
    if (M.has_shared) LS_TRY(run_experts(M.glu_alpha, M.glu_up_offset, M.shared, h2_, sgu_, sact_, sdn_, T, nullptr, nullptr, 1));
    if (into_stream) return ntk_moe_combine(x_, mix_, dn_, where_, wts_, M.has_shared ? sdn_ : nullptr, sgate, T, M.top, W, stream_);
    return ntk_moe_sum(ff_, dn_, where_, wts_, M.has_shared ? sdn_ : nullptr, sgate, T, M.top, W, stream_);
}

// up, the polynomial activation over every token's row of ff values, down -> ff_ (the activation runs in place in the up product's buffer)
int LayerStackModel::run_dense_ff(const StackLayer& L, int T) {
    const DenseFeedForward& D = L.ffn;
    const int W = info_.width;
    LS_TRY(ntk_dense_linear(zf_, D.ff, h2_, W, D.up.ptr, D.up.dtype, T, D.ff, W, 0, stream_));
    LS_TRY(ntk_polynorm(zf_, D.ff, zf_, D.ff, D.act, T, D.ff, eps_, stream_));
    return ntk_dense_linear(ff_, W, zf_, D.ff, D.down.ptr, D.down.dtype, T, W, D.ff, 0, stream_);
}

// the dense clipped gated unit (the experts' unit with one member): gate and up in one product (decoding: the activation inside its launch), down -> ff_
int LayerStackModel::run_clipped_ff(const StackLayer& L, int T) {
    return run_experts(kGluAlpha, 1.0f, L.cff, h2_, gu2_, zf_, ff_, T, nullptr, nullptr, 1);
}

// the delta rule with per-head gates: one product for [q | k | v | gate | beta | decay], the short convolutions of q, k and v (+ silu) with their carried
// inputs, the recurrence (unit q and k, decay and write strength formed from their raw projections in its pre-pass), unit norm per head with the shared
// weight and the silu gate, output projection -> mix_.  state = [S | the convolutions' last inputs]
int LayerStackModel::run_gated_delta(const StackLayer& L, float* state, int T, int pos0) {
    const GatedDeltaMixer& m = L.gdl;
    const int W = info_.width, na = (int)m.in.out_f, nc = m.channels(), hv = m.heads * m.vdim;
    LS_TRY(ntk_dense_linear(a_, na, h1_, W, m.in.ptr, m.in.dtype, T, na, W, 0, stream_));
    ntk_gated_recurrence_desc d{};
    if (T == 1) {   // a decoded token: the convolutions run inside the recurrence's pre-pass
        d.q = a_; d.ldq = na; d.k = a_ + m.k_off; d.ldk = na; d.v = a_ + m.v_off; d.ldv = na;
        d.conv_w = m.conv; d.conv_state = state + m.recurrent_floats(); d.conv_taps = m.taps;
    } else {
        LS_TRY(ntk_causal_conv_act(cv_, nc, a_, na, m.conv, state + m.recurrent_floats(), m.taps, 1, pos0, T, nc, stream_));
        d.q = cv_; d.ldq = nc; d.k = cv_ + m.k_off; d.ldk = nc; d.v = cv_ + m.v_off; d.ldv = nc;
    }
    d.out = att_; d.ldo = hv;
    d.wz = a_ + m.a_off; d.ldw = na; d.wb = m.dt_bias; d.decay_form = NTK_DECAY_EXP_SOFTPLUS; d.decay_rates = m.rates;
    d.az = a_ + m.b_off; d.lda = na; d.unit_eps = kUnitKeyEps;
    d.G = m.kv_heads; d.unit_q = 1; d.unit_k = 1; d.head_gates = 1; d.write_gated = 1;
    d.state = state; d.H = m.heads; d.dn = m.dim; d.dv = m.vdim; d.q_scale = 1.0f / std::sqrt((float)m.dim); d.pos0 = pos0; d.T = T; d.scratch = rscratch_;
    LS_TRY(ntk_gated_recurrence(&d, stream_));
    LS_TRY(ntk_head_rmsnorm_gate(att_, hv, att_, hv, m.norm, 0, a_ + m.g_off, na, 2, 1.0f, T, m.heads, m.vdim, eps_, stream_));
    return ntk_dense_linear(mix_, W, att_, hv, m.o.ptr, m.o.dtype, T, W, hv, 0, stream_);
}

// the seam in front of a sublayer of the scaled form: what the stream is still owed joins it (RMS norm, weight, the residual factor), then the norm of the row
int LayerStackModel::rms_seam(const NormW& nw, float* out, int T) {
    const int W = info_.width;
    const int st = ntk_rms_seam(out, W, x_, W, owed_.y, W, owed_.nb.w, residual_mult_, nw.w, T, W, eps_, stream_);
    owed_.y = nullptr;
    return st;
}

int LayerStackModel::scaled_layer(const Run& run, const StackLayer& L, int slot, int T, int pos0) {
    LS_TRY(rms_seam(L.norm1, h1_, T));
    if (L.mixer == kMixWindow) LS_TRY(run_window(L, run.cache + (size_t)slot * opt_.max_context * L.att.row(), T, pos0));
    else if (L.mixer == kMixLatent) LS_TRY(run_mixer(L, run.cache + (size_t)slot * opt_.max_context * L.mix.row(), T, pos0, true));
    else LS_TRY(run_gated_delta(L, run.state + (size_t)slot * L.gdl.state_floats(), T, pos0));
    owed_ = Owed{mix_, L.norm1b};
    if (!L.has_mlp) return NTK_OK;
    LS_TRY(rms_seam(L.norm2, h2_, T));
    LS_TRY(run_clipped_ff(L, T));
    owed_ = Owed{ff_, L.norm2b};
    return NTK_OK;
}

// gated linear attention: one product for [q | k | v | gate | a1 | residual gate], the decay's second projection, the recurrence (decay formed from its raw
// projection on the way in), unit norm per head with the shared weight and the silu gate, output projection -> mix_
int LayerStackModel::run_gla(const StackLayer& L, float* state, int T, int pos0) {
    const GlaMixer& m = L.gla;
    const int W = info_.width, na = (int)m.in.out_f, hq = m.heads * m.dim, hv = m.heads * m.vdim;
    LS_TRY(ntk_dense_linear(a_, na, h1_, W, m.in.ptr, m.in.dtype, T, na, W, 0, stream_));
    LS_TRY(ntk_dense_linear(zq_, hq, a_ + m.a_off, na, m.a2.ptr, m.a2.dtype, T, hq, m.rank, 0, stream_));
    ntk_gated_recurrence_desc d{};
    d.out = att_; d.ldo = hv; d.q = a_; d.ldq = na; d.k = a_ + m.k_off; d.ldk = na; d.v = a_ + m.v_off; d.ldv = na;
    d.wz = zq_; d.ldw = hq; d.wb = m.a2_b; d.decay_form = NTK_DECAY_SIGMOID_ROOT; d.decay_param = m.tau;
    d.state = state; d.H = m.heads; d.dn = m.dim; d.dv = m.vdim; d.q_scale = 1.0f / std::sqrt((float)m.dim); d.pos0 = pos0; d.T = T; d.scratch = rscratch_;
    LS_TRY(ntk_gated_recurrence(&d, stream_));
    LS_TRY(ntk_head_rmsnorm_gate(att_, hv, att_, hv, m.norm, 0, a_ + m.g_off, na, 2, 1.0f, T, m.heads, m.vdim, eps_, stream_));
    return ntk_dense_linear(mix_, W, att_, hv, m.o.ptr, m.o.dtype, T, W, hv, 0, stream_);
}

// two mixers over the same input: one product for all their projections and the residual gate; left: biases and the query temperature on the way into the
// cache, attention with the distance bias, sigmoid gate; right: the decay's second projection, the delta-rule recurrence, unit norm per head, weight and
// sigmoid gate; both results side by side (each times its fixed weight) through ONE output product -> mix_
int LayerStackModel::run_parallel(const StackLayer& L, float* cache, float* state, int T, int pos0) {
    const ParallelMixer& m = L.par;
    const BiasedAttention& a = m.left;
    const DeltaMixer& r = m.right;
    const int W = info_.width, na = (int)m.in.out_f, hv = a.heads * a.vdim, hd = r.heads * r.dim, no = hv + hd;
    LS_TRY(ntk_dense_linear(a_, na, h1_, W, m.in.ptr, m.in.dtype, T, na, W, 0, stream_));
    // ---- left
    ntk_rotary rot{nullptr, 1.0f, 0};
    LS_TRY(ntk_window_prepare_biased(cache, a.row(), a_ + a.q_off, na, a_ + a.k_off, na, a_ + a.v_off, na, a.heads, a.kv_heads, 1, a.dim, a.vdim, &rot, a.q_b, a.k_b, a.v_b,
                                     a.temp_coef, a.temp_every, pos0, T, stream_));
    ntk_window_attention_desc d{};
    d.out = att_; d.ldo = no; d.q = a_ + a.q_off; d.ldq = na; d.cache = cache; d.row = a.row(); d.H = a.heads; d.G = a.kv_heads; d.maps = 1; d.dn = a.dim; d.dv = a.vdim;
    d.pos0 = pos0; d.T = T; d.window = 0; d.scale = a.scale; d.out_scale = 1.0f; d.eps = eps_; d.scratch = wscratch_;
    d.rel = a.rel; d.bucket_of = a.bucket_of; d.n_dist = opt_.max_context;
    LS_TRY(ntk_window_attention(&d, stream_));
    LS_TRY(ntk_sigmoid_gate_scaled(att_, no, a_ + a.g_off, na, nullptr, m.left_scale, T, hv, stream_));
    // ---- right
    LS_TRY(ntk_tanh_rows(a_ + r.w1_off, na, T, r.rank, stream_));
    LS_TRY(ntk_dense_linear(zq_, hd, a_ + r.w1_off, na, r.w2.ptr, r.w2.dtype, T, hd, r.rank, 0, stream_));
    ntk_gated_recurrence_desc g{};
    g.out = att_ + hv; g.ldo = no; g.q = a_ + r.r_off; g.ldq = na; g.k = a_ + r.k_off; g.ldk = na; g.v = a_ + r.v_off; g.ldv = na;
    g.wz = zq_; g.ldw = hd; g.wb = r.w0; g.decay_form = NTK_DECAY_EXP_SIGMOID; g.decay_param = kDeltaDecayRate;
    g.az = a_ + r.a_off; g.lda = na; g.ab = r.a_b; g.unit_eps = kUnitKeyEps;
    g.state = state; g.H = r.heads; g.dn = r.dim; g.dv = r.dim; g.q_scale = 1.0f; g.pos0 = pos0; g.T = T; g.scratch = rscratch_;
    LS_TRY(ntk_gated_recurrence(&g, stream_));
    LS_TRY(ntk_head_rmsnorm_gate(att_ + hv, no, att_ + hv, no, r.norm, r.dim, a_ + r.g_off, na, 1, m.right_scale, T, r.heads, r.dim, eps_, stream_));
    return ntk_dense_linear(mix_, W, att_, no, m.o.ptr, m.o.dtype, T, W, no, 0, stream_);
}

// gate and up (decoding: the gated unit inside the product's launch) and the residual gate's rows, down -> ff_; the residual gate stays in gu2_ behind them
int LayerStackModel::run_gated_ff(const StackLayer& L, int T) {
    const GatedFeedForward& G = L.gff;
    const int W = info_.width, n2 = (int)G.in.out_f, ff = G.ff;
    if (T <= ntk_dense_few_rows()) {
        ntk_dense_desc d{};
        d.Y = zf_; d.ldy = ff; d.X = h2_; d.ldx = W; d.W = G.in.ptr; d.wdtype = G.in.dtype; d.G = 1; d.row_div = 1; d.T = T; d.N = 2 * ff; d.K = W;
        d.glu_ff = ff; d.glu_limit = INFINITY; d.glu_alpha = kGeluAlpha; d.glu_cubic = kGeluCubic; d.glu_up_offset = 0.0f;
        LS_TRY(ntk_dense(&d, stream_));
        const size_t es = G.in.dtype == NTK_DT_BF16 ? 2 : 4;
        LS_TRY(ntk_dense_linear(gu2_ + 2 * ff, n2, h2_, W, (const char*)G.in.ptr + (size_t)2 * ff * W * es, G.in.dtype, T, W, W, 0, stream_));
    } else {
        LS_TRY(ntk_dense_linear(gu2_, n2, h2_, W, G.in.ptr, G.in.dtype, T, n2, W, 0, stream_));
        LS_TRY(ntk_glu_cubic(zf_, gu2_, n2, T, ff, INFINITY, kGeluAlpha, kGeluCubic, 0.0f, stream_));
    }
    return ntk_dense_linear(ff_, W, zf_, ff, G.down.ptr, G.down.dtype, T, W, ff, 0, stream_);
}

// A layer of the gated form.  h1_ holds the first norm of the stream already (the embedding's launch or the previous layer's last seam wrote it).  Every
// seam is one launch: gated residual sum, after the layer's last sublayer the weighted sum over all layer results so far, and the norm that follows.
int LayerStackModel::gated_layer(size_t r, const StackLayer& L, int slot, int T, int pos0) {
    const int W = info_.width;
    const Run& run = runs_[r];
    const NormW* next = r + 1 < runs_.size() ? &layers_[(size_t)runs_[r + 1].layer].norm1 : nullptr;
    float* state = run.state + (size_t)slot * L.state_floats();
    int na, rg_off;
    const float* yb = nullptr;
    if (L.mixer == kMixGla) {
        LS_TRY(run_gla(L, state, T, pos0));
        na = (int)L.gla.in.out_f; rg_off = L.gla.rg_off;
    } else {
        LS_TRY(run_parallel(L, run.cache + (size_t)slot * opt_.max_context * L.par.left.row(), state, T, pos0));
        na = (int)L.par.in.out_f; rg_off = L.par.rg_off; yb = L.par.o_b;
    }
    auto depth = [&](ntk_gated_seam_desc& d) {     // the layer's result joins the others; what goes on is their weighted sum, normed for the next layer
        d.hist = results_; d.hist_stride = (long long)chunk_ * W; d.n_hist = run.layer + 2; d.coef = L.depth;
        if (next) { d.h = h1_; d.ldh = W; d.nw = next->w; d.nb = next->b; d.alpha = next->alpha; }
    };
    ntk_gated_seam_desc d{};
    d.x = x_; d.ldx = W; d.y = mix_; d.ldy = W; d.yb = yb; d.g = a_ + rg_off; d.ldg = na; d.gb = L.rg1_b; d.T = T; d.n = W;
    if (!L.has_mlp) { depth(d); return ntk_gated_seam(&d, stream_); }
    d.h = h2_; d.ldh = W; d.nw = L.norm2.w; d.nb = L.norm2.b; d.alpha = L.norm2.alpha;
    LS_TRY(ntk_gated_seam(&d, stream_));
    LS_TRY(run_gated_ff(L, T));
    ntk_gated_seam_desc e{};
    e.x = x_; e.ldx = W; e.y = ff_; e.ldy = W; e.g = gu2_ + 2 * L.gff.ff; e.ldg = (int)L.gff.in.out_f; e.gb = L.rg2_b; e.T = T; e.n = W;
    depth(e);
    return ntk_gated_seam(&e, stream_);
}

// out = h + conv(h), h = layer norm of the stream: the carried inputs in front of the portion's, the convolution, and the portion's last inputs carried on
// The sublayer output that the stream has not taken yet (owed_) goes in first, in the same launch: the norm after one sublayer and the norm before the next
// read the same row.  One token: one launch for the whole seam.
int LayerStackModel::norm_conv(const NormW& nw, const float* canon, float* conv_state, float* out, int T, int pos0) {
    const int W = info_.width;
    const int st = ntk_sandwich_norm_conv(out, W, x_, W, owed_.y, W, owed_.nb.w, owed_.nb.b, nw.w, nw.b, canon, conv_state, hist_, taps_, pos0, T, W, eps_, stream_);
    owed_.y = nullptr;
    return st;
}

// x += norm(owed sublayer output), on its own: after the last layer run, and after every one while the stream is being captured
int LayerStackModel::settle(int T) {
    if (!owed_.y) return NTK_OK;
    const int W = info_.width;
    const int st = form_.scaled ? ntk_rms_seam(nullptr, 0, x_, W, owed_.y, W, owed_.nb.w, residual_mult_, nullptr, T, W, eps_, stream_)
                                : ntk_layernorm(x_, W, owed_.y, W, owed_.nb.w, owed_.nb.b, T, W, eps_, 1, stream_);
    owed_.y = nullptr;
    return st;
}

int LayerStackModel::sequential_layer(const Run& run, const StackLayer& L, int slot, int T, int pos0) {
    const int W = info_.width;
    float* conv = run.conv ? run.conv + (size_t)slot * 2 * (taps_ - 1) * W : nullptr;
    LS_TRY(norm_conv(L.norm1, L.canon1, conv, h1_, T, pos0));
    if (L.mixer == kMixWindow) LS_TRY(run_window(L, run.cache + (size_t)slot * opt_.max_context * L.att.row(), T, pos0));
    else LS_TRY(run_lightning(L, run.state + (size_t)slot * L.lin.state_floats(), T, pos0));
    owed_ = Owed{mix_, L.norm1b};
    if (!L.has_mlp) return NTK_OK;
    LS_TRY(norm_conv(L.norm2, L.canon2, conv ? conv + (size_t)(taps_ - 1) * W : nullptr, h2_, T, pos0));
    if (L.mlp_kind == kMlpMoe) LS_TRY(run_moe(L, T, false));
    else LS_TRY(run_dense_ff(L, T));
    owed_ = Owed{ff_, L.norm2b};
    return NTK_OK;
}

int LayerStackModel::parallel_layer(const Run& run, const StackLayer& L, int slot, int T, int pos0) {
    const int W = info_.width;
    if (T > ntk_dense_few_rows()) {
        LS_TRY(ntk_rmsnorm_offset(h1_, L.norm1.w, L.has_mlp ? h2_ : nullptr, L.has_mlp ? L.norm2.w : nullptr, W, x_, W, T, W, eps_, 1.0f, stream_));
    } else if (L.has_mlp) {   // decoding: the mixer's norm runs inside its first product (run_mixer); the feed-forward's input has three readers
        LS_TRY(ntk_rmsnorm_offset(h2_, L.norm2.w, nullptr, nullptr, W, x_, W, T, W, eps_, 1.0f, stream_));
    }
    float* cache = run.cache + (size_t)slot * opt_.max_context * L.mix.row();
    LS_TRY(run_mixer(L, cache, T, pos0));
    if (L.has_mlp) return run_moe(L, T, true);
    return ntk_residual_add(x_, mix_, nullptr, T * W, stream_);
}

int LayerStackModel::portion(int slot, const int* tokens_dev, int T, int pos0, const int* want_dev, int n_want, float* logits_out) {
    const int W = info_.width;
    // (the embedding is kept beside the stream only where a repeated span is entered through a projection of both)
    const bool keep_embedding = has_loop_ && form_.loop_projection;
    if (form_.gated) {
        // token row + position row, the embedding's norm; the result is the first of the layer results; then the first layer's norm
        LS_TRY(ntk_embed_positions(x_, results_, embed_.ptr, pos_.ptr, embed_.dtype, tokens_dev, T, info_.vocab, W, pos0, n_positions_, embed_norm_.w, embed_norm_.b,
                                   embed_norm_.alpha, stream_));
        const NormW& n1 = layers_[(size_t)runs_[0].layer].norm1;
        LS_TRY(ntk_dyt(h1_, W, x_, W, n1.w, n1.b, n1.alpha, T, W, stream_));
    } else
    LS_TRY(ntk_embed_dense_scaled(keep_embedding ? x0_ : x_, embed_.ptr, embed_.dtype, tokens_dev, T, info_.vocab, W, embed_scale_, stream_));
    bool x_is_x0 = keep_embedding;   // until the first layer run writes x_
    owed_.y = nullptr;
    for (size_t r = 0; r < runs_.size(); ++r) {
        const Run& run = runs_[r];
        const StackLayer& L = layers_[(size_t)run.layer];
        if (x_is_x0 && !run.enters) { LS_TRY(ntk_rows_copy(x_, x0_, (long long)T * W, stream_)); x_is_x0 = false; }
        if (run.enters) {
            LS_TRY(ntk_concat_rows(cat_, x_is_x0 ? x0_ : x_, x0_, T, W, stream_));
            LS_TRY(ntk_dense_linear(x_, W, cat_, 2 * W, loop_in_.ptr, loop_in_.dtype, T, W, 2 * W, 0, stream_));
            x_is_x0 = false;
        }
        if (form_.gated) {
            LS_TRY(gated_layer(r, L, slot, T, pos0));
        } else if (form_.scaled) {
            LS_TRY(scaled_layer(run, L, slot, T, pos0));
            if (r + 1 == runs_.size() || (capture_ && capture_buf_)) LS_TRY(settle(T));
        } else if (form_.sequential) {
            LS_TRY(sequential_layer(run, L, slot, T, pos0));
            if (r + 1 == runs_.size() || (capture_ && capture_buf_)) LS_TRY(settle(T));
        } else {
            LS_TRY(parallel_layer(run, L, slot, T, pos0));
        }
        if (capture_ && capture_buf_) LS_TRY(ntk_rows_copy(capture_buf_ + r * (size_t)T * W, x_, (long long)T * W, stream_));
    }
    if (n_want > 0) {
        // the wanted rows only: gather, norm, head
        const float* xs = x_is_x0 ? x0_ : x_;
        const float* rows = xs;                       // a single decoded token is its own gather
        if (!(T == 1 && n_want == 1)) { LS_TRY(ntk_embed_dense(xw_, xs, NTK_DT_F32, want_dev, n_want, T, W, stream_)); rows = xw_; }
        ntk_dense_desc d{};
        d.Y = logits_out; d.ldy = info_.vocab; d.X = rows; d.ldx = W; d.W = head_.ptr; d.wdtype = head_.dtype; d.G = 1; d.row_div = 1; d.T = n_want;
        d.N = info_.vocab; d.K = W;
        if (form_.gated) { LS_TRY(ntk_dyt(hn_, W, rows, W, final_norm_.w, final_norm_.b, final_norm_.alpha, n_want, W, stream_)); d.X = hn_; }
        else if (final_norm_.b) { LS_TRY(ntk_layernorm(hn_, W, rows, W, final_norm_.w, final_norm_.b, n_want, W, eps_, 0, stream_)); d.X = hn_; }
        else if (n_want <= ntk_dense_few_rows()) { d.norm_w = final_norm_.w; d.norm_eps = eps_; d.norm_offset = norm_offset_; }   // the output norm inside the head's launch
        else { LS_TRY(ntk_rmsnorm_offset(hn_, final_norm_.w, nullptr, nullptr, W, rows, W, n_want, W, eps_, norm_offset_, stream_)); d.X = hn_; }
        LS_TRY(ntk_dense(&d, stream_));
        if (logit_softcap_ > 0.0f) LS_TRY(ntk_softcap_rows(logits_out, info_.vocab, logit_softcap_, n_want, info_.vocab, stream_));
        if (logit_scale_ != 1.0f) LS_TRY(ntk_scale(logits_out, (long long)n_want * info_.vocab, logit_scale_, stream_));
    }
    return NTK_OK;
}

float* LayerStackModel::forward(int slot, const int* tokens, int n, const int* want, int n_want) {
    if (!slots_.live(slot)) { err_ = "forward: the slot is not live"; return nullptr; }
    if (n <= 0 || !tokens || n_want < 0 || (n_want && !want)) { err_ = "forward: no tokens"; return nullptr; }
    const int pos0 = slots_.length(slot);
    if (pos0 + n > opt_.max_context) { err_ = "forward: the slot's " + std::to_string(opt_.max_context) + " positions are used up"; return nullptr; }
    for (int i = 0; i < n_want; ++i)
        if (want[i] < 0 || want[i] >= n || (i && want[i] < want[i - 1])) { err_ = "forward: wanted places must be ascending and inside the portion"; return nullptr; }
    const size_t need = (size_t)std::max(n_want, 1);
    if (need > logits_rows_) {
        if (ntk_stream_synchronize(stream_) != NTK_OK) return nullptr;
        if (logits_) nt_hip_free(logits_);
        logits_rows_ = need;
        logits_ = (float*)nt_hip_malloc(logits_rows_ * (size_t)info_.vocab * sizeof(float));
        if (!logits_) { logits_rows_ = 0; err_ = "out of device memory (logits)"; return nullptr; }
    }
    if (capture_) {
        const size_t cf = runs_.size() * (size_t)n * info_.width;
        if (n > chunk_) { err_ = "capture: the portion must fit one internal pass"; return nullptr; }
        if (cf > capture_floats_) {
            ntk_stream_synchronize(stream_);
            if (capture_buf_) nt_hip_free(capture_buf_);
            capture_buf_ = (float*)nt_hip_malloc(cf * sizeof(float));
            capture_floats_ = capture_buf_ ? cf : 0;
            if (!capture_buf_) { err_ = "out of device memory (capture)"; return nullptr; }
        }
        capture_T_ = n;
    }
    int done_want = 0;
    for (int at = 0; at < n; at += chunk_) {
        const int T = std::min(chunk_, n - at);
        int w1 = done_want;
        while (w1 < n_want && want[w1] < at + T) ++w1;
        std::vector<int> rel((size_t)std::max(w1 - done_want, 1));
        for (int i = done_want; i < w1; ++i) rel[(size_t)(i - done_want)] = want[i] - at;
        // the pinned staging area is free once the previous pass's copy has run: wait for the stream (idle already after a copy_logits), then one
        // stream-ordered copy brings the tokens and the wanted places
        if (ntk_stream_synchronize(stream_) != NTK_OK) { err_ = "forward: the stream failed"; return nullptr; }
        memcpy(h_stage_, tokens + at, (size_t)T * sizeof(int));
        const int nw = w1 - done_want;
        if (nw > 0) memcpy(h_stage_ + chunk_, rel.data(), (size_t)nw * sizeof(int));
        if (ntk_memcpy_h2d_async(tokens_dev_, h_stage_, (size_t)(nw > 0 ? chunk_ + nw : T) * sizeof(int), stream_) != NTK_OK) { err_ = "forward: the copy of the tokens failed"; return nullptr; }
        const int st = portion(slot, tokens_dev_, T, pos0 + at, want_dev_, w1 - done_want, logits_ + (size_t)done_want * info_.vocab);
        if (st != NTK_OK) { if (err_.empty()) err_ = std::string("forward: ") + ntk_status_string(st); return nullptr; }
        done_want = w1;
    }
    slots_.set_length(slot, pos0 + n);
    last_rows_ = n_want;
    return logits_;
}

int LayerStackModel::copy_logits(float* host, int rows) {
    if (!host || rows < 0 || rows > last_rows_) return NTK_E_SHAPE;
    LS_TRY(ntk_stream_synchronize(stream_));
    if (rows) nt_hip_memcpy_d2h(host, logits_, (size_t)rows * info_.vocab * sizeof(float));
    return NTK_OK;
}

int LayerStackModel::copy_capture(float* host) {
    if (!capture_buf_ || !capture_T_) return NTK_E_NULL;
    LS_TRY(ntk_stream_synchronize(stream_));
    nt_hip_memcpy_d2h(host, capture_buf_, runs_.size() * (size_t)capture_T_ * info_.width * sizeof(float));
    return NTK_OK;
}

int LayerStackModel::sync() { return ntk_stream_synchronize(stream_); }

}  // namespace nt
