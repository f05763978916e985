"""Plain float64 restatement of the Tubazen family (the gated form of the layer stack), one function per mechanism, for the tests: numpy only, loops
over tokens where the mechanism is a recurrence, nothing shared with the product.

Notation.  x [T, W] is the stream, h a sublayer's input, W* matrices stored [out, in] and applied as h @ W.T.
  dyt(x)        = tanh(alpha x) * w + b                                   (a norm without row sums)
  embedding     X_0 = dyt_e(E[token] + P[position])
  layer i       h = dyt_1(x);  x' = x + mixer(h) * sigmoid(Rg1 h + c1);  h' = dyt_2(x');  X_(i+1) = x' + ff(h') * sigmoid(Rg2 h' + c2)
                what goes on: x = sum_{j <= i+1} depth_i[j] X_j
  logits        head @ dyt_f(x) * logit_scale
"""
import json
import math
import os
import struct

import numpy as np

F = np.float64


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def dyt(x, w, b, alpha):
    return np.tanh(alpha * x) * w + b


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


# ---------------------------------------------------------------------------------------------------------------- attention with a bias by distance
def distance_bucket(n, rows, reach):
    """rows of the bias table: the first rows // 2 distances own a row each; farther ones share the remaining rows on a logarithmic scale that ends at
    `reach`; everything beyond sits in the last row"""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(reach / half) * (rows - half))))


def query_temperature(p, coef, every):
    return 1.0 + coef * math.log(math.floor((p + 1) / every) + 1.0)


def biased_attention(h, w, pre, mx, pos0=0, past=None):
    """h [T, W] at positions pos0 ..; past = (k, v) of the positions before -> (out [T, W], (k, v) of all positions so far)"""
    T = h.shape[0]
    H, G, dn, dv = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).reshape(T, H, dn)
    k = (h @ w[pre + "k"].T + w[pre + "k.b"]).reshape(T, G, dn)
    v = (h @ w[pre + "v"].T + w[pre + "v.b"]).reshape(T, G, dv)
    if past is not None:
        k, v = np.concatenate([past[0], k]), np.concatenate([past[1], v])
    qt = mx.get("q_temp")
    rel = w[pre + "rel"]
    out = np.zeros((T, H, dv), F)
    for t in range(T):
        p = pos0 + t
        temp = query_temperature(p, qt["coef"], qt["every"]) if qt else 1.0
        for hh in range(H):
            g = hh // (H // G)
            s = (k[:p + 1, g] @ (q[t, hh] * temp)) * mx["scale"]
            s = s + np.array([rel[distance_bucket(p - j, rel.shape[0], mx["bias_max"]), hh] for j in range(p + 1)])
            e = np.exp(s - s.max())
            out[t, hh] = (e / e.sum()) @ v[:p + 1, g]
    out = out.reshape(T, H * dv) * sigmoid(h @ w[pre + "g"].T)
    return out @ w[pre + "o"].T + w[pre + "o.b"], (k, v)


# ---------------------------------------------------------------------------------------------------------------- recurrences
def decay_recurrence(q, k, v, decay, removal=None, unit_eps=1e-6, state=None):
    """S_t = diag(decay_t) S_(t-1) - (removal_t * u_t)(u_t^T S_(t-1)) + k_t v_t^T, o_t = S_t^T q_t, u_t = k_t / sqrt(|k_t|^2 + unit_eps); all [T, H, .];
    removal None: no second term -> (o [T, H, dv], S [H, dn, dv])"""
    T, H, dn = k.shape
    dv = v.shape[2]
    S = np.zeros((H, dn, dv), F) if state is None else np.array(state, F)
    o = np.zeros((T, H, dv), F)
    for t in range(T):
        for hh in range(H):
            old = S[hh]
            new = decay[t, hh][:, None] * old + np.outer(k[t, hh], v[t, hh])
            if removal is not None:
                u = k[t, hh] / math.sqrt(float(k[t, hh] @ k[t, hh]) + unit_eps)
                new = new - np.outer(removal[t, hh] * u, u @ old)
            S[hh] = new
            o[t, hh] = new.T @ q[t, hh]
    return o, S


def gla(h, w, pre, mx, eps, state=None):
    T = h.shape[0]
    H, dn, dv = mx["heads"], mx["dim"], mx["vdim"]
    q = (h @ w[pre + "q"].T).reshape(T, H, dn) * dn ** -0.5
    k = (h @ w[pre + "k"].T).reshape(T, H, dn)
    v = (h @ w[pre + "v"].T).reshape(T, H, dv)
    z = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "a2.b"]
    decay = (sigmoid(z) ** (1.0 / mx["tau"])).reshape(T, H, dn)
    o, S = decay_recurrence(q, k, v, decay, state=state)
    o = unit_rms(o, eps) * w[pre + "norm"]
    g = h @ w[pre + "g"].T
    return (o.reshape(T, H * dv) * (g * sigmoid(g))) @ w[pre + "o"].T, S


def delta_rule(h, w, pre, mx, eps, state=None):
    T = h.shape[0]
    H, d = mx["heads"], mx["dim"]
    r = (h @ w[pre + "r"].T).reshape(T, H, d)
    k = (h @ w[pre + "k"].T).reshape(T, H, d)
    v = (h @ w[pre + "v"].T).reshape(T, H, d)
    decay = np.exp(-math.exp(-0.5) * sigmoid(np.tanh(h @ w[pre + "w1"].T) @ w[pre + "w2"].T + w[pre + "w0"])).reshape(T, H, d)
    removal = sigmoid(h @ w[pre + "a"].T + w[pre + "a.b"]).reshape(T, H, d)
    o, S = decay_recurrence(r, k, v, decay, removal, 1e-6, state)
    o = unit_rms(o, eps).reshape(T, H * d) * w[pre + "norm"] * sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T, S


def gated_ff(h, w, pre):
    return (gelu_tanh(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


# ---------------------------------------------------------------------------------------------------------------- the model
def forward(cfg, w, tokens, return_layers=False):
    """logits [T, vocab] of a whole sequence (and the stream after every layer [layers, T, W])"""
    w = {k: np.asarray(v, F) for k, v in w.items()}
    tokens = np.asarray(tokens)
    T, eps = len(tokens), cfg["norm"]["eps"]
    x = dyt(w["embed"][tokens] + w["pos"][:T], w["embed.norm"], w["embed.norm.b"], w["embed.norm.alpha"])
    results, streams = [x], []
    for i, L in enumerate(cfg["layers"]):
        p = "l%d." % i
        h = dyt(x, w[p + "norm1"], w[p + "norm1.b"], w[p + "norm1.alpha"])
        if L["type"] == "gla":
            m, _ = gla(h, w, p + "mix.", L["mixer"], eps)
        else:
            mm = L["mixer"]
            left, _ = biased_attention(h, w, p + "mix.left.", mm["left"])
            right, _ = delta_rule(h, w, p + "mix.right.", mm["right"], eps)
            m = mm["left_scale"] * left + mm["right_scale"] * right
        x = x + m * sigmoid(h @ w[p + "rg1"].T + w[p + "rg1.b"])
        if L.get("mlp"):
            h = dyt(x, w[p + "norm2"], w[p + "norm2.b"], w[p + "norm2.alpha"])
            x = x + gated_ff(h, w, p + "mlp.") * sigmoid(h @ w[p + "rg2"].T + w[p + "rg2.b"])
        results.append(x)
        x = sum(w[p + "dwa"][j] * results[j] for j in range(i + 2))
        streams.append(x)
    logits = dyt(x, w["final.norm"], w["final.norm.b"], w["final.norm.alpha"]) @ w["head"].T * cfg.get("logit_scale", 1.0)
    return (logits, np.stack(streams)) if return_layers else logits


def greedy(cfg, w, prompt, n):
    toks, out = list(prompt), []
    for _ in range(n):
        out.append(int(np.argmax(forward(cfg, w, toks)[-1])))
        toks.append(out[-1])
    return out


# ---------------------------------------------------------------------------------------------------------------- configurations and weights
def bf16_round(a):
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def small_config(layers=("parallel", "gla"), mlps=(True, True), width=40, vocab=72, positions=600, heads=6, kv_heads=2, dim=10, vdim=14, buckets=10, bias_max=37,
                 temp=(0.5, 16), scale=None, rheads=3, rdim=12, left_scale=0.8, right_scale=0.5, gheads=2, gdim=9, gvdim=11, tau=4.0, ff=52, eps=1e-5,
                 logit_scale=1.5):
    """sizes that all differ, so that a swapped pair shows.  mlps: per layer, True or None"""
    ls = []
    for t, m in zip(layers, mlps):
        if t == "parallel":
            left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "bias_max": bias_max, "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
            if temp is not None:
                left["q_temp"] = {"coef": temp[0], "every": temp[1]}
            mx = {"left": left, "right": {"heads": rheads, "dim": rdim}, "left_scale": left_scale, "right_scale": right_scale}
        else:
            mx = {"heads": gheads, "dim": gdim, "vdim": gvdim, "tau": tau}
        ls.append({"type": t, "mixer": mx, "mlp": {"kind": "dense", "ff": ff} if m else None})
    cfg = {"architecture": "Tubazen", "layers": ls, "norm": {"eps": eps}, "logit_scale": logit_scale, "max_positions": positions, "vocab": vocab, "width": width}
    cfg["_buckets"] = buckets          # (rows of the bias tables: a tensor's shape in the folder, kept here for tensor_shapes; not written to config.json)
    cfg["_ranks"] = (5, 7)             # low ranks of the decay projections (gla, delta rule): tensor shapes too
    return cfg


def tensor_shapes(cfg):
    W, V = cfg["width"], cfg["vocab"]
    B, (ra, rw) = cfg.get("_buckets", 8), cfg.get("_ranks", (4, 4))
    s = {"embed": (V, W), "pos": (cfg["max_positions"], W), "head": (V, W)}
    def norm(name):
        s[name], s[name + ".b"], s[name + ".alpha"] = (W,), (W,), ()
    norm("embed.norm")
    norm("final.norm")
    for i, L in enumerate(cfg["layers"]):
        p, mx = "l%d." % i, L["mixer"]
        norm(p + "norm1")
        s[p + "rg1"], s[p + "rg1.b"], s[p + "dwa"] = (W, W), (W,), (i + 2,)
        if L["type"] == "gla":
            H, dn, dv = mx["heads"], mx["dim"], mx["vdim"]
            q = p + "mix."
            s[q + "q"], s[q + "k"], s[q + "v"], s[q + "g"], s[q + "o"], s[q + "norm"] = (H * dn, W), (H * dn, W), (H * dv, W), (H * dv, W), (W, H * dv), (dv,)
            s[q + "a1"], s[q + "a2"], s[q + "a2.b"] = (ra, W), (H * dn, ra), (H * dn,)
        else:
            l, r = mx["left"], mx["right"]
            H, G, dn, dv = l["heads"], l.get("kv_heads", l["heads"]), l["dim"], l["vdim"]
            q = p + "mix.left."
            s[q + "q"], s[q + "q.b"], s[q + "k"], s[q + "k.b"], s[q + "v"], s[q + "v.b"] = (H * dn, W), (H * dn,), (G * dn, W), (G * dn,), (G * dv, W), (G * dv,)
            s[q + "rel"], s[q + "g"], s[q + "o"], s[q + "o.b"] = (B, H), (H * dv, W), (W, H * dv), (W,)
            q, hd = p + "mix.right.", r["heads"] * r["dim"]
            for nm in ("r", "k", "v", "g", "a"):
                s[q + nm] = (hd, W)
            s[q + "a.b"], s[q + "w1"], s[q + "w2"], s[q + "w0"], s[q + "norm"], s[q + "o"] = (hd,), (rw, W), (hd, rw), (hd,), (hd,), (W, hd)
        if L.get("mlp"):
            norm(p + "norm2")
            ff = L["mlp"]["ff"]
            s[p + "mlp.gate"], s[p + "mlp.up"], s[p + "mlp.down"], s[p + "rg2"], s[p + "rg2.b"] = (ff, W), (ff, W), (W, ff), (W, W), (W,)
    return s


def random_weights(cfg, seed, gain=1.0):
    """bfloat16-representable values: matrices ~ N(0, gain / in), norm weights around one, alphas around one, depth weights around an average with a
    preference for the newest result, decays spread over (0, 1)"""
    g = np.random.default_rng(seed)
    w = {}
    for name, shp in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if last == "alpha":
            v = np.array(0.6 + 0.8 * g.random())
        elif last == "dwa":
            n = shp[0]
            v = 0.5 / n + 0.2 * g.standard_normal(n) / n
            v[-1] += 0.6
        elif len(shp) == 1 and last in ("norm", "norm1", "norm2"):
            v = 1.0 + 0.2 * g.standard_normal(shp)
        elif name == "embed" or name == "pos":
            v = g.standard_normal(shp) * (1.0 if name == "embed" else 0.5)
        elif last == "rel":
            v = g.standard_normal(shp)
        elif last == "w0":
            v = g.standard_normal(shp) * 1.5
        elif name.endswith("a2.b"):
            v = 2.0 + g.standard_normal(shp) * 1.5
        elif len(shp) == 1:
            v = 0.3 * g.standard_normal(shp)
        else:
            v = g.standard_normal(shp) * gain / math.sqrt(shp[-1])
        w[name] = bf16_round(np.asarray(v, np.float32))
    return w


def save_model(folder, cfg, w):
    """config.json (without the keys that only describe tensor shapes) + model.safetensors (bfloat16) written by hand"""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump({k: v for k, v in cfg.items() if not k.startswith("_")}, f)
    header, blobs, at = {}, [], 0
    for name, t in w.items():
        raw = (np.ascontiguousarray(t, np.float32).view(np.uint32) >> 16).astype(np.uint16).tobytes()
        header[name] = {"dtype": "BF16", "shape": list(np.shape(t)), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for b in blobs:
            f.write(b)
