"""Plain float64 restatement of the Fifotar family (the scaled-sandwich form of the layer stack), one function per mechanism, for the tests: numpy only,
loops over tokens where a mechanism is a recurrence, nothing shared with the product.

Notation.  x [T, W] is the stream, h a sublayer's input, matrices are stored [out, in] and applied as h @ M.T, m = residual_mult.
  rms(x; w)     = x / sqrt(mean(x^2) + eps) * w
  embedding     x = E[token] * embedding.scale
  layer         x += m * rms(mixer(rms(x; n1)); n1b)        x += m * rms(ff(rms(x; n2)); n2b)   (the second only where the layer has a feed-forward)
  logits        z = E @ rms(x; final);  cap * tanh(z / cap)
  mixers        chunked_attention (no positions; capped scores; a sink in the softmax; values blended with the first such layer's; elementwise gate)
                latent_attention  (queries through a normed latent; one normed latent + one rotated key part per position; half-split rotation with
                                   blended frequencies; per-head gate)
                gated_delta       (short causal convolutions + silu on q, k, v; unit q and k; scalar decay per head; delta-rule write; gated unit norm)
  feed-forward  down(act(min(gate h, L)) * (clamp(up h, -L, L) + 1)),  act(g) = g * sigmoid(1.702 g)
"""
import json
import math
import os
import struct

import numpy as np

F = np.float64
UNIT_EPS = 1e-6
GLU_SLOPE = 1.702


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.maximum(z, 0.0) + np.log1p(np.exp(-np.abs(z)))


def rms(x, w, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


# ---------------------------------------------------------------------------------------------------------------- chunked attention with a sink
def sees_chunk(i, j, size):
    """query position i, key position j; size None or 0: plain causal"""
    return j <= i and (not size or i // size == j // size)


def capped(s, cap):
    return cap * np.tanh(s / cap) if cap else s


def sink_softmax(s):
    """exp(s_j) / (1 + sum exp(s)): a silent extra key of score 0 that carries no value"""
    m = max(0.0, float(np.max(s))) if len(s) else 0.0
    e = np.exp(s - m)
    return e / (math.exp(-m) + e.sum())


def attend(q, k, v, pos0, scale, size=None, cap=None, sink=True):
    """q [T, H, dn] at positions pos0 ..; k [P, G, dn], v [P, G, dv] of positions 0 .. P - 1 -> [T, H, dv]"""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]), F)
    for t in range(T):
        p = pos0 + t
        js = [j for j in range(p + 1) if sees_chunk(p, j, size)]
        for hh in range(H):
            g = hh // (H // G)
            s = capped((k[js, g] @ q[t, hh]) * scale, cap)
            if sink:
                wts = sink_softmax(s)
            else:
                e = np.exp(s - s.max())
                wts = e / e.sum()
            out[t, hh] = wts @ v[js, g]
    return out


def chunked_attention(h, w, pre, mx, pos0=0, past=None, v_first=None):
    """h [T, W] at positions pos0 ..; past = (k, v) of earlier positions; v_first [T, G, dv]: the first blending layer's values of the same tokens (None in
    that layer itself or without blending) -> (out [T, W], (k, v) so far, this layer's raw values [T, G, dv])"""
    T = h.shape[0]
    H, G, dn, dv = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
    q = (h @ w[pre + "q"].T).reshape(T, H, dn)
    k = (h @ w[pre + "k"].T).reshape(T, G, dn)
    v = (h @ w[pre + "v"].T).reshape(T, G, dv)
    v_own = v
    if v_first is not None:
        lam = float(w[pre + "vmix"])
        v = (1.0 - lam) * v + lam * v_first
    if past is not None:
        k, v = np.concatenate([past[0], k]), np.concatenate([past[1], v])
    out = attend(q, k, v, pos0, mx["scale"], (mx.get("mask") or {}).get("size"), mx.get("softcap"))
    out = out.reshape(T, H * dv) * sigmoid(h @ w[pre + "g"].T)
    return out @ w[pre + "o"].T, (k, v), v_own


# ---------------------------------------------------------------------------------------------------------------- latent attention
def blended_frequencies(rot):
    """(f [dims / 2], magnitude): base^(-2i/dims), and with 'scaling' a blend between f and f / factor along a ramp over the pair index"""
    dims, base = rot["dims"], rot["base"]
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)], F)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    def where(turns):
        return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(where(sc["fast"])), 0)
    hi = min(math.ceil(where(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate_halves(x, pos, freq, mag, dims):
    """x [..., n]: entry i < dims/2 is paired with entry i + dims/2; the rest passes"""
    half = dims // 2
    a = pos * freq
    c, s = np.cos(a) * mag, np.sin(a) * mag
    y = np.array(x, F)
    u, v = x[..., :half], x[..., half:dims]
    y[..., :half] = u * c - v * s
    y[..., half:dims] = v * c + u * s
    return y


def latent_attention(h, w, pre, mx, eps, pos0=0, past=None):
    """past = (latents [P, R], rotated key parts [P, dr]) -> (out [T, W], (latents, key parts) so far)"""
    T = h.shape[0]
    H, dn, dr, dv, R = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    freq, mag = blended_frequencies(mx["rot"])
    dims = mx["rot"]["dims"]
    cq = rms(h @ w[pre + "dq"].T, w[pre + "dq.norm"], eps)
    q = (cq @ w[pre + "uq"].T).reshape(T, H, dn + dr)
    kv = h @ w[pre + "dkv"].T
    lat = rms(kv[:, :R], w[pre + "dkv.norm"], eps)
    kr = np.stack([rotate_halves(kv[t, R:], pos0 + t, freq, mag, dims) for t in range(T)])
    if past is not None:
        lat, kr = np.concatenate([past[0], lat]), np.concatenate([past[1], kr])
    kn = (lat @ w[pre + "uk"].T).reshape(-1, H, dn)
    vv = (lat @ w[pre + "uv"].T).reshape(-1, H, dv)
    gate = sigmoid(h @ w[pre + "g"].T)           # [T, H]
    out = np.zeros((T, H, dv), F)
    for t in range(T):
        p = pos0 + t
        for hh in range(H):
            qr = rotate_halves(q[t, hh, dn:], p, freq, mag, dims)
            s = (kn[:p + 1, hh] @ q[t, hh, :dn] + kr[:p + 1] @ qr) * mx["scale"]
            e = np.exp(s - s.max())
            out[t, hh] = (e / e.sum()) @ vv[:p + 1, hh] * gate[t, hh]
    return out.reshape(T, H * dv) @ w[pre + "o"].T, (lat, kr)


# ---------------------------------------------------------------------------------------------------------------- gated delta rule
def short_conv(z, taps_w, carried=None):
    """z [T, C]; taps_w [C, K], column K - 1 weighs the present token; carried [K - 1, C]: the inputs before this portion (zeros at a sequence's start)
    -> (silu(conv) [T, C], the last K - 1 inputs)"""
    K = taps_w.shape[1]
    if carried is None:
        carried = np.zeros((K - 1, z.shape[1]), F)
    full = np.concatenate([carried, z])
    y = np.zeros_like(z)
    for t in range(z.shape[0]):
        for j in range(K):
            y[t] += taps_w[:, j] * full[t + j]
    return silu(y), full[full.shape[0] - (K - 1):]


def unit(x):
    return x / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) + UNIT_EPS)


def delta_walk(q, k, v, beta, decay, state=None):
    """q, k [T, H, dn] (already unit / scaled), v [T, H, dv], beta, decay [T, H]: S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q"""
    T, H, dn = k.shape
    dv = v.shape[2]
    S = np.zeros((H, dn, dv), F) if state is None else np.array(state, F)
    o = np.zeros((T, H, dv), F)
    for t in range(T):
        for hh in range(H):
            S[hh] *= decay[t, hh]
            u = beta[t, hh] * (v[t, hh] - S[hh].T @ k[t, hh])
            S[hh] += np.outer(k[t, hh], u)
            o[t, hh] = S[hh].T @ q[t, hh]
    return o, S


def gated_delta(h, w, pre, mx, eps, carry=None):
    """carry = (S [H, dn, dv], conv inputs of q, k, v) -> (out [T, W], carry)"""
    T = h.shape[0]
    H, G, dn, dv = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
    S, cq, ck, cv = carry if carry is not None else (None, None, None, None)
    q, cq = short_conv(h @ w[pre + "q"].T, w[pre + "q.conv"], cq)
    k, ck = short_conv(h @ w[pre + "k"].T, w[pre + "k.conv"], ck)
    v, cv = short_conv(h @ w[pre + "v"].T, w[pre + "v.conv"], cv)
    q = unit(q.reshape(T, G, dn)) * dn ** -0.5
    k = unit(k.reshape(T, G, dn))
    share = np.arange(H) // (H // G)
    q, k = q[:, share], k[:, share]
    beta = sigmoid(h @ w[pre + "b"].T)
    decay = np.exp(-np.exp(w[pre + "A_log"]) * softplus(h @ w[pre + "a"].T + w[pre + "dt_bias"]))
    o, S = delta_walk(q, k, v.reshape(T, H, dv), beta, decay, S)
    o = o / np.sqrt(np.mean(o * o, axis=-1, keepdims=True) + eps) * w[pre + "norm"]
    o = o.reshape(T, H * dv) * silu(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T, (S, cq, ck, cv)


# ---------------------------------------------------------------------------------------------------------------- feed-forward
def clipped_unit(h, w, pre, ml):
    L = ml["limit"]
    g = np.minimum(h @ w[pre + "gate"].T, L)
    u = np.clip(h @ w[pre + "up"].T, -L, L)
    return (g * sigmoid(GLU_SLOPE * g) * (u + 1.0)) @ w[pre + "down"].T


# ---------------------------------------------------------------------------------------------------------------- the model
class Sequence:
    """what a sequence carries from portion to portion: its length and, per layer, keys / values, latents or a state"""

    def __init__(self, cfg):
        self.n = 0
        self.per_layer = [None] * len(cfg["layers"])


def forward(cfg, w, tokens, seq=None, layers_out=None):
    """tokens appended to seq (a new sequence if None) -> logits [T, vocab]; layers_out (a list) receives the stream after every layer"""
    seq = seq if seq is not None else Sequence(cfg)
    eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    E = w["embed"]
    x = E[np.asarray(tokens)] * cfg["embedding"]["scale"]
    v_first = None
    seen_blend = False
    for i, L in enumerate(cfg["layers"]):
        p = "l%d." % i
        mx = L["mixer"]
        h = rms(x, w[p + "norm1"], eps)
        if L["type"] == "attention":
            blend = bool(mx.get("v_mix"))
            y, seq.per_layer[i], v_own = chunked_attention(h, w, p + "mix.", mx, seq.n, seq.per_layer[i], v_first if (blend and seen_blend) else None)
            if blend and not seen_blend:
                v_first, seen_blend = v_own, True
        elif L["type"] == "latent_attention":
            y, seq.per_layer[i] = latent_attention(h, w, p + "mix.", mx, eps, seq.n, seq.per_layer[i])
        elif L["type"] == "delta":
            y, seq.per_layer[i] = gated_delta(h, w, p + "mix.", mx, eps, seq.per_layer[i])
        else:
            raise ValueError(L["type"])
        x = x + m * rms(y, w[p + "norm1b"], eps)
        if L.get("mlp"):
            y = clipped_unit(rms(x, w[p + "norm2"], eps), w, p + "mlp.", L["mlp"])
            x = x + m * rms(y, w[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    seq.n += len(tokens)
    z = rms(x, w["final.norm"], eps) @ E.T
    cap = cfg.get("logit_softcap")
    return (cap * np.tanh(z / cap) if cap else z), seq


def greedy(cfg, w, prompt, n):
    """n tokens, each the argmax of the last position's logits"""
    logits, seq = forward(cfg, w, prompt)
    out = []
    for _ in range(n):
        out.append(int(np.argmax(logits[-1])))
        logits, seq = forward(cfg, w, [out[-1]], seq)
    return out


# ---------------------------------------------------------------------------------------------------------------- configurations and folders
def attention_layer(heads=4, kv_heads=2, dim=8, vdim=8, size=16, softcap=20.0, v_mix=True, ff=24, limit=2.0, scale=None):
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if size:
        mx["mask"] = {"size": size}
    if softcap:
        mx["softcap"] = softcap
    if v_mix:
        mx["v_mix"] = True
    return {"type": "attention", "mixer": mx, "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def latent_layer(heads=3, dim=8, rot_dim=4, vdim=8, kv_rank=12, q_rank=16, base=10000.0, scaling=None, ff=24, limit=2.0, scale=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = scaling
    mx = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "rot": rot,
          "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    return {"type": "latent_attention", "mixer": mx, "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def delta_layer(heads=4, kv_heads=2, dim=8, vdim=8, conv=4, ff=0, limit=2.0):
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}
    return {"type": "delta", "mixer": mx, "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def config(layers, vocab=61, width=32, eps=1e-5, mult=0.6, embed_scale=None, logit_softcap=25.0):
    cfg = {"architecture": "Fifotar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
           "embedding": {"scale": embed_scale if embed_scale is not None else math.sqrt(width)}, "layers": layers}
    if logit_softcap:
        cfg["logit_softcap"] = logit_softcap
    return cfg


def shapes_of(cfg):
    W, out = cfg["width"], {}
    out["embed"] = (cfg["vocab"], W)
    out["final.norm"] = (W,)
    for i, L in enumerate(cfg["layers"]):
        p, mx = "l%d." % i, L["mixer"]
        out[p + "norm1"] = out[p + "norm1b"] = (W,)
        if L["type"] == "attention":
            H, G, dn, dv = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
            out[p + "mix.q"], out[p + "mix.k"], out[p + "mix.v"] = (H * dn, W), (G * dn, W), (G * dv, W)
            out[p + "mix.g"], out[p + "mix.o"] = (H * dv, W), (W, H * dv)
            if mx.get("v_mix"):
                out[p + "mix.vmix"] = ()
        elif L["type"] == "latent_attention":
            H, dn, dr, dv, R, Q = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"], mx["q_rank"]
            out[p + "mix.dq"], out[p + "mix.dq.norm"], out[p + "mix.uq"] = (Q, W), (Q,), (H * (dn + dr), Q)
            out[p + "mix.dkv"], out[p + "mix.dkv.norm"] = (R + dr, W), (R,)
            out[p + "mix.uk"], out[p + "mix.uv"] = (H * dn, R), (H * dv, R)
            out[p + "mix.g"], out[p + "mix.o"] = (H, W), (W, H * dv)
        else:
            H, G, dn, dv, K = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"], mx["conv"]
            for nm, rows in (("q", G * dn), ("k", G * dn), ("v", H * dv)):
                out[p + "mix." + nm] = (rows, W)
                out[p + "mix." + nm + ".conv"] = (rows, K)
            out[p + "mix.b"] = out[p + "mix.a"] = (H, W)
            out[p + "mix.A_log"] = out[p + "mix.dt_bias"] = (H,)
            out[p + "mix.norm"] = (dv,)
            out[p + "mix.g"], out[p + "mix.o"] = (H * dv, W), (W, H * dv)
        if L.get("mlp"):
            ff = L["mlp"]["ff"]
            out[p + "norm2"] = out[p + "norm2b"] = (W,)
            out[p + "mlp.gate"] = out[p + "mlp.up"] = (ff, W)
            out[p + "mlp.down"] = (W, ff)
    return out


def to_bf16(a):
    """round to the nearest bfloat16 (ties to even), returned as float64"""
    b = np.asarray(a, np.float32).view(np.uint32).astype(np.uint64)
    b = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16) << 16
    return b.astype(np.uint32).view(np.float32).astype(F)


def random_weights(cfg, seed=1, gain=1.0):
    rng = np.random.default_rng(seed)
    w = {}
    for name, shp in shapes_of(cfg).items():
        last = name.split(".")[-1]
        if "norm" in last:
            a = 1.0 + 0.2 * rng.standard_normal(shp)
        elif last == "vmix":
            a = np.array(rng.uniform(0.2, 0.7))
        elif last == "A_log":
            a = rng.uniform(-3.0, 0.5, shp)
        elif last == "dt_bias":
            a = rng.uniform(-2.0, 1.0, shp)
        elif last == "conv":
            a = rng.standard_normal(shp) * 0.5
        elif name == "embed":
            a = rng.standard_normal(shp) / math.sqrt(shp[1])
        else:
            a = rng.standard_normal(shp) * gain / math.sqrt(shp[-1])
        w[name] = to_bf16(a)
    return w


def save_model(folder, cfg, w):
    """config.json + model.safetensors (bfloat16)"""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    header, blobs, at = {}, [], 0
    for name in sorted(w):
        a = np.asarray(w[name], np.float32)
        bits = (a.view(np.uint32) >> 16).astype(np.uint16)
        raw = bits.tobytes()
        header[name] = {"dtype": "BF16", "shape": list(a.shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    hj = json.dumps(header).encode()
    hj += b" " * ((8 - len(hj) % 8) % 8)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for b in blobs:
            f.write(b)


def load_model(folder):
    """(config, weights as float64) of a folder written by save_model or any bfloat16 / float32 safetensors file"""
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    with open(os.path.join(folder, "model.safetensors"), "rb") as f:
        n = struct.unpack("<Q", f.read(8))[0]
        header = json.loads(f.read(n))
        data = f.read()
    w = {}
    for name, t in header.items():
        if name == "__metadata__":
            continue
        lo, hi = t["data_offsets"]
        if t["dtype"] == "BF16":
            a = (np.frombuffer(data[lo:hi], np.uint16).astype(np.uint32) << 16).view(np.float32)
        elif t["dtype"] == "F32":
            a = np.frombuffer(data[lo:hi], np.float32)
        else:
            continue
        w[name] = a.astype(F).reshape(t["shape"])
    return cfg, w
