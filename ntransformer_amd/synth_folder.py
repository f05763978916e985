"""Seeded synthetic model folders (config.json + model.safetensors, bfloat16) for the layer-list families: the counterpart of the seeded GGUF
generator (csrc/engine/synth.cpp) for benchmarks that need real-sized layers without a checkpoint.  Values come from one random pool that is
repeated to fill a tensor -- timing does not care, and gigabytes are written in seconds."""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Dict, Tuple

import numpy as np

PRESETS = {
    # name: width, heads, dim, rot_dim, vdim, kv_rank, q_rank, window, experts, top, ff, shared_ff, vocab
    "tiny": dict(width=192, heads=4, dim=24, rot_dim=8, vdim=40, kv_rank=64, q_rank=80, window=48, experts=6, top=2, ff=112, shared_ff=160, vocab=1024),
    "lite": dict(width=2048, heads=16, dim=128, rot_dim=64, vdim=128, kv_rank=512, q_rank=768, window=1024, experts=64, top=6, ff=1408, shared_ff=2816, vocab=32000),
    "mid": dict(width=4096, heads=32, dim=128, rot_dim=64, vdim=128, kv_rank=512, q_rank=1536, window=2048, experts=32, top=4, ff=2048, shared_ff=4096, vocab=64000),
}


def fabolorn_config(preset: str, layers: int = 2, loop_times: int = 1) -> dict:
    p = PRESETS[preset]
    ls = []
    for k in range(layers):
        windowed = k % 2 == 1
        mx = {"heads": p["heads"], "dim": p["dim"], "rot_dim": p["rot_dim"], "vdim": p["vdim"], "kv_rank": p["kv_rank"],
              "scale": 1.0 / math.sqrt(p["dim"] + p["rot_dim"]), "rot": {"base": 1000000.0, "dims": p["rot_dim"]}}
        if windowed:
            mx["mask"] = {"size": p["window"]}
        else:
            mx["q_rank"] = p["q_rank"]
            mx["rot"]["scaling"] = {"factor": 8.0, "original": 4096, "fast": 16.0, "slow": 2.0}
        ml = {"kind": "moe", "expert": {"ff": p["ff"], "limit": 7.0}, "router": {"experts": p["experts"], "top": p["top"]},
              "shared": {"ff": p["shared_ff"], "limit": 7.0}}
        ls.append({"type": "latent_attention_2" if windowed else "latent_attention", "mixer": mx, "mlp": ml})
    cfg = {"architecture": "Fabolorn", "layers": ls, "norm": {"eps": 1e-5}, "vocab": p["vocab"], "width": p["width"]}
    if loop_times > 1:
        cfg["loop"] = {"start": 0, "stop": layers, "times": loop_times}
    return cfg


def fabolorn_shapes(cfg: dict) -> Dict[str, Tuple[int, ...]]:
    W, V = cfg["width"], cfg["vocab"]
    s: Dict[str, Tuple[int, ...]] = {"embed": (V, W), "final.norm": (W,), "head": (V, W)}
    if cfg.get("loop"):
        s["loop.in"] = (W, 2 * W)
    for i, L in enumerate(cfg["layers"]):
        p, mx, ml = "l%d." % i, L["mixer"], L.get("mlp")
        H, dn, dr, dv, R = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
        s[p + "norm1"] = (W,)
        if "q_rank" in mx:
            s[p + "mix.dq"], s[p + "mix.dq.norm"], s[p + "mix.uq"] = (mx["q_rank"], W), (mx["q_rank"],), (H * (dn + dr), mx["q_rank"])
        else:
            s[p + "mix.q"] = (H * (dn + dr), W)
        s[p + "mix.dkv"], s[p + "mix.dkv.norm"] = (R + dr, W), (R,)
        s[p + "mix.uk"], s[p + "mix.uv"], s[p + "mix.g"], s[p + "mix.o"] = (H * dn, R), (H * dv, R), (H * dv, W), (W, H * dv)
        if ml:
            s[p + "norm2"] = (W,)
            ff = ml["expert"]["ff"]
            for e in range(ml["router"]["experts"]):
                q = "%smlp.e%d." % (p, e)
                s[q + "gate"], s[q + "up"], s[q + "down"] = (ff, W), (ff, W), (W, ff)
            s[p + "mlp.router"] = (ml["router"]["experts"], W)
            if ml.get("shared"):
                sf = ml["shared"]["ff"]
                s[p + "mlp.shared.gate"], s[p + "mlp.shared.up"], s[p + "mlp.shared.down"], s[p + "mlp.shared.sg"] = (sf, W), (sf, W), (W, sf), (1, W)
    return s


def nizorax_config(preset: str, layers: int = 2, dense_only: bool = False) -> dict:
    """the sequential family at the preset's width, heads, experts and vocabulary: attention layers (two score maps of half the preset's key size each,
    four query heads per key/value head, the preset's window) alternate with lightning layers; every third layer (dense_only: every layer) has the dense
    feed-forward at the mixture's active width, the others the mixture (groups of eight experts, half of the groups open)"""
    p = PRESETS[preset]
    H, dn = p["heads"], p["dim"] + p["rot_dim"]
    ls = []
    for k in range(layers):
        if k % 2 == 0:
            mx = {"heads": H, "kv_heads": max(H // 4, 1), "dim": dn // 2, "vdim": p["vdim"], "diff": 0.8, "scale": 1.0 / math.sqrt(dn // 2),
                  "mask": {"size": p["window"]}, "rot": {"base": 1000000.0, "dims": dn // 4, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 4096}}}
            t = "attention"
        else:
            mx = {"heads": H, "dim": dn // 2 if dn // 2 <= 128 else 128, "vdim": p["vdim"], "decay": [1.0 - 2.0 ** (-5.0 - 3.0 * h / max(H - 1, 1)) for h in range(H)]}
            t = "lightning"
        if k % 3 == 2 or dense_only:
            ml = {"kind": "dense", "ff": p["top"] * p["ff"] + p["shared_ff"]}
        else:
            per = 8 if p["experts"] % 8 == 0 and p["experts"] >= 16 else 1
            ml = {"kind": "moe", "expert": {"ff": p["ff"]}, "router": {"experts": p["experts"], "top": p["top"], "scale": 2.0}, "shared": {"ff": p["shared_ff"]}}
            if per > 1:
                ml["router"]["groups"] = {"count": p["experts"] // per, "keep": max(p["experts"] // per // 2, 1)}
        ls.append({"type": t, "mixer": mx, "mlp": ml})
    return {"architecture": "Nizorax", "layers": ls, "norm": {"eps": 1e-5}, "canon": {"taps": 4}, "embedding": {"scale": math.sqrt(p["width"])},
            "logit_scale": 1.0 / math.sqrt(p["width"]), "vocab": p["vocab"], "width": p["width"]}


def nizorax_shapes(cfg: dict) -> Dict[str, Tuple[int, ...]]:
    W, V, taps = cfg["width"], cfg["vocab"], cfg["canon"]["taps"]
    s: Dict[str, Tuple[int, ...]] = {"embed": (V, W), "final.norm": (W,), "final.norm.b": (W,), "head": (V, W)}
    for i, L in enumerate(cfg["layers"]):
        p, mx, ml = "l%d." % i, L["mixer"], L.get("mlp")
        for nm in ("norm1", "norm1b") + (("norm2", "norm2b") if ml else ()):
            s[p + nm], s[p + nm + ".b"] = (W,), (W,)
        s[p + "canon1"] = (W, taps)
        if ml:
            s[p + "canon2"] = (W, taps)
        H, dn, dv = mx["heads"], mx["dim"], mx["vdim"]
        if L["type"] == "attention":
            G = mx.get("kv_heads", H)
            s[p + "mix.q"], s[p + "mix.k"], s[p + "mix.v"], s[p + "mix.o"] = (H * 2 * dn, W), (G * 2 * dn, W), (G * dv, W), (W, H * dv)
            for nm in ("lq1", "lk1", "lq2", "lk2"):
                s[p + "mix." + nm] = (dn,)
        else:
            s[p + "mix.q"], s[p + "mix.k"], s[p + "mix.v"], s[p + "mix.g"] = (H * dn, W), (H * dn, W), (H * dv, W), (H * dv, W)
            s[p + "mix.o"], s[p + "mix.norm"] = (W, H * dv), (H * dv,)
        if ml and ml["kind"] == "dense":
            s[p + "mlp.up"], s[p + "mlp.down"], s[p + "mlp.act"] = (ml["ff"], W), (W, ml["ff"]), (4,)
        elif ml:
            ff = ml["expert"]["ff"]
            for e in range(ml["router"]["experts"]):
                q = "%smlp.e%d." % (p, e)
                s[q + "gate"], s[q + "up"], s[q + "down"] = (ff, W), (ff, W), (W, ff)
            s[p + "mlp.router"] = (ml["router"]["experts"], W)
            if ml.get("shared"):
                sf = ml["shared"]["ff"]
                s[p + "mlp.shared.gate"], s[p + "mlp.shared.up"], s[p + "mlp.shared.down"] = (sf, W), (sf, W), (W, sf)
    return s


def tubazen_config(preset: str, layers: int = 2, positions: int = 8192) -> dict:
    """the gated family at the preset's width, heads and vocabulary: layers with two mixers side by side (attention over four query heads per key/value
    head with a distance-bias table of 32 rows, beside a delta-rule recurrence with 64-entry keys) alternate with gated-linear-attention layers (keys 96,
    the preset's value size); every layer has the gated feed-forward with the bytes of a two-matrix feed-forward at the mixture's active width"""
    p = PRESETS[preset]
    H, dn = p["heads"], p["dim"]
    ff = (p["top"] * p["ff"] + p["shared_ff"]) * 2 // 3
    ff -= ff % 64
    ls = []
    for k in range(layers):
        if k % 2 == 0:
            left = {"heads": H, "kv_heads": max(H // 4, 1), "dim": dn, "vdim": p["vdim"], "bias_max": 4096, "scale": 1.0 / math.sqrt(dn), "q_temp": {"coef": 0.1, "every": 512}}
            mx = {"left": left, "right": {"heads": H, "dim": max(dn // 2, 8)}, "left_scale": 0.8, "right_scale": 0.5}
            t = "parallel"
        else:
            mx = {"heads": H, "dim": max(3 * dn // 4, 8), "vdim": p["vdim"], "tau": 16.0}
            t = "gla"
        ls.append({"type": t, "mixer": mx, "mlp": {"kind": "dense", "ff": max(ff, 64)}})
    return {"architecture": "Tubazen", "layers": ls, "norm": {"eps": 1e-5}, "logit_scale": 1.0 / math.sqrt(p["width"]), "max_positions": positions,
            "vocab": p["vocab"], "width": p["width"]}


def tubazen_shapes(cfg: dict, buckets: int = 32, rank: int = 64) -> Dict[str, Tuple[int, ...]]:
    W, V = cfg["width"], cfg["vocab"]
    rank = min(rank, max(W // 8, 4))
    s: Dict[str, Tuple[int, ...]] = {"embed": (V, W), "pos": (cfg["max_positions"], W), "head": (V, W)}
    for nm in ("embed.norm", "final.norm"):
        s[nm], s[nm + ".b"], s[nm + ".alpha"] = (W,), (W,), ()
    for i, L in enumerate(cfg["layers"]):
        p, mx, ml = "l%d." % i, L["mixer"], L.get("mlp")
        for nm in ("norm1",) + (("norm2",) if ml else ()):
            s[p + nm], s[p + nm + ".b"], s[p + nm + ".alpha"] = (W,), (W,), ()
        s[p + "rg1"], s[p + "rg1.b"], s[p + "dwa"] = (W, W), (W,), (i + 2,)
        if L["type"] == "gla":
            H, dn, dv, q = mx["heads"], mx["dim"], mx["vdim"], p + "mix."
            s[q + "q"], s[q + "k"], s[q + "v"], s[q + "g"], s[q + "o"], s[q + "norm"] = (H * dn, W), (H * dn, W), (H * dv, W), (H * dv, W), (W, H * dv), (dv,)
            s[q + "a1"], s[q + "a2"], s[q + "a2.b"] = (rank, W), (H * dn, rank), (H * dn,)
        else:
            l, r = mx["left"], mx["right"]
            H, G, dn, dv, q = l["heads"], l.get("kv_heads", l["heads"]), l["dim"], l["vdim"], p + "mix.left."
            s[q + "q"], s[q + "q.b"], s[q + "k"], s[q + "k.b"], s[q + "v"], s[q + "v.b"] = (H * dn, W), (H * dn,), (G * dn, W), (G * dn,), (G * dv, W), (G * dv,)
            s[q + "rel"], s[q + "g"], s[q + "o"], s[q + "o.b"] = (buckets, H), (H * dv, W), (W, H * dv), (W,)
            q, hd = p + "mix.right.", r["heads"] * r["dim"]
            for nm in ("r", "k", "v", "g", "a"):
                s[q + nm] = (hd, W)
            s[q + "a.b"], s[q + "w1"], s[q + "w2"], s[q + "w0"], s[q + "norm"], s[q + "o"] = (hd,), (rank, W), (hd, rank), (hd,), (hd,), (W, hd)
        if ml:
            s[p + "mlp.gate"], s[p + "mlp.up"], s[p + "mlp.down"], s[p + "rg2"], s[p + "rg2.b"] = (ml["ff"], W), (ml["ff"], W), (W, ml["ff"]), (W, W), (W,)
    return s


def fifotar_config(preset: str, layers: int = 4, mlp_everywhere: bool = True) -> dict:
    """the scaled family at the preset's width, heads and vocabulary: chunked attention (four query heads per key/value head, chunks of the preset's window,
    capped scores, blended values), the per-head delta rule (two value heads per key head, keys and values of the preset's sizes, four taps) and latent
    attention (the preset's ranks) in the order attention, delta, latent, delta; the clipped gated feed-forward with the bytes of the gated family's"""
    p = PRESETS[preset]
    H, dn, dv = p["heads"], p["dim"], p["vdim"]
    ff = (p["top"] * p["ff"] + p["shared_ff"]) * 2 // 3
    ff -= ff % 64
    ls = []
    for k in range(layers):
        if k % 4 == 0:
            mx = {"heads": H, "kv_heads": max(H // 4, 1), "dim": dn, "vdim": dv, "scale": 1.0 / math.sqrt(dn), "softcap": 40.0, "mask": {"size": p["window"]}, "v_mix": True}
            t = "attention"
        elif k % 4 == 2:
            mx = {"heads": H, "dim": dn, "rot_dim": p["rot_dim"], "vdim": dv, "kv_rank": p["kv_rank"], "q_rank": p["q_rank"], "scale": 1.0 / math.sqrt(dn + p["rot_dim"]),
                  "rot": {"base": 1000000.0, "dims": p["rot_dim"], "scaling": {"factor": 8.0, "original": 4096, "fast": 16.0, "slow": 2.0}}}
            t = "latent_attention"
        else:
            mx = {"heads": H, "kv_heads": max(H // 2, 1), "dim": dn, "vdim": dv, "conv": 4}
            t = "delta"
        has_mlp = mlp_everywhere or t != "delta"
        ls.append({"type": t, "mixer": mx, "mlp": {"kind": "dense", "ff": max(ff, 64), "limit": 7.0} if has_mlp else None})
    return {"architecture": "Fifotar", "layers": ls, "norm": {"eps": 1e-5}, "embedding": {"scale": math.sqrt(p["width"])}, "residual_mult": 0.7, "logit_softcap": 25.0,
            "vocab": p["vocab"], "width": p["width"]}


def fifotar_shapes(cfg: dict) -> Dict[str, Tuple[int, ...]]:
    W, V = cfg["width"], cfg["vocab"]
    s: Dict[str, Tuple[int, ...]] = {"embed": (V, W), "final.norm": (W,)}
    for i, L in enumerate(cfg["layers"]):
        p, mx, ml = "l%d." % i, L["mixer"], L.get("mlp")
        for nm in ("norm1", "norm1b") + (("norm2", "norm2b") if ml else ()):
            s[p + nm] = (W,)
        q = p + "mix."
        H, dn, dv = mx["heads"], mx["dim"], mx["vdim"]
        if L["type"] == "attention":
            G = mx.get("kv_heads", H)
            s[q + "q"], s[q + "k"], s[q + "v"], s[q + "g"], s[q + "o"] = (H * dn, W), (G * dn, W), (G * dv, W), (H * dv, W), (W, H * dv)
            if mx.get("v_mix"):
                s[q + "vmix"] = ()
        elif L["type"] == "latent_attention":
            dr, R, Q = mx["rot_dim"], mx["kv_rank"], mx["q_rank"]
            s[q + "dq"], s[q + "dq.norm"], s[q + "uq"] = (Q, W), (Q,), (H * (dn + dr), Q)
            s[q + "dkv"], s[q + "dkv.norm"], s[q + "uk"], s[q + "uv"] = (R + dr, W), (R,), (H * dn, R), (H * dv, R)
            s[q + "g"], s[q + "o"] = (H, W), (W, H * dv)
        else:
            G, K = mx.get("kv_heads", H), mx.get("conv", 1)
            for nm, rows in (("q", G * dn), ("k", G * dn), ("v", H * dv)):
                s[q + nm], s[q + nm + ".conv"] = (rows, W), (rows, K)
            s[q + "b"], s[q + "a"], s[q + "A_log"], s[q + "dt_bias"] = (H, W), (H, W), (H,), (H,)
            s[q + "norm"], s[q + "g"], s[q + "o"] = (dv,), (H * dv, W), (W, H * dv)
        if ml:
            s[p + "mlp.gate"], s[p + "mlp.up"], s[p + "mlp.down"] = (ml["ff"], W), (ml["ff"], W), (W, ml["ff"])
    return s


def shapes_of(cfg: dict) -> Dict[str, Tuple[int, ...]]:
    arch = cfg.get("architecture")
    return (nizorax_shapes(cfg) if arch == "Nizorax" else tubazen_shapes(cfg) if arch == "Tubazen" else fifotar_shapes(cfg) if arch == "Fifotar" else
            fabolorn_shapes(cfg))


def _bf16(a: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def write_folder(folder: str, cfg: dict, seed: int = 20260925) -> int:
    """-> bytes of model.safetensors"""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    shapes = shapes_of(cfg)
    g = np.random.default_rng(seed)
    pool = g.standard_normal(1 << 22).astype(np.float32)
    header, at = {}, 0
    for name, shp in shapes.items():
        n = int(np.prod(shp)) * 2
        header[name] = {"dtype": "BF16", "shape": list(shp), "data_offsets": [at, at + n]}
        at += n
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for k, (name, shp) in enumerate(shapes.items()):
            n = int(np.prod(shp))
            if len(shp) == 0 or name.endswith(".dwa"):       # a norm's slope around one; depth weights: an average over the results so far
                vals = (1.0 + 0.1 * pool[:1]) if len(shp) == 0 else (1.0 / n + 0.01 * pool[:n])
                if name.endswith(".vmix"):                    # a blend weight between zero and one
                    vals = np.array([0.5], np.float32)
                f.write(_bf16(vals).tobytes())
                continue
            if len(shp) == 1:
                around_one = name.endswith(".norm") and name != "final.norm"
                if cfg.get("architecture") == "Tubazen":
                    around_one = name.rsplit(".", 1)[-1] in ("norm", "norm1", "norm2")
                if cfg.get("architecture") == "Nizorax":     # layer-norm weights around one, biases / lambda vectors / activation numbers small
                    around_one = name.rsplit(".", 1)[-1] in ("norm", "norm1", "norm2", "norm1b", "norm2b")
                if cfg.get("architecture") == "Fifotar":     # every norm weight is stored plain; decay rates and biases small
                    around_one = "norm" in name.rsplit(".", 1)[-1]
                vals = 0.1 * pool[:n] + (1.0 if around_one else 0.0)
                f.write(_bf16(vals).tobytes())
                continue
            scale = 1.0 if name == "embed" else 1.0 / math.sqrt(shp[-1])
            block = _bf16(np.roll(pool, 7919 * k) * scale).tobytes()
            left = n * 2
            while left > 0:
                f.write(block[:min(left, len(block))])
                left -= len(block)
    return at
