"""Host side of the Tubazen family (no GPU): the folder reader and the registry know the family, and the float64 restatement's own invariants -- the
things the GPU tests lean on: causality, what every mechanism carries across a cut (cached keys and values, both recurrent states), the bucket map of
the distance bias, the query temperature's steps, the synthetic folders of the benchmark."""
import ctypes as C
import json
import math
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import tubazen_oracle as O  # noqa: E402
from ntransformer_amd import _lib  # noqa: E402


def describe(path):
    L = _lib.lib()
    L.nt_model_folder_describe.argtypes = [C.c_char_p, C.c_char_p, C.c_int]
    n = L.nt_model_folder_describe(path.encode(), None, 0)
    assert n >= 0
    buf = C.create_string_buffer(n + 1)
    assert L.nt_model_folder_describe(path.encode(), buf, n + 1) == n
    return json.loads(buf.value.decode())


def test_a_written_folder_is_described_and_its_family_is_built_in(tmp_path):
    cfg = O.small_config(layers=("parallel", "gla", "gla"), mlps=(True, None, True))
    w = O.random_weights(cfg, 3)
    O.save_model(str(tmp_path / "m"), cfg, w)
    d = describe(str(tmp_path / "m"))
    assert d["architecture"] == "Tubazen" and d["family_built_in"] is True and {"Tubazen", "Nizorax", "Fabolorn"} <= set(d["families"])
    got = {t["name"]: tuple(t["shape"]) for t in d["tensors"]}
    assert got == {k: tuple(np.shape(v)) for k, v in w.items()}
    assert "l1.norm2" not in got and "l1.rg2" not in got and got["l2.dwa"] == (4,) and got["embed.norm.alpha"] == ()
    assert "_buckets" not in json.load(open(tmp_path / "m" / "config.json"))


def test_causality_and_shapes():
    cfg = O.small_config(layers=("parallel", "gla", "parallel"), mlps=(True, None, True))
    w = O.random_weights(cfg, 2)
    toks = [int(t) for t in np.random.default_rng(0).integers(0, cfg["vocab"], 14)]
    lg, st = O.forward(cfg, w, toks, return_layers=True)
    assert st.shape == (3, 14, cfg["width"]) and lg.shape == (14, cfg["vocab"])
    assert np.allclose(lg[:9], O.forward(cfg, w, toks[:9]), atol=1e-10)


def test_every_mechanism_carries_what_a_cut_needs():
    cfg = O.small_config()
    w = {k: np.asarray(v, np.float64) for k, v in O.random_weights(cfg, 4).items()}
    g = np.random.default_rng(5)
    h = g.standard_normal((13, cfg["width"]))
    eps = cfg["norm"]["eps"]
    mx = cfg["layers"][0]["mixer"]
    whole, _ = O.biased_attention(h, w, "l0.mix.left.", mx["left"])
    a, past = O.biased_attention(h[:5], w, "l0.mix.left.", mx["left"])
    b, past = O.biased_attention(h[5:6], w, "l0.mix.left.", mx["left"], 5, past)
    c, _ = O.biased_attention(h[6:], w, "l0.mix.left.", mx["left"], 6, past)
    assert np.allclose(np.concatenate([a, b, c]), whole, atol=1e-12)
    for fn, pre, m in ((O.delta_rule, "l0.mix.right.", mx["right"]), (O.gla, "l1.mix.", cfg["layers"][1]["mixer"])):
        whole, S = fn(h, w, pre, m, eps)
        a, st = fn(h[:4], w, pre, m, eps)
        b, st = fn(h[4:], w, pre, m, eps, st)
        assert np.allclose(np.concatenate([a, b]), whole, atol=1e-12) and np.allclose(st, S, atol=1e-12)


def test_the_recurrence_forgets_per_channel_and_removes_along_the_unit_key():
    q = np.array([[[1.0, 0.0]], [[1.0, 0.0]], [[0.0, 1.0]]])
    k = np.array([[[2.0, 1.0]], [[0.0, 0.0]], [[0.0, 0.0]]])
    v = np.ones((3, 1, 1))
    decay = np.array([[[0.5, 1.0]]] * 3)
    o, S = O.decay_recurrence(q, k, v, decay)
    assert np.allclose(o[:, 0, 0], [2.0, 1.0, 1.0]) and np.allclose(S[0, :, 0], [0.5, 1.0])       # channel 0 halves every step, channel 1 keeps
    # removal at rate one along a unit key takes that direction out of the OLD state, before the token's own write
    k2 = np.array([[[3.0, 0.0]], [[1e-9, 0.0]]])
    o, S = O.decay_recurrence(np.array([[[1.0, 0.0]]] * 2), k2, np.ones((2, 1, 1)), np.ones((2, 1, 2)), np.ones((2, 1, 2)), unit_eps=1e-30)
    assert abs(o[0, 0, 0] - 3.0) < 1e-12 and abs(o[1, 0, 0]) < 1e-8


def test_bucket_map_and_temperature_steps():
    rows, reach = 12, 80
    b = [O.distance_bucket(n, rows, reach) for n in range(200)]
    assert b[:6] == list(range(6)) and b[6] == 6 and all(x <= y for x, y in zip(b, b[1:]))
    assert (b[51], b[52]) == (10, 11) and b[reach] == rows - 1 and b[199] == rows - 1      # the last row starts at 6 * (80 / 6)^(5 / 6) = 51.9
    assert [O.distance_bucket(n, 2, 5) for n in range(4)] == [0, 1, 1, 1]
    t = [O.query_temperature(p, 0.5, 8) for p in range(20)]
    assert t[0] == 1.0 and t[6] == 1.0 and abs(t[7] - (1 + 0.5 * math.log(2))) < 1e-15 and t[14] == t[7] and t[15] > t[14]


def test_gelu_is_a_sigmoid_gate_with_a_cubic_term():
    z = np.linspace(-6, 6, 101)
    alpha = 2 * math.sqrt(2 / math.pi)
    assert np.allclose(O.gelu_tanh(z), z * O.sigmoid(alpha * (z + 0.044715 * z ** 3)), atol=1e-14)


def test_synthetic_folders_of_the_benchmark_have_the_family_s_tensors(tmp_path):
    from ntransformer_amd import synth_folder as S
    cfg = S.tubazen_config("tiny", layers=3)
    S.write_folder(str(tmp_path / "s"), cfg)
    d = describe(str(tmp_path / "s"))
    assert d["architecture"] == "Tubazen" and d["family_built_in"] is True
    got = {t["name"]: tuple(t["shape"]) for t in d["tensors"]}
    assert got == S.shapes_of(cfg)
    assert {L["type"] for L in cfg["layers"]} == {"parallel", "gla"} and "l0.mix.left.rel" in got and "l1.mix.a2.b" in got
