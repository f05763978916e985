"""Host side of the Fifotar family (no GPU): the folder reader and the registry know the family, and the float64 restatement's own invariants -- the things
the GPU tests lean on: causality, what every mechanism carries across a cut (cached keys and values, latents, the state and the convolutions' inputs), the
chunk mask, the sink, the delta rule's replacement of a key's value, the blended frequencies, the synthetic folders of the benchmark."""
import ctypes as C
import json
import math
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import fifotar_oracle as O  # noqa: E402
from ntransformer_amd import _lib  # noqa: E402


def describe(path):
    L = _lib.lib()
    L.nt_model_folder_describe.argtypes = [C.c_char_p, C.c_char_p, C.c_int]
    n = L.nt_model_folder_describe(path.encode(), None, 0)
    assert n >= 0
    buf = C.create_string_buffer(n + 1)
    assert L.nt_model_folder_describe(path.encode(), buf, n + 1) == n
    return json.loads(buf.value.decode())


def small():
    return O.config([O.attention_layer(size=6), O.delta_layer(), O.latent_layer(), O.attention_layer(size=5), O.delta_layer(ff=12)])


def test_a_written_folder_is_described_and_its_family_is_built_in(tmp_path):
    cfg = small()
    w = O.random_weights(cfg, 3)
    O.save_model(str(tmp_path / "m"), cfg, w)
    d = describe(str(tmp_path / "m"))
    assert d["architecture"] == "Fifotar" and d["family_built_in"] is True and {"Fifotar", "Tubazen", "Nizorax", "Fabolorn"} <= set(d["families"])
    got = {t["name"]: tuple(t["shape"]) for t in d["tensors"]}
    assert got == {k: tuple(np.shape(v)) for k, v in w.items()}
    assert "l1.norm2" not in got and "head" not in got and got["l0.mix.vmix"] == () and got["l1.mix.q.conv"] == (16, 4) and got["l2.mix.g"] == (3, 32)
    c2, w2 = O.load_model(str(tmp_path / "m"))
    assert c2 == cfg and all(np.array_equal(w[k], w2[k]) for k in w)


def test_causality_and_cuts_of_the_whole_model():
    cfg = small()
    w = O.random_weights(cfg, 2)
    toks = [int(t) for t in np.random.default_rng(0).integers(0, cfg["vocab"], 17)]
    streams = []
    lg, _ = O.forward(cfg, w, toks, layers_out=streams)
    assert len(streams) == 5 and streams[0].shape == (17, cfg["width"]) and lg.shape == (17, cfg["vocab"])
    assert np.allclose(lg[:9], O.forward(cfg, w, toks[:9])[0], atol=1e-10)
    seq, parts = None, []
    for a, b in ((0, 5), (5, 6), (6, 8), (8, 17)):
        o, seq = O.forward(cfg, w, toks[a:b], seq)
        parts.append(o)
    assert np.allclose(np.concatenate(parts), lg, atol=1e-9) and seq.n == 17
    assert np.abs(lg).max() < cfg["logit_softcap"]


def test_chunk_mask_and_sink():
    assert [j for j in range(8) if O.sees_chunk(7, j, 4)] == [4, 5, 6, 7] and [j for j in range(9) if O.sees_chunk(8, j, 4)] == [8]
    assert [j for j in range(4) if O.sees_chunk(2, j, None)] == [0, 1, 2]
    s = np.array([0.0, math.log(2.0)])
    assert np.allclose(O.sink_softmax(s), [0.25, 0.5])
    assert O.sink_softmax(np.array([-800.0])).sum() < 1e-300 and abs(O.sink_softmax(np.array([800.0])).sum() - 1.0) < 1e-12
    assert abs(O.capped(np.array([1000.0]), 7.0)[0] - 7.0) < 1e-9 and O.capped(np.array([0.3]), None)[0] == 0.3


def test_the_delta_rule_replaces_and_decays():
    e0 = np.array([1.0, 0.0])
    q = np.tile(e0, (3, 1)).reshape(3, 1, 2)
    k = q.copy()
    v = np.array([[[1.0]], [[5.0]], [[0.0]]])
    beta = np.array([[1.0], [1.0], [0.0]])
    o, S = O.delta_walk(q, k, v, beta, np.array([[1.0], [1.0], [0.5]]))
    assert np.allclose(o[:, 0, 0], [1.0, 5.0, 2.5]) and np.allclose(S[0, :, 0], [2.5, 0.0])     # replaced, not summed; then halved without a write
    o, _ = O.delta_walk(q, k, v, np.full((3, 1), 0.5), np.ones((3, 1)))
    assert np.allclose(o[:2, 0, 0], [0.5, 0.5 + 0.5 * (5.0 - 0.5)])                              # half of the way from what is there to the new value


def test_short_convolution_carries_its_last_inputs():
    g = np.random.default_rng(1)
    z, cw = g.standard_normal((9, 3)), g.standard_normal((3, 4))
    whole, last = O.short_conv(z, cw)
    a, c = O.short_conv(z[:2], cw)
    b, c = O.short_conv(z[2:], cw, c)
    assert np.allclose(np.concatenate([a, b]), whole) and np.allclose(c, last) and np.allclose(last, z[-3:])
    assert np.allclose(whole[0], O.silu(cw[:, 3] * z[0]))


def test_blended_frequencies_and_the_half_split_pairs():
    f, mag = O.blended_frequencies({"base": 100.0, "dims": 8})
    assert np.allclose(f, [1.0, 100 ** -0.25, 0.1, 100 ** -0.75]) and mag == 1.0
    f2, mag2 = O.blended_frequencies({"base": 100.0, "dims": 8, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}})
    assert abs(mag2 - (0.1 * math.log(4.0) + 1.0)) < 1e-15 and f2[0] == f[0] and abs(f2[3] - f[3] / 4.0) < 1e-15 and f[1] / 4 < f2[1] < f[1]
    x = np.arange(1.0, 11.0)
    y = O.rotate_halves(x, 3, f, 1.0, 8)
    a = 3 * f[1]
    assert np.allclose([y[1], y[5]], [x[1] * math.cos(a) - x[5] * math.sin(a), x[5] * math.cos(a) + x[1] * math.sin(a)]) and np.array_equal(y[8:], x[8:])


def test_synthetic_folders_of_the_benchmark_have_the_family_s_tensors(tmp_path):
    from ntransformer_amd import synth_folder as S
    cfg = S.fifotar_config("tiny", layers=4)
    S.write_folder(str(tmp_path / "s"), cfg)
    d = describe(str(tmp_path / "s"))
    assert d["architecture"] == "Fifotar" and d["family_built_in"] is True
    got = {t["name"]: tuple(t["shape"]) for t in d["tensors"]}
    assert got == S.shapes_of(cfg)
    assert [L["type"] for L in cfg["layers"]] == ["attention", "delta", "latent_attention", "delta"] and "l0.mix.vmix" in got and "l1.mix.A_log" in got and "head" not in got
