"""The Tubazen family (the gated form of the layer stack: dynamic-tanh norms, gated residuals, a weighted sum over all layer results, learned positions;
mixers: softmax attention with projection biases, a query temperature and a bias by bucketed distance beside a delta-rule recurrence, and gated linear
attention; a gelu gated feed-forward) against tests/tubazen_oracle.py -- a float64 restatement that shares nothing with the product.  Every test makes its
own small configuration and random bf16-representable weights, writes them as a model folder and runs them through the C API (the engine's step function,
slot cache and state and kernels); the operator tests call include/ntk_layers.h directly.

Error measure: rms of the difference over rms of the reference.  float32 mode is held to 2e-4 (observed ~1e-6), bfloat16 mode to 4e-2."""
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import tubazen_oracle as O  # noqa: E402

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {"float32": 2e-4, "bfloat16": 4e-2}


def rel(got, ref):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    return float(np.sqrt(np.mean((got - ref) ** 2)) / (np.sqrt(np.mean(ref ** 2)) + 1e-30))


def row_err(got, ref):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    return np.sqrt(np.mean((got - ref) ** 2, axis=1)) / np.sqrt(np.mean(ref ** 2))


def make(tmp_path, cfg, seed=1, name="m", gain=1.0):
    w = O.random_weights(cfg, seed, gain)
    folder = str(tmp_path / name)
    O.save_model(folder, cfg, w)
    return folder, w


def engine_for(folder, dtype="float32", ctx=512, slots=1):
    from ntransformer_amd.engine import Engine
    e = Engine()
    e.load_folder(folder, max_context=ctx, dtype=dtype, slots=slots)
    return e


def tokens_for(cfg, n, seed=0):
    return [int(t) for t in np.random.default_rng(seed).integers(0, cfg["vocab"], n)]


def f32(a):
    return np.asarray(a, np.float32)


MIXED = dict(layers=("parallel", "gla", "gla", "parallel"), mlps=(True, True, None, True))


# ====================================================================================================================== operators
def test_dynamic_tanh_norm_and_the_embedding_with_positions():
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(1)
    x = f32(g.standard_normal((7, 130)) * 2)
    w, b = f32(1 + 0.2 * g.standard_normal(130)), f32(0.3 * g.standard_normal(130))
    assert rel(Lr.dyt(x, w, b, 0.7), O.dyt(x.astype(np.float64), w, b, 0.7)) < 1e-6
    big = f32(np.array([[1e4, -1e4, 0.0, 1e-8]]))                       # saturation and the origin
    assert np.abs(Lr.dyt(big, np.ones(4, np.float32), np.zeros(4, np.float32), 1.0) - np.array([[1, -1, 0, 1e-8]])).max() < 1e-6
    E, P = O.bf16_round(g.standard_normal((50, 130))), O.bf16_round(0.5 * g.standard_normal((40, 130)))
    toks = [3, 49, 0, 3, 17]
    for dtype in ("float32", "bfloat16"):
        ref = E[toks] + P[11:16]
        assert rel(Lr.embed_positions(E, P, toks, 11, dtype=dtype), ref) < 1e-7                                    # positions count from the slot's length
        assert rel(Lr.embed_positions(E, P, toks, 11, w, b, 1.3, dtype=dtype), O.dyt(ref.astype(np.float64), w, b, 1.3)) < 1e-6
    assert np.abs(Lr.embed_positions(E, P, toks[:1], 0) - (E[3] + P[0])).max() < 1e-7                              # the first position is 0


def test_the_seam_gated_residual_depth_average_and_next_norm():
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(2)
    T, n = 5, 70
    x, y, gz = (f32(g.standard_normal((T, n))) for _ in range(3))
    yb, gb = f32(0.3 * g.standard_normal(n)), f32(g.standard_normal(n))
    r = x.astype(np.float64) + (y + yb) * O.sigmoid(gz.astype(np.float64) + gb)
    got, _, h = Lr.gated_seam(x, y, gz, yb, gb, norm=(np.ones(n, np.float32), np.zeros(n, np.float32), 0.5))
    assert rel(got, r) < 1e-6 and rel(h, np.tanh(0.5 * r)) < 1e-6
    got, _, _ = Lr.gated_seam(x, y, gz)                                                                          # no biases, no norm
    assert rel(got, x + y * O.sigmoid(gz.astype(np.float64))) < 1e-6
    for n_hist in (1, 2, 5):       # the newest result lands in the last entry; what goes on is the weighted sum of all of them
        hist = f32(g.standard_normal((n_hist, T, n)))
        coef = f32(g.standard_normal(n_hist))
        nw, nb = f32(1 + 0.1 * g.standard_normal(n)), f32(0.1 * g.standard_normal(n))
        got, hh, h = Lr.gated_seam(x, y, gz, yb, gb, hist=hist.copy(), coef=coef, norm=(nw, nb, 0.9))
        want = sum(coef[j] * hist[j].astype(np.float64) for j in range(n_hist - 1)) + coef[-1] * r
        assert rel(hh[-1], r) < 1e-6 and np.array_equal(hh[:-1], hist[:-1])
        assert rel(got, want) < 1e-6 and rel(h, O.dyt(want, nw, nb, 0.9)) < 1e-6


def test_gelu_gated_unit_alone_and_inside_the_few_row_product():
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(3)
    ff, K = 37, 64
    alpha, cubic = 2 * math.sqrt(2 / math.pi), 0.044715
    gu = f32(g.standard_normal((6, 2 * ff + 9)) * 3)                         # rows longer than 2 ff: what lies behind is not read
    ref = O.gelu_tanh(gu[:, :ff].astype(np.float64)) * gu[:, ff:2 * ff]
    assert rel(Lr.glu_cubic(gu, ff, alpha, cubic), ref) < 1e-6
    x = f32(g.standard_normal((3, K)))
    wm = O.bf16_round(g.standard_normal((2 * ff, K)) / 4)
    z = x.astype(np.float64) @ wm.T
    for dtype in ("float32", "bfloat16"):
        got = Lr.dense(x, wm, dtype, glu_limit=float("inf"), glu_alpha=alpha, glu_up_offset=0.0, glu_cubic=cubic)
        assert rel(got, O.gelu_tanh(z[:, :ff]) * z[:, ff:]) < 1e-5


@pytest.mark.parametrize("H,dv", [(1, 1), (3, 14), (2, 64), (2, 200)])
def test_unit_norm_per_head_with_weight_gate_and_scale(H, dv):
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(H * dv)
    x, gz = f32(g.standard_normal((4, H * dv)) * 5), f32(g.standard_normal((4, H * dv)))
    u = O.unit_rms(x.astype(np.float64).reshape(4, H, dv), 1e-3)
    shared, own = f32(1 + 0.2 * g.standard_normal(dv)), f32(1 + 0.2 * g.standard_normal(H * dv))
    silu = gz * O.sigmoid(gz.astype(np.float64))
    assert rel(Lr.head_rmsnorm_gate(x, shared, H, dv, 1e-3, gz, act=2), (u * shared).reshape(4, -1) * silu) < 1e-6
    assert rel(Lr.head_rmsnorm_gate(x, own, H, dv, 1e-3, gz, act=1, scale=0.5, per_head=True), u.reshape(4, -1) * own * O.sigmoid(gz.astype(np.float64)) * 0.5) < 1e-6
    assert rel(Lr.head_rmsnorm_gate(x, shared, H, dv, 1e-3), (u * shared).reshape(4, -1)) < 1e-6
    tiny = f32(np.full((1, H * dv), 1e-6))                                   # eps inside the root decides here
    assert rel(Lr.head_rmsnorm_gate(tiny, np.ones(dv, np.float32), H, dv, 1e-3), tiny / math.sqrt(1e-12 + 1e-3)) < 1e-5


def test_biases_and_query_temperature_on_the_way_into_the_cache():
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(5)
    H, G, dn, dv, T, pos0, every = 4, 2, 6, 5, 40, 3, 8
    q, k, v = f32(g.standard_normal((T, H * dn))), f32(g.standard_normal((T, G * dn))), f32(g.standard_normal((T, G * dv)))
    qb, kb, vb = f32(g.standard_normal(H * dn)), f32(g.standard_normal(G * dn)), f32(g.standard_normal(G * dv))
    cache, qq = Lr.window_prepare_biased(q, k, v, H, G, dn, dv, pos0, qb, kb, vb, temp_coef=0.5, temp_every=every)
    temp = np.array([O.query_temperature(pos0 + t, 0.5, every) for t in range(T)])
    assert rel(qq, (q + qb) * temp[:, None]) < 1e-6
    assert rel(cache[pos0:, :G * dn], k + kb) < 1e-7 and rel(cache[pos0:, G * dn:], v + vb) < 1e-7
    # the temperature steps where (p + 1) / every passes an integer: p = every - 2 and every - 1 differ, every - 1 and every do not
    t_of = lambda p: Lr.window_prepare_biased(np.ones((1, dn), np.float32), np.zeros((1, dn), np.float32), np.zeros((1, dv), np.float32), 1, 1, dn, dv, p,
                                              temp_coef=0.5, temp_every=every)[1][0, 0]
    assert t_of(every - 2) == 1.0 and abs(t_of(every - 1) - (1 + 0.5 * math.log(2))) < 1e-6 and t_of(every) == t_of(every - 1) and t_of(0) == 1.0
    cache, qq = Lr.window_prepare_biased(q, k, v, H, G, dn, dv, pos0)                 # nothing optional: a copy
    assert np.array_equal(qq, q) and np.array_equal(cache[pos0:, :G * dn], k)


def _attention_reference(q, K, V, H, G, pos0, scale, rel_table, reach):
    T, dn, dv = q.shape[0], K.shape[2], V.shape[2]
    out = np.zeros((T, H, dv))
    qh = q.reshape(T, H, dn).astype(np.float64)
    for t in range(T):
        p = pos0 + t
        for h in range(H):
            s = K[:p + 1, h // (H // G)] @ qh[t, h] * scale
            if rel_table is not None:
                s = s + np.array([rel_table[O.distance_bucket(p - j, rel_table.shape[0], reach), h] for j in range(p + 1)])
            e = np.exp(s - s.max())
            out[t, h] = (e / e.sum()) @ V[:p + 1, h // (H // G)]
    return out.reshape(T, H * dv)


@pytest.mark.parametrize("H,G,dn,dv,buckets,reach", [(4, 2, 12, 20, 10, 37), (3, 3, 5, 3, 9, 300), (6, 1, 70, 130, 32, 240), (1, 1, 8, 8, 2, 5)])
@pytest.mark.parametrize("pos0,T", [(0, 50), (130, 1), (125, 6), (60, 23)])
def test_attention_with_a_bias_by_bucketed_distance(H, G, dn, dv, buckets, reach, pos0, T):
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(H + dn + pos0)
    n = pos0 + T
    K, V = f32(g.standard_normal((n, G, dn))), f32(g.standard_normal((n, G, dv)))
    q = f32(g.standard_normal((T, H * dn)))
    table = f32(g.standard_normal((buckets, H)) * 2)
    cache = np.concatenate([K.reshape(n, -1), V.reshape(n, -1)], axis=1)
    bucket_of = np.array([O.distance_bucket(d, buckets, reach) for d in range(n + 5)], np.int32)
    ref = _attention_reference(q, K.astype(np.float64), V.astype(np.float64), H, G, pos0, 0.3, table.astype(np.float64), reach)
    for split in (True, False):
        assert rel(Lr.window_attention(q, cache, H, G, 1, dn, dv, pos0, 0, 0.3, split=split, rel=table, bucket_of=bucket_of), ref) < 2e-6
    # a table of distances shorter than the sequence: everything beyond its end shares its last entry
    short = bucket_of[:max(reach + 1, buckets)] if n > reach + 1 else bucket_of
    assert rel(Lr.window_attention(q, cache, H, G, 1, dn, dv, pos0, 0, 0.3, rel=table, bucket_of=short), ref) < 2e-6


def test_bucket_borders_one_row_of_the_table_at_a_time():
    """all keys and values alike except their index in one value column; a table with ONE large entry pulls the weights onto the distances of that bucket:
    the weighted mean of the key indices must be the mean over exactly the bucket's distances, for a decoded token and inside a portion"""
    from ntransformer_amd import layers as Lr
    buckets, reach, n = 12, 80, 300
    bucket_of = np.array([O.distance_bucket(d, buckets, reach) for d in range(n)], np.int32)
    assert bucket_of[5] == 5 and bucket_of[6] == 6 and (bucket_of[51], bucket_of[52]) == (10, 11) and bucket_of[n - 1] == buckets - 1
    K = np.zeros((n, 1, 4), np.float32)
    V = np.zeros((n, 1, 2), np.float32)
    V[:, 0, 0] = np.arange(n)
    cache = np.concatenate([K.reshape(n, -1), V.reshape(n, -1)], axis=1)
    for b in range(buckets):
        table = np.zeros((buckets, 1), np.float32)
        table[b] = 60.0
        dist = np.nonzero(bucket_of == b)[0]
        for pos0, T in ((n - 1, 1), (n - 7, 7), (0, n)):
            out = Lr.window_attention(np.zeros((T, 4), np.float32), cache, 1, 1, 1, 4, 2, pos0, 0, 1.0, rel=table, bucket_of=bucket_of)
            for t in (0, T - 1):
                p = pos0 + t
                d = dist[dist <= p]
                if len(d):
                    assert abs(out[t, 0] - np.mean(p - d)) < 1e-3, (b, pos0, t)


def test_a_towering_far_key_is_found_at_every_place_of_the_walk():
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(8)
    H, G, dn, dv, n = 2, 1, 16, 8, 1300
    K, V = f32(g.standard_normal((n, G, dn))), f32(g.standard_normal((n, G, dv)))
    q = f32(g.standard_normal((1, H * dn)))
    table = f32(g.standard_normal((8, H)))
    bucket_of = np.array([O.distance_bucket(d, 8, 100) for d in range(n)], np.int32)
    for far in (0, 1, 63, 64, 65, 640, 1235, 1298, 1299):
        K2 = K.copy()
        K2[far, 0] = q[0, :dn] * 4                                          # head 0's score at `far` stands far above the rest
        cache = np.concatenate([K2.reshape(n, -1), V.reshape(n, -1)], axis=1)
        out = Lr.window_attention(q, cache, H, G, 1, dn, dv, n - 1, 0, 1.0, rel=table, bucket_of=bucket_of)
        assert np.abs(out[0, :dv] - V[far, 0]).max() < 1e-3, far
        assert rel(out, _attention_reference(q, K2.astype(np.float64), V.astype(np.float64), H, G, n - 1, 1.0, table.astype(np.float64), 100)) < 2e-6


def _recurrence_inputs(g, T, H, dn, dv, spread=1.0):
    return (f32(g.standard_normal((T, H * dn))), f32(g.standard_normal((T, H * dn))), f32(g.standard_normal((T, H * dv))), f32(g.standard_normal((T, H * dn)) * spread),
            f32(g.standard_normal((T, H * dn))), f32(g.standard_normal(H * dn)), f32(g.standard_normal(H * dn)))


SHAPES = [(2, 9, 11), (1, 1, 1), (3, 12, 12), (2, 48, 32), (1, 130, 70), (1, 300, 5), (2, 64, 64), (1, 600, 9)]


@pytest.mark.parametrize("H,dn,dv", SHAPES)
@pytest.mark.parametrize("delta", [False, True])
def test_decay_recurrence_whole_in_portions_and_token_by_token(H, dn, dv, delta):
    """gated linear attention (decay = sigmoid^(1/tau) per key channel) and the delta rule (decay = exp(-c sigmoid), removal along the unit key): whole,
    portions that cut anywhere (also inside a staged batch of tokens) and single tokens give the same sums; a sequence's start reads no state"""
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(H * dn + dv + delta)
    T = 45
    q, k, v, wz, az, wb, ab = _recurrence_inputs(g, T, H, dn, dv, 2.0)
    z = (wz + wb).astype(np.float64).reshape(T, H, dn)
    if delta:
        kw = dict(decay_form=Lr.DECAY_EXP_SIGMOID, decay_param=0.6, wb=wb, az=az, ab=ab, unit_eps=1e-6)
        decay, removal = np.exp(-0.6 * O.sigmoid(z)), O.sigmoid((az + ab).astype(np.float64)).reshape(T, H, dn)
    else:
        kw = dict(decay_form=Lr.DECAY_SIGMOID_ROOT, decay_param=3.0, wb=wb, q_scale=0.25)
        decay, removal = O.sigmoid(z) ** (1 / 3.0), None
    qs = q.astype(np.float64).reshape(T, H, dn) * (1.0 if delta else 0.25)
    ref, S = O.decay_recurrence(qs, k.astype(np.float64).reshape(T, H, dn), v.astype(np.float64).reshape(T, H, dv), decay, removal, 1e-6)
    ref = ref.reshape(T, H * dv)
    out, st = Lr.gated_recurrence(q, k, v, wz, H, dn, dv, 0, **kw)          # (the state buffer starts full of NaN: position 0 must not read it)
    assert rel(out, ref) < 2e-6 and rel(st, S) < 2e-6
    out2, st2 = Lr.gated_recurrence(q, k, v, wz, H, dn, dv, 0, prepass=False, **kw)   # the per-token vectors formed inside the walk instead of ahead of it
    assert np.abs(out2 - out).max() <= 1e-6 * np.abs(ref).max() and rel(st2, S) < 2e-6
    for cuts in ([1] * T, [2, 9, 3, 8, 17, 1, 5], [16, 16, 13], [44, 1]):
        parts, at, st = [], 0, None
        for n in cuts:
            o, st = Lr.gated_recurrence(q[at:at + n], k[at:at + n], v[at:at + n], wz[at:at + n], H, dn, dv, at, state=st, **dict(kw, az=az[at:at + n] if delta else None))
            parts.append(o)
            at += n
        assert at == T
        assert rel(np.concatenate(parts), ref) < 2e-6 and rel(st, S) < 2e-6
        assert np.abs(np.concatenate(parts) - out).max() <= 1e-6 * np.abs(ref).max()      # the same sums in the same order, whatever the cut


@pytest.mark.parametrize("H,dn,dv", [(2, 9, 11), (3, 64, 64), (1, 128, 70), (2, 96, 128), (1, 130, 20)])
@pytest.mark.parametrize("delta", [False, True])
def test_long_portions_walk_in_segments_side_by_side(H, dn, dv, delta):
    """portions long enough to be cut into segments that start from nothing and are settled afterwards (the state handed from segment to segment, every
    output given what the state at its segment's start still owed it) against the walk in turn and the oracle; from a sequence's start and from a state;
    lengths that leave a short last segment; heads too wide for segments stay in turn"""
    from ntransformer_amd import layers as Lr
    g = np.random.default_rng(H * dn + dv + delta)
    T0, T = 37, 333
    q, k, v, wz, az, wb, ab = _recurrence_inputs(g, T0 + T, H, dn, dv, 2.0)
    z = (wz + wb).astype(np.float64).reshape(-1, H, dn)
    if delta:
        kw = dict(decay_form=Lr.DECAY_EXP_SIGMOID, decay_param=0.6, wb=wb, ab=ab, unit_eps=1e-6)
        decay, removal = np.exp(-0.6 * O.sigmoid(z)), O.sigmoid((az + ab).astype(np.float64)).reshape(-1, H, dn)
    else:
        kw = dict(decay_form=Lr.DECAY_SIGMOID_ROOT, decay_param=8.0, wb=wb)
        decay, removal = O.sigmoid(z) ** (1 / 8.0), None
    ref, S = O.decay_recurrence(q.astype(np.float64).reshape(-1, H, dn), k.astype(np.float64).reshape(-1, H, dn), v.astype(np.float64).reshape(-1, H, dv), decay, removal, 1e-6)
    ref = ref.reshape(-1, H * dv)
    run = lambda a, b, st, **more: Lr.gated_recurrence(q[a:b], k[a:b], v[a:b], wz[a:b], H, dn, dv, a, state=st, az=az[a:b] if delta else None, **dict(kw, **more))
    whole, st = run(0, T0 + T, None)
    assert rel(whole, ref) < 3e-6 and rel(st, S) < 3e-6
    turn, st2 = run(0, T0 + T, None, prepass=False)
    assert rel(whole, turn) < 3e-6 and rel(st, st2) < 3e-6
    head, st = run(0, T0, None)
    tail, st = run(T0, T0 + T, st)                                          # the first segment starts from the sequence's state
    assert rel(np.concatenate([head, tail]), ref) < 3e-6 and rel(st, S) < 3e-6
    for n in (128, 129, 191):                                               # two segments of 64, of 65, of 96 and 95
        part, _ = run(0, n, None)
        assert rel(part, ref[:n]) < 3e-6, n


def test_decay_forms_at_their_ends_and_a_given_decay():
    from ntransformer_amd import layers as Lr
    T, H, dn, dv = 6, 1, 4, 3
    g = np.random.default_rng(11)
    q, k, v = f32(g.standard_normal((T, dn))), f32(g.standard_normal((T, dn))), f32(g.standard_normal((T, dv)))
    run = lambda wz, **kw: Lr.gated_recurrence(q, k, v, f32(wz), H, dn, dv, 0, **kw)[0]
    ref = lambda decay: O.decay_recurrence(q.astype(np.float64).reshape(T, 1, dn), k.astype(np.float64).reshape(T, 1, dn), v.astype(np.float64).reshape(T, 1, dv),
                                           decay.reshape(T, 1, dn))[0].reshape(T, dv)
    given = g.random((T, dn))
    assert rel(run(given), ref(given)) < 2e-6                                # decay handed over as it is (0: forget everything, 1: keep everything)
    assert rel(run(np.ones((T, dn))), ref(np.ones((T, dn)))) < 2e-6 and rel(run(np.zeros((T, dn))), ref(np.zeros((T, dn)))) < 2e-6
    z = np.array([[-90.0, -20.0, 0.0, 30.0]] * T)                            # sigmoid^(1/tau) far out on both sides: exp(z / tau) on the left, 1 on the right
    want = np.exp(-np.logaddexp(0.0, -z) / 16.0)
    assert rel(run(z, decay_form=Lr.DECAY_SIGMOID_ROOT, decay_param=16.0), ref(want)) < 2e-6
    assert rel(run(z, decay_form=Lr.DECAY_EXP_SIGMOID, decay_param=0.6), ref(np.exp(-0.6 * O.sigmoid(z)))) < 2e-6


def test_a_key_is_remembered_over_hundreds_of_tokens_and_removed_by_its_own_direction():
    """one channel never decays and carries a key from the first token; every later query finds its value.  With the removal term a later token whose unit
    key points the same way, at rate one, takes exactly that value out again"""
    from ntransformer_amd import layers as Lr
    T, dn, dv = 700, 8, 4
    g = np.random.default_rng(12)
    k = f32(g.standard_normal((T, dn)) * 0.01)
    k[:, 0] = 0.0
    k[0] = 0.0
    k[0, 0] = 3.0                                                            # only the first token writes channel 0
    v = f32(g.standard_normal((T, dv)))
    q = np.zeros((T, dn), np.float32)
    q[:, 0] = 1.0
    wz = f32(np.full((T, dn), -2.0))
    wz[:, 0] = 40.0                                                          # sigmoid(40)^(1/tau) = 1 in F32
    out, _ = Lr.gated_recurrence(q, k, v, wz, 1, dn, dv, 0, decay_form=Lr.DECAY_SIGMOID_ROOT, decay_param=2.0)
    assert np.abs(out - 3.0 * v[0]).max() < 1e-5
    parts, st = [], None
    for at in range(0, T, 97):                                               # ... also across portions
        o, st = Lr.gated_recurrence(q[at:at + 97], k[at:at + 97], v[at:at + 97], wz[at:at + 97], 1, dn, dv, at, decay_form=Lr.DECAY_SIGMOID_ROOT, decay_param=2.0, state=st)
        parts.append(o)
    assert np.abs(np.concatenate(parts) - 3.0 * v[0]).max() < 1e-5
    # removal: decay 1 everywhere (given), token 500 has key e_0 * tiny (its own write is negligible) and removal rate sigmoid(+40) = 1 on channel 0
    k2, az = k.copy(), f32(np.full((T, dn), -40.0))
    k2[1:] = 0.0
    k2[500, 0] = 1e-3
    v2 = v.copy()
    v2[500] = 0.0
    az[500, 0] = 40.0
    out, _ = Lr.gated_recurrence(q, k2, v2, np.ones((T, dn), np.float32), 1, dn, dv, 0, az=az, unit_eps=1e-12)
    assert np.abs(out[:500] - 3.0 * v[0]).max() < 1e-5 and np.abs(out[500:]).max() < 1e-4


# ====================================================================================================================== whole models
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_with_the_stream_after_every_layer(tmp_path, dtype):
    cfg = O.small_config(**MIXED)
    folder, w = make(tmp_path, cfg, seed=2)
    toks = tokens_for(cfg, 40, seed=3)
    ref, streams = O.forward(cfg, w, toks, return_layers=True)
    e = engine_for(folder, dtype)
    assert e.layer_runs == 4
    e.seq_capture(True)
    s = e.seq_acquire()
    got = e.seq_forward(s, toks)
    cap = e.seq_captured(len(toks))
    for i in range(4):
        assert rel(cap[i], streams[i]) < TOL[dtype], i
    assert rel(got, ref) < TOL[dtype]
    e.seq_capture(False)
    e.seq_release(s)
    s = e.seq_acquire()
    some = e.seq_forward(s, toks, want=[0, 7, 39])                           # wanted places only
    assert rel(some, ref[[0, 7, 39]]) < TOL[dtype]
    e.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_against_token_by_token_and_portions(tmp_path, dtype):
    """the same sequence whole, one token at a time and in portions down to two tokens: same logits at every position.  150 tokens, a bias table that reaches
    to distance 90 and a query temperature that steps every 32 positions: portions start and end on both sides of every such edge, of the attention's 64-key
    chunks, of the recurrence's token batches and of the switch between the few-row and the tiled products"""
    cfg = O.small_config(bias_max=90, buckets=16, temp=(0.7, 32), **MIXED)
    folder, w = make(tmp_path, cfg, seed=3)
    e = engine_for(folder, dtype)
    toks = tokens_for(cfg, 150, seed=4)
    ref = O.forward(cfg, w, toks)
    s = e.seq_acquire()
    whole = e.seq_forward(s, toks)
    e.seq_release(s)
    assert rel(whole, ref) < TOL[dtype] and row_err(whole, ref).max() < 3 * TOL[dtype]
    s = e.seq_acquire()
    one = np.concatenate([e.seq_forward(s, toks[i:i + 1]) for i in range(len(toks))])
    e.seq_release(s)
    assert rel(one, ref) < TOL[dtype] and row_err(one, ref).max() < 3 * TOL[dtype]
    s = e.seq_acquire()
    parts, at = [], 0
    for n in [2, 9, 3, 8, 17, 2, 30, 1, 5, 64, 2, 7]:
        parts.append(e.seq_forward(s, toks[at:at + n]))
        at += n
    assert at == len(toks) and e.seq_length(s) == at
    cut = np.concatenate(parts)
    assert rel(cut, ref) < TOL[dtype] and row_err(cut, ref).max() < 3 * TOL[dtype]
    if dtype == "float32":
        assert rel(one, whole) < 1e-5 and rel(cut, whole) < 1e-5
    e.close()


def test_first_tokens_of_a_sequence(tmp_path):
    cfg = O.small_config(**MIXED)
    folder, w = make(tmp_path, cfg, seed=5)
    e = engine_for(folder)
    for n in (1, 2, 3):
        toks = tokens_for(cfg, n, seed=n)
        s = e.seq_acquire()
        assert rel(e.seq_forward(s, toks), O.forward(cfg, w, toks)) < TOL["float32"]
        e.seq_release(s)
    e.close()


def test_two_slots_side_by_side_and_a_slot_used_again(tmp_path):
    """two sequences advance in turn, each alone would give the same; a freed slot (cache rows and both kinds of state of a longer sequence still there) is
    taken by a shorter one; a sequence with recurrent state can be cut back to its start only"""
    cfg = O.small_config(**MIXED)
    folder, w = make(tmp_path, cfg, seed=6)
    e = engine_for(folder, slots=2)
    ta, tb = tokens_for(cfg, 60, 1), tokens_for(cfg, 33, 2)
    ra, rb = O.forward(cfg, w, ta), O.forward(cfg, w, tb)
    a, b = e.seq_acquire(), e.seq_acquire()
    assert a != b
    with pytest.raises(Exception):
        e.seq_acquire()
    got_a, got_b = [], []
    cuts_a, cuts_b = [20, 1, 1, 30, 8], [2, 1, 25, 5]
    ia = ib = 0
    for k in range(5):
        got_a.append(e.seq_forward(a, ta[ia:ia + cuts_a[k]])); ia += cuts_a[k]
        if k < 4:
            got_b.append(e.seq_forward(b, tb[ib:ib + cuts_b[k]])); ib += cuts_b[k]
    assert rel(np.concatenate(got_a), ra) < TOL["float32"] and rel(np.concatenate(got_b), rb) < TOL["float32"]
    e.seq_release(a)
    c = e.seq_acquire()
    assert c == a
    tc = tokens_for(cfg, 9, 3)
    assert rel(e.seq_forward(c, tc), O.forward(cfg, w, tc)) < TOL["float32"]
    with pytest.raises(Exception):
        e.seq_truncate(c, 4)
    e.seq_truncate(c, 0)
    assert rel(e.seq_forward(c, tb[:5]), rb[:5]) < TOL["float32"]
    e.close()


OTHER = {
    "one of everything": dict(layers=("parallel",), mlps=(None,), heads=1, kv_heads=1, dim=1, vdim=1, rheads=1, rdim=1, buckets=2, bias_max=3, width=8, vocab=5, temp=None),
    "all sizes equal, scales one": dict(layers=("gla", "parallel"), mlps=(True, True), heads=4, kv_heads=4, dim=16, vdim=16, rheads=4, rdim=16, gheads=4, gdim=16, gvdim=16,
                                        width=16, vocab=16, ff=16, buckets=16, bias_max=16.5, left_scale=1.0, right_scale=1.0, logit_scale=1.0, tau=1.0, temp=(1.0, 1)),
    "multiples of nothing": dict(layers=("gla", "gla", "parallel"), mlps=(None, True, True), heads=3, kv_heads=1, dim=7, vdim=5, rheads=5, rdim=3, gheads=3, gdim=13, gvdim=7,
                                 width=23, vocab=31, ff=29, buckets=7, bias_max=55, tau=0.5, temp=(0.3, 7)),
    "wide heads": dict(layers=("parallel", "gla"), mlps=(True, None), heads=2, kv_heads=1, dim=96, vdim=136, rheads=1, rdim=140, gheads=1, gdim=264, gvdim=72, width=64,
                       vocab=50, ff=40, buckets=32, bias_max=200, tau=16.0),
    "nothing but recurrences without feed-forward": dict(layers=("gla", "gla"), mlps=(None, None)),
}


@pytest.mark.parametrize("name", sorted(OTHER))
def test_other_sizes(tmp_path, name):
    cfg = O.small_config(**OTHER[name])
    folder, w = make(tmp_path, cfg, seed=7)
    toks = tokens_for(cfg, 70, seed=8)
    ref, streams = O.forward(cfg, w, toks, return_layers=True)
    for dtype in ("float32", "bfloat16"):
        e = engine_for(folder, dtype)
        e.seq_capture(True)
        s = e.seq_acquire()
        got = e.seq_forward(s, toks[:61])
        assert rel(e.seq_captured(61)[-1], streams[-1][:61]) < TOL[dtype]
        e.seq_capture(False)
        tail = np.concatenate([e.seq_forward(s, toks[61:63])] + [e.seq_forward(s, [t]) for t in toks[63:]])
        assert rel(np.concatenate([got, tail]), ref) < TOL[dtype], dtype
        e.close()


def test_long_decoding_and_a_prompt_longer_than_one_internal_pass(tmp_path):
    cfg = O.small_config(positions=1300, bias_max=500, buckets=24, temp=(0.5, 128), layers=("parallel", "gla"), mlps=(True, True))
    folder, w = make(tmp_path, cfg, seed=9)
    toks = tokens_for(cfg, 1100, seed=10)
    e = engine_for(folder, ctx=1300)
    s = e.seq_acquire()
    got = e.seq_forward(s, toks, want=[0, 1023, 1024, 1099])                # 1100 tokens: two internal passes
    ref = O.forward(cfg, w, toks)
    assert rel(got, ref[[0, 1023, 1024, 1099]]) < TOL["float32"]
    e.seq_release(s)
    s = e.seq_acquire()
    e.seq_forward(s, toks[:900], want=[])
    dec = np.concatenate([e.seq_forward(s, [t]) for t in toks[900:]])       # 200 tokens one by one, the temperature stepping at 1023 -> 1024 on the way
    assert rel(dec, ref[900:]) < TOL["float32"] and row_err(dec, ref[900:]).max() < 3 * TOL["float32"]
    with pytest.raises(Exception):                                          # the position table ends at 1300
        e.seq_forward(s, toks[:300])
    e.close()


def test_more_positions_asked_for_than_the_table_has(tmp_path):
    cfg = O.small_config(positions=50, layers=("parallel",), mlps=(True,))
    folder, w = make(tmp_path, cfg, seed=11)
    e = engine_for(folder, ctx=512)
    s = e.seq_acquire()
    toks = tokens_for(cfg, 50, seed=1)
    assert rel(e.seq_forward(s, toks), O.forward(cfg, w, toks)) < TOL["float32"]
    with pytest.raises(Exception):
        e.seq_forward(s, [1])
    e.close()


def test_greedy_generation_through_the_engine_and_the_command_line(tmp_path):
    cfg = O.small_config(**MIXED)
    folder, w = make(tmp_path, cfg, seed=15, gain=2.0)
    prompt = tokens_for(cfg, 12, seed=16)
    want = O.greedy(cfg, w, prompt, 10)
    e = engine_for(folder)
    assert e.is_sequence_model and e.vocab_size == cfg["vocab"] and e.hidden_size == cfg["width"] and e.n_layers == 4
    assert e.generate_tokens(prompt, 10, temperature=0.0, stop_at_eos=False) == want
    assert e.generate_tokens(prompt, 10, temperature=0.0, stop_at_eos=False) == want      # the slot came back, its old state is not read
    a = e.generate_tokens(prompt, 8, temperature=0.9, top_k=20, top_p=0.95, seed=5, stop_at_eos=False)
    assert a == e.generate_tokens(prompt, 8, temperature=0.9, top_k=20, top_p=0.95, seed=5, stop_at_eos=False) and len(a) == 8
    assert rel(e.forward(prompt[:8], 0), O.forward(cfg, w, prompt[:8])[-1]) < TOL["float32"]
    assert rel(e.forward(prompt[8:], 8), O.forward(cfg, w, prompt)[-1]) < TOL["float32"]
    e.close()
    cli = os.path.join(ROOT, "ntransformer_amd", "ntransformer")
    r = subprocess.run([cli, "-m", folder, "--dtype", "float32", "--tokens", ",".join(map(str, prompt)), "-n", "10", "-t", "0", "--repeat-penalty", "1"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [int(t) for t in r.stdout.strip().splitlines()[-1].split(",")] == want


def test_trace_runner_replays_steps(tmp_path):
    cfg = O.small_config(**MIXED)
    folder, w = make(tmp_path, cfg, seed=17)
    ta, tb = tokens_for(cfg, 20, 1), tokens_for(cfg, 6, 2)
    ra, rb = O.forward(cfg, w, ta), O.forward(cfg, w, tb)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": ta[:13], "want": [0, 12]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": ta[13:15], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": ta[15:], "want": [4]}], "end": ["a"]},
        {"step": 3, "entries": [{"id": "b", "tokens": tb, "want": [5]}], "end": ["b"]},
    ]
    V = cfg["vocab"]
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / ("out_" + dtype)
        out.mkdir()
        r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out), "--max-tokens", "20"],
                           input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
        assert r.returncode == 0, r.stderr[-2000:]
        assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done %d" % k for k in range(4)]
        assert not (out / "1.f32").exists()
        assert rel(np.fromfile(out / "0.f32", np.float32).reshape(-1, V), ra[[0, 12]]) < TOL[dtype]
        assert rel(np.fromfile(out / "2.f32", np.float32).reshape(-1, V), ra[[19]]) < TOL[dtype]
        assert rel(np.fromfile(out / "3.f32", np.float32).reshape(-1, V), rb[[5]]) < TOL[dtype]


@pytest.mark.parametrize("bad", ["mixer type", "tensor", "kv_heads", "kind", "tau"])
def test_refused_folders(tmp_path, bad):
    from ntransformer_amd.engine import Engine
    cfg = O.small_config(**MIXED)
    w = O.random_weights(cfg, 1)
    if bad == "mixer type": cfg["layers"][1]["type"] = "lightning"
    elif bad == "tensor": del w["l0.mix.left.rel"]
    elif bad == "kv_heads": cfg["layers"][0]["mixer"]["left"]["kv_heads"] = 4
    elif bad == "kind": cfg["layers"][0]["mlp"]["kind"] = "moe"
    else: cfg["layers"][1]["mixer"]["tau"] = 0.0
    folder = str(tmp_path / "bad")
    O.save_model(folder, cfg, w)
    e = Engine()
    with pytest.raises(Exception):
        e.load_folder(folder, max_context=64, dtype="float32")
    e.close()
