"""Python view of include/ntk_layers.h: the operators of the layer-list model families, numpy in / numpy out (every call uploads its
operands, launches on the library's compute stream and downloads the result -- for tests and micro-benchmarks, not a serving path).
Weights are passed as float arrays and stored as bfloat16 (dtype="bfloat16", rounded to nearest even) or float32 on the device."""
from __future__ import annotations

import ctypes as C
from typing import Optional

import numpy as np

from . import _lib
from ._lib import check
from .ops import DeviceBuffer

DT_F32, DT_BF16 = 0, 9


class DenseDesc(C.Structure):
    _fields_ = [("Y", C.c_void_p), ("ldy", C.c_int), ("X", C.c_void_p), ("ldx", C.c_int), ("W", C.c_void_p), ("wstride", C.c_longlong), ("wdtype", C.c_int),
                ("offsets", C.c_void_p), ("G", C.c_int), ("rows", C.c_void_p), ("row_div", C.c_int), ("T", C.c_int), ("N", C.c_int), ("K", C.c_int),
                ("accumulate", C.c_int), ("glu_ff", C.c_int), ("glu_limit", C.c_float), ("glu_alpha", C.c_float),
                ("norm_w", C.c_void_p), ("norm_eps", C.c_float), ("norm_offset", C.c_float), ("glu_up_offset", C.c_float), ("glu_cubic", C.c_float)]


class Rotary(C.Structure):
    _fields_ = [("freq", C.c_void_p), ("mag", C.c_float), ("dims", C.c_int), ("layout", C.c_int)]


ROT_NEIGHBOURS, ROT_HALVES = 0, 1
MASK_SLIDING, MASK_CHUNKS = 0, 1


class WindowPrepareDesc(C.Structure):
    _fields_ = [("cache", C.c_void_p), ("row", C.c_int), ("q", C.c_void_p), ("ldq", C.c_int), ("k", C.c_void_p), ("ldk", C.c_int), ("v", C.c_void_p), ("ldv", C.c_int),
                ("H", C.c_int), ("G", C.c_int), ("maps", C.c_int), ("dn", C.c_int), ("dv", C.c_int), ("rot", C.POINTER(Rotary)),
                ("qb", C.c_void_p), ("kb", C.c_void_p), ("vb", C.c_void_p), ("temp_coef", C.c_float), ("temp_every", C.c_double),
                ("v_other", C.c_void_p), ("ld_other", C.c_int), ("v_blend", C.c_float), ("v_keep", C.c_void_p), ("ld_keep", C.c_int), ("pos0", C.c_int), ("T", C.c_int)]


class WindowAttentionDesc(C.Structure):
    _fields_ = [("out", C.c_void_p), ("ldo", C.c_int), ("q", C.c_void_p), ("ldq", C.c_int), ("cache", C.c_void_p), ("row", C.c_int),
                ("H", C.c_int), ("G", C.c_int), ("maps", C.c_int), ("dn", C.c_int), ("dv", C.c_int), ("pos0", C.c_int), ("T", C.c_int), ("window", C.c_int),
                ("scale", C.c_float), ("lam", C.c_float), ("sub_norm", C.c_int), ("eps", C.c_float), ("out_scale", C.c_float), ("scratch", C.c_void_p),
                ("rel", C.c_void_p), ("bucket_of", C.c_void_p), ("n_dist", C.c_int), ("mask_mode", C.c_int), ("softcap", C.c_float), ("sink", C.c_int),
                ("gate", C.c_void_p), ("ldg", C.c_int)]


class GatedSeamDesc(C.Structure):
    _fields_ = [("x", C.c_void_p), ("ldx", C.c_int), ("y", C.c_void_p), ("ldy", C.c_int), ("yb", C.c_void_p), ("g", C.c_void_p), ("ldg", C.c_int), ("gb", C.c_void_p),
                ("hist", C.c_void_p), ("hist_stride", C.c_longlong), ("n_hist", C.c_int), ("coef", C.c_void_p),
                ("h", C.c_void_p), ("ldh", C.c_int), ("nw", C.c_void_p), ("nb", C.c_void_p), ("alpha", C.c_float), ("T", C.c_int), ("n", C.c_int)]


class GatedRecurrenceDesc(C.Structure):
    _fields_ = [("out", C.c_void_p), ("ldo", C.c_int), ("q", C.c_void_p), ("ldq", C.c_int), ("k", C.c_void_p), ("ldk", C.c_int), ("v", C.c_void_p), ("ldv", C.c_int),
                ("wz", C.c_void_p), ("ldw", C.c_int), ("wb", C.c_void_p), ("decay_form", C.c_int), ("decay_param", C.c_float),
                ("az", C.c_void_p), ("lda", C.c_int), ("ab", C.c_void_p), ("unit_eps", C.c_float), ("state", C.c_void_p),
                ("H", C.c_int), ("dn", C.c_int), ("dv", C.c_int), ("q_scale", C.c_float), ("pos0", C.c_int), ("T", C.c_int), ("scratch", C.c_void_p),
                ("G", C.c_int), ("unit_q", C.c_int), ("unit_k", C.c_int), ("head_gates", C.c_int), ("write_gated", C.c_int), ("decay_rates", C.c_void_p),
                ("conv_w", C.c_void_p), ("conv_state", C.c_void_p), ("conv_taps", C.c_int)]


DECAY_GIVEN, DECAY_SIGMOID_ROOT, DECAY_EXP_SIGMOID, DECAY_EXP_SOFTPLUS = 0, 1, 2, 3


class RouteDesc(C.Structure):
    _fields_ = [("score", C.c_int), ("groups", C.c_int), ("keep", C.c_int), ("group_top", C.c_int), ("renorm", C.c_int), ("scale", C.c_float)]


def _bind():
    L = _lib.lib()
    if getattr(L, "_layers_bound", False):
        return L
    vp, i, f, ll = C.c_void_p, C.c_int, C.c_float, C.c_longlong
    L.ntk_dense.argtypes = [C.POINTER(DenseDesc), vp]
    L.ntk_dense_linear.argtypes = [vp, i, vp, i, vp, i, i, i, i, i, vp]
    L.ntk_embed_dense.argtypes = [vp, vp, i, vp, i, i, i, vp]
    L.ntk_rmsnorm_offset.argtypes = [vp, vp, vp, vp, i, vp, i, i, i, f, f, vp]
    L.ntk_concat_rows.argtypes = [vp, vp, vp, i, i, vp]
    L.ntk_sigmoid_gate.argtypes = [vp, i, vp, i, i, i, vp]
    L.ntk_rows_copy.argtypes = [vp, vp, ll, vp]
    L.ntk_residual_add.argtypes = [vp, vp, vp, i, vp]
    L.ntk_latent_prepare.argtypes = [vp, i, vp, i, vp, f, i, i, vp, i, i, i, C.POINTER(Rotary), i, i, vp]
    L.ntk_latent_attention_scratch.argtypes = [i, i, i, i]
    L.ntk_latent_attention_scratch.restype = C.c_size_t
    L.ntk_latent_attention.argtypes = [vp, i, vp, i, vp, i, vp, i, vp, i, i, i, i, i, i, i, i, i, i, i, f, vp, vp]
    L.ntk_latent_fold_query.argtypes = [vp, vp, i, vp, i, i, i, i, i, i, vp]
    L.ntk_latent_unfold_value.argtypes = [vp, i, vp, vp, i, vp, i, i, i, i, i, vp]
    L.ntk_moe_route.argtypes = [vp, vp, vp, vp, i, vp, vp, i, i, i, i, vp]
    L.ntk_moe_group.argtypes = [vp, vp, vp, vp, i, i, i, vp]
    L.ntk_clipped_glu.argtypes = [vp, vp, i, i, f, f, vp]
    L.ntk_moe_combine.argtypes = [vp, vp, vp, vp, vp, vp, vp, i, i, i, vp]
    L.ntk_embed_dense_scaled.argtypes = [vp, vp, i, vp, i, i, i, f, vp]
    L.ntk_scale.argtypes = [vp, ll, f, vp]
    L.ntk_layernorm.argtypes = [vp, i, vp, i, vp, vp, i, i, f, i, vp]
    L.ntk_layernorm_history.argtypes = [vp, vp, i, vp, vp, vp, i, i, i, i, f, vp]
    L.ntk_causal_conv_mix.argtypes = [vp, i, vp, vp, vp, i, i, i, vp]
    L.ntk_sandwich_norm_conv.argtypes = [vp, i, vp, i, vp, i, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, f, vp]
    L.ntk_polynorm.argtypes = [vp, i, vp, i, vp, i, i, f, vp]
    L.ntk_gated_rmsnorm.argtypes = [vp, i, vp, i, vp, vp, i, i, i, f, vp]
    L.ntk_window_prepare.argtypes = [vp, i, vp, i, vp, i, vp, i, i, i, i, i, i, C.POINTER(Rotary), i, i, vp]
    L.ntk_window_attention_scratch.argtypes = [i, i, i, i, i]
    L.ntk_window_attention_scratch.restype = C.c_size_t
    L.ntk_window_attention.argtypes = [C.POINTER(WindowAttentionDesc), vp]
    L.ntk_lightning_attention.argtypes = [vp, i, vp, i, vp, i, vp, i, vp, vp, i, i, i, i, i, i, vp, vp]
    L.ntk_lightning_attention_scratch.argtypes = [i, i, i, i]
    L.ntk_lightning_attention_scratch.restype = C.c_size_t
    L.ntk_moe_route_ex.argtypes = [vp, vp, vp, vp, i, vp, vp, i, i, i, i, C.POINTER(RouteDesc), vp]
    L.ntk_glu.argtypes = [vp, vp, i, i, f, f, f, vp]
    L.ntk_moe_sum.argtypes = [vp, vp, vp, vp, vp, vp, i, i, i, vp]
    L.ntk_dyt.argtypes = [vp, i, vp, i, vp, vp, f, i, i, vp]
    L.ntk_embed_positions.argtypes = [vp, vp, vp, vp, i, vp, i, i, i, i, i, vp, vp, f, vp]
    L.ntk_sigmoid_gate_scaled.argtypes = [vp, i, vp, i, vp, f, i, i, vp]
    L.ntk_tanh_rows.argtypes = [vp, i, i, i, vp]
    L.ntk_head_rmsnorm_gate.argtypes = [vp, i, vp, i, vp, i, vp, i, i, f, i, i, i, f, vp]
    L.ntk_gated_seam.argtypes = [C.POINTER(GatedSeamDesc), vp]
    L.ntk_window_prepare_biased.argtypes = [vp, i, vp, i, vp, i, vp, i, i, i, i, i, i, C.POINTER(Rotary), vp, vp, vp, f, C.c_double, i, i, vp]
    L.ntk_gated_recurrence.argtypes = [C.POINTER(GatedRecurrenceDesc), vp]
    L.ntk_gated_recurrence_scratch.argtypes = [i, i, i, i, i]
    L.ntk_gated_recurrence_scratch.restype = C.c_size_t
    L.ntk_glu_cubic.argtypes = [vp, vp, i, i, i, f, f, f, f, vp]
    L.ntk_rms_seam.argtypes = [vp, i, vp, i, vp, i, vp, f, vp, i, i, f, vp]
    L.ntk_causal_conv_act.argtypes = [vp, i, vp, i, vp, vp, i, i, i, i, i, vp]
    L.ntk_softcap_rows.argtypes = [vp, i, f, i, i, vp]
    L.ntk_head_gate.argtypes = [vp, i, vp, i, i, i, i, vp]
    L.ntk_latent_unfold_value_ex.argtypes = [vp, i, vp, vp, i, vp, i, i, i, i, i, i, vp]
    L.ntk_window_prepare_ex.argtypes = [C.POINTER(WindowPrepareDesc), vp]
    L.ntk_gated_recurrence_scratch_ex.argtypes = [C.POINTER(GatedRecurrenceDesc)]
    L.ntk_gated_recurrence_scratch_ex.restype = C.c_size_t
    L._layers_bound = True
    return L


def to_bf16_bits(a: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return (u >> 16).astype(np.uint16)


def from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


def weight_buffer(w: np.ndarray, dtype: str) -> tuple:
    """(DeviceBuffer, NTK_DT_*) of a weight array in the given storage"""
    if dtype == "bfloat16":
        return DeviceBuffer.from_numpy(to_bf16_bits(w)), DT_BF16
    if dtype == "float32":
        return DeviceBuffer.from_numpy(np.ascontiguousarray(w, np.float32)), DT_F32
    raise ValueError(dtype)


def _f(a) -> DeviceBuffer:
    return DeviceBuffer.from_numpy(np.ascontiguousarray(a, np.float32))


def _i(a) -> DeviceBuffer:
    return DeviceBuffer.from_numpy(np.ascontiguousarray(a, np.int32))


def dense(x: np.ndarray, w: np.ndarray, dtype: str = "float32", offsets=None, rows=None, row_div: int = 1, n_rows: Optional[int] = None,
          y0: Optional[np.ndarray] = None, glu_limit: Optional[float] = None, glu_alpha: float = 1.702, norm_w: Optional[np.ndarray] = None,
          norm_eps: float = 1e-6, norm_offset: float = 0.0, glu_up_offset: float = 1.0, glu_cubic: float = 0.0) -> np.ndarray:
    """y[r] = x[src(r)] . w[g(r)]^T; w [N, K] or a stack [G, N, K] with `offsets` [G + 1]; rows: source row per output row (divided by row_div);
    y0: start values to accumulate onto."""
    L = _bind()
    w = np.asarray(w)
    stacked = w.ndim == 3
    N, K = w.shape[-2], w.shape[-1]
    T = int(n_rows if n_rows is not None else (len(rows) if rows is not None else x.shape[0]))
    xb, (wb, wdt) = _f(x), weight_buffer(w, dtype)
    yb = _f(y0) if y0 is not None else DeviceBuffer.zeros(max(T, 1) * N * 4)
    ob = _i(offsets) if offsets is not None else None
    rb = _i(rows) if rows is not None else None
    d = DenseDesc(yb.ptr, N, xb.ptr, x.shape[1], wb.ptr, N * K if stacked else 0, wdt, ob.ptr if ob else None, w.shape[0] if stacked else 1,
                  rb.ptr if rb else None, row_div, T, N, K, int(y0 is not None), 0, 0.0, 0.0, None, 0.0, 0.0, glu_up_offset, glu_cubic)
    nb = _f(norm_w) if norm_w is not None else None
    if nb is not None:          # fused RMS norm of the activation rows (few rows)
        d.norm_w, d.norm_eps, d.norm_offset = nb.ptr, norm_eps, norm_offset
    if glu_limit is not None:   # fused clipped GLU (few rows): N / 2 outputs per row
        d.glu_ff, d.glu_limit, d.glu_alpha, d.ldy = N // 2, glu_limit, glu_alpha, N // 2
        check(L.ntk_dense(C.byref(d), None), "ntk_dense")
        return yb.numpy(np.float32, T * (N // 2)).reshape(T, N // 2)
    check(L.ntk_dense(C.byref(d), None), "ntk_dense")
    return yb.numpy(np.float32, T * N).reshape(T, N)


def rmsnorm_offset(x: np.ndarray, w1: np.ndarray, w2: Optional[np.ndarray], eps: float, offset: float):
    L = _bind()
    T, n = x.shape
    xb, w1b = _f(x), _f(w1)
    y1 = DeviceBuffer.zeros(T * n * 4)
    y2 = DeviceBuffer.zeros(T * n * 4) if w2 is not None else None
    w2b = _f(w2) if w2 is not None else None
    check(L.ntk_rmsnorm_offset(y1.ptr, w1b.ptr, y2.ptr if y2 else None, w2b.ptr if w2b else None, n, xb.ptr, n, T, n, eps, offset, None), "ntk_rmsnorm_offset")
    a = y1.numpy(np.float32, T * n).reshape(T, n)
    return (a, y2.numpy(np.float32, T * n).reshape(T, n)) if y2 else a


def latent_prepare(kv: np.ndarray, norm_w: np.ndarray, eps: float, kv_rank: int, rot_dim: int, q: Optional[np.ndarray], heads: int, freq: np.ndarray, mag: float,
                   dims: int, pos0: int, cache: Optional[np.ndarray] = None, cache_rows: Optional[int] = None, layout: int = ROT_NEIGHBOURS):
    """-> (cache [rows, kv_rank + rot_dim] with rows pos0.. filled, q rotated)"""
    L = _bind()
    T, row = kv.shape[0], kv_rank + rot_dim
    n = cache_rows or (pos0 + T)
    cb = _f(cache) if cache is not None else DeviceBuffer.zeros(n * row * 4)
    kb, nb, fb = _f(kv), _f(norm_w), DeviceBuffer.from_numpy(np.ascontiguousarray(freq, np.float64))
    qb = _f(q) if q is not None else None
    qd = q.shape[1] // heads if q is not None else rot_dim
    rot = Rotary(fb.ptr, mag, dims, layout)
    check(L.ntk_latent_prepare(cb.ptr, row, kb.ptr, kv.shape[1], nb.ptr, eps, kv_rank, rot_dim, qb.ptr if qb else None, q.shape[1] if q is not None else 0, heads, qd,
                               C.byref(rot), pos0, T, None), "ntk_latent_prepare")
    return cb.numpy(np.float32, n * row).reshape(n, row), (qb.numpy(np.float32, q.size).reshape(q.shape) if qb else None)


def latent_attention(q: np.ndarray, cache: np.ndarray, kv_rank: int, rot_dim: int, heads: int, pos0: int, window: int, scale: float,
                     K: Optional[np.ndarray] = None, V: Optional[np.ndarray] = None, key0: int = 0) -> np.ndarray:
    """expanded form when K [nkeys, H * dn] and V [nkeys, H * dv] are given (q [T, H * (dn + dr)]), else the shared form (q [T, H * (R + dr)])"""
    L = _bind()
    T, row = q.shape[0], kv_rank + rot_dim
    qb, cb = _f(q), _f(cache)
    if K is not None:
        dn, dv = K.shape[1] // heads, V.shape[1] // heads
        kb, vb = _f(K), _f(V)
        out = DeviceBuffer.zeros(T * heads * dv * 4)
        check(L.ntk_latent_attention(out.ptr, heads * dv, qb.ptr, q.shape[1], kb.ptr, K.shape[1], vb.ptr, V.shape[1], cb.ptr, row, kv_rank, rot_dim, heads, dn, dv, 0,
                                     pos0, T, key0, window, scale, None, None), "ntk_latent_attention")
        return out.numpy(np.float32, T * heads * dv).reshape(T, heads * dv)
    nkeys = pos0 + T
    sc = DeviceBuffer.zeros(max(int(L.ntk_latent_attention_scratch(T, heads, kv_rank, nkeys)), 1) * 4)
    out = DeviceBuffer.zeros(T * heads * kv_rank * 4)
    check(L.ntk_latent_attention(out.ptr, heads * kv_rank, qb.ptr, q.shape[1], None, 0, None, 0, cb.ptr, row, kv_rank, rot_dim, heads, 0, 0, 1, pos0, T, 0, window,
                                 scale, sc.ptr, None), "ntk_latent_attention")
    return out.numpy(np.float32, T * heads * kv_rank).reshape(T, heads * kv_rank)


def latent_fold_query(q: np.ndarray, w_uk: np.ndarray, heads: int, dn: int, dr: int, dtype: str = "float32") -> np.ndarray:
    L = _bind()
    T, R = q.shape[0], w_uk.shape[1]
    qb, (wb, wdt) = _f(q), weight_buffer(w_uk, dtype)
    out = DeviceBuffer.zeros(T * heads * (R + dr) * 4)
    check(L.ntk_latent_fold_query(out.ptr, qb.ptr, q.shape[1], wb.ptr, wdt, T, heads, dn, dr, R, None), "ntk_latent_fold_query")
    return out.numpy(np.float32, T * heads * (R + dr)).reshape(T, heads * (R + dr))


def latent_unfold_value(lat: np.ndarray, w_uv: np.ndarray, heads: int, gate: Optional[np.ndarray] = None, dtype: str = "float32", head_gate: bool = False) -> np.ndarray:
    """head_gate: gate [T, heads] (one number per head) instead of [T, heads * dv]"""
    L = _bind()
    T, R = lat.shape[0], w_uv.shape[1]
    dv = w_uv.shape[0] // heads
    lb, (wb, wdt) = _f(lat), weight_buffer(w_uv, dtype)
    gb = _f(gate) if gate is not None else None
    out = DeviceBuffer.zeros(T * heads * dv * 4)
    check(L.ntk_latent_unfold_value_ex(out.ptr, heads * dv, lb.ptr, wb.ptr, wdt, gb.ptr if gb else None, gate.shape[1] if gate is not None else 0, int(head_gate), T, heads,
                                       dv, R, None), "ntk_latent_unfold_value")
    return out.numpy(np.float32, T * heads * dv).reshape(T, heads * dv)


def moe_route(h: np.ndarray, w_router: np.ndarray, top: int, shared_gate_w: Optional[np.ndarray] = None):
    L = _bind()
    T, n = h.shape
    E = w_router.shape[0]
    hb, wb = _f(h), _f(w_router)
    sb = _f(shared_gate_w) if shared_gate_w is not None else None
    ids, wts, sg = DeviceBuffer.zeros(T * top * 4), DeviceBuffer.zeros(T * top * 4), DeviceBuffer.zeros(T * 4)
    check(L.ntk_moe_route(ids.ptr, wts.ptr, sg.ptr if sb else None, hb.ptr, n, wb.ptr, sb.ptr if sb else None, T, n, E, top, None), "ntk_moe_route")
    return ids.numpy(np.int32, T * top).reshape(T, top), wts.numpy(np.float32, T * top).reshape(T, top), (sg.numpy(np.float32, T) if sb else None)


def moe_group(ids: np.ndarray, E: int):
    L = _bind()
    T, top = ids.shape
    ib = _i(ids)
    off, order, where = DeviceBuffer.zeros((E + 1) * 4), DeviceBuffer.zeros(T * top * 4), DeviceBuffer.zeros(T * top * 4)
    check(L.ntk_moe_group(off.ptr, order.ptr, where.ptr, ib.ptr, T, top, E, None), "ntk_moe_group")
    return off.numpy(np.int32, E + 1), order.numpy(np.int32, T * top), where.numpy(np.int32, T * top)


def clipped_glu(gu: np.ndarray, limit: float, alpha: float = 1.702) -> np.ndarray:
    L = _bind()
    rows, ff = gu.shape[0], gu.shape[1] // 2
    gb = _f(gu)
    out = DeviceBuffer.zeros(rows * ff * 4)
    check(L.ntk_clipped_glu(out.ptr, gb.ptr, rows, ff, limit, alpha, None), "ntk_clipped_glu")
    return out.numpy(np.float32, rows * ff).reshape(rows, ff)


def moe_combine(x, mix, d, where, wts, shared=None, sgate=None) -> np.ndarray:
    L = _bind()
    T, n = x.shape
    top = wts.shape[1]
    xb, db, wb, tb = _f(x), _f(d), _i(where), _f(wts)
    mb = _f(mix) if mix is not None else None
    sb = _f(shared) if shared is not None else None
    gb = _f(sgate) if sgate is not None else None
    check(L.ntk_moe_combine(xb.ptr, mb.ptr if mb else None, db.ptr, wb.ptr, tb.ptr, sb.ptr if sb else None, gb.ptr if gb else None, T, top, n, None), "ntk_moe_combine")
    return xb.numpy(np.float32, T * n).reshape(T, n)


# ---------------------------------------------------------------------------------------------------------------- sequential-form operators
def layernorm(x: np.ndarray, w: np.ndarray, b: Optional[np.ndarray], eps: float, onto: Optional[np.ndarray] = None) -> np.ndarray:
    """(x - mean) / sqrt(var + eps) * w + b per row; onto: start values the result is added to"""
    L = _bind()
    T, n = x.shape
    xb, wb = _f(x), _f(w)
    bb = _f(b) if b is not None else None
    yb = _f(onto) if onto is not None else DeviceBuffer.zeros(T * n * 4)
    check(L.ntk_layernorm(yb.ptr, n, xb.ptr, n, wb.ptr, bb.ptr if bb else None, T, n, eps, int(onto is not None), None), "ntk_layernorm")
    return yb.numpy(np.float32, T * n).reshape(T, n)


def norm_conv(x: np.ndarray, w: np.ndarray, b: np.ndarray, eps: float, canon: np.ndarray, state: Optional[np.ndarray], pos0: int):
    """h = layer norm of x; -> (h + causal convolution of h with the carried inputs in front, the new carried inputs [taps - 1, n])"""
    L = _bind()
    T, n = x.shape
    taps = canon.shape[1]
    xb, wb, bb, cb = _f(x), _f(w), _f(b), _f(canon)
    sb = _f(state) if state is not None else DeviceBuffer.zeros(max(taps - 1, 1) * n * 4)
    hist, out = DeviceBuffer.zeros((T + taps - 1) * n * 4), DeviceBuffer.zeros(T * n * 4)
    check(L.ntk_layernorm_history(hist.ptr, xb.ptr, n, wb.ptr, bb.ptr, sb.ptr, taps, pos0, T, n, eps, None), "ntk_layernorm_history")
    check(L.ntk_causal_conv_mix(out.ptr, n, hist.ptr, cb.ptr, sb.ptr, taps, T, n, None), "ntk_causal_conv_mix")
    return out.numpy(np.float32, T * n).reshape(T, n), sb.numpy(np.float32, max(taps - 1, 1) * n).reshape(-1, n)[:taps - 1]


def sandwich_norm_conv(x: np.ndarray, w: np.ndarray, b: np.ndarray, eps: float, canon: np.ndarray, state: Optional[np.ndarray], pos0: int,
                       owed: Optional[np.ndarray] = None, owed_w: Optional[np.ndarray] = None, owed_b: Optional[np.ndarray] = None):
    """the seam between two sublayers in one call: x += layer norm of `owed`; h = layer norm of x; -> (h + conv(h), x, the new carried inputs)"""
    L = _bind()
    T, n = x.shape
    taps = canon.shape[1]
    xb, wb, bb, cb = _f(x), _f(w), _f(b), _f(canon)
    sb = _f(state) if state is not None else DeviceBuffer.zeros(max(taps - 1, 1) * n * 4)
    ob, owb, obb = (_f(owed), _f(owed_w), _f(owed_b)) if owed is not None else (None, None, None)
    hist, out = DeviceBuffer.zeros((T + taps - 1) * n * 4), DeviceBuffer.zeros(T * n * 4)
    check(L.ntk_sandwich_norm_conv(out.ptr, n, xb.ptr, n, ob.ptr if ob else None, n, owb.ptr if ob else None, obb.ptr if ob else None, wb.ptr, bb.ptr, cb.ptr, sb.ptr,
                                   hist.ptr, taps, pos0, T, n, eps, None), "ntk_sandwich_norm_conv")
    return (out.numpy(np.float32, T * n).reshape(T, n), xb.numpy(np.float32, T * n).reshape(T, n),
            sb.numpy(np.float32, max(taps - 1, 1) * n).reshape(-1, n)[:taps - 1])


def polynorm(z: np.ndarray, coef, eps: float) -> np.ndarray:
    L = _bind()
    T, n = z.shape
    zb, cb = _f(z), _f(np.asarray(coef, np.float32))
    out = DeviceBuffer.zeros(T * n * 4)
    check(L.ntk_polynorm(out.ptr, n, zb.ptr, n, cb.ptr, T, n, eps, None), "ntk_polynorm")
    return out.numpy(np.float32, T * n).reshape(T, n)


def gated_rmsnorm(x: np.ndarray, w: np.ndarray, g: Optional[np.ndarray], eps: float) -> np.ndarray:
    L = _bind()
    T, n = x.shape
    xb, wb = _f(x), _f(w)
    gb = _f(g) if g is not None else None
    out = DeviceBuffer.zeros(T * n * 4)
    check(L.ntk_gated_rmsnorm(out.ptr, n, xb.ptr, n, wb.ptr, gb.ptr if gb else None, n, T, n, eps, None), "ntk_gated_rmsnorm")
    return out.numpy(np.float32, T * n).reshape(T, n)


def window_prepare(q: np.ndarray, k: np.ndarray, v: np.ndarray, H: int, G: int, maps: int, dn: int, dv: int, freq: np.ndarray, dims: int, pos0: int,
                   cache: Optional[np.ndarray] = None, cache_rows: Optional[int] = None):
    """-> (cache [rows, G * (maps * dn + dv)] with rows pos0 .. filled, q rotated)"""
    L = _bind()
    T, row = q.shape[0], G * (maps * dn + dv)
    n = cache_rows or (pos0 + T)
    cb = _f(cache) if cache is not None else DeviceBuffer.zeros(n * row * 4)
    qb, kb, vb = _f(q), _f(k), _f(v)
    fb = DeviceBuffer.from_numpy(np.ascontiguousarray(freq if len(freq) else [0.0], np.float64))
    rot = Rotary(fb.ptr, 1.0, dims)
    check(L.ntk_window_prepare(cb.ptr, row, qb.ptr, q.shape[1], kb.ptr, k.shape[1], vb.ptr, v.shape[1], H, G, maps, dn, dv, C.byref(rot), pos0, T, None), "ntk_window_prepare")
    return cb.numpy(np.float32, n * row).reshape(n, row), qb.numpy(np.float32, q.size).reshape(q.shape)


def window_prepare_biased(q, k, v, H: int, G: int, dn: int, dv: int, pos0: int, qb=None, kb=None, vb=None, temp_coef: float = 0.0, temp_every: float = 1.0,
                          cache: Optional[np.ndarray] = None, cache_rows: Optional[int] = None):
    """no rotation, one score map: q = (q + qb) * temperature(position), k + kb and v + vb into the cache rows -> (cache, q)"""
    L = _bind()
    T, row = q.shape[0], G * (dn + dv)
    n = cache_rows or (pos0 + T)
    cb = _f(cache) if cache is not None else DeviceBuffer.zeros(n * row * 4)
    qd, kd, vd = _f(q), _f(k), _f(v)
    bq, bk, bv = (_f(x) if x is not None else None for x in (qb, kb, vb))
    rot = Rotary(None, 1.0, 0)
    check(L.ntk_window_prepare_biased(cb.ptr, row, qd.ptr, q.shape[1], kd.ptr, k.shape[1], vd.ptr, v.shape[1], H, G, 1, dn, dv, C.byref(rot), bq.ptr if bq else None,
                                      bk.ptr if bk else None, bv.ptr if bv else None, temp_coef, temp_every, pos0, T, None), "ntk_window_prepare_biased")
    return cb.numpy(np.float32, n * row).reshape(n, row), qd.numpy(np.float32, q.size).reshape(q.shape)


def window_attention(q: np.ndarray, cache: np.ndarray, H: int, G: int, maps: int, dn: int, dv: int, pos0: int, window: int, scale: float, lam: float = 0.0,
                     sub_norm: bool = False, eps: float = 1e-6, out_scale: float = 1.0, split: bool = True, rel: Optional[np.ndarray] = None,
                     bucket_of: Optional[np.ndarray] = None, chunks: bool = False, softcap: float = 0.0, sink: bool = False, gate: Optional[np.ndarray] = None) -> np.ndarray:
    """q [T, H * maps * dn] (rotated), cache rows [G][maps][dn] keys | [G][dv] values; split: long key ranges of few rows may be cut into merged parts;
    rel [buckets, H] with bucket_of [distances]: a bias by distance on the scaled score"""
    L = _bind()
    T, row = q.shape[0], G * (maps * dn + dv)
    qb, cb = _f(q), _f(cache)
    out = DeviceBuffer.zeros(T * H * dv * 4)
    sc = DeviceBuffer.zeros(max(int(L.ntk_window_attention_scratch(T, H, maps, dv, pos0 + T)), 1) * 4) if split else None
    d = WindowAttentionDesc(out.ptr, H * dv, qb.ptr, q.shape[1], cb.ptr, row, H, G, maps, dn, dv, pos0, T, window, scale, lam, int(sub_norm), eps, out_scale,
                            sc.ptr if sc else None, None, None, 0)
    if rel is not None:
        rb, bb = _f(rel), _i(bucket_of)
        d.rel, d.bucket_of, d.n_dist = rb.ptr, bb.ptr, len(bucket_of)
    d.mask_mode, d.softcap, d.sink = (MASK_CHUNKS if chunks else MASK_SLIDING), softcap, int(sink)
    if gate is not None:        # [T, H * dv]: an elementwise sigmoid gate on the result
        gb = _f(gate)
        d.gate, d.ldg = gb.ptr, gate.shape[1]
    check(L.ntk_window_attention(C.byref(d), None), "ntk_window_attention")
    return out.numpy(np.float32, T * H * dv).reshape(T, H * dv)


def lightning_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, decay, H: int, dn: int, dv: int, pos0: int, state: Optional[np.ndarray] = None, silu: bool = True,
                        side_by_side: bool = True):
    """-> (out [T, H * dv], state [H, dn, dv]); state: what an earlier portion left (ignored when pos0 == 0); side_by_side: give the scratch that lets the
    chunks of a long portion run in parallel"""
    L = _bind()
    T = q.shape[0]
    qb, kb, vb = _f(q), _f(k), _f(v)
    with np.errstate(divide="ignore"):
        lb = _f(np.log(np.asarray(decay, np.float64)))
    sb = _f(state) if state is not None else DeviceBuffer.from_numpy(np.full(H * dn * dv, np.nan, np.float32))
    out = DeviceBuffer.zeros(T * H * dv * 4)
    ns = int(L.ntk_lightning_attention_scratch(T, H, dn, dv)) if side_by_side else 0
    scr = DeviceBuffer.from_numpy(np.full(ns, np.nan, np.float32)) if ns else None
    check(L.ntk_lightning_attention(out.ptr, H * dv, qb.ptr, q.shape[1], kb.ptr, k.shape[1], vb.ptr, v.shape[1], lb.ptr, sb.ptr, H, dn, dv, int(silu), pos0, T,
                                    scr.ptr if scr else None, None), "ntk_lightning_attention")
    return out.numpy(np.float32, T * H * dv).reshape(T, H * dv), sb.numpy(np.float32, H * dn * dv).reshape(H, dn, dv)


def moe_route_ex(h: np.ndarray, w_router: np.ndarray, top: int, score: int = 1, groups: int = 1, keep: int = 1, group_top: int = 2, renorm: bool = False,
                 scale: float = 1.0):
    L = _bind()
    T, n = h.shape
    E = w_router.shape[0]
    hb, wb = _f(h), _f(w_router)
    ids, wts = DeviceBuffer.zeros(T * top * 4), DeviceBuffer.zeros(T * top * 4)
    r = RouteDesc(score, groups, keep, group_top, int(renorm), scale)
    check(L.ntk_moe_route_ex(ids.ptr, wts.ptr, None, hb.ptr, n, wb.ptr, None, T, n, E, top, C.byref(r), None), "ntk_moe_route_ex")
    return ids.numpy(np.int32, T * top).reshape(T, top), wts.numpy(np.float32, T * top).reshape(T, top)


def glu(gu: np.ndarray, limit: float = float("inf"), alpha: float = 1.0, up_offset: float = 0.0) -> np.ndarray:
    L = _bind()
    rows, ff = gu.shape[0], gu.shape[1] // 2
    gb = _f(gu)
    out = DeviceBuffer.zeros(rows * ff * 4)
    check(L.ntk_glu(out.ptr, gb.ptr, rows, ff, limit, alpha, up_offset, None), "ntk_glu")
    return out.numpy(np.float32, rows * ff).reshape(rows, ff)


def moe_sum(d, where, wts, shared=None, sgate=None) -> np.ndarray:
    L = _bind()
    T, top = wts.shape
    n = d.shape[1]
    db, wb, tb = _f(d), _i(where), _f(wts)
    sb = _f(shared) if shared is not None else None
    gb = _f(sgate) if sgate is not None else None
    out = DeviceBuffer.zeros(T * n * 4)
    check(L.ntk_moe_sum(out.ptr, db.ptr, wb.ptr, tb.ptr, sb.ptr if sb else None, gb.ptr if gb else None, T, top, n, None), "ntk_moe_sum")
    return out.numpy(np.float32, T * n).reshape(T, n)


def dyt(x: np.ndarray, w: np.ndarray, b: Optional[np.ndarray], alpha: float) -> np.ndarray:
    L = _bind()
    T, n = x.shape
    xb, wb = _f(x), _f(w)
    bb = _f(b) if b is not None else None
    out = DeviceBuffer.zeros(T * n * 4)
    check(L.ntk_dyt(out.ptr, n, xb.ptr, n, wb.ptr, bb.ptr if bb else None, alpha, T, n, None), "ntk_dyt")
    return out.numpy(np.float32, T * n).reshape(T, n)


def embed_positions(table: np.ndarray, pos_table: np.ndarray, tokens, pos0: int, w=None, b=None, alpha: float = 0.0, dtype: str = "float32") -> np.ndarray:
    L = _bind()
    T, (V, W) = len(tokens), table.shape
    (tb, dt), (pb, _) = weight_buffer(table, dtype), weight_buffer(pos_table, dtype)
    ib = _i(tokens)
    wb, bb = (_f(x) if x is not None else None for x in (w, b))
    out = DeviceBuffer.zeros(T * W * 4)
    check(L.ntk_embed_positions(out.ptr, None, tb.ptr, pb.ptr, dt, ib.ptr, T, V, W, pos0, pos_table.shape[0], wb.ptr if wb else None, bb.ptr if bb else None, alpha,
                                None), "ntk_embed_positions")
    return out.numpy(np.float32, T * W).reshape(T, W)


def sigmoid_gate_scaled(y: np.ndarray, g: np.ndarray, gb=None, scale: float = 1.0) -> np.ndarray:
    L = _bind()
    T, n = y.shape
    yb, gd = _f(y), _f(g)
    bb = _f(gb) if gb is not None else None
    check(L.ntk_sigmoid_gate_scaled(yb.ptr, n, gd.ptr, n, bb.ptr if bb else None, scale, T, n, None), "ntk_sigmoid_gate_scaled")
    return yb.numpy(np.float32, T * n).reshape(T, n)


def head_rmsnorm_gate(x: np.ndarray, w: np.ndarray, H: int, dv: int, eps: float, g=None, act: int = 0, scale: float = 1.0, per_head: bool = False) -> np.ndarray:
    """w [dv] (shared by the heads) or, per_head, [H * dv]; act 0 none, 1 sigmoid(g), 2 silu(g)"""
    L = _bind()
    T = x.shape[0]
    xb, wb = _f(x), _f(w)
    gb = _f(g) if g is not None else None
    out = DeviceBuffer.zeros(T * H * dv * 4)
    check(L.ntk_head_rmsnorm_gate(out.ptr, H * dv, xb.ptr, H * dv, wb.ptr, dv if per_head else 0, gb.ptr if gb else None, H * dv, act,
                                  scale, T, H, dv, eps, None), "ntk_head_rmsnorm_gate")
    return out.numpy(np.float32, T * H * dv).reshape(T, H * dv)


def gated_seam(x, y=None, g=None, yb=None, gb=None, hist=None, coef=None, norm=None):
    """x [T, n] stream, y / g a sublayer's result and gate pre-activations; hist [n_hist, T, n] (its last entry is overwritten with the new layer result) with
    coef [n_hist]; norm = (w, b, alpha) -> (x, hist, h)"""
    L = _bind()
    T, n = x.shape
    xb = _f(x)
    bufs = {k: (_f(v) if v is not None else None) for k, v in dict(y=y, g=g, yb=yb, gb=gb, hist=hist, coef=coef).items()}
    p = lambda k: bufs[k].ptr if bufs[k] else None
    hb = DeviceBuffer.zeros(T * n * 4) if norm is not None else None
    nw, nb = (_f(norm[0]), _f(norm[1])) if norm is not None else (None, None)
    d = GatedSeamDesc(xb.ptr, n, p("y"), n, p("yb"), p("g"), n, p("gb"), p("hist"), T * n, 0 if hist is None else hist.shape[0], p("coef"),
                      hb.ptr if hb else None, n, nw.ptr if nw else None, nb.ptr if nb else None, norm[2] if norm is not None else 0.0, T, n)
    check(L.ntk_gated_seam(C.byref(d), None), "ntk_gated_seam")
    return (xb.numpy(np.float32, T * n).reshape(T, n), bufs["hist"].numpy(np.float32, hist.size).reshape(hist.shape) if hist is not None else None,
            hb.numpy(np.float32, T * n).reshape(T, n) if hb else None)


def gated_recurrence(q, k, v, wz, H: int, dn: int, dv: int, pos0: int, decay_form: int = DECAY_GIVEN, decay_param: float = 1.0, wb=None, az=None, ab=None,
                     unit_eps: float = 1e-6, q_scale: float = 1.0, state: Optional[np.ndarray] = None, prepass: bool = True, G: int = 0, unit_q: bool = False,
                     unit_k: bool = False, head_gates: bool = False, write_gated: bool = False, decay_rates=None, conv_w=None, conv_state=None):
    """-> (out [T, H * dv], state [H, dn, dv]); az: the removal rate's raw projection (None: no removal term); state: what an earlier portion left (ignored when
    pos0 == 0; by default full of NaN so that a read at the start would show); prepass: give the scratch that lets longer portions form their per-token vectors
    in a launch of their own"""
    L = _bind()
    T = q.shape[0]
    qb, kb, vb, zb = _f(q), _f(k), _f(v), _f(wz)
    wbb, azb, abb = (_f(x) if x is not None else None for x in (wb, az, ab))
    sb = _f(state) if state is not None else DeviceBuffer.from_numpy(np.full(H * dn * dv, np.nan, np.float32))
    out = DeviceBuffer.zeros(T * H * dv * 4)
    d = GatedRecurrenceDesc(out.ptr, H * dv, qb.ptr, q.shape[1], kb.ptr, k.shape[1], vb.ptr, v.shape[1], zb.ptr, wz.shape[1], wbb.ptr if wbb else None, decay_form,
                            decay_param, azb.ptr if azb else None, az.shape[1] if az is not None else 0, abb.ptr if abb else None, unit_eps, sb.ptr, H, dn, dv, q_scale,
                            pos0, T, None)
    rb = _f(decay_rates) if decay_rates is not None else None
    d.G, d.unit_q, d.unit_k, d.head_gates, d.write_gated, d.decay_rates = G, int(unit_q), int(unit_k), int(head_gates), int(write_gated), rb.ptr if rb else None
    cwb = csb = None
    if conv_w is not None:      # one token whose raw q, k, v pass their short convolutions inside the pre-pass; the carried inputs come back as a third result
        taps, nch = conv_w.shape[1], conv_w.shape[0]
        cwb = _f(conv_w)
        csb = _f(conv_state) if conv_state is not None and np.size(conv_state) else DeviceBuffer.from_numpy(np.full(max(taps - 1, 1) * nch, np.nan, np.float32))
        d.conv_w, d.conv_state, d.conv_taps = cwb.ptr, csb.ptr, taps
    ns = int(L.ntk_gated_recurrence_scratch_ex(C.byref(d))) if prepass else 0
    scr = DeviceBuffer.from_numpy(np.full(ns, np.nan, np.float32)) if ns else None
    if scr:
        d.scratch = scr.ptr
    check(L.ntk_gated_recurrence(C.byref(d), None), "ntk_gated_recurrence")
    if csb is not None:
        taps, nch = conv_w.shape[1], conv_w.shape[0]
        return (out.numpy(np.float32, T * H * dv).reshape(T, H * dv), sb.numpy(np.float32, H * dn * dv).reshape(H, dn, dv),
                csb.numpy(np.float32, max(taps - 1, 1) * nch).reshape(max(taps - 1, 1), nch)[:taps - 1])
    return out.numpy(np.float32, T * H * dv).reshape(T, H * dv), sb.numpy(np.float32, H * dn * dv).reshape(H, dn, dv)


def glu_cubic(gu: np.ndarray, ff: int, alpha: float, cubic: float, limit: float = float("inf"), up_offset: float = 0.0) -> np.ndarray:
    """gu rows may be longer than 2 * ff (what lies behind the up values is ignored)"""
    L = _bind()
    rows = gu.shape[0]
    gb = _f(gu)
    out = DeviceBuffer.zeros(rows * ff * 4)
    check(L.ntk_glu_cubic(out.ptr, gb.ptr, gu.shape[1], rows, ff, limit, alpha, cubic, up_offset, None), "ntk_glu_cubic")
    return out.numpy(np.float32, rows * ff).reshape(rows, ff)


def window_prepare_ex(q, k, v, H: int, G: int, dn: int, dv: int, pos0: int, freq=None, dims: int = 0, layout: int = ROT_NEIGHBOURS, v_other=None, v_blend: float = 0.0,
                      keep: bool = False, cache: Optional[np.ndarray] = None, cache_rows: Optional[int] = None):
    """one score map: rotation by `layout`, values blended with v_other [T, G * dv] on their way into the cache rows -> (cache, q, the values as they came if keep)"""
    L = _bind()
    T, row = q.shape[0], G * (dn + dv)
    n = cache_rows or (pos0 + T)
    cb = _f(cache) if cache is not None else DeviceBuffer.zeros(n * row * 4)
    qd, kd, vd = _f(q), _f(k), _f(v)
    fb = DeviceBuffer.from_numpy(np.ascontiguousarray(freq if freq is not None and len(freq) else [0.0], np.float64))
    rot = Rotary(fb.ptr, 1.0, dims, layout)
    ob = _f(v_other) if v_other is not None else None
    kb = DeviceBuffer.zeros(T * G * dv * 4) if keep else None
    d = WindowPrepareDesc()
    d.cache, d.row, d.q, d.ldq, d.k, d.ldk, d.v, d.ldv = cb.ptr, row, qd.ptr, q.shape[1], kd.ptr, k.shape[1], vd.ptr, v.shape[1]
    d.H, d.G, d.maps, d.dn, d.dv, d.rot, d.temp_every, d.pos0, d.T = H, G, 1, dn, dv, C.pointer(rot), 1.0, pos0, T
    if ob:
        d.v_other, d.ld_other, d.v_blend = ob.ptr, G * dv, v_blend
    if kb:
        d.v_keep, d.ld_keep = kb.ptr, G * dv
    check(L.ntk_window_prepare_ex(C.byref(d), None), "ntk_window_prepare_ex")
    return (cb.numpy(np.float32, n * row).reshape(n, row), qd.numpy(np.float32, q.size).reshape(q.shape),
            kb.numpy(np.float32, T * G * dv).reshape(T, G * dv) if kb else None)


def rms_seam(x: np.ndarray, w: Optional[np.ndarray], eps: float, add_y: Optional[np.ndarray] = None, add_w: Optional[np.ndarray] = None, mult: float = 1.0):
    """x += mult * rms(add_y) * add_w (if add_y), h = rms(x) * w (if w) -> (x, h or None)"""
    L = _bind()
    T, n = x.shape
    xb = _f(x)
    yb, awb, wb = (_f(a) if a is not None else None for a in (add_y, add_w, w))
    hb = DeviceBuffer.zeros(T * n * 4) if w is not None else None
    check(L.ntk_rms_seam(hb.ptr if hb else None, n, xb.ptr, n, yb.ptr if yb else None, n, awb.ptr if awb else None, mult, wb.ptr if wb else None, T, n, eps, None), "ntk_rms_seam")
    return xb.numpy(np.float32, T * n).reshape(T, n), (hb.numpy(np.float32, T * n).reshape(T, n) if hb else None)


def causal_conv_act(x: np.ndarray, w: np.ndarray, pos0: int, state: Optional[np.ndarray] = None, act: int = 1, n: Optional[int] = None):
    """x [T, >= n] (the first n columns are the channels), w [n, taps], state [taps - 1, n] (by default full of NaN) -> (y [T, n], state)"""
    L = _bind()
    T, taps = x.shape[0], w.shape[1]
    n = n or w.shape[0]
    xb, wb = _f(x), _f(w)
    sb = _f(state) if state is not None and np.size(state) else DeviceBuffer.from_numpy(np.full(max(taps - 1, 1) * n, np.nan, np.float32))
    yb = DeviceBuffer.zeros(T * n * 4)
    check(L.ntk_causal_conv_act(yb.ptr, n, xb.ptr, x.shape[1], wb.ptr, sb.ptr, taps, act, pos0, T, n, None), "ntk_causal_conv_act")
    return yb.numpy(np.float32, T * n).reshape(T, n), sb.numpy(np.float32, max(taps - 1, 1) * n).reshape(max(taps - 1, 1), n)[:taps - 1]


def softcap_rows(x: np.ndarray, cap: float) -> np.ndarray:
    L = _bind()
    T, n = x.shape
    xb = _f(x)
    check(L.ntk_softcap_rows(xb.ptr, n, cap, T, n, None), "ntk_softcap_rows")
    return xb.numpy(np.float32, T * n).reshape(T, n)


def head_gate(y: np.ndarray, g: np.ndarray, H: int) -> np.ndarray:
    """y [T, H * dv] times sigmoid(g [T, H]) per head"""
    L = _bind()
    T, dv = y.shape[0], y.shape[1] // H
    yb, gb = _f(y), _f(g)
    check(L.ntk_head_gate(yb.ptr, y.shape[1], gb.ptr, g.shape[1], T, H, dv, None), "ntk_head_gate")
    return yb.numpy(np.float32, y.size).reshape(y.shape)
