"""ctypes view of the CPU oracle (oracle/moe_oracle.c).

Test infrastructure only: imported by tests/, by the smoke check and by the
benchmark's CPU-baseline leg.  bfloat16 arrays are numpy uint16 arrays holding the raw
bits; indices are uint32.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmoe_oracle.so")

SCORE_SOFTMAX_TOPK_RENORM = 0
SCORE_SOFTMAX_TOPK = 1
SCORE_TOPK_SOFTMAX = 2


def build(force=False):
    """Compile the oracle with gcc (oracle/Makefile)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "libmoe_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return _SO


class Config(C.Structure):
    _fields_ = [(n, C.c_int32) for n in
                ("hidden", "n_experts", "top_k", "intermediate", "bits", "group_size", "score_mode")]


class QMat(C.Structure):
    _fields_ = [("w", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p)]


class Weights(C.Structure):
    _fields_ = [("router_w", C.c_void_p), ("router_bias", C.c_void_p),
                ("gate", QMat), ("up", QMat), ("down", QMat)]


class DebugOut(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in
                ("topk_idx", "topk_w", "counts", "offsets", "perm", "inv_perm")]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.orc_last_error.restype = C.c_char_p
        _lib.orc_expf.restype = C.c_float
        _lib.orc_expf.argtypes = [C.c_float]
        _lib.orc_f32_to_bf16.restype = C.c_uint16
        _lib.orc_f32_to_bf16.argtypes = [C.c_float]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _chk(rc):
    if rc != 0:
        raise RuntimeError(lib().orc_last_error().decode())


def _c(a, dt):
    a = np.ascontiguousarray(a)
    assert a.dtype == dt, (a.dtype, dt)
    return a


def f32_to_bf16(a):
    a = _c(np.asarray(a, dtype=np.float32), np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().orc_f32_to_bf16_n(_p(a), _p(out), C.c_int64(a.size))
    return out


def bf16_to_f32(a):
    a = _c(a, np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().orc_bf16_to_f32_n(_p(a), _p(out), C.c_int64(a.size))
    return out


def expf(x):
    return float(lib().orc_expf(C.c_float(x)))


def quantize(w, bits=4, group=64, scale_dtype="bf16"):
    w = _c(np.asarray(w, np.float32), np.float32)
    rows, cols = w.shape
    if group <= 0 or cols % group:
        _chk(lib().orc_quantize(_p(w), C.c_int64(rows), C.c_int64(cols), bits, group, None, None, None))
    q = np.empty((rows, cols * bits // 32), np.uint32)
    sdt = np.uint16 if scale_dtype == "bf16" else np.float32
    s = np.empty((rows, cols // group), sdt)
    b = np.empty((rows, cols // group), sdt)
    fn = lib().orc_quantize if scale_dtype == "bf16" else lib().orc_quantize_f32
    _chk(fn(_p(w), C.c_int64(rows), C.c_int64(cols), bits, group, _p(q), _p(s), _p(b)))
    return q, s, b


def dequantize(q, s, b, bits=4, group=64):
    q = _c(q, np.uint32)
    rows = q.shape[0]
    cols = q.shape[1] * 32 // bits
    out = np.empty((rows, cols), np.float32)
    if s.dtype == np.uint16:
        fn = lib().orc_dequantize
    else:
        fn = lib().orc_dequantize_f32
        s, b = _c(s, np.float32), _c(b, np.float32)
    _chk(fn(_p(q), _p(np.ascontiguousarray(s)), _p(np.ascontiguousarray(b)), C.c_int64(rows),
            C.c_int64(cols), bits, group, _p(out)))
    return out


def router_logits(x, wg, bias=None, f32seq=False):
    x, wg = _c(x, np.uint16), _c(wg, np.uint16)
    T, H = x.shape
    E = wg.shape[0]
    if bias is not None:
        bias = _c(bias, np.float32)
    g = np.empty((T, E), np.uint16)
    fn = lib().orc_router_logits_f32seq if f32seq else lib().orc_router_logits
    fn(_p(x), _p(wg), _p(bias), C.c_int64(T), H, E, _p(g))
    return g


def softmax(g):
    g = _c(g, np.uint16)
    T, E = g.shape
    p = np.empty((T, E), np.uint16)
    lib().orc_softmax(_p(g), C.c_int64(T), E, _p(p))
    return p


def topk(v, k):
    v = _c(v, np.uint16)
    T, E = v.shape
    inds = np.empty((T, k), np.uint32)
    lib().orc_topk(_p(v), C.c_int64(T), E, k, _p(inds))
    return inds


def scores(g, p, inds, score_mode):
    T, E = g.shape
    k = inds.shape[1]
    sc = np.empty((T, k), np.uint16)
    lib().orc_scores(_p(_c(g, np.uint16)), _p(None if p is None else _c(p, np.uint16)),
                     _p(_c(inds, np.uint32)), C.c_int64(T), E, k, score_mode, _p(sc))
    return sc


def route(cfg, router_w, router_bias, x):
    x = _c(x, np.uint16)
    T = x.shape[0]
    inds = np.empty((T, cfg.top_k), np.uint32)
    sc = np.empty((T, cfg.top_k), np.uint16)
    if router_bias is not None:
        router_bias = _c(router_bias, np.float32)
    lib().orc_route(C.byref(cfg), _p(_c(router_w, np.uint16)), _p(router_bias), _p(x),
                    C.c_int64(T), _p(inds), _p(sc))
    return inds, sc


def dispatch(flat, E):
    flat = np.ascontiguousarray(np.asarray(flat).reshape(-1).astype(np.uint32))
    P = flat.size
    counts = np.empty(E, np.uint32)
    offsets = np.empty(E + 1, np.uint32)
    perm = np.empty(P, np.uint32)
    inv = np.empty(P, np.uint32)
    _chk(lib().orc_dispatch(_p(flat), C.c_int64(P), E, _p(counts), _p(offsets), _p(perm), _p(inv)))
    return counts, offsets, perm, inv


def gather_qmm(x, w, s, b, lhs, rhs, bits=4, group=64, n_threads=8, want="f32", transpose=True):
    """x: uint16 [x_batch, M, K]; w: uint32 [E, N, K*bits/32] (transpose=False: [E, K, N*bits/32]);
    returns [n_idx, M, N]."""
    x, w = _c(x, np.uint16), _c(w, np.uint32)
    s, b = _c(s, np.uint16), _c(b, np.uint16)
    xb, M, K = x.shape
    E, N = w.shape[0], w.shape[1]
    if not transpose:
        N = w.shape[2] * 32 // bits
        rhs = np.ascontiguousarray(np.asarray(rhs).reshape(-1).astype(np.uint32))
        if lhs is not None:
            lhs = np.ascontiguousarray(np.asarray(lhs).reshape(-1).astype(np.uint32))
        n_idx = rhs.size
        yf = np.empty((n_idx, M, N), np.float32) if want == "f32" else None
        yb = np.empty((n_idx, M, N), np.uint16) if want == "bf16" else None
        _chk(lib().orc_gather_qmm_nt(_p(x), _p(w), _p(s), _p(b), _p(lhs), _p(rhs), C.c_int64(n_idx),
                                     C.c_int64(xb), M, N, K, E, bits, group, _p(yf), _p(yb)))
        return yf if want == "f32" else yb
    rhs = np.ascontiguousarray(np.asarray(rhs).reshape(-1).astype(np.uint32))
    if lhs is not None:
        lhs = np.ascontiguousarray(np.asarray(lhs).reshape(-1).astype(np.uint32))
    n_idx = rhs.size
    yf = np.empty((n_idx, M, N), np.float32) if want == "f32" else None
    yb = np.empty((n_idx, M, N), np.uint16) if want == "bf16" else None
    _chk(lib().orc_gather_qmm(_p(x), _p(w), _p(s), _p(b), _p(lhs), _p(rhs), C.c_int64(n_idx),
                              C.c_int64(xb), M, N, K, E, bits, group, _p(yf), _p(yb), n_threads))
    return yf if want == "f32" else yb


def swiglu_bf16(gate, up):
    gate, up = _c(gate, np.uint16), _c(up, np.uint16)
    out = np.empty(gate.shape, np.uint16)
    lib().orc_swiglu_bf16(_p(gate), _p(up), C.c_int64(gate.size), _p(out))
    return out


def swiglu_f32(gate, up):
    gate, up = _c(gate, np.float32), _c(up, np.float32)
    out = np.empty(gate.shape, np.uint16)
    lib().orc_swiglu_f32(_p(gate), _p(up), C.c_int64(gate.size), _p(out))
    return out


def combine(y, sc, inv_perm, strict=False):
    y, sc = _c(y, np.uint16), _c(sc, np.uint16)
    T, k = sc.shape
    H = y.shape[-1]
    if inv_perm is not None:
        inv_perm = _c(inv_perm, np.uint32)
    out = np.empty((T, H), np.uint16)
    lib().orc_combine(_p(y), _p(sc), _p(inv_perm), C.c_int64(T), k, H, int(strict), _p(out))
    return out


def rms_norm(x, weight, eps=1e-5):
    x, weight = _c(x, np.uint16), _c(weight, np.uint16)
    T, H = x.shape
    out = np.empty((T, H), np.uint16)
    lib().orc_rms_norm(_p(x), _p(weight), C.c_float(eps), C.c_int64(T), H, _p(out))
    return out


def make_config(hidden, n_experts, top_k, intermediate, bits=4, group_size=64, score_mode=0):
    return Config(hidden, n_experts, top_k, intermediate, bits, group_size, score_mode)


def moe_forward(cfg, weights, x, strict=False, n_threads=8, debug=True, norm_weight=None, eps=1e-5):
    """weights: dict with router_w (uint16 [E,H]), router_bias (float32 [E] or None) and
    gate/up/down each a (w uint32, scales uint16, biases uint16) tuple.
    With norm_weight (uint16 [H]) the result is x + moe(rms_norm(x, norm_weight, eps)).
    Returns (out uint16 [T,H], dict of routing arrays)."""
    x = _c(x, np.uint16)
    T = x.shape[0]
    P = T * cfg.top_k
    keep = []

    def qm(t):
        arrs = [np.ascontiguousarray(a) for a in t]
        keep.extend(arrs)
        return QMat(*[_p(a) for a in arrs])

    rw = _c(weights["router_w"], np.uint16)
    rb = weights.get("router_bias")
    if rb is not None:
        rb = _c(rb, np.float32)
    W = Weights(_p(rw), _p(rb), qm(weights["gate"]), qm(weights["up"]), qm(weights["down"]))
    out = np.empty((T, cfg.hidden), np.uint16)
    d = dict(topk_idx=np.empty((T, cfg.top_k), np.uint32), topk_w=np.empty((T, cfg.top_k), np.uint16),
             counts=np.empty(cfg.n_experts, np.uint32), offsets=np.empty(cfg.n_experts + 1, np.uint32),
             perm=np.empty(P, np.uint32), inv_perm=np.empty(P, np.uint32))
    dbg = DebugOut(*[_p(d[n]) for n in ("topk_idx", "topk_w", "counts", "offsets", "perm", "inv_perm")])
    if norm_weight is None:
        _chk(lib().orc_moe_forward(C.byref(cfg), C.byref(W), _p(x), C.c_int64(T), _p(out),
                                   C.byref(dbg) if debug else None, int(strict), int(n_threads)))
    else:
        nw = _c(norm_weight, np.uint16)
        _chk(lib().orc_moe_forward_residual(C.byref(cfg), C.byref(W), _p(x), _p(nw), C.c_float(eps),
                                            C.c_int64(T), _p(out), C.byref(dbg) if debug else None,
                                            int(strict), int(n_threads)))
    return out, d
