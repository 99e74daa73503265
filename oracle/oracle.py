"""numpy front end of oracle/liboracle.so (see attention_oracle.c for what it restates).

TEST INFRASTRUCTURE ONLY -- the checker, never the thing measured or shipped.
Inputs are uint16 bit patterns of fp16 / bf16 values, outputs are float64.
"""
import ctypes
import math
import os

import numpy as np

from .build import LIB_PATH, build_oracle

DTYPE_CODE = {"fp16": 0, "bf16": 1}
_lib = None

_u16p = ctypes.POINTER(ctypes.c_uint16)
_f64p = ctypes.POINTER(ctypes.c_double)
_i64p = ctypes.POINTER(ctypes.c_int64)
_i32p = ctypes.POINTER(ctypes.c_int)


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        build_oracle()
    lib = ctypes.CDLL(LIB_PATH)
    lib.oracle_attention_rows.restype = ctypes.c_int
    lib.oracle_attention_rows.argtypes = [_u16p, _u16p, _u16p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int64,
                                          ctypes.c_int, ctypes.c_double, ctypes.c_int, _i64p, ctypes.c_int64, _f64p, _f64p]
    lib.oracle_ring_rows.restype = ctypes.c_int
    lib.oracle_ring_rows.argtypes = [_u16p, _u16p, _u16p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, _i32p,
                                     ctypes.c_int, ctypes.c_double, ctypes.c_int, ctypes.c_int, ctypes.c_int, _i32p,
                                     _i64p, ctypes.c_int64, _f64p, _f64p, _f64p, _f64p]
    lib.oracle_block_partial.restype = ctypes.c_int
    lib.oracle_block_partial.argtypes = [_u16p, _u16p, _u16p, ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
                                         ctypes.c_double, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                         _f64p, _f64p]
    lib.oracle_merge.restype = ctypes.c_int
    lib.oracle_merge.argtypes = [_f64p, _f64p, ctypes.c_int, ctypes.c_int64, ctypes.c_int, _f64p, _f64p]
    lib.oracle_round_array.restype = None
    lib.oracle_round_array.argtypes = [_f64p, _u16p, ctypes.c_int64, ctypes.c_int]
    lib.oracle_widen_array.restype = None
    lib.oracle_widen_array.argtypes = [_u16p, _f64p, ctypes.c_int64, ctypes.c_int]
    lib.oracle_num_threads.restype = ctypes.c_int
    lib.oracle_num_threads.argtypes = []
    _lib = lib
    return lib


def _u16(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint16, a.dtype
    return a


def _p(a, t):
    return a.ctypes.data_as(t)


def num_threads():
    return load().oracle_num_threads()


def widen(bits, dtype):
    """uint16 bit patterns -> float64 values (exact)."""
    bits = _u16(bits)
    out = np.empty(bits.shape, dtype=np.float64)
    load().oracle_widen_array(_p(bits, _u16p), _p(out, _f64p), bits.size, DTYPE_CODE[dtype])
    return out


def round_to(x, dtype):
    """float64 -> uint16 bit patterns of `dtype`, round-to-nearest-even."""
    x = np.ascontiguousarray(x, dtype=np.float64)
    out = np.empty(x.shape, dtype=np.uint16)
    load().oracle_round_array(_p(x, _f64p), _p(out, _u16p), x.size, DTYPE_CODE[dtype])
    return out


def default_scale(d):
    return 1.0 / math.sqrt(d)


def attention_rows(q, k, v, dtype, causal=False, scale=None, rows=None):
    """Direct softmax(scale QK^T [+causal]) V and LSE for the given flat rows (all if None).

    q, k, v: uint16 [B, H, S, d].  Returns (O [n, d] f64, LSE [n] f64)."""
    q, k, v = _u16(q), _u16(k), _u16(v)
    assert q.shape == k.shape == v.shape, "q, k, v must have the same [B, H, S, d] shape"
    B, H, S, d = q.shape
    scale = default_scale(d) if scale is None else scale
    if rows is None:
        n, rp = B * H * S, None
    else:
        rows = np.ascontiguousarray(rows, dtype=np.int64)
        n, rp = rows.size, _p(rows, _i64p)
    o = np.empty((n, d), dtype=np.float64)
    lse = np.empty((n,), dtype=np.float64)
    rc = load().oracle_attention_rows(_p(q, _u16p), _p(k, _u16p), _p(v, _u16p), DTYPE_CODE[dtype], B, H, S, d,
                                      float(scale), int(bool(causal)), rp, n, _p(o, _f64p), _p(lse, _f64p))
    if rc != 0:
        raise RuntimeError("oracle_attention_rows failed")
    return o, lse


def ring_rows(q, k, v, dtype, seqlen, rows, causal=False, scale=None, tile=64, round_p=False, order=None,
              want_parts=False):
    """Ring form (per-chunk online-softmax partials merged in ring order) for flat rows."""
    q, k, v = _u16(q), _u16(k), _u16(v)
    B, H, S, d = q.shape
    P = len(seqlen)
    assert sum(seqlen) == S
    scale = default_scale(d) if scale is None else scale
    rows = np.ascontiguousarray(rows, dtype=np.int64)
    n = rows.size
    sl = np.ascontiguousarray(seqlen, dtype=np.int32)
    o = np.empty((n, d), dtype=np.float64)
    lse = np.empty((n,), dtype=np.float64)
    po = np.empty((n, P, d), dtype=np.float64) if want_parts else None
    pl = np.empty((n, P), dtype=np.float64) if want_parts else None
    ordp = None
    if order is not None:
        orda = np.ascontiguousarray(order, dtype=np.int32)
        ordp = _p(orda, _i32p)
    rc = load().oracle_ring_rows(_p(q, _u16p), _p(k, _u16p), _p(v, _u16p), DTYPE_CODE[dtype], B, H, P, _p(sl, _i32p), d,
                                 float(scale), int(bool(causal)), int(tile), int(bool(round_p)), ordp, _p(rows, _i64p), n,
                                 _p(o, _f64p), _p(lse, _f64p), _p(po, _f64p) if want_parts else None,
                                 _p(pl, _f64p) if want_parts else None)
    if rc != 0:
        raise RuntimeError("oracle_ring_rows failed")
    return (o, lse, po, pl) if want_parts else (o, lse)


def block_partial(q, k, v, dtype, mask_mode=0, diag_offset=0, scale=None, tile=64, round_p=False):
    """Partial (O, LSE) of one head's Q chunk [cq, d] against one KV chunk [ck, d]."""
    q, k, v = _u16(q), _u16(k), _u16(v)
    cq, d = q.shape
    ck = k.shape[0]
    scale = default_scale(d) if scale is None else scale
    o = np.empty((cq, d), dtype=np.float64)
    lse = np.empty((cq,), dtype=np.float64)
    rc = load().oracle_block_partial(_p(q, _u16p), _p(k, _u16p), _p(v, _u16p), DTYPE_CODE[dtype], cq, ck, d, float(scale),
                                     int(mask_mode), int(diag_offset), int(tile), int(bool(round_p)), _p(o, _f64p),
                                     _p(lse, _f64p))
    if rc != 0:
        raise RuntimeError("oracle_block_partial failed")
    return o, lse


def merge(o_parts, lse_parts):
    """n-way merge: o_parts [n, rows, d], lse_parts [n, rows] (float64) -> (O [rows, d], LSE [rows])."""
    o_parts = np.ascontiguousarray(o_parts, dtype=np.float64)
    lse_parts = np.ascontiguousarray(lse_parts, dtype=np.float64)
    n, rows, d = o_parts.shape
    o = np.empty((rows, d), dtype=np.float64)
    lse = np.empty((rows,), dtype=np.float64)
    rc = load().oracle_merge(_p(o_parts, _f64p), _p(lse_parts, _f64p), n, rows, d, _p(o, _f64p), _p(lse, _f64p))
    if rc != 0:
        raise RuntimeError("oracle_merge failed")
    return o, lse
