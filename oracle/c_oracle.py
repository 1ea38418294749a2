"""ctypes loader for oracle/libmta_oracle.so, the brute-force C checker.  TEST INFRASTRUCTURE ONLY.

Inputs and outputs are float32 numpy arrays; arithmetic inside is double.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmta_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "mta_oracle.c")):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libmta_oracle.so"])
    return _SO


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


_i64 = ctypes.c_int64


def conv2d(x, w, causal: bool):
    x, w = _f32(x), _f32(w)
    n, c, h, wd = x.shape
    c2, r, s = w.shape
    assert c2 == c
    y = np.empty_like(x)
    _load().oracle_conv2d(_p(x), _p(w), _p(y), _i64(n), _i64(c), _i64(h), _i64(wd), r, s, int(causal))
    return y


def headmix(x, w, causal: bool, fill: float):
    x, w = _f32(x), _f32(w)
    n, c, p, q = x.shape
    assert w.shape == (c, c)
    y = np.empty_like(x)
    _load().oracle_headmix(_p(x), _p(w), _p(y), _i64(n), _i64(c), _i64(p), _i64(q), int(causal),
                           ctypes.c_float(fill))
    return y


def mta_forward(q, k, v, w_pre, wpsm, w_post, wposm, mask=None):
    """``mask``: None = causal, else an additive (B,H,S,S) array of 0 / -inf."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    w_pre, wpsm, w_post, wposm = _f32(w_pre), _f32(wpsm), _f32(w_post), _f32(wposm)
    b, h, s, d = q.shape
    out = np.empty((b, s, h, d), dtype=np.float32)
    if mask is not None:
        mask = _f32(mask)
        assert mask.shape == (b, h, s, s)
    rc = _load().oracle_mta_forward(_p(q), _p(k), _p(v), _p(w_pre), _p(wpsm), _p(w_post), _p(wposm),
                                    _p(mask) if mask is not None else None, _p(out), _i64(b), _i64(h), _i64(s), _i64(d),
                                    w_pre.shape[1], w_pre.shape[2], w_post.shape[1], w_post.shape[2])
    assert rc == 0
    return out


def conv_attention(q, k, v, w, causal: bool, scale: float):
    q, k, v, w = _f32(q), _f32(k), _f32(v), _f32(w)
    b, h, s, d = q.shape
    o = np.empty_like(q)
    rc = _load().oracle_conv_attention(_p(q), _p(k), _p(v), _p(w), _p(o), _i64(b), _i64(h), _i64(s),
                                       _i64(d), w.shape[1], w.shape[2], int(causal), ctypes.c_float(scale))
    assert rc == 0
    return o


def conv2d_bwd(x, w, dy, causal: bool):
    """(dx float32, dw float64) from the C restatement of the reference's backward kernels."""
    x, w, dy = _f32(x), _f32(w), _f32(dy)
    n, c, h, wd = x.shape
    _, r, s = w.shape
    dx = np.empty_like(x)
    dw = np.empty((c, r, s), dtype=np.float64)
    _load().oracle_conv2d_bwd(_p(x), _p(w), _p(dy), _p(dx), _p(dw), _i64(n), _i64(c), _i64(h), _i64(wd), r, s, int(causal))
    return dx, dw


def headmix_bwd(x, w, dy, causal: bool):
    x, w, dy = _f32(x), _f32(w), _f32(dy)
    n, c, p, q = x.shape
    dx = np.empty_like(x)
    dw = np.empty((c, c), dtype=np.float64)
    _load().oracle_headmix_bwd(_p(x), _p(w), _p(dy), _p(dx), _p(dw), _i64(n), _i64(c), _i64(p), _i64(q), int(causal))
    return dx, dw
