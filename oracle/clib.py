"""ctypes front end of the C restatement (oracle/c/libmrx_oracle.so).

TEST INFRASTRUCTURE: imported only by tests, smoke() and bench.py's cpu_baseline.
Build with ``make -C oracle``.  ``precision`` selects the running-state type:
"f64" (parity checker) or "f32" (timed CPU baseline).
"""
from __future__ import annotations

import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "c", "libmrx_oracle.so")
_lib = None


def available() -> bool:
    return os.path.exists(_PATH)


def lib():
    global _lib
    if _lib is None:
        if not available():
            raise RuntimeError(f"{_PATH} missing: run `make -C oracle`")
        _lib = ctypes.CDLL(_PATH)
        _lib.orc_num_threads.restype = ctypes.c_int
    return _lib


def num_threads() -> int:
    return int(lib().orc_num_threads())


def set_num_threads(n: int) -> None:
    lib().orc_set_num_threads(ctypes.c_int(int(n)))


def _f(x):
    return None if x is None else np.ascontiguousarray(x, dtype=np.float32)


def _p(x):
    return None if x is None else x.ctypes.data_as(ctypes.c_void_p)


def _d(done):
    return np.ascontiguousarray(np.asarray(done) != 0, dtype=np.uint8)


def _i(*xs):
    return [ctypes.c_int64(int(x)) for x in xs]


def diag_scan_fwd(a, b, done, h0=None, precision="f64"):
    a, b, h0, done = _f(a), _f(b), _f(h0), _d(done)
    B, T, D = b.shape
    assert a.shape == b.shape
    h = np.empty_like(b)
    hl = np.empty((B, D), np.float32)
    Pl = np.empty((B, D), np.float32)
    getattr(lib(), f"orc_diag_scan_fwd_{precision}")(
        _p(a), _p(b), _p(done), _p(h0), _p(h), _p(hl), _p(Pl), *_i(B, T, D))
    return h, hl, Pl


def diag_scan_bwd(a, h, done, h0, g, g_last=None, precision="f64"):
    a, h, h0, g, g_last, done = _f(a), _f(h), _f(h0), _f(g), _f(g_last), _d(done)
    B, T, D = g.shape
    da, db = np.empty_like(g), np.empty_like(g)
    dh0 = np.empty((B, D), np.float32)
    getattr(lib(), f"orc_diag_scan_bwd_{precision}")(
        _p(a), _p(h), _p(done), _p(h0), _p(g), _p(g_last), _p(da), _p(db), _p(dh0),
        *_i(B, T, D))
    return da, db, dh0


def linear_attn_fwd(q, k, v, done, S0=None, fmap=0, precision="f64"):
    q, k, v, S0, done = _f(q), _f(k), _f(v), _f(S0), _d(done)
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    o = np.empty((B, T, H, dv), np.float32)
    Sl = np.empty((B, H, dv, dk), np.float32)
    getattr(lib(), f"orc_linear_attn_fwd_{precision}")(
        _p(q), _p(k), _p(v), _p(done), _p(S0), _p(o), _p(Sl), *_i(B, T, H, dk, dv),
        ctypes.c_int(int(fmap)))
    return o, Sl


def linear_attn_bwd(q, k, v, done, S0, do, dS_last=None, fmap=0, precision="f64"):
    q, k, v, S0, do, dS_last, done = _f(q), _f(k), _f(v), _f(S0), _f(do), _f(dS_last), _d(done)
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    dq, dk_, dv_ = np.empty_like(q), np.empty_like(k), np.empty_like(v)
    dS0 = np.empty((B, H, dv, dk), np.float32)
    getattr(lib(), f"orc_linear_attn_bwd_{precision}")(
        _p(q), _p(k), _p(v), _p(done), _p(S0), _p(do), _p(dS_last), _p(dq), _p(dk_),
        _p(dv_), _p(dS0), *_i(B, T, H, dk, dv), ctypes.c_int(int(fmap)))
    return dq, dk_, dv_, dS0


def delta_rule_fwd(q, k, v, beta, done, S0=None, precision="f64"):
    q, k, v, beta, S0, done = _f(q), _f(k), _f(v), _f(beta), _f(S0), _d(done)
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    o = np.empty((B, T, H, dv), np.float32)
    Sl = np.empty((B, H, dv, dk), np.float32)
    getattr(lib(), f"orc_delta_rule_fwd_{precision}")(
        _p(q), _p(k), _p(v), _p(beta), _p(done), _p(S0), _p(o), _p(Sl),
        *_i(B, T, H, dk, dv))
    return o, Sl


def delta_rule_bwd(q, k, v, beta, done, S0, do, dS_last=None, precision="f64"):
    q, k, v, beta, S0, do, dS_last, done = (
        _f(q), _f(k), _f(v), _f(beta), _f(S0), _f(do), _f(dS_last), _d(done))
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    dq, dk_, dv_ = np.empty_like(q), np.empty_like(k), np.empty_like(v)
    db = np.empty((B, T, H), np.float32)
    dS0 = np.empty((B, H, dv, dk), np.float32)
    getattr(lib(), f"orc_delta_rule_bwd_{precision}")(
        _p(q), _p(k), _p(v), _p(beta), _p(done), _p(S0), _p(do), _p(dS_last),
        _p(dq), _p(dk_), _p(dv_), _p(db), _p(dS0), *_i(B, T, H, dk, dv))
    return dq, dk_, dv_, db, dS0
