"""Pins the C restatement (fwd + analytic bwd) against the NumPy / torch-fp64 oracle."""
import numpy as np
import pytest

from oracle import clib
from oracle import grad as G
from oracle import memoroid as M

pytestmark = pytest.mark.skipif(not clib.available(), reason="run `make -C oracle`")
RNG = np.random.default_rng(13)


def f32(*s):
    return RNG.standard_normal(s).astype(np.float32)


def close(x, y, tol, name=""):
    err = np.abs(np.asarray(x, np.float64) - y).max() / max(np.abs(y).max(), 1e-30)
    assert err <= tol, f"{name}: rel err {err:.3e} > {tol}"


@pytest.mark.parametrize("prec,tol", [("f64", 2e-7), ("f32", 2e-5)])
def test_c_diag_scan(prec, tol):
    B, T, D = 3, 70, 19
    a = RNG.uniform(0.9, 0.999, (B, T, D)).astype(np.float32)
    b, h0 = f32(B, T, D), f32(B, D)
    d = RNG.random((B, T)) < 0.05
    d[1, 0] = True
    h, hl, Pl = clib.diag_scan_fwd(a, b, d, h0, prec)
    rh, rhl, rPl = M.diag_scan(a, b, d, h0)
    close(h, rh, tol, "h"); close(hl, rhl, tol, "h_last"); close(Pl, rPl, tol, "P_last")
    g, gl = f32(B, T, D), f32(B, D)
    da, db, dh0 = clib.diag_scan_bwd(a, rh.astype(np.float32), d, h0, g, gl, prec)
    ag = G.diag_scan_grads(a, b, d, h0, g, gl)
    close(da, ag["da"], 5 * tol, "da"); close(db, ag["db"], 5 * tol, "db"); close(dh0, ag["dh0"], 5 * tol, "dh0")


@pytest.mark.parametrize("prec,tol", [("f64", 3e-7), ("f32", 3e-5)])
@pytest.mark.parametrize("fmap", [0, 1])
def test_c_linear_attention(prec, tol, fmap):
    B, T, H, dk, dv = 2, 50, 2, 8, 6
    q, k, v, S0 = f32(B, T, H, dk), f32(B, T, H, dk), f32(B, T, H, dv), f32(B, H, dv, dk)
    do, dSl = f32(B, T, H, dv), f32(B, H, dv, dk)
    d = RNG.random((B, T)) < 0.08
    name = "elu1" if fmap else "none"
    ag = G.linear_attention_grads(q, k, v, d, S0, do, dSl, name)
    o, Sl = clib.linear_attn_fwd(q, k, v, d, S0, fmap, prec)
    close(o, ag["o"], tol, "o"); close(Sl, ag["S_last"], tol, "S_last")
    dq, dk_, dv_, dS0 = clib.linear_attn_bwd(q, k, v, d, S0, do, dSl, fmap, prec)
    close(dq, ag["dq"], tol, "dq"); close(dk_, ag["dk"], tol, "dk")
    close(dv_, ag["dv"], tol, "dv"); close(dS0, ag["dS0"], tol, "dS0")


@pytest.mark.parametrize("prec,tol", [("f64", 3e-7), ("f32", 5e-5)])
def test_c_delta_rule(prec, tol):
    B, T, H, dk, dv = 2, 60, 2, 8, 6
    q, k, v, S0 = f32(B, T, H, dk), f32(B, T, H, dk), f32(B, T, H, dv), f32(B, H, dv, dk)
    k /= np.linalg.norm(k, axis=-1, keepdims=True)
    beta = M.sigmoid(f32(B, T, H)).astype(np.float32)
    do, dSl = f32(B, T, H, dv), f32(B, H, dv, dk)
    d = RNG.random((B, T)) < 0.06
    d[0, 0] = True
    ag = G.delta_rule_grads(q, k, v, beta, d, S0, do, dSl)
    o, Sl = clib.delta_rule_fwd(q, k, v, beta, d, S0, prec)
    close(o, ag["o"], tol, "o"); close(Sl, ag["S_last"], tol, "S_last")
    dq, dk_, dv_, db, dS0 = clib.delta_rule_bwd(q, k, v, beta, d, S0, do, dSl, prec)
    close(dq, ag["dq"], tol, "dq"); close(dk_, ag["dk"], tol, "dk"); close(dv_, ag["dv"], tol, "dv")
    close(db, ag["dbeta"], tol, "dbeta"); close(dS0, ag["dS0"], tol, "dS0")


def test_c_null_optionals():
    B, T, H, d = 1, 5, 1, 4
    q, k, v = f32(B, T, H, d), f32(B, T, H, d), f32(B, T, H, d)
    dn = np.zeros((B, T), bool)
    o, _ = clib.linear_attn_fwd(q, k, v, dn, None)
    close(o, M.linear_attention(q, k, v, dn)[0], 1e-6)
