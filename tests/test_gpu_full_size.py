"""The benchmark configurations at their full sizes, through the C ABI.

The C oracle (fp64 state, OpenMP over the sequences) does configuration 4's whole batch in well
under a second, so configurations 2, 4 and 5 are compared with it outright; on top of that,
properties that hold at any size: split invariance (two calls with the carried state equal one),
linearity of the backward pass in the incoming gradients, the two routes to the triangular factors."""
import numpy as np
import pytest
import torch

from oracle import clib
from oracle import memoroid as M
from gpu_util import TOL_BF16, TOL_F32, bf16_round, dev, relerr

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _cfg4(B=64, T=1024, H=8, p_seed=4):
    x = M.make_inputs(p_seed, (B, T, H, 64))
    xb = {n: bf16_round(x[n]) for n in ("q", "k", "v", "beta")}
    do = bf16_round(np.random.default_rng(1).standard_normal(x["v"].shape).astype(np.float32))
    return x, xb, do


def test_config4_delta_rule_full_batch_against_the_c_oracle():
    from memorax_amd import kernels as K
    x, xb, do = _cfg4()
    print("case full cfg4 delta rule fwd+bwd", flush=True)
    tq, tk, tv, tb, tdo = (dev(a, BF) for a in (xb["q"], xb["k"], xb["v"], xb["beta"], do))
    dn = dev(x["done"])
    o, Sl, chk = K.delta_rule_fwd(tq, tk, tv, tb, dn)
    got = K.delta_rule_bwd(tq, tk, tv, tb, dn, chk, tdo)
    ro, rSl = clib.delta_rule_fwd(xb["q"], xb["k"], xb["v"], xb["beta"], x["done"])
    ref = clib.delta_rule_bwd(xb["q"], xb["k"], xb["v"], xb["beta"], x["done"], None, do)
    errs = {"o": relerr(o, ro), "S_last": relerr(Sl, rSl)}
    errs.update({n: relerr(g, r) for n, g, r in zip(("dq", "dk", "dv", "dbeta", "dS0"), got, ref)})
    assert all(e <= TOL_BF16 for e in errs.values()), errs


def test_config5_shape_delta_rule_against_the_c_oracle():
    """One block of configuration 5: 1024 environments x 4 heads, T = 128, resets every hundred steps
    (more sequences than two per compute unit: the sequential kernel inverts in place)."""
    from memorax_amd import kernels as K
    rng = np.random.default_rng(1005)
    shp = (1024, 128, 4, 64)
    x = {"q": rng.standard_normal(shp).astype(np.float32), "k": rng.standard_normal(shp).astype(np.float32),
         "v": rng.standard_normal(shp).astype(np.float32),
         "beta": (1.0 / (1.0 + np.exp(-rng.standard_normal(shp[:3])))).astype(np.float32),
         "done": rng.random(shp[:2]) < 0.01}
    x["k"] /= np.linalg.norm(x["k"], axis=-1, keepdims=True)
    xb = {n: bf16_round(x[n]) for n in ("q", "k", "v", "beta")}
    do = bf16_round(np.random.default_rng(2).standard_normal(x["v"].shape).astype(np.float32))
    print("case full cfg5 delta rule fwd+bwd", flush=True)
    tq, tk, tv, tb, tdo = (dev(a, BF) for a in (xb["q"], xb["k"], xb["v"], xb["beta"], do))
    dn = dev(x["done"])
    o, Sl, chk = K.delta_rule_fwd(tq, tk, tv, tb, dn)
    got = K.delta_rule_bwd(tq, tk, tv, tb, dn, chk, tdo)
    ro, rSl = clib.delta_rule_fwd(xb["q"], xb["k"], xb["v"], xb["beta"], x["done"])
    ref = clib.delta_rule_bwd(xb["q"], xb["k"], xb["v"], xb["beta"], x["done"], None, do)
    errs = {"o": relerr(o, ro), "S_last": relerr(Sl, rSl)}
    errs.update({n: relerr(g, r) for n, g, r in zip(("dq", "dk", "dv", "dbeta", "dS0"), got, ref)})
    assert all(e <= TOL_BF16 for e in errs.values()), errs


def test_config2_linear_attention_full_batch_against_the_c_oracle():
    from memorax_amd import kernels as K
    x = M.make_inputs(2, (64, 256, 4, 64))
    do = np.random.default_rng(0).standard_normal(x["v"].shape).astype(np.float32)
    print("case full cfg2 linear attention fwd+bwd", flush=True)
    tq, tk, tv, tdo = (dev(a) for a in (x["q"], x["k"], x["v"], do))
    o, Sl, chk = K.linear_attn_fwd(tq, tk, tv, dev(x["done"]), None, 1)
    got = K.linear_attn_bwd(tq, tk, tv, dev(x["done"]), chk, tdo, None, 1)
    ro, rSl = clib.linear_attn_fwd(x["q"], x["k"], x["v"], x["done"], None, 1)
    ref = clib.linear_attn_bwd(x["q"], x["k"], x["v"], x["done"], None, do, None, 1)
    errs = {"o": relerr(o, ro), "S_last": relerr(Sl, rSl)}
    errs.update({n: relerr(g, r) for n, g, r in zip(("dq", "dk", "dv", "dS0"), got, ref)})
    assert all(e <= TOL_F32 for e in errs.values()), errs


def test_config4_split_invariance_is_exact():
    """Steps [0, 512) and then [512, 1024) from the carried fp32 state give the outputs and the final
    state of one call bit for bit (the split falls on a chunk boundary)."""
    from memorax_amd import kernels as K
    x, xb, _ = _cfg4()
    tq, tk, tv, tb = (dev(a, BF) for a in (xb["q"], xb["k"], xb["v"], xb["beta"]))
    dn = dev(x["done"])
    o, Sl, _ = K.delta_rule_fwd(tq, tk, tv, tb, dn, save_chk=False)
    h = 512
    a = [t[:, :h].contiguous() for t in (tq, tk, tv, tb, dn)]
    b = [t[:, h:].contiguous() for t in (tq, tk, tv, tb, dn)]
    o1, S1, _ = K.delta_rule_fwd(*a, save_chk=False)
    o2, S2, _ = K.delta_rule_fwd(*b, S1, save_chk=False)
    assert torch.equal(torch.cat((o1, o2), dim=1), o) and torch.equal(S2, Sl)


def test_config4_backward_is_linear_in_the_incoming_gradients():
    from memorax_amd import kernels as K
    x, xb, do = _cfg4()
    tq, tk, tv, tb = (dev(a, BF) for a in (xb["q"], xb["k"], xb["v"], xb["beta"]))
    dn = dev(x["done"])
    g = torch.Generator(device="cuda").manual_seed(9)
    d1 = dev(do, BF)
    d2 = torch.randn(d1.shape, device="cuda", generator=g).to(BF)
    s1 = torch.randn((64, 8, 64, 64), device="cuda", generator=g)
    s2 = torch.randn((64, 8, 64, 64), device="cuda", generator=g)
    _, _, chk = K.delta_rule_fwd(tq, tk, tv, tb, dn)
    ga = K.delta_rule_bwd(tq, tk, tv, tb, dn, chk, d1, s1)
    gb = K.delta_rule_bwd(tq, tk, tv, tb, dn, chk, d2, s2)
    gs = K.delta_rule_bwd(tq, tk, tv, tb, dn, chk, (d1.float() + d2.float()).to(BF), s1 + s2)
    for n, u, v_, w in zip(("dq", "dk", "dv", "dbeta", "dS0"), ga, gb, gs):
        assert relerr(w, (u.float() + v_.float()).cpu().numpy()) <= TOL_BF16, n


def test_config3_linear_attention_full_size_properties():
    """Configuration 3 (B=256, T=4096, H=8, bf16, no resets; 1 GiB per tensor) is too large for the
    CPU oracle in a test: split invariance (exact) and linearity of the backward at full size, and the
    first two batch rows against the C oracle."""
    from memorax_amd import kernels as K
    B, T, H = 256, 4096, 8
    g = torch.Generator(device="cuda").manual_seed(1003)
    q, k, v, d1, d2 = ((torch.randn((B, T, H, 64), device="cuda", generator=g) / 8).to(BF) for _ in range(5))
    dn = torch.zeros((B, T), device="cuda", dtype=torch.uint8)
    print("case full cfg3 linear attention", flush=True)
    o, Sl, chk = K.linear_attn_fwd(q, k, v, dn, None, 0)
    h = T // 2
    o1, S1, _ = K.linear_attn_fwd(q[:, :h].contiguous(), k[:, :h].contiguous(), v[:, :h].contiguous(), dn[:, :h].contiguous(),
                                  None, 0, save_chk=False)
    o2, S2, _ = K.linear_attn_fwd(q[:, h:].contiguous(), k[:, h:].contiguous(), v[:, h:].contiguous(), dn[:, h:].contiguous(),
                                  S1, 0, save_chk=False)
    assert torch.equal(o[:, :h], o1) and torch.equal(o[:, h:], o2) and torch.equal(S2, Sl)
    del o1, o2
    ga = K.linear_attn_bwd(q, k, v, dn, chk, d1, None, 0)
    gb = K.linear_attn_bwd(q, k, v, dn, chk, d2, None, 0)
    gs = K.linear_attn_bwd(q, k, v, dn, chk, (d1.float() + d2.float()).to(BF), None, 0)
    for n, u, w_, s_ in zip(("dq", "dk", "dv"), ga, gb, gs):
        err = float((s_.float() - (u.float() + w_.float())).abs().max() / (u.float() + w_.float()).abs().max())
        assert err <= TOL_BF16, (n, err)
    nb = 2
    xs = [t[:nb].float().cpu().numpy() for t in (q, k, v, d1)]
    ro, rSl = clib.linear_attn_fwd(xs[0], xs[1], xs[2], np.zeros((nb, T), bool), None, 0)
    ref = clib.linear_attn_bwd(xs[0], xs[1], xs[2], np.zeros((nb, T), bool), None, xs[3], None, 0)
    assert relerr(o[:nb], ro) <= TOL_BF16 and relerr(Sl[:nb], rSl) <= TOL_BF16
    for n, u, r in zip(("dq", "dk", "dv"), ga, ref):
        assert relerr(u[:nb], r) <= TOL_BF16, n


def test_config5_scan_shape_against_the_oracle():
    """The diagonal scan at configuration 5's shape (1024, 128, 256), resets every hundred steps:
    forward and backward against the NumPy oracle (streaming kernels: enough columns to fill the chip)."""
    from memorax_amd import kernels as K
    shape = (1024, 128, 256)
    rng = np.random.default_rng(1005)
    a = rng.uniform(0.9, 0.999, shape).astype(np.float32)
    b = rng.standard_normal(shape).astype(np.float32)
    g = rng.standard_normal(shape).astype(np.float32)
    done = rng.random(shape[:2]) < 0.01
    print("case full cfg5 scan", flush=True)
    h, hl, Pl = K.linear_scan_fwd(dev(a), dev(b), dev(done))
    rh, rhl, rPl = M.diag_scan(a, b, done)
    assert relerr(h, rh) <= TOL_F32 and relerr(hl, rhl) <= TOL_F32 and relerr(Pl, rPl) <= TOL_F32
    da, db, _ = K.linear_scan_bwd(dev(a), h, dev(done), None, dev(g), None)
    rda, rdb, _ = M.diag_scan_bwd(a, rh, done, g)
    assert relerr(da, rda) <= TOL_F32 and relerr(db, rdb) <= TOL_F32


def test_scan_sweep_shape_properties():
    """512 x 1024 x 1024 fp32 (2 GiB per tensor), the shape the scan's bandwidth is quoted on: split
    invariance at full size and one batch row against the oracle."""
    from memorax_amd import kernels as K
    B, T, D = 512, 1024, 1024
    g = torch.Generator(device="cuda").manual_seed(7)
    a = torch.rand((B, T, D), device="cuda", generator=g) * 0.099 + 0.9
    b = torch.randn((B, T, D), device="cuda", generator=g)
    done = torch.rand((B, T), device="cuda", generator=g) < 0.002
    print("case scan sweep shape", flush=True)
    h, hl, Pl = K.linear_scan_fwd(a, b, done)
    s = 500  # not a multiple of anything the kernels block by
    h1, hl1, Pl1 = K.linear_scan_fwd(a[:, :s].contiguous(), b[:, :s].contiguous(), done[:, :s].contiguous())
    h2, hl2, Pl2 = K.linear_scan_fwd(a[:, s:].contiguous(), b[:, s:].contiguous(), done[:, s:].contiguous(), hl1, Pl1)
    err = float((torch.cat((h1, h2), dim=1) - h).abs().max() / h.abs().max())
    assert err <= 1e-6 and float((hl2 - hl).abs().max()) <= 1e-5 * float(hl.abs().max()), err
    rh, rhl, rPl = M.diag_scan(a[:1].cpu().numpy(), b[:1].cpu().numpy(), done[:1].cpu().numpy())
    assert relerr(h[:1], rh) <= TOL_F32 and relerr(hl[:1], rhl) <= TOL_F32 and relerr(Pl[:1], rPl) <= TOL_F32


def test_config5_mingru_shape_against_the_oracle():
    """The MinGRU recurrence with the gate arithmetic inside the kernels at configuration 5's shape
    (1024, 128, 256): states against the oracle's log-space route (the reference's formulation),
    gradients against the closed form over the oracle's reverse scan."""
    from memorax_amd import kernels as K
    shape = (1024, 128, 256)
    rng = np.random.default_rng(2005)
    z = (2 * rng.standard_normal(shape)).astype(np.float32)
    x = (2 * rng.standard_normal(shape)).astype(np.float32)
    g = rng.standard_normal(shape).astype(np.float32)
    done = rng.random(shape[:2]) < 0.01
    print("case full cfg5 mingru", flush=True)
    h, hl, _ = K.mingru_scan_fwd(dev(z), dev(x), dev(done))
    dz, dx, _ = K.mingru_scan_bwd(dev(z), dev(x), h, dev(done), None, dev(g))
    nxt, rh = M.mingru_scan(z, x, done)
    assert relerr(h, rh) <= TOL_F32 and relerr(hl, np.exp(nxt[0][:, 0])) <= TOL_F32
    a, b = M.mingru_linear_coeffs(z, x)
    da, lam, _ = M.diag_scan_bwd(a, rh, done, g)
    z64, x64 = z.astype(np.float64), x.astype(np.float64)
    s = M.sigmoid(z64)
    rdz = s * (1 - s) * (np.where(x64 >= 0, x64 + 0.5, M.sigmoid(x64)) * lam - da)
    rdx = lam * s * np.where(x64 >= 0, 1.0, M.sigmoid(x64) * (1 - M.sigmoid(x64)))
    assert relerr(dz, rdz) <= TOL_F32 and relerr(dx, rdx) <= TOL_F32
