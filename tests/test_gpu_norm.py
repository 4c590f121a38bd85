"""GPU parity of linear attention with the fused normalised read-out (through the C ABI)
against the oracle recurrence (forward) and its torch-fp64 autograd (backward)."""
import numpy as np
import pytest
import torch

from oracle import grad as G
from oracle import memoroid as M
from gpu_util import TOL_BF16, TOL_F32, attn_inputs, bf16_round, dev, relerr

pytestmark = pytest.mark.gpu

SHAPES = [(1, 64, 1), (2, 128, 2), (1, 1, 1), (2, 7, 1), (1, 65, 2), (2, 200, 3), (1, 33, 1)]


def _inputs(B, T, H, p, seed, dtype, z_scale=1.0):
    x = attn_inputs(B, T, H, p=p, seed=seed, scale=1.0 / 8)
    rng = np.random.default_rng(seed + 1)
    x["z0"] = (np.abs(rng.standard_normal((B, H, 64))) * z_scale).astype(np.float32)
    x["do"] = rng.standard_normal((B, T, H, 64)).astype(np.float32)
    x["dSl"] = (rng.standard_normal((B, H, 64, 64)) * 0.1).astype(np.float32)
    x["dzl"] = (rng.standard_normal((B, H, 64)) * 0.1).astype(np.float32)
    if dtype == "bf16":
        for n in ("q", "k", "v", "do"):
            x[n] = bf16_round(x[n])
    return x


def _td(dtype):
    return torch.bfloat16 if dtype == "bf16" else torch.float32


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.05])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_normalised_fwd(shape, p, dtype):
    from memorax_amd import kernels as K
    B, T, H = shape
    x = _inputs(B, T, H, p, B * 100 + T + H + 3, dtype)
    print(f"case la_norm_fwd shape={shape} p={p} dtype={dtype}", flush=True)
    td = _td(dtype)
    o, den, Sl, zl, chk = K.linear_attn_norm_fwd(dev(x["q"], td), dev(x["k"], td), dev(x["v"], td), dev(x["done"]),
                                                 dev(x["S0"]), dev(x["z0"]), 1, 1e-6)
    ro, rden, rS, rz = M.normalised_linear_attention(x["q"], x["k"], x["v"], x["done"], x["S0"], x["z0"], "elu1", 1e-6)
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    assert relerr(o, ro) <= tol, relerr(o, ro)
    rden = rden.transpose(0, 2, 1)  # the kernels keep the denominators as (B,H,T)
    assert relerr(den, rden) <= tol, relerr(den, rden)
    assert relerr(Sl, rS) <= (1e-5 if dtype == "f32" else tol)
    assert relerr(zl, rz) <= (1e-5 if dtype == "f32" else tol)
    # the state leaf equals what the un-normalised entry point returns, bit for bit
    _, Sl2, _ = K.linear_attn_fwd(dev(x["q"], td), dev(x["k"], td), dev(x["v"], td), dev(x["done"]), dev(x["S0"]), 1)
    assert torch.equal(Sl, Sl2)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.05])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_normalised_bwd(shape, p, dtype):
    from memorax_amd import kernels as K
    B, T, H = shape
    x = _inputs(B, T, H, p, B * 100 + T + H + 17, dtype)
    print(f"case la_norm_bwd shape={shape} p={p} dtype={dtype}", flush=True)
    td = _td(dtype)
    tq, tk, tv, tdo = (dev(x[n], td) for n in ("q", "k", "v", "do"))
    o, den, Sl, zl, chk = K.linear_attn_norm_fwd(tq, tk, tv, dev(x["done"]), dev(x["S0"]), dev(x["z0"]), 1, 1e-6)
    got = K.linear_attn_norm_bwd(tq, tk, tv, dev(x["done"]), chk, o, den, tdo, dev(x["dSl"]), dev(x["dzl"]), 1, 1e-6)
    ref = G.normalised_linear_attention_grads(x["q"], x["k"], x["v"], x["done"], x["S0"], x["z0"], x["do"],
                                              x["dSl"], x["dzl"], "elu1", 1e-6)
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    errs = {n: relerr(g, ref[n]) for n, g in zip(("dq", "dk", "dv", "dS0", "dz0"), got)}
    assert all(e <= tol for e in errs.values()), errs


@pytest.mark.parametrize("shape", [(2, 128, 2), (1, 65, 2), (2, 200, 3), (1, 1, 1)])
@pytest.mark.parametrize("p", [0.0, 0.05])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_sums_of_squares_out_of_the_epilogue_and_their_gradient(shape, p, dtype):
    """ss[b,h,t] = |o[b,t,h]|^2 written by the forward kernel from its output tile (what the RMS norm
    over the heads, linear_attention.py:114, needs from each head) equals the sum of squares of the
    outputs as stored; and the backward call given d_ss returns the gradients of
    L = <do, o> + <dS_last, S_last> + <dz_last, z_last> + <d_ss, ss> (torch-fp64 autograd)."""
    from memorax_amd import kernels as K
    B, T, H = shape
    x = _inputs(B, T, H, p, B * 100 + T + H + 31, dtype)
    rng = np.random.default_rng(5)
    d_ss = rng.standard_normal((B, T, H)).astype(np.float32)
    print(f"case la_norm_ss shape={shape} p={p} dtype={dtype}", flush=True)
    td = _td(dtype)
    tq, tk, tv, tdo = (dev(x[n], td) for n in ("q", "k", "v", "do"))
    o, den, Sl, zl, chk, ss = K.linear_attn_norm_fwd(tq, tk, tv, dev(x["done"]), dev(x["S0"]), dev(x["z0"]), 1, 1e-6,
                                                     want_ss=True)
    assert ss.shape == (B, H, T) and ss.dtype == torch.float32
    want = o.float().square().sum(-1).transpose(1, 2)      # of the outputs as stored
    assert relerr(ss, want.cpu().numpy()) <= 1e-6
    o2 = K.linear_attn_norm_fwd(tq, tk, tv, dev(x["done"]), dev(x["S0"]), dev(x["z0"]), 1, 1e-6)[0]
    assert torch.equal(o, o2)                              # asking for ss changes nothing else
    got = K.linear_attn_norm_bwd(tq, tk, tv, dev(x["done"]), chk, o, den, tdo, dev(x["dSl"]), dev(x["dzl"]), 1, 1e-6,
                                 d_ss=dev(np.ascontiguousarray(d_ss.transpose(0, 2, 1))))
    ref = G.normalised_linear_attention_grads(x["q"], x["k"], x["v"], x["done"], x["S0"], x["z0"], x["do"],
                                              x["dSl"], x["dzl"], "elu1", 1e-6, d_ss=d_ss)
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    errs = {n: relerr(g, ref[n]) for n, g in zip(("dq", "dk", "dv", "dS0", "dz0"), got)}
    assert all(e <= tol for e in errs.values()), errs
    # d_ss = 0 is the call without it
    z = K.linear_attn_norm_bwd(tq, tk, tv, dev(x["done"]), chk, o, den, tdo, dev(x["dSl"]), dev(x["dzl"]), 1, 1e-6,
                               d_ss=torch.zeros_like(ss))
    n = K.linear_attn_norm_bwd(tq, tk, tv, dev(x["done"]), chk, o, den, tdo, dev(x["dSl"]), dev(x["dzl"]), 1, 1e-6)
    for a, b_ in zip(z, n):
        assert relerr(a, b_.float().cpu().numpy()) <= (4e-3 if dtype == "bf16" else 1e-6)


def test_sums_of_squares_do_not_cross_episodes():
    """A NaN in the outputs of one episode (poisoned values before a reset) leaves ss and every gradient
    of the later episode finite: the d_ss term joins dout by select on live rows only."""
    from memorax_amd import kernels as K
    B, T, H = 1, 96, 1
    x = _inputs(B, T, H, 0.0, 77, "f32")
    x["done"][0, 40] = True
    x["v"][0, 10] = np.nan
    tq, tk, tv, tdo = (dev(x[n]) for n in ("q", "k", "v", "do"))
    o, den, Sl, zl, chk, ss = K.linear_attn_norm_fwd(tq, tk, tv, dev(x["done"]), None, None, 1, 1e-6, want_ss=True)
    assert torch.isfinite(ss[0, 0, 40:]).all() and torch.isnan(ss[0, 0, 10:40]).all()
    d_ss = torch.ones_like(ss)
    got = K.linear_attn_norm_bwd(tq, tk, tv, dev(x["done"]), chk, o, den, tdo, None, None, 1, 1e-6, d_ss=d_ss)
    for g in got[:3]:
        assert torch.isfinite(g[0, 40:]).all()


def test_normalised_clamp_and_plain_feature_map():
    """No feature map, so that denominators of either sign occur: rows under the clamp take
    den = eps and pass no gradient through the denominator.  fp32 only: the seed keeps every
    denominator 1.7e-3 away from the kink, far more than the fp32 kernel's error."""
    from memorax_amd import kernels as K
    B, T, H = 2, 150, 2
    x = _inputs(B, T, H, 0.03, 78, "f32", z_scale=0.05)
    eps = 0.05
    ro, rden, rS, rz = M.normalised_linear_attention(x["q"], x["k"], x["v"], x["done"], x["S0"], x["z0"], "none", eps)
    rden = rden.transpose(0, 2, 1)  # the kernels keep the denominators as (B,H,T)
    frac = float((rden == eps).mean())
    assert 0.3 < frac < 0.7, frac
    tq, tk, tv, tdo = (dev(x[n]) for n in ("q", "k", "v", "do"))
    o, den, Sl, zl, chk = K.linear_attn_norm_fwd(tq, tk, tv, dev(x["done"]), dev(x["S0"]), dev(x["z0"]), 0, eps)
    assert ((den.cpu().numpy() == np.float32(eps)) == (rden == eps)).all()
    assert relerr(den, rden) <= TOL_F32 and relerr(o, ro) <= TOL_F32, (relerr(den, rden), relerr(o, ro))
    got = K.linear_attn_norm_bwd(tq, tk, tv, dev(x["done"]), chk, o, den, tdo, dev(x["dSl"]), dev(x["dzl"]), 0, eps)
    ref = G.normalised_linear_attention_grads(x["q"], x["k"], x["v"], x["done"], x["S0"], x["z0"], x["do"],
                                              x["dSl"], x["dzl"], "none", eps)
    errs = {n: relerr(g, ref[n]) for n, g in zip(("dq", "dk", "dv", "dS0", "dz0"), got)}
    assert all(e <= TOL_F32 for e in errs.values()), errs


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_normalised_fully_clamped_equals_plain_attention_over_eps(dtype):
    """With eps above every denominator the read-out is the un-normalised kernel's divided by eps,
    and z only carries the gradient handed in for z_last."""
    from memorax_amd import kernels as K
    B, T, H = 2, 130, 2
    x = _inputs(B, T, H, 0.03, 31, dtype)
    td = _td(dtype)
    eps = float(2 ** 20)   # a power of two (the division is exact) above every denominator (~64 T)
    tq, tk, tv, tdo = (dev(x[n], td) for n in ("q", "k", "v", "do"))
    dn = dev(x["done"])
    o, den, Sl, zl, chk = K.linear_attn_norm_fwd(tq, tk, tv, dn, dev(x["S0"]), dev(x["z0"]), 1, eps)
    assert (den == eps).all()
    o0, Sl0, chk0 = K.linear_attn_fwd(tq, tk, tv, dn, dev(x["S0"]), 1)
    assert torch.equal(o.float(), o0.float() / eps) and torch.equal(Sl, Sl0)
    got = K.linear_attn_norm_bwd(tq, tk, tv, dn, chk, o, den, tdo, dev(x["dSl"]), dev(x["dzl"]), 1, eps)
    ref = G.normalised_linear_attention_grads(x["q"], x["k"], x["v"], x["done"], x["S0"], x["z0"], x["do"],
                                              x["dSl"], x["dzl"], "elu1", eps)
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    errs = {n: relerr(g, ref[n]) for n, g in zip(("dq", "dk", "dv", "dS0", "dz0"), got)}
    assert all(e <= tol for e in errs.values()), errs


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_normalised_split_invariance(dtype):
    """Two calls chained through the carry (S, z) reproduce one call over the whole sequence."""
    from memorax_amd import kernels as K
    B, T, H = 2, 192, 2
    x = _inputs(B, T, H, 0.02, 5, dtype)
    td = _td(dtype)
    tq, tk, tv = (dev(x[n], td) for n in ("q", "k", "v"))
    dn = dev(x["done"])
    o, den, Sl, zl, _ = K.linear_attn_norm_fwd(tq, tk, tv, dn, dev(x["S0"]), dev(x["z0"]), 1, 1e-6, save_chk=False)
    cut = 128   # a multiple of both chunk sizes: the two calls then do the same arithmetic
    o1, _, S1, z1, _ = K.linear_attn_norm_fwd(tq[:, :cut].contiguous(), tk[:, :cut].contiguous(),
                                              tv[:, :cut].contiguous(), dn[:, :cut].contiguous(),
                                              dev(x["S0"]), dev(x["z0"]), 1, 1e-6, save_chk=False)
    o2, _, S2, z2, _ = K.linear_attn_norm_fwd(tq[:, cut:].contiguous(), tk[:, cut:].contiguous(),
                                              tv[:, cut:].contiguous(), dn[:, cut:].contiguous(), S1, z1, 1, 1e-6,
                                              save_chk=False)
    tol = 1e-5 if dtype == "f32" else TOL_BF16
    assert relerr(torch.cat([o1, o2], 1), o.float().cpu().numpy()) <= tol
    assert relerr(S2, Sl.cpu().numpy()) <= tol and relerr(z2, zl.cpu().numpy()) <= tol


def test_normalised_poison_does_not_cross_episodes():
    """NaN in one episode must not reach another (rows of other episodes are removed by select,
    and their denominators are never divided into live rows)."""
    from memorax_amd import kernels as K
    B, T, H = 1, 100, 1
    x = _inputs(B, T, H, 0.0, 9, "f32")
    done = np.zeros((B, T), bool)
    done[0, 40] = True
    done[0, 70] = True
    clean = {n: dev(x[n]) for n in ("q", "k", "v", "do")}
    bad = {n: t.clone() for n, t in clean.items()}
    for n in ("q", "k", "v", "do"):
        bad[n][0, 40:70] = float("nan")
    outs = []
    for inp in (clean, bad):
        o, den, Sl, zl, chk = K.linear_attn_norm_fwd(inp["q"], inp["k"], inp["v"], dev(done), dev(x["S0"]),
                                                     dev(x["z0"]), 1, 1e-6)
        g = K.linear_attn_norm_bwd(inp["q"], inp["k"], inp["v"], dev(done), chk, o, den, inp["do"], dev(x["dSl"]),
                                   dev(x["dzl"]), 1, 1e-6)
        outs.append((o, Sl, zl) + tuple(g))
    keep = np.ones(T, bool)
    keep[40:70] = False
    for a, b in zip(outs[0], outs[1]):
        if a.dim() == 4 and a.shape[1] == T:
            assert torch.equal(a[:, keep], b[:, keep])
        else:
            assert torch.equal(a, b)
    assert torch.isnan(outs[1][0][0, 40:70]).all()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_normalised_functional_autograd_and_step(dtype):
    from memorax_amd import functional as F
    B, T, H = 2, 70, 2
    x = _inputs(B, T, H, 0.04, 21, dtype)
    td = _td(dtype)
    q, k, v = (dev(x[n], td).requires_grad_() for n in ("q", "k", "v"))
    S0, z0 = dev(x["S0"]).requires_grad_(), dev(x["z0"]).requires_grad_()
    o, Sl, zl = F.normalised_linear_attention(q, k, v, dev(x["done"]), S0, z0, "elu1", 1e-6)
    loss = (o.float() * dev(x["do"])).sum() + (Sl * dev(x["dSl"])).sum() + (zl * dev(x["dzl"])).sum()
    loss.backward()
    ref = G.normalised_linear_attention_grads(x["q"], x["k"], x["v"], x["done"], x["S0"], x["z0"], x["do"],
                                              x["dSl"], x["dzl"], "elu1", 1e-6)
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    errs = {n: relerr(t.grad, ref[n]) for n, t in (("dq", q), ("dk", k), ("dv", v), ("dS0", S0), ("dz0", z0))}
    assert all(e <= tol for e in errs.values()), errs
    assert relerr(o, ref["o"]) <= tol
    # acting: T = 1 without gradients goes through the single-step kernel and agrees with the chunked kernel
    with torch.no_grad():
        q1, k1, v1 = (t.detach()[:, :1].contiguous() for t in (q, k, v))
        d1 = dev(x["done"])[:, :1].contiguous()
        a = F.normalised_linear_attention(q1, k1, v1, d1, S0.detach(), z0.detach(), "elu1", 1e-6)
    from memorax_amd import kernels as K
    b = K.linear_attn_norm_fwd(q1, k1, v1, d1, S0.detach(), z0.detach(), 1, 1e-6, save_chk=False)
    # (bf16: the chunked kernel rounds phi(k) to bf16 before the products, the step kernel does not)
    tol1 = 1e-5 if dtype == "f32" else TOL_BF16
    assert relerr(a[0], b[0].float().cpu().numpy()) <= tol1
    assert relerr(a[1], b[2].cpu().numpy()) <= tol1 and relerr(a[2], b[3].cpu().numpy()) <= tol1


def test_normalised_rejects_bad_arguments():
    from memorax_amd import _lib
    lib = _lib.load()
    t = torch.zeros(64 * 64 * 4, device="cuda")
    p = t.data_ptr()
    fwd = lambda den, dk, dt, ss=None: lib.mrx_linear_attn_norm_fwd(None, p, p, p, p, None, None, p, den, ss, None, None, None,
                                                                    None, 1, 4, 1, dk, 64, dt, 0, 1, 1e-6)
    assert fwd(p, 64, 0) == 0
    assert fwd(None, 64, 0) == -1     # den is required
    assert fwd(p, 72, 0) == -2        # unsupported head dim
    assert fwd(p, 64, 2) == -2        # complex64
    assert fwd(p, 64, 0, p + 2) == -1  # ss must be aligned to its element size
    bwd = lambda zc, dss=None: lib.mrx_linear_attn_norm_bwd(None, p, p, p, p, p, p, zc, p, p, p, dss, None, None, p, p, p,
                                                            None, None, 1, 4, 1, 64, 64, 0, 0, 1, 1e-6)
    assert bwd(None) == -1            # z_chk is required
    assert bwd(p, p + 2) == -1        # d_ss must be aligned to its element size
    torch.cuda.synchronize()


def test_normalised_constant_values_come_back_at_full_size():
    """Size-independent property at configuration 3's per-sequence shape (T = 4096, bf16): without a
    carry the normalised read-out is a convex combination of the episode's values, so values that
    are constant along time come back unchanged, resets or not."""
    from memorax_amd import kernels as K
    B, T, H = 8, 4096, 8
    g = torch.Generator(device="cuda").manual_seed(11)
    bf = torch.bfloat16
    q, k = (torch.randn((B, T, H, 64), device="cuda", generator=g).div_(8).to(bf) for _ in range(2))
    c = torch.randn((B, 1, H, 64), device="cuda", generator=g).to(bf)
    v = c.expand(B, T, H, 64).contiguous()
    done = torch.rand((B, T), device="cuda", generator=g) < 0.002
    o, den, Sl, zl, _ = K.linear_attn_norm_fwd(q, k, v, done, None, None, 1, 1e-6, save_chk=False)
    err = (o.float() - v.float()).abs().max() / v.float().abs().max()
    assert float(err) <= TOL_BF16, float(err)
    assert float(den.min()) > 0.5   # phi > 0: every denominator is at least one key's worth
