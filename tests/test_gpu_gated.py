"""GPU parity of gated linear attention (the Mamba cell's algebra), forward and backward, through
the C ABI against the oracle (NumPy recurrence, torch-fp64 autograd for the gradients)."""
import numpy as np
import pytest
import torch

from oracle import grad as G
from oracle import memoroid as M
from gpu_util import TOL_BF16, TOL_F32, attn_inputs, bf16_round, dev, relerr

pytestmark = pytest.mark.gpu

SHAPES = [(1, 64, 1), (2, 128, 2), (1, 1, 1), (2, 7, 1), (1, 65, 2), (2, 200, 3), (1, 33, 1)]


def _inputs(B, T, H, p, seed, dtype, strong=False):
    x = attn_inputs(B, T, H, p=p, seed=seed, scale=1.0 / 8)
    rng = np.random.default_rng(seed + 99)
    x["g"] = (-np.abs(rng.standard_normal((B, T, H))) * (3.0 if strong else 0.2)).astype(np.float32)
    if dtype == "bf16":
        for n in ("q", "k", "v"):
            x[n] = bf16_round(x[n])
    return x


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.05])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("fmap", [0, 1])
def test_gated_linear_attention_fwd(shape, p, dtype, fmap):
    from memorax_amd import kernels as K
    B, T, H = shape
    x = _inputs(B, T, H, p, B * 100 + T + H, dtype)
    print(f"case gla_fwd shape={shape} p={p} dtype={dtype} fmap={fmap}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    o, Sl, chk = K.gated_linear_attn_fwd(dev(x["q"], td), dev(x["k"], td), dev(x["v"], td), dev(x["g"]),
                                         dev(x["done"]), dev(x["S0"]), fmap)
    ro, rSl = M.gated_linear_attention(x["q"], x["k"], x["v"], x["g"], x["done"], x["S0"], "elu1" if fmap else "none")
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    assert relerr(o, ro) <= tol, relerr(o, ro)
    assert relerr(Sl, rSl) <= tol, relerr(Sl, rSl)


def test_gated_strong_decay_and_zero_decay():
    """Log-decays down to about -10 per step (exp(G) underflows inside a chunk) stay finite and
    accurate; g = 0 reproduces plain linear attention bit for bit."""
    from memorax_amd import kernels as K
    B, T, H = 2, 150, 2
    x = _inputs(B, T, H, 0.02, 7, "f32", strong=True)
    args = [dev(x[n]) for n in ("q", "k", "v")]
    o, Sl, _ = K.gated_linear_attn_fwd(*args, dev(x["g"]), dev(x["done"]), dev(x["S0"]), 0)
    ro, rSl = M.gated_linear_attention(x["q"], x["k"], x["v"], x["g"], x["done"], x["S0"])
    assert torch.isfinite(o).all() and relerr(o, ro) <= TOL_F32 and relerr(Sl, rSl) <= TOL_F32
    o0, S0l, _ = K.gated_linear_attn_fwd(*args, torch.zeros((B, T, H), device="cuda"), dev(x["done"]), dev(x["S0"]), 0)
    o1, S1l, _ = K.linear_attn_fwd(*args, dev(x["done"]), dev(x["S0"]), 0)
    assert torch.equal(o0, o1) and torch.equal(S0l, S1l)


@pytest.mark.parametrize("shape", [(1, 64, 1), (2, 100, 2), (1, 1, 1), (2, 7, 1), (1, 130, 2)])
@pytest.mark.parametrize("p", [0.0, 0.06])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("fmap", [0, 1])
def test_gated_linear_attention_bwd(shape, p, dtype, fmap):
    from memorax_amd import kernels as K
    B, T, H = shape
    x = _inputs(B, T, H, p, B * 10 + T + H + 3, dtype)
    rng = np.random.default_rng(5)
    do = (rng.standard_normal(x["v"].shape) / 8).astype(np.float32)
    dSl = (rng.standard_normal(x["S0"].shape) * 0.1).astype(np.float32)
    if dtype == "bf16":
        do = bf16_round(do)
    print(f"case gla_bwd shape={shape} p={p} dtype={dtype} fmap={fmap}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    q, k, v, g, dn, S0 = dev(x["q"], td), dev(x["k"], td), dev(x["v"], td), dev(x["g"]), dev(x["done"]), dev(x["S0"])
    o, Sl, chk = K.gated_linear_attn_fwd(q, k, v, g, dn, S0, fmap)
    dq, dk, dv, dg, dS0 = K.gated_linear_attn_bwd(q, k, v, g, dn, chk, dev(do, td), dev(dSl), fmap, S_last=Sl)
    r = G.gated_linear_attention_grads(x["q"], x["k"], x["v"], x["g"], x["done"], x["S0"], do, dSl,
                                       "elu1" if fmap else "none")
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    for name, got in (("dq", dq), ("dk", dk), ("dv", dv), ("dS0", dS0)):
        assert relerr(got, r[name]) <= tol, (name, relerr(got, r[name]))
    # dg_t is a sum of differences q.dq - k.dk whose diagonal parts cancel: the error scales with
    # the terms, not with the result
    terms = np.abs((x["q"] * r["dq"]).sum(-1)) + np.abs((x["k"] * r["dk"]).sum(-1))
    scale = np.abs(r["dg"]).max() + terms.max()
    err = np.abs(dg.float().cpu().numpy() - r["dg"]).max() / scale
    assert err <= (tol if dtype == "bf16" else 5 * tol), ("dg", err)


def test_gated_autograd_function_and_split_invariance():
    from memorax_amd import gated_linear_attention
    B, T, H = 2, 96, 2
    x = _inputs(B, T, H, 0.03, 21, "f32")
    q, k, v, g = (dev(x[n]).requires_grad_(True) for n in ("q", "k", "v", "g"))
    dn, S0 = dev(x["done"]), dev(x["S0"]).requires_grad_(True)
    o, Sl = gated_linear_attention(q, k, v, g, dn, S0, "elu1")
    do = torch.randn_like(o) / 8
    dSl = torch.randn_like(Sl) * 0.1
    ((o * do).sum() + (Sl * dSl).sum()).backward()
    r = G.gated_linear_attention_grads(x["q"], x["k"], x["v"], x["g"], x["done"], x["S0"],
                                       do.cpu().numpy(), dSl.cpu().numpy(), "elu1")
    for name, t in (("dq", q), ("dk", k), ("dv", v), ("dg", g), ("dS0", S0)):
        assert relerr(t.grad, r[name]) <= 5 * TOL_F32, (name, relerr(t.grad, r[name]))
    with torch.no_grad():
        o1, S1 = gated_linear_attention(q[:, :40], k[:, :40], v[:, :40], g[:, :40], dn[:, :40], S0, "elu1")
        o2, S2 = gated_linear_attention(q[:, 40:], k[:, 40:], v[:, 40:], g[:, 40:], dn[:, 40:], S1, "elu1")
    assert relerr(torch.cat([o1, o2], 1), o.detach().cpu().numpy()) <= TOL_F32
    assert relerr(S2, Sl.detach().cpu().numpy()) <= TOL_F32


def test_gated_poison_does_not_cross_episodes():
    """NaN in one episode (inputs, log-decays, output gradient) leaves every other episode's
    outputs and gradients bit-identical, including dg (reverse reset-aware sum of the row dots)."""
    from memorax_amd import kernels as K
    B, T, H = 1, 200, 2
    x = attn_inputs(B, T, H, p=0.0, seed=17, scale=1.0 / 8)
    rng = np.random.default_rng(18)
    g = (-np.abs(rng.standard_normal((B, T, H))) * 0.1).astype(np.float32)
    do = rng.standard_normal((B, T, H, 64)).astype(np.float32)
    dSl = (rng.standard_normal((B, H, 64, 64)) * 0.1).astype(np.float32)
    done = np.zeros((B, T), bool)
    done[0, 70] = True
    done[0, 130] = True
    clean = dict(q=dev(x["q"]), k=dev(x["k"]), v=dev(x["v"]), g=dev(g), do=dev(do))
    bad = {n: t.clone() for n, t in clean.items()}
    for n in bad:
        bad[n][0, 70:130] = float("nan")
    outs = []
    for inp in (clean, bad):
        o, Sl, chk = K.gated_linear_attn_fwd(inp["q"], inp["k"], inp["v"], inp["g"], dev(done), dev(x["S0"]), 1)
        gr = K.gated_linear_attn_bwd(inp["q"], inp["k"], inp["v"], inp["g"], dev(done), chk, inp["do"], dev(dSl), 1,
                                     S_last=Sl)
        outs.append((o, Sl) + tuple(gr))
    keep = np.ones(T, bool)
    keep[70:130] = False
    for name, a, b_ in zip(("o", "S_last", "dq", "dk", "dv", "dg", "dS0"), outs[0], outs[1]):
        if a.dim() >= 3 and a.shape[1] == T:
            a, b_ = a[:, keep], b_[:, keep]
        assert torch.equal(a, b_), name


def test_gated_with_zero_log_decay_is_linear_attention_at_full_size():
    """Size-independent property at configuration 3's per-sequence shape: g = 0 reduces the gated
    kernels to the plain ones (same products, decay factors exactly 1)."""
    from memorax_amd import kernels as K
    B, T, H = 8, 4096, 8
    gen = torch.Generator(device="cuda").manual_seed(12)
    bf = torch.bfloat16
    q, k, v, do = (torch.randn((B, T, H, 64), device="cuda", generator=gen).div_(8).to(bf) for _ in range(4))
    done = torch.rand((B, T), device="cuda", generator=gen) < 0.002
    g0 = torch.zeros((B, T, H), device="cuda")
    o, Sl, chk = K.gated_linear_attn_fwd(q, k, v, g0, done, None, 1)
    dq, dk, dv, dg, _ = K.gated_linear_attn_bwd(q, k, v, g0, done, chk, do, None, 1, want_dS0=False)
    o2, Sl2, chk2 = K.linear_attn_fwd(q, k, v, done, None, 1)
    dq2, dk2, dv2, _ = K.linear_attn_bwd(q, k, v, done, chk2, do, None, 1, want_dS0=False)
    assert relerr(Sl, Sl2.cpu().numpy()) <= 1e-5
    # bf16 outputs: the gated kernels add the two terms of dV and dK in the other order, so a result may
    # round to the neighbouring bf16 value (2^-8 relative); and their backward takes the state entering
    # a chunk from a bf16 checkpoint where the plain kernel walks it back in fp32 (another 2^-9 on dq)
    for a, b_ in ((o, o2), (dq, dq2), (dk, dk2), (dv, dv2)):
        assert relerr(a, b_.float().cpu().numpy()) <= 2.0 ** -7
    assert torch.isfinite(dg).all()
