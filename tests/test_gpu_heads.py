"""GPU parity of the differentiable ops at head dims other than the kernels' own (zero-padded
keys, value blocks and key blocks as extra heads) against the oracle at the native dims."""
import numpy as np
import pytest
import torch

from oracle import grad as G
from gpu_util import TOL_BF16, TOL_F32, bf16_round, dev, relerr

pytestmark = pytest.mark.gpu


def _data(B, T, H, dk, dv, seed, dtype):
    r = np.random.default_rng(seed)
    x = dict(q=r.standard_normal((B, T, H, dk)) / np.sqrt(dk), k=r.standard_normal((B, T, H, dk)) / np.sqrt(dk),
             v=r.standard_normal((B, T, H, dv)), do=r.standard_normal((B, T, H, dv)),
             S0=r.standard_normal((B, H, dv, dk)) * 0.1, z0=np.abs(r.standard_normal((B, H, dk))),
             g=-np.abs(r.standard_normal((B, T, H))) * 0.2, beta=1 / (1 + np.exp(-r.standard_normal((B, T, H)))),
             dSl=r.standard_normal((B, H, dv, dk)) * 0.1)
    x = {n: a.astype(np.float32) for n, a in x.items()}
    x["done"] = r.random((B, T)) < 0.04
    if dtype == "bf16":
        for n in ("q", "k", "v", "do", "beta"):
            x[n] = bf16_round(x[n])
    return x


@pytest.mark.parametrize("dk,dv", [(16, 16), (32, 32), (64, 128), (16, 80)])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("op", ["linear", "normalised", "gated", "delta"])
def test_other_head_dims(dk, dv, dtype, op):
    from memorax_amd import functional as F
    B, T, H = 2, 75, 2
    x = _data(B, T, H, dk, dv, dk * 7 + dv, dtype)
    print(f"case heads op={op} dk={dk} dv={dv} dtype={dtype}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    if op == "delta":
        x["k"] = x["k"] / np.linalg.norm(x["k"], axis=-1, keepdims=True)
        if dtype == "bf16":
            x["k"] = bf16_round(x["k"])
    q, k, v = (dev(x[n], td).requires_grad_() for n in ("q", "k", "v"))
    S0 = dev(x["S0"]).requires_grad_()
    done = dev(x["done"])
    extra = {}
    if op == "linear":
        o, Sl = F.linear_attention(q, k, v, done, S0, "elu1")
        ref = G.linear_attention_grads(x["q"], x["k"], x["v"], x["done"], x["S0"], x["do"], x["dSl"], "elu1")
    elif op == "normalised":
        z0 = dev(x["z0"]).requires_grad_()
        o, Sl, zl = F.normalised_linear_attention(q, k, v, done, S0, z0, "elu1", 1e-6)
        ref = G.normalised_linear_attention_grads(x["q"], x["k"], x["v"], x["done"], x["S0"], x["z0"], x["do"],
                                                  x["dSl"], None, "elu1", 1e-6)
        extra = {"dz0": z0}
        assert zl.shape == (B, H, dk) and relerr(zl, ref["z_last"]) <= (1e-5 if dtype == "f32" else TOL_BF16)
    elif op == "gated":
        g = dev(x["g"]).requires_grad_()
        o, Sl = F.gated_linear_attention(q, k, v, g, done, S0, "elu1")
        ref = G.gated_linear_attention_grads(x["q"], x["k"], x["v"], x["g"], x["done"], x["S0"], x["do"], x["dSl"], "elu1")
        extra = {"dg": g}
    else:
        beta = dev(x["beta"], td).requires_grad_()
        o, Sl = F.delta_rule(q, k, v, beta, done, S0)
        ref = G.delta_rule_grads(x["q"], x["k"], x["v"], x["beta"], x["done"], x["S0"], x["do"], x["dSl"])
        extra = {"dbeta": beta}
    assert o.shape == (B, T, H, dv) and Sl.shape == (B, H, dv, dk)
    ((o.float() * dev(x["do"])).sum() + (Sl * dev(x["dSl"])).sum()).backward()
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    errs = {"o": relerr(o, ref["o"]), "S_last": relerr(Sl, ref["S_last"])}
    for n, t in dict(dq=q, dk=k, dv=v, dS0=S0, **extra).items():
        assert t.grad.shape == t.shape
        errs[n] = relerr(t.grad, ref[n])
    assert all(e <= tol for e in errs.values()), errs


@pytest.mark.parametrize("dk,dv", [(128, 64), (96, 40), (130, 16)])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("op", ["linear", "gated"])
def test_key_dims_above_64_run_as_key_blocks_whose_outputs_add_up(dk, dv, dtype, op):
    """o = sum over 64-wide key blocks of S[:, block] q[block]: plain and gated linear attention, outputs,
    state and every gradient against the oracle at the native dims."""
    from memorax_amd import functional as F
    B, T, H = 2, 75, 2
    x = _data(B, T, H, dk, dv, dk * 3 + dv, dtype)
    print(f"case key blocks op={op} dk={dk} dv={dv} dtype={dtype}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    q, k, v = (dev(x[n], td).requires_grad_() for n in ("q", "k", "v"))
    S0 = dev(x["S0"]).requires_grad_()
    done = dev(x["done"])
    extra = {}
    if op == "linear":
        o, Sl = F.linear_attention(q, k, v, done, S0, "elu1")
        ref = G.linear_attention_grads(x["q"], x["k"], x["v"], x["done"], x["S0"], x["do"], x["dSl"], "elu1")
    else:
        g = dev(x["g"]).requires_grad_()
        o, Sl = F.gated_linear_attention(q, k, v, g, done, S0, "elu1")
        ref = G.gated_linear_attention_grads(x["q"], x["k"], x["v"], x["g"], x["done"], x["S0"], x["do"], x["dSl"], "elu1")
        extra = {"dg": g}
    assert o.shape == (B, T, H, dv) and Sl.shape == (B, H, dv, dk)
    ((o.float() * dev(x["do"])).sum() + (Sl * dev(x["dSl"])).sum()).backward()
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    errs = {"o": relerr(o, ref["o"]), "S_last": relerr(Sl, ref["S_last"])}
    for n, t in dict(dq=q, dk=k, dv=v, dS0=S0, **extra).items():
        assert t.grad.shape == t.shape
        errs[n] = relerr(t.grad, ref[n])
    assert all(e <= tol for e in errs.values()), errs
    with pytest.raises(ValueError):  # the normalised read-out and the delta rule couple the key features
        F.normalised_linear_attention(q, k, v, done, None, None, "elu1", 1e-6)
    with pytest.raises(ValueError):
        F.delta_rule(q, k, v, dev(x["beta"], td), done, None)


def test_linear_attention_model_at_the_reference_guides_head_dim():
    """LinearAttentionCell(features=64, num_heads=4, head_dim=16), the configuration of the
    reference's guide (docs/source/guides/sequence_models.md:128)."""
    from memorax_amd import sequence_models as sm
    from oracle import memoroid as M
    torch.manual_seed(0)
    B, T, Fe, H, d = 2, 40, 64, 4, 16
    cell = sm.LinearAttentionCell(Fe, d, H).cuda()
    model = sm.LinearAttention(cell)
    x = torch.randn(B, T, Fe, device="cuda")
    done = torch.rand(B, T, device="cuda") < 0.05
    carry, y = model(x, done)
    assert carry[0].shape == (B, 1, H, d, d) and carry[1].shape == (B, 1, H, d)
    npf = lambda t: t.detach().double().cpu().numpy()  # noqa: E731
    hv = lambda t: npf(t).reshape(B, T, H, d)          # noqa: E731
    ro, rden, rS, rz = M.normalised_linear_attention(hv(cell.query(x)), hv(cell.key(x)), hv(cell.value(x)),
                                                     npf(done.float()), None, None, "elu1", 1e-6)
    out = ro.reshape(B, T, H * d)
    out = out / np.sqrt((out ** 2).mean(-1, keepdims=True) + 1e-6) * npf(cell.norm.scale)
    ry = out @ npf(cell.output_projection.weight).T + npf(cell.output_projection.bias)
    assert relerr(y, ry) <= 2e-4
    assert relerr(carry[0][:, 0], rS) <= 1e-4 and relerr(carry[1][:, 0], rz) <= 1e-4
    # acting from the carried state: one step (T = 1, no gradients)
    with torch.no_grad():
        c2, y2 = model(x[:, :1], done[:, :1], carry)
    assert c2[0].shape == carry[0].shape and torch.isfinite(y2).all()
    y.pow(2).mean().backward()
    assert cell.key.weight.grad.abs().sum() > 0


def test_extra_leading_axes_fold_into_the_batch():
    """What jax.vmap over seeds adds around the reference's calls: a leading axis on every argument."""
    import memorax_amd as mx
    g = torch.Generator(device="cuda").manual_seed(0)
    S, B, T, H, d = 3, 2, 70, 2, 64
    q, k, v = (torch.randn((S, B, T, H, d), device="cuda", generator=g) / 8 for _ in range(3))
    beta = torch.rand((S, B, T, H), device="cuda", generator=g)
    done = torch.rand((S, B, T), device="cuda", generator=g) < 0.05
    S0 = torch.randn((S, B, H, d, d), device="cuda", generator=g) * 0.1
    kn = torch.nn.functional.normalize(k, dim=-1)
    o, Sl = mx.delta_rule(q, kn, v, beta, done, S0)
    assert o.shape == (S, B, T, H, d) and Sl.shape == (S, B, H, d, d)
    for s in range(S):
        o1, S1 = mx.delta_rule(q[s], kn[s], v[s], beta[s], done[s], S0[s])
        assert torch.equal(o[s], o1) and torch.equal(Sl[s], S1)
    o, Sl = mx.linear_attention(q, k, v, done, None, "elu1")
    o1, S1 = mx.linear_attention(q[1], k[1], v[1], done[1], None, "elu1")
    assert torch.equal(o[1], o1) and torch.equal(Sl[1], S1)
    a = torch.rand((S, B, T, 48), device="cuda", generator=g) * 0.1 + 0.9
    b = torch.randn((S, B, T, 48), device="cuda", generator=g).requires_grad_()
    lam = torch.rand((48,), device="cuda", generator=g)     # a time-invariant decay carries no leading axes
    h, hl, Pl = mx.linear_scan(a, b, done)
    h1, hl1, _ = mx.linear_scan(a[2], b[2], done[2])
    assert h.shape == (S, B, T, 48) and torch.equal(h[2], h1) and torch.equal(hl[2], hl1)
    h, _, _ = mx.linear_scan(lam, b, done)
    h2, _, _ = mx.linear_scan(lam, b[0], done[0])
    assert torch.equal(h[0], h2)
    h.sum().backward()
    assert b.grad.shape == b.shape
    hm, _, _ = mx.mingru_scan(a, b.detach(), done)
    hm1, _, _ = mx.mingru_scan(a[1], b.detach()[1], done[1])
    assert torch.equal(hm[1], hm1)
