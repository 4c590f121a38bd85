"""Host logic that maps other head dims onto what the kernels take: d_k = d_v = 64 or 32, and for the
linear-attention family any narrower head of whole 16-byte segments (CPU: the oracle recurrences stand in
for the kernels, so the test pins the padding/blocking algebra itself)."""
import numpy as np
import pytest
import torch

from oracle import grad as G
from memorax_amd.functional import _Heads


def _rand(*s, seed=0):
    return torch.from_numpy(np.random.default_rng(seed).standard_normal(s))


@pytest.mark.parametrize("dk,dv", [(16, 16), (32, 64), (64, 96), (16, 130), (64, 64), (32, 32), (33, 20), (24, 8), (15, 16), (16, 31),
                                   (128, 64), (96, 40), (130, 130), (48, 48), (40, 64), (64, 24)])
@pytest.mark.parametrize("op", ["linear", "normalised", "gated", "delta"])
def test_padding_and_value_blocks_reproduce_the_native_recurrence(dk, dv, op):
    B, T, H = 2, 9, 2
    q, k, v = _rand(B, T, H, dk, seed=1), _rand(B, T, H, dk, seed=2), _rand(B, T, H, dv, seed=3)
    S0, z0 = _rand(B, H, dv, dk, seed=4), _rand(B, H, dk, seed=5).abs()
    g, beta = -_rand(B, T, H, seed=6).abs() * 0.3, torch.sigmoid(_rand(B, T, H, seed=7))
    done = torch.from_numpy(np.random.default_rng(8).random((B, T)) < 0.2)
    fm = "none" if op == "delta" else "elu1"
    narrow = True  # the kernels take narrower heads as they are
    split_k = op in ("linear", "gated")  # outputs linear in the state: key features beyond 64 run as further blocks
    if dk > 64 and not split_k:
        with pytest.raises(ValueError):
            _Heads(q, v, 0 if op == "delta" else 1, narrow=narrow, split_k=split_k)
        return
    hd = _Heads(q, v, 0 if op == "delta" else 1, narrow=narrow, split_k=split_k)
    w = 32 if dk <= 32 else 64  # the 32-wide kernels serve keys of up to 32 features
    seg = 16 // q.element_size()
    kw = dk if narrow and dk <= w and dk % seg == 0 else w
    vw = dv if narrow and dv <= w and dv % seg == 0 else w
    nkb = -(-dk // kw)
    assert hd.hd == w and (hd.kw, hd.vw) == (kw, vw) and hd.native == (dk == kw and dv == vw)
    assert hd.nb == -(-dv // vw) and hd.nkb == nkb and (nkb == 1 or dk > 64)
    kfm = "elu1" if hd.fmap else "none"   # the feature map the kernel would be asked to apply
    qq, kk, vv, SS = hd.qk(q), hd.qk(k), hd.v(v), hd.state_in(S0)
    nh = H * hd.nb * nkb
    assert qq.shape == (B, T, nh, kw) and vv.shape == (B, T, nh, vw) and SS.shape == (B, nh, vw, kw)
    if op == "linear":
        o, Sl = G.linear_attention_t(qq, kk, vv, done, SS, kfm)
        ro, rS = G.linear_attention_t(q, k, v, done, S0, fm)
    elif op == "normalised":
        o, Sl, zl = G.normalised_linear_attention_t(qq, kk, vv, done, SS, hd.z_in(z0), kfm)
        ro, rS, rz = G.normalised_linear_attention_t(q, k, v, done, S0, z0, fm)
        np.testing.assert_allclose(hd.z_out(zl).numpy(), rz.numpy(), rtol=1e-12, atol=1e-12)
    elif op == "gated":
        o, Sl = G.gated_linear_attention_t(qq, kk, vv, hd.per_head(g), done, SS, kfm)
        ro, rS = G.gated_linear_attention_t(q, k, v, g, done, S0, fm)
    else:
        o, Sl = G.delta_rule_t(qq, kk, vv, hd.per_head(beta), done, SS)
        ro, rS = G.delta_rule_t(q, k, v, beta, done, S0)
    np.testing.assert_allclose(hd.out(o).numpy(), ro.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(hd.state_out(Sl).numpy(), rS.numpy(), rtol=1e-12, atol=1e-12)


def test_key_dim_above_the_kernel_head_dim_is_refused():
    with pytest.raises(ValueError):
        _Heads(torch.zeros(1, 1, 1, 65), torch.zeros(1, 1, 1, 64))
