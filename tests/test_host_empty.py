"""No sequences (B = 0) or no time steps (T = 0): the reference's scan hands the carry back unchanged
(memoroid.py:60-91 scans the carry prepended to zero elements), and so do the differentiable ops --
without launching anything, which is why this runs on the CPU."""
import pytest
import torch

from memorax_amd import functional as F


@pytest.mark.parametrize("B,T", [(0, 5), (3, 0)])
def test_bf16_scans_without_steps_carry_float32_like_the_kernels(B, T):
    D = 8
    a, b = torch.rand(B, T, D).bfloat16(), torch.randn(B, T, D).bfloat16()
    done = torch.zeros(B, T, dtype=torch.bool)
    for op in (F.linear_scan, F.mingru_scan):
        h, h_last, P_last = op(a, b, done)
        assert h.dtype == torch.bfloat16 and h_last.dtype == torch.float32 and P_last.dtype == torch.float32
        h0, P0 = torch.randn(B, D), torch.rand(B, D)
        h, h_last, P_last = op(a, b, done, h0, P0)
        assert h_last.dtype == torch.float32 and torch.equal(h_last, h0) and torch.equal(P_last, P0)


@pytest.mark.parametrize("B,T", [(0, 5), (3, 0), (0, 0)])
def test_scans_without_steps_return_the_carry(B, T):
    D = 6
    a, b = torch.rand(B, T, D), torch.randn(B, T, D)
    done = torch.zeros(B, T, dtype=torch.bool)
    h0, P0 = torch.randn(B, D, requires_grad=True), torch.rand(B, D)
    for op in (F.linear_scan, F.mingru_scan):
        h, h_last, P_last = op(a, b, done, h0, P0)
        assert h.shape == (B, T, D) and torch.equal(h_last, h0) and torch.equal(P_last, P0)
        h_last.sum().backward()
        assert torch.equal(h0.grad, torch.ones_like(h0))
        h0.grad = None
        h, h_last, P_last = op(a, b, done)
        assert h_last.shape == (B, D) and not h_last.any() and P_last.shape == (B, D) and (P_last == 1).all()


@pytest.mark.parametrize("B,T", [(0, 5), (3, 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_ops_without_steps_return_the_state(B, T, dtype):
    H, dk, dv = 2, 16, 24
    q, k, v = torch.randn(B, T, H, dk).to(dtype), torch.randn(B, T, H, dk).to(dtype), torch.randn(B, T, H, dv).to(dtype)
    g, beta = -torch.rand(B, T, H), torch.rand(B, T, H).to(dtype)
    done = torch.zeros(B, T, dtype=torch.bool)
    S0 = torch.randn(B, H, dv, dk, requires_grad=True)
    z0 = torch.rand(B, H, dk)
    calls = [lambda S: F.linear_attention(q, k, v, done, S, "elu1"),
             lambda S: F.gated_linear_attention(q, k, v, g, done, S),
             lambda S: F.delta_rule(q, k, v, beta, done, S),
             lambda S: F.deltanet(q, k, v, beta, done, S),
             lambda S: F.normalised_linear_attention(q, k, v, done, S, z0)[:2]]
    for call in calls:
        o, S_last = call(S0)
        assert o.shape == (B, T, H, dv) and o.dtype == dtype
        assert S_last.dtype == torch.float32 and torch.equal(S_last, S0)
        S_last.sum().backward()
        assert torch.equal(S0.grad, torch.ones_like(S0))
        S0.grad = None
        o, S_last = call(None)
        assert S_last.shape == (B, H, dv, dk) and not S_last.any()
    o, S_last, z_last = F.normalised_linear_attention(q, k, v, done, S0, z0)
    assert torch.equal(z_last, z0)
    assert F.normalised_linear_attention(q, k, v, done)[2].shape == (B, H, dk)


def test_sensitivities_without_steps_are_unchanged():
    B, T, H = 2, 0, 3
    sens = {"w": torch.randn(B, 1, H, 4)}
    out = F.propagate_sensitivities(torch.rand(B, T, H), {"w": torch.randn(B, T, H, 4)}, sens, torch.zeros(B, T, dtype=torch.bool))
    assert torch.equal(out["w"], sens["w"])
