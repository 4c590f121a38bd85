"""Tensors of more than 2^31 elements: element offsets of the last batch rows do not fit 32 bits
(byte offsets do not fit 32 bits long before that).  Each kernel family runs once at such a size
through the C ABI and its last two batch rows are compared with the oracle."""
import numpy as np
import pytest
import torch

from oracle import clib
from oracle import memoroid as M
from gpu_util import TOL_BF16, TOL_F32, relerr

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
NB = 2  # batch rows compared with the oracle: the last ones


def _rows(t):
    return t[-NB:].float().cpu().numpy()


def test_delta_rule_beyond_32_bit_offsets():
    from memorax_amd import kernels as K
    B, T, H = 528, 8192, 8
    assert (B - NB) * T * H * 64 > 2**31
    g = torch.Generator(device="cuda").manual_seed(31)
    print("case large offsets delta rule", (B, T, H), flush=True)
    q, v, do = (torch.randn((B, T, H, 64), device="cuda", generator=g).to(BF) for _ in range(3))
    k = torch.nn.functional.normalize(torch.randn((B, T, H, 64), device="cuda", generator=g), dim=-1).to(BF)
    beta = torch.sigmoid(torch.randn((B, T, H), device="cuda", generator=g)).to(BF)
    done = torch.rand((B, T), device="cuda", generator=g) < 0.002
    o, Sl, chk = K.delta_rule_fwd(q, k, v, beta, done)
    got = K.delta_rule_bwd(q, k, v, beta, done, chk, do)
    torch.cuda.synchronize()
    xs = [_rows(t) for t in (q, k, v, beta)]
    dn = done[-NB:].cpu().numpy()
    ro, rSl = clib.delta_rule_fwd(*xs, dn)
    ref = clib.delta_rule_bwd(*xs, dn, None, _rows(do))
    errs = {"o": relerr(o[-NB:], ro), "S_last": relerr(Sl[-NB:], rSl)}
    errs.update({n: relerr(u[-NB:], r) for n, u, r in zip(("dq", "dk", "dv", "dbeta", "dS0"), got, ref)})
    assert all(e <= TOL_BF16 for e in errs.values()), errs


def test_linear_attention_beyond_32_bit_offsets():
    from memorax_amd import kernels as K
    B, T, H = 528, 8192, 8
    g = torch.Generator(device="cuda").manual_seed(32)
    print("case large offsets linear attention", (B, T, H), flush=True)
    q, k, v, do = ((torch.randn((B, T, H, 64), device="cuda", generator=g) / 8).to(BF) for _ in range(4))
    done = torch.rand((B, T), device="cuda", generator=g) < 0.002
    o, Sl, chk = K.linear_attn_fwd(q, k, v, done, None, 1)
    got = K.linear_attn_bwd(q, k, v, done, chk, do, None, 1)
    torch.cuda.synchronize()
    xs = [_rows(t) for t in (q, k, v)]
    dn = done[-NB:].cpu().numpy()
    ro, rSl = clib.linear_attn_fwd(*xs, dn, None, 1)
    ref = clib.linear_attn_bwd(*xs, dn, None, _rows(do), None, 1)
    errs = {"o": relerr(o[-NB:], ro), "S_last": relerr(Sl[-NB:], rSl)}
    errs.update({n: relerr(u[-NB:], r) for n, u, r in zip(("dq", "dk", "dv", "dS0"), got, ref)})
    assert all(e <= TOL_BF16 for e in errs.values()), errs


def test_diagonal_scan_beyond_32_bit_offsets():
    from memorax_amd import kernels as K
    B, T, D = 520, 1024, 4096
    assert (B - NB) * T * D > 2**31
    g = torch.Generator(device="cuda").manual_seed(33)
    print("case large offsets scan", (B, T, D), flush=True)
    a = torch.rand((B, T, D), device="cuda", generator=g) * 0.099 + 0.9
    b = torch.randn((B, T, D), device="cuda", generator=g)
    gr = torch.randn((B, T, D), device="cuda", generator=g)
    done = torch.rand((B, T), device="cuda", generator=g) < 0.002
    h, hl, Pl = K.linear_scan_fwd(a, b, done)
    da, db, _ = K.linear_scan_bwd(a, h, done, None, gr, None)
    last = K.linear_scan_last(a, b, done)
    torch.cuda.synchronize()
    an, bn, gn, dn = _rows(a), _rows(b), _rows(gr), done[-NB:].cpu().numpy()
    rh, rhl, rPl = M.diag_scan(an, bn, dn)
    rda, rdb, _ = M.diag_scan_bwd(an, rh, dn, gn)
    errs = {"h": relerr(h[-NB:], rh), "h_last": relerr(hl[-NB:], rhl), "P_last": relerr(Pl[-NB:], rPl),
            "da": relerr(da[-NB:], rda), "db": relerr(db[-NB:], rdb), "last": relerr(last[-NB:], rhl)}
    assert all(e <= TOL_F32 for e in errs.values()), errs


def test_delta_rule_sequence_longer_than_the_factor_kernel_covers():
    """One sequence of more steps than the chunk-parallel factor kernel's grid covers: the call falls
    back to the in-kernel inverse instead of failing, and since the recurrence is causal its first
    steps equal a call on those steps alone (same kernel, bit for bit)."""
    from memorax_amd import kernels as K
    T, n = 4 * 65535 * 32 + 32, 2048
    g = torch.Generator(device="cuda").manual_seed(34)
    print("case long sequence delta rule", T, flush=True)
    q, v = (torch.randn((1, T, 1, 64), device="cuda", generator=g).to(BF) for _ in range(2))
    k = torch.nn.functional.normalize(torch.randn((1, T, 1, 64), device="cuda", generator=g), dim=-1).to(BF)
    beta = torch.sigmoid(torch.randn((1, T, 1), device="cuda", generator=g)).to(BF)
    done = torch.rand((1, T), device="cuda", generator=g) < 0.002
    o, Sl, chk = K.delta_rule_fwd(q, k, v, beta, done)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(o.float()).all()) and bool(torch.isfinite(Sl).all())
    o1, _, _ = K.delta_rule_fwd(q[:, :n].contiguous(), k[:, :n].contiguous(), v[:, :n].contiguous(),
                                beta[:, :n].contiguous(), done[:, :n].contiguous(), save_chk=False, tm_scratch=False)
    assert torch.equal(o[:, :n], o1)
