"""GPU parity of the linear-attention family on heads narrower than the library's two builds (d_k, d_v <= 32
on the 32-wide kernels, anything else up to 64 on the 64-wide ones; whole 16-byte segments, d_k and d_v
independent): the kernels take such rows as they lie in memory and pad inside; results against the oracle
at the same head dims."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import grad as G
from gpu_util import TOL_BF16, TOL_F32, bf16_round, dev, relerr

pytestmark = pytest.mark.gpu

# (d_k, d_v): the reference guides' head_dim 16, unequal widths either way, one full and one narrow side
DIMS = [(16, 16), (8, 24), (24, 8), (32, 16), (16, 32), (48, 48), (40, 64), (64, 24), (16, 56)]
DIMS_F32_ONLY = [(12, 20), (4, 4)]  # whole 16-byte segments of float32 only
SHAPES = [(3, 1, 2), (2, 65, 1), (2, 200, 3), (1, 1100, 2)]


def _inputs(shape, dk, dv, p, dtype, seed):
    B, T, H = shape
    rng = np.random.default_rng(seed)
    x = {n: (rng.standard_normal((B, T, H, d)) / 4).astype(np.float32)
         for n, d in (("q", dk), ("k", dk), ("v", dv), ("do", dv))}
    x["do"] *= 4
    x["done"] = rng.random((B, T)) < p
    x["S0"] = (rng.standard_normal((B, H, dv, dk)) * 0.1).astype(np.float32)
    x["dSl"] = (rng.standard_normal((B, H, dv, dk)) * 0.1).astype(np.float32)
    x["g"] = (-np.abs(rng.standard_normal((B, T, H))) * 0.2).astype(np.float32)
    x["z0"] = np.abs(rng.standard_normal((B, H, dk))).astype(np.float32)
    x["dzl"] = (rng.standard_normal((B, H, dk)) * 0.1).astype(np.float32)
    if dtype == "bf16":
        for n in ("q", "k", "v", "do"):
            x[n] = bf16_round(x[n])
    return x


def _check(got, ref, names, tol):
    errs = {n: relerr(g, ref[n]) for n, g in zip(names, got)}
    assert all(e <= tol for e in errs.values()), errs


def _cases():
    return [(d, "f32") for d in DIMS + DIMS_F32_ONLY] + [(d, "bf16") for d in DIMS]


@pytest.mark.parametrize("dims,dtype", _cases())
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.06])
@pytest.mark.parametrize("par", [False, True])
def test_linear_attention(dims, dtype, shape, p, par):
    from memorax_amd import kernels as K
    dk, dv = dims
    x = _inputs(shape, dk, dv, p, dtype, seed=sum(shape) + dk + 3)
    print(f"case narrow la dk={dk} dv={dv} shape={shape} p={p} dtype={dtype} chunk_parallel={par}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    tq, tk, tv, tdo = (dev(x[n], td) for n in ("q", "k", "v", "do"))
    for fm, name in ((1, "elu1"), (0, "none")):
        o, Sl, chk = K.linear_attn_fwd(tq, tk, tv, dev(x["done"]), dev(x["S0"]), fm, chunk_parallel=par)
        assert o.shape == (shape[0], shape[1], shape[2], dv) and Sl.shape == (shape[0], shape[2], dv, dk)
        ref = G.linear_attention_grads(x["q"], x["k"], x["v"], x["done"], x["S0"], x["do"], x["dSl"], name)
        _check((o, Sl), ref, ("o", "S_last"), tol)
        got = K.linear_attn_bwd(tq, tk, tv, dev(x["done"]), chk, tdo, dev(x["dSl"]), fm)
        _check(got, ref, ("dq", "dk", "dv", "dS0"), tol)


@pytest.mark.parametrize("dims,dtype", _cases())
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.06])
def test_gated_and_normalised_linear_attention(dims, dtype, shape, p):
    from memorax_amd import kernels as K
    dk, dv = dims
    x = _inputs(shape, dk, dv, p, dtype, seed=sum(shape) + dk + 5)
    print(f"case narrow gated/norm dk={dk} dv={dv} shape={shape} p={p} dtype={dtype}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    tq, tk, tv, tdo = (dev(x[n], td) for n in ("q", "k", "v", "do"))
    dn = dev(x["done"])
    o, Sl, S_chk = K.gated_linear_attn_fwd(tq, tk, tv, dev(x["g"]), dn, dev(x["S0"]), 1)
    ref = G.gated_linear_attention_grads(x["q"], x["k"], x["v"], x["g"], x["done"], x["S0"], x["do"], x["dSl"], "elu1")
    _check((o, Sl), ref, ("o", "S_last"), tol)
    got = K.gated_linear_attn_bwd(tq, tk, tv, dev(x["g"]), dn, S_chk, tdo, dev(x["dSl"]), 1, S_last=Sl)
    _check(got, ref, ("dq", "dk", "dv", "dg", "dS0"), tol)
    o, den, Sl, zl, chk = K.linear_attn_norm_fwd(tq, tk, tv, dn, dev(x["S0"]), dev(x["z0"]), 1, 1e-6)
    ref = G.normalised_linear_attention_grads(x["q"], x["k"], x["v"], x["done"], x["S0"], x["z0"], x["do"], x["dSl"],
                                              x["dzl"], "elu1", 1e-6)
    _check((o, Sl, zl), ref, ("o", "S_last", "z_last"), tol)
    got = K.linear_attn_norm_bwd(tq, tk, tv, dn, chk, o, den, tdo, dev(x["dSl"]), dev(x["dzl"]), 1, 1e-6)
    # bf16: the gradients carry the rounding of the denominators twice (the same numbers, bit for bit, as the
    # full-width kernels give on zero-padded heads: test_narrow_heads_equal_zero_padded_heads_bit_for_bit)
    _check(got, ref, ("dq", "dk", "dv", "dS0", "dz0"), tol * (1.5 if dtype == "bf16" else 1.0))


@pytest.mark.parametrize("dims", [(16, 16), (8, 24), (40, 64), (48, 24)])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_narrow_heads_equal_zero_padded_heads_bit_for_bit(dims, dtype):
    """What the narrow instances pad inside is what a caller would pad outside: with the feature map applied
    beforehand (phi(0) = 1 would count otherwise), a narrow call and the same call on zero-padded q, k, v,
    states and gradients at the build's full width give identical bits -- normalised read-out (forward and
    backward) and gated linear attention."""
    from memorax_amd import kernels as K
    dk, dv = dims
    W = 32 if max(dk, dv) <= 32 else 64
    shape = (2, 200, 3)
    x = _inputs(shape, dk, dv, 0.05, dtype, seed=77)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    print(f"case narrow vs padded dk={dk} dv={dv} dtype={dtype}", flush=True)
    pad = lambda t, n: torch.nn.functional.pad(t, (0, n)).contiguous()
    pad2 = lambda t: torch.nn.functional.pad(t, (0, W - dk, 0, W - dv)).contiguous()
    fq, fk = ((torch.nn.functional.elu(dev(x[n])) + 1).to(td) for n in ("q", "k"))
    tv, tdo = dev(x["v"], td), dev(x["do"], td)
    dn, S0, z0, dSl, dzl, g = dev(x["done"]), dev(x["S0"]), dev(x["z0"]), dev(x["dSl"]), dev(x["dzl"]), dev(x["g"])

    def norm(q, k, v, do, S0, z0, dSl, dzl):
        o, den, Sl, zl, chk = K.linear_attn_norm_fwd(q, k, v, dn, S0, z0, 0, 1e-6)
        return (o, den, Sl, zl) + tuple(K.linear_attn_norm_bwd(q, k, v, dn, chk, o, den, do, dSl, dzl, 0, 1e-6))

    def gated(q, k, v, do, S0, z0, dSl, dzl):
        o, Sl, chk = K.gated_linear_attn_fwd(q, k, v, g, dn, S0, 0)
        return (o, Sl) + tuple(K.gated_linear_attn_bwd(q, k, v, g, dn, chk, do, dSl, 0, S_last=Sl))

    cut = {"k": lambda t: t[..., :dk], "v": lambda t: t[..., :dv], "s": lambda t: t[..., :dv, :dk], "": lambda t: t}
    for fn, kinds in ((norm, ("v", "", "s", "k", "k", "k", "v", "s", "k")), (gated, ("v", "s", "k", "k", "v", "", "s"))):
        a = fn(fq, fk, tv, tdo, S0, z0, dSl, dzl)
        b = fn(pad(fq, W - dk), pad(fk, W - dk), pad(tv, W - dv), pad(tdo, W - dv), pad2(S0), pad(z0, W - dk), pad2(dSl),
               pad(dzl, W - dk))
        assert len(a) == len(kinds)
        for i, (ta, tb, kd) in enumerate(zip(a, b, kinds)):
            assert torch.equal(ta, cut[kd](tb)), (fn.__name__, i)


@pytest.mark.parametrize("dims,dtype", _cases())
def test_single_steps_roll_out_to_the_sequence_results(dims, dtype):
    from memorax_amd import kernels as K
    dk, dv = dims
    B, T, H = 3, 11, 2
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    print(f"case narrow steps dk={dk} dv={dv} dtype={dtype}", flush=True)
    x = _inputs((B, T, H), dk, dv, 0.2, dtype, seed=21)
    q, k, v, done = dev(x["q"], td), dev(x["k"], td), dev(x["v"], td), dev(x["done"])
    for normalise in (True, False):
        S, z, outs = dev(x["S0"]), dev(x["z0"]) if normalise else None, []
        for t in range(T):
            o, S, z = K.linear_attn_step(q[:, t].contiguous(), k[:, t].contiguous(), v[:, t].contiguous(),
                                         done[:, t].contiguous(), S, z, "elu1", normalise)
            outs.append(o)
        args = [torch.from_numpy(x[n]).double() for n in ("q", "k", "v")] + [torch.from_numpy(x["done"]),
                                                                              torch.from_numpy(x["S0"]).double()]
        if normalise:
            ro, rS, rz = (a.numpy() for a in G.normalised_linear_attention_t(*args, torch.from_numpy(x["z0"]).double(), "elu1"))
            assert relerr(z, rz) <= tol
        else:
            ro, rS = (a.numpy() for a in G.linear_attention_t(*args, "elu1"))
        assert outs[0].shape == (B, H, dv) and S.shape == (B, H, dv, dk)
        assert relerr(torch.stack(outs, 1), ro) <= tol and relerr(S, rS) <= tol


def _delta_inputs(shape, dk, dv, p, dtype, seed):
    B, T, H = shape
    rng = np.random.default_rng(seed)
    x = {"q": rng.standard_normal((B, T, H, dk)).astype(np.float32), "v": rng.standard_normal((B, T, H, dv)).astype(np.float32),
         "do": rng.standard_normal((B, T, H, dv)).astype(np.float32)}
    kk = rng.standard_normal((B, T, H, dk)).astype(np.float32)
    x["k"] = kk / np.linalg.norm(kk, axis=-1, keepdims=True)
    x["beta"] = (1 / (1 + np.exp(-rng.standard_normal((B, T, H))))).astype(np.float32)
    x["kr"] = (x["k"] * (0.5 + rng.random((B, T, H, 1)))).astype(np.float32)   # raw keys and gate pre-activations
    x["br"] = (rng.standard_normal((B, T, H)) * 1.5).astype(np.float32)
    x["done"] = rng.random((B, T)) < p
    x["S0"] = (rng.standard_normal((B, H, dv, dk)) * 0.1).astype(np.float32)
    x["dSl"] = (rng.standard_normal((B, H, dv, dk)) * 0.1).astype(np.float32)
    if dtype == "bf16":
        for n in ("q", "k", "v", "do", "beta", "kr", "br"):
            x[n] = bf16_round(x[n])
    return x


def _delta_cases():
    # every width on the short shapes; the long sequence (35 chunks) on one width per build
    short = [(d, t, s) for d, t in _cases() for s in [(3, 1, 2), (2, 65, 1), (2, 200, 3)]]
    return short + [(d, t, (1, 1100, 2)) for d in [(16, 16), (40, 64)] for t in ("f32", "bf16")]


@pytest.mark.parametrize("dims,dtype,shape", _delta_cases())
@pytest.mark.parametrize("p", [0.0, 0.06])
@pytest.mark.parametrize("path", ["parallel", "inline"])
def test_delta_rule_and_deltanet(dims, dtype, shape, p, path):
    from memorax_amd import kernels as K
    dk, dv = dims
    x = _delta_inputs(shape, dk, dv, p, dtype, seed=sum(shape) + dk + 9)
    print(f"case narrow delta dk={dk} dv={dv} shape={shape} p={p} dtype={dtype} factors={path}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    tq, tk, tv, tb, tdo = (dev(x[n], td) for n in ("q", "k", "v", "beta", "do"))
    dn = dev(x["done"])
    o, Sl, chk = K.delta_rule_fwd(tq, tk, tv, tb, dn, dev(x["S0"]), factor_path=path)
    assert o.shape == (shape[0], shape[1], shape[2], dv) and Sl.shape == (shape[0], shape[2], dv, dk)
    ref = G.delta_rule_grads(x["q"], x["k"], x["v"], x["beta"], x["done"], x["S0"], x["do"], x["dSl"])
    _check((o, Sl), ref, ("o", "S_last"), tol)
    got = K.delta_rule_bwd(tq, tk, tv, tb, dn, chk, tdo, dev(x["dSl"]))
    _check(got, ref, ("dq", "dk", "dv", "dbeta", "dS0"), tol)
    # the cell's prologue inside the kernels: raw keys and gate pre-activations
    tk2, tb2 = dev(x["kr"], td), dev(x["br"], td)
    o, Sl, chk = K.delta_rule_fwd(tq, tk2, tv, tb2, dn, dev(x["S0"]), prologue=True, factor_path=path)
    ref = G.deltanet_grads(x["q"], x["kr"], x["v"], x["br"], x["done"], x["S0"], x["do"], x["dSl"])
    _check((o, Sl), ref, ("o", "S_last"), tol)
    got = K.delta_rule_bwd(tq, tk2, tv, tb2, dn, chk, tdo, dev(x["dSl"]), prologue=True)
    _check(got, ref, ("dq", "dk", "dv", "dbeta", "dS0"), tol)


@pytest.mark.parametrize("dims", [(16, 16), (8, 24), (40, 64), (48, 24)])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_narrow_delta_rule_equals_zero_padded_heads_bit_for_bit(dims, dtype):
    """Zero key features change neither k k^T nor the key norm, zero value features add zero rows to the state:
    a narrow call and the same call on zero-padded arrays at the build's full width give identical bits, with
    either factor path, with and without the prologue, forward, backward and single steps."""
    from memorax_amd import kernels as K
    dk, dv = dims
    W = 32 if max(dk, dv) <= 32 else 64
    shape = (2, 200, 3)
    x = _delta_inputs(shape, dk, dv, 0.05, dtype, seed=78)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    print(f"case narrow delta vs padded dk={dk} dv={dv} dtype={dtype}", flush=True)
    pad = lambda t, n: torch.nn.functional.pad(t, (0, n)).contiguous()
    pad2 = lambda t: torch.nn.functional.pad(t, (0, W - dk, 0, W - dv)).contiguous()
    tq, tv, tdo = dev(x["q"], td), dev(x["v"], td), dev(x["do"], td)
    dn, S0, dSl = dev(x["done"]), dev(x["S0"]), dev(x["dSl"])
    cut = {"k": lambda t: t[..., :dk], "v": lambda t: t[..., :dv], "s": lambda t: t[..., :dv, :dk], "": lambda t: t}
    for pro, kn, bn in ((False, "k", "beta"), (True, "kr", "br")):
        tk, tb = dev(x[kn], td), dev(x[bn], td)
        for path in ("parallel", "inline"):
            def run(q, k, v, do, S0, dSl):
                o, Sl, chk = K.delta_rule_fwd(q, k, v, tb, dn, S0, prologue=pro, factor_path=path)
                return (o, Sl) + tuple(K.delta_rule_bwd(q, k, v, tb, dn, chk, do, dSl, prologue=pro))
            a = run(tq, tk, tv, tdo, S0, dSl)
            b = run(pad(tq, W - dk), pad(tk, W - dk), pad(tv, W - dv), pad(tdo, W - dv), pad2(S0), pad2(dSl))
            for i, (ta, tb_, kd) in enumerate(zip(a, b, ("v", "s", "k", "k", "v", "", "s"))):
                assert torch.equal(ta, cut[kd](tb_)), (pro, path, i)
    tk, tb = dev(x["k"], td), dev(x["beta"], td)
    o1, S1 = K.delta_rule_step(tq[:, 0].contiguous(), tk[:, 0].contiguous(), tv[:, 0].contiguous(), tb[:, 0].contiguous(),
                               dn[:, 0].contiguous(), S0)
    o2, S2 = K.delta_rule_step(pad(tq[:, 0], W - dk), pad(tk[:, 0], W - dk), pad(tv[:, 0], W - dv), tb[:, 0].contiguous(),
                               dn[:, 0].contiguous(), pad2(S0))
    assert torch.equal(o1, o2[..., :dv]) and torch.equal(S1, S2[..., :dv, :dk])


def test_what_is_not_a_narrow_head_is_refused():
    from memorax_amd import _lib
    lib = _lib.load()
    P = lambda t: ctypes.c_void_p(t.data_ptr())

    def la(dk, dv, dtype):
        td = torch.bfloat16 if dtype else torch.float32
        q = torch.zeros((1, 4, 1, dk), dtype=td, device="cuda")
        v = torch.zeros((1, 4, 1, dv), dtype=td, device="cuda")
        dn = torch.zeros((1, 4), dtype=torch.uint8, device="cuda")
        o = torch.empty_like(v)
        return lib.mrx_linear_attn_fwd(None, P(q), P(q), P(v), P(dn), None, P(o), None, None, 1, 4, 1, dk, dv, dtype, 0, 0)

    assert la(16, 16, 0) == 0 and la(16, 16, 1) == 0 and la(12, 4, 0) == 0
    assert la(12, 16, 1) == -2       # 12 bf16 are one and a half segments
    assert la(6, 16, 0) == -2 and la(16, 10, 0) == -2
    assert la(16, 64, 0) == 0 and la(64, 16, 1) == 0 and la(48, 48, 0) == 0 and la(32, 40, 1) == 0  # the 64-wide kernels
    assert la(72, 64, 0) == -2 and la(64, 128, 0) == -2 and la(36, 36, 1) == -2
    # the delta rule: the same widths; the variant with the static scratch array stays at 64
    q = torch.zeros((1, 4, 1, 16), device="cuda")
    dn = torch.zeros((1, 4), dtype=torch.uint8, device="cuda")
    beta = torch.zeros((1, 4, 1), device="cuda")
    o = torch.empty_like(q)
    assert lib.mrx_delta_rule_fwd(None, P(q), P(q), P(q), P(beta), P(dn), None, P(o), None, None, None, 1, 4, 1, 16, 16, 0, 0, 0, 0) == 0
    assert lib.mrx_delta_rule_fwd(None, P(q), P(q), P(q), P(beta), P(dn), None, P(o), None, None, None, 1, 4, 1, 16, 6, 0, 0, 0, 0) == -2
    assert lib.mrx_delta_rule_fwd_noalloc(None, P(q), P(q), P(q), P(beta), P(dn), None, P(o), None, 1, 4, 1, 16, 16, 0, 0) == -2
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_reference_default_head_dim_at_scale(dtype):
    """1024 environments x 128 steps x 8 heads x 16 features (the Mamba cell's default heads, mamba.py:36-38):
    two calls over [0, 64) and [64, 128) with the state carried equal one call bit for bit (chunk boundaries
    coincide), the backward is linear in the incoming gradient, and two batch rows match the oracle."""
    from memorax_amd import kernels as K
    B, T, H, d = 1024, 128, 8, 16
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    g = torch.Generator(device="cuda").manual_seed(5)
    q, k, v, do = (torch.randn((B, T, H, d), device="cuda", generator=g).div_(4).to(td) for _ in range(4))
    glog = -torch.rand((B, T, H), device="cuda", generator=g) * 0.3
    done = torch.rand((B, T), device="cuda", generator=g) < 0.01
    S0 = torch.randn((B, H, d, d), device="cuda", generator=g) * 0.1
    print(f"case narrow at scale dtype={dtype}", flush=True)
    o, Sl, chk = K.gated_linear_attn_fwd(q, k, v, glog, done, S0, 1)
    h = T // 2
    o1, S1, _ = K.gated_linear_attn_fwd(q[:, :h].contiguous(), k[:, :h].contiguous(), v[:, :h].contiguous(),
                                        glog[:, :h].contiguous(), done[:, :h].contiguous(), S0, 1, save_chk=False)
    o2, S2, _ = K.gated_linear_attn_fwd(q[:, h:].contiguous(), k[:, h:].contiguous(), v[:, h:].contiguous(),
                                        glog[:, h:].contiguous(), done[:, h:].contiguous(), S1, 1, save_chk=False)
    assert torch.equal(torch.cat([o1, o2], 1), o) and torch.equal(S2, Sl)
    g1 = K.gated_linear_attn_bwd(q, k, v, glog, done, chk, do, None, 1, S_last=Sl)
    g2 = K.gated_linear_attn_bwd(q, k, v, glog, done, chk, (do.float() * 2).to(td), None, 1, S_last=Sl)
    for a, b in zip(g1, g2):  # doubling is exact in either dtype
        assert torch.equal((a.float() * 2).to(a.dtype), b)
    rows = [3, B - 1]
    x = {n: t[rows].float().cpu().numpy() for n, t in (("q", q), ("k", k), ("v", v), ("do", do))}
    ref = G.gated_linear_attention_grads(x["q"], x["k"], x["v"], glog[rows].cpu().numpy(), done[rows].cpu().numpy(),
                                         S0[rows].cpu().numpy(), x["do"], None, "elu1")
    got = dict(zip(("dq", "dk", "dv", "dg", "dS0"), g1))
    errs = {"o": relerr(o[rows], ref["o"]), "S_last": relerr(Sl[rows], ref["S_last"])}
    errs.update({n: relerr(got[n][rows], ref[n]) for n in got})
    assert all(e <= tol for e in errs.values()), errs
