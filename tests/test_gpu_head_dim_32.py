"""GPU parity of the library's second build of the chunked and single-step kernels (d_k = d_v = 32),
called through the same public entry points, against the oracle at that head dim."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import grad as G
from oracle import memoroid as M
from gpu_util import TOL_BF16, TOL_F32, attn_inputs, bf16_round, dev, relerr

pytestmark = pytest.mark.gpu

D = 32
# (B, T, H): single rows and chunks, ragged ends, several chunks, a long sequence
# (every tensor of a case holds several rows: a lone bf16 scalar such as dbeta of one step has no scale
# to be judged against)
SHAPES = [(3, 1, 2), (2, 7, 1), (1, 64, 2), (2, 65, 1), (2, 200, 3), (1, 1100, 2)]


def _inputs(shape, p, dtype, seed, delta=False):
    B, T, H = shape
    x = attn_inputs(B, T, H, d=D, p=p, seed=seed, delta=delta, scale=None if delta else 1.0 / 6)
    rng = np.random.default_rng(seed + 1)
    x["do"] = rng.standard_normal((B, T, H, D)).astype(np.float32)
    x["dSl"] = (rng.standard_normal((B, H, D, D)) * 0.1).astype(np.float32)
    x["g"] = (-np.abs(rng.standard_normal((B, T, H))) * 0.2).astype(np.float32)
    x["z0"] = np.abs(rng.standard_normal((B, H, D))).astype(np.float32)
    if dtype == "bf16":
        for n in ("q", "k", "v", "do") + (("beta",) if delta else ()):
            x[n] = bf16_round(x[n])
    return x


def _check(got, ref, names, tol):
    errs = {n: relerr(g, ref[n]) for n, g in zip(names, got)}
    assert all(e <= tol for e in errs.values()), errs


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.06])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("par", [False, True])
def test_linear_attention(shape, p, dtype, par):
    from memorax_amd import kernels as K
    x = _inputs(shape, p, dtype, seed=sum(shape) + 3)
    print(f"case hd32 la shape={shape} p={p} dtype={dtype} chunk_parallel={par}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    tq, tk, tv, tdo = (dev(x[n], td) for n in ("q", "k", "v", "do"))
    o, Sl, chk = K.linear_attn_fwd(tq, tk, tv, dev(x["done"]), dev(x["S0"]), 1, chunk_parallel=par)
    assert Sl.shape == (shape[0], shape[2], D, D)
    ref = G.linear_attention_grads(x["q"], x["k"], x["v"], x["done"], x["S0"], x["do"], x["dSl"], "elu1")
    _check((o, Sl), ref, ("o", "S_last"), tol)
    got = K.linear_attn_bwd(tq, tk, tv, dev(x["done"]), chk, tdo, dev(x["dSl"]), 1)
    _check(got, ref, ("dq", "dk", "dv", "dS0"), tol)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.06])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_gated_and_normalised_linear_attention(shape, p, dtype):
    from memorax_amd import kernels as K
    x = _inputs(shape, p, dtype, seed=sum(shape) + 5)
    print(f"case hd32 gated/norm shape={shape} p={p} dtype={dtype}", flush=True)
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
                                              None, "elu1", 1e-6)
    _check((o, Sl, zl), ref, ("o", "S_last", "z_last"), tol)
    got = K.linear_attn_norm_bwd(tq, tk, tv, dn, chk, o, den, tdo, dev(x["dSl"]), None, 1, 1e-6)
    _check(got, ref, ("dq", "dk", "dv", "dS0", "dz0"), tol)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.06])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("path", ["parallel", "inline"])
def test_delta_rule_and_deltanet(shape, p, dtype, path):
    from memorax_amd import kernels as K
    x = _inputs(shape, p, dtype, seed=sum(shape) + 9, delta=True)
    print(f"case hd32 delta shape={shape} p={p} dtype={dtype} factors={path}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    tq, tk, tv, tb, tdo = (dev(x[n], td) for n in ("q", "k", "v", "beta", "do"))
    dn = dev(x["done"])
    o, Sl, chk = K.delta_rule_fwd(tq, tk, tv, tb, dn, dev(x["S0"]), factor_path=path)
    ref = G.delta_rule_grads(x["q"], x["k"], x["v"], x["beta"], x["done"], x["S0"], x["do"], x["dSl"])
    _check((o, Sl), ref, ("o", "S_last"), tol)
    got = K.delta_rule_bwd(tq, tk, tv, tb, dn, chk, tdo, dev(x["dSl"]))
    _check(got, ref, ("dq", "dk", "dv", "dbeta", "dS0"), tol)
    # the cell's prologue inside the kernels: raw keys and gate pre-activations
    rng = np.random.default_rng(7)
    kr = (x["k"] * (0.5 + rng.random(x["k"].shape[:-1] + (1,)))).astype(np.float32)
    br = (rng.standard_normal(x["beta"].shape) * 1.5).astype(np.float32)
    if dtype == "bf16":
        kr, br = bf16_round(kr), bf16_round(br)
    tk2, tb2 = dev(kr, td), dev(br, td)
    o, Sl, chk = K.delta_rule_fwd(tq, tk2, tv, tb2, dn, dev(x["S0"]), prologue=True, factor_path=path)
    ref = G.deltanet_grads(x["q"], kr, x["v"], br, x["done"], x["S0"], x["do"], x["dSl"])
    _check((o, Sl), ref, ("o", "S_last"), tol)
    got = K.delta_rule_bwd(tq, tk2, tv, tb2, dn, chk, tdo, dev(x["dSl"]), prologue=True)
    _check(got, ref, ("dq", "dk", "dv", "dbeta", "dS0"), tol)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_single_steps_roll_out_to_the_sequence_results(dtype):
    from memorax_amd import kernels as K
    B, T, H = 3, 11, 2
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    print(f"case hd32 steps dtype={dtype}", flush=True)
    x = _inputs((B, T, H), 0.2, dtype, seed=21)
    q, k, v, done = dev(x["q"], td), dev(x["k"], td), dev(x["v"], td), dev(x["done"])
    S, z, outs = dev(x["S0"]), dev(x["z0"]), []
    for t in range(T):
        o, S, z = K.linear_attn_step(q[:, t].contiguous(), k[:, t].contiguous(), v[:, t].contiguous(),
                                     done[:, t].contiguous(), S, z, "elu1", True)
        outs.append(o)
    ro, rS, rz = (a.numpy() for a in G.normalised_linear_attention_t(
        *(torch.from_numpy(x[n]).double() for n in ("q", "k", "v")), torch.from_numpy(x["done"]),
        torch.from_numpy(x["S0"]).double(), torch.from_numpy(x["z0"]).double(), "elu1"))
    assert relerr(torch.stack(outs, 1), ro) <= tol and relerr(S, rS) <= tol and relerr(z, rz) <= tol
    x = _inputs((B, T, H), 0.2, dtype, seed=22, delta=True)
    q, k, v, beta = (dev(x[n], td) for n in ("q", "k", "v", "beta"))
    done = dev(x["done"])
    S, outs = dev(x["S0"]), []
    for t in range(T):
        o, S = K.delta_rule_step(q[:, t].contiguous(), k[:, t].contiguous(), v[:, t].contiguous(),
                                 beta[:, t].contiguous(), done[:, t].contiguous(), S)
        outs.append(o)
    ro, rS = M.delta_rule(x["q"], x["k"], x["v"], x["beta"], x["done"], x["S0"])
    assert relerr(torch.stack(outs, 1), ro) <= tol and relerr(S, rS) <= tol


def test_other_head_dims_are_still_refused_and_the_static_scratch_variant_is_64_only():
    from memorax_amd import _lib
    lib = _lib.load()
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    for d in (72, 128):  # narrower heads: tests/test_gpu_narrow_heads.py
        q = torch.zeros((1, 4, 1, d), device="cuda")
        dn = torch.zeros((1, 4), dtype=torch.uint8, device="cuda")
        o = torch.empty_like(q)
        assert lib.mrx_linear_attn_fwd(None, P(q), P(q), P(q), P(dn), None, P(o), None, None, 1, 4, 1, d, d, 0, 0, 0) == -2
    q = torch.zeros((1, 4, 1, 32), device="cuda")
    dn = torch.zeros((1, 4), dtype=torch.uint8, device="cuda")
    beta = torch.zeros((1, 4, 1), device="cuda")
    o = torch.empty_like(q)
    assert lib.mrx_linear_attn_fwd(None, P(q), P(q), P(q), P(dn), None, P(o), None, None, 1, 4, 1, 32, 32, 0, 0, 0) == 0
    # nothing is launched on a refusal
    assert lib.mrx_delta_rule_fwd(None, P(q), P(q), P(q), P(beta), P(dn), None, P(o), None, None, None, 1, 4, 1, 32, 72, 0, 0, 0, 0) == -2
    assert lib.mrx_delta_rule_fwd_noalloc(None, P(q), P(q), P(q), P(beta), P(dn), None, P(o), None, 1, 4, 1, 32, 32, 0, 0) == -2
    torch.cuda.synchronize()
