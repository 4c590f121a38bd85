"""GPU parity of the chunked backward kernels (through the C ABI) against the
torch-fp64 autograd oracle (small shapes) and the C oracle (benchmark shapes)."""
import numpy as np
import pytest
import torch

from oracle import clib
from oracle import grad as G
from oracle import memoroid as M
from gpu_util import TOL_BF16, TOL_F32, attn_inputs, bf16_round, dev, relerr

pytestmark = pytest.mark.gpu

SHAPES = [(1, 64, 1), (2, 128, 2), (1, 1, 1), (2, 7, 1), (1, 65, 2), (2, 200, 3), (1, 33, 1)]


def _check(got, ref, tol, names):
    errs = {n: relerr(g, ref[n]) for n, g in zip(names, got)}
    bad = {n: e for n, e in errs.items() if not e <= tol}
    assert not bad, f"rel errs {errs}"


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.05])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("fmap", [0, 1])
def test_linear_attention_bwd(shape, p, dtype, fmap):
    from memorax_amd import kernels as K
    B, T, H = shape
    x = attn_inputs(B, T, H, p=p, seed=B * 100 + T + H + 31, scale=1.0 / 8)
    rng = np.random.default_rng(T)
    do = rng.standard_normal((B, T, H, 64)).astype(np.float32)
    dSl = (rng.standard_normal((B, H, 64, 64)) * 0.1).astype(np.float32)
    print(f"case la_bwd shape={shape} p={p} dtype={dtype} fmap={fmap}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    if dtype == "bf16":
        for n in ("q", "k", "v"):
            x[n] = bf16_round(x[n])
        do = bf16_round(do)
    tq, tk, tv, tdo = (dev(a, td) for a in (x["q"], x["k"], x["v"], do))
    o, Sl, chk = K.linear_attn_fwd(tq, tk, tv, dev(x["done"]), dev(x["S0"]), fmap)
    got = K.linear_attn_bwd(tq, tk, tv, dev(x["done"]), chk, tdo, dev(dSl), fmap)
    ref = G.linear_attention_grads(x["q"], x["k"], x["v"], x["done"], x["S0"], do, dSl,
                                   "elu1" if fmap else "none")
    _check(got, ref, TOL_BF16 if dtype == "bf16" else TOL_F32, ("dq", "dk", "dv", "dS0"))


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.05])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_delta_rule_bwd(shape, p, dtype):
    from memorax_amd import kernels as K
    B, T, H = shape
    x = attn_inputs(B, T, H, p=p, seed=B * 100 + T + H + 57, delta=True)
    rng = np.random.default_rng(T + 1)
    do = rng.standard_normal((B, T, H, 64)).astype(np.float32)
    dSl = (rng.standard_normal((B, H, 64, 64)) * 0.1).astype(np.float32)
    print(f"case delta_bwd shape={shape} p={p} dtype={dtype}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    if dtype == "bf16":
        do = bf16_round(do)
        for n in ("q", "k", "v", "beta"):
            x[n] = bf16_round(x[n])
    tq, tk, tv, tb, tdo = (dev(a, td) for a in (x["q"], x["k"], x["v"], x["beta"], do))
    o, Sl, chk = K.delta_rule_fwd(tq, tk, tv, tb, dev(x["done"]), dev(x["S0"]))
    got = K.delta_rule_bwd(tq, tk, tv, tb, dev(x["done"]), chk, tdo, dev(dSl))
    ref = G.delta_rule_grads(x["q"], x["k"], x["v"], x["beta"], x["done"], x["S0"], do, dSl)
    _check(got, ref, TOL_BF16 if dtype == "bf16" else TOL_F32, ("dq", "dk", "dv", "dbeta", "dS0"))


@pytest.mark.parametrize("done_dtype", ["uint8", "float32"])
def test_chunk_kernels_done_dtypes(done_dtype):
    """done as uint8 or float32 (memoroid.py:67 casts it to float) gives identical results."""
    from memorax_amd import kernels as K
    x = attn_inputs(2, 130, 2, p=0.04, seed=11, delta=True)
    args = [dev(x[n]) for n in ("q", "k", "v", "beta")]
    ref = K.delta_rule_fwd(*args, dev(x["done"]))
    dd = x["done"].astype(np.uint8) if done_dtype == "uint8" else x["done"].astype(np.float32) * 3.5
    got = K.delta_rule_fwd(*args, dev(dd))
    assert torch.equal(got[0], ref[0]) and torch.equal(got[1], ref[1])
    do = torch.ones_like(ref[0])
    g1 = K.delta_rule_bwd(*args, dev(x["done"]), ref[2], do)
    g2 = K.delta_rule_bwd(*args, dev(dd), got[2], do)
    assert all(torch.equal(a, b) for a, b in zip(g1, g2))


def test_bwd_reset_isolation():
    """A poisoned (NaN) gradient / value on one side of a reset stays on that side."""
    from memorax_amd import kernels as K
    B, T, H = 1, 192, 1
    x = attn_inputs(B, T, H, seed=5, delta=True)
    x["done"][:] = False
    x["done"][0, 100] = True
    for n in ("q", "k", "v", "beta"):
        x[n] = bf16_round(x[n])
    do = bf16_round(np.random.default_rng(2).standard_normal((B, T, H, 64)).astype(np.float32))
    do[0, 150] = np.nan      # poison in the later episode: gradient, key and gate
    x["k"][0, 120] = np.nan
    x["beta"][0, 110] = np.nan
    bf = torch.bfloat16
    tq, tk, tv, tb, tdo = (dev(a, bf) for a in (x["q"], x["k"], x["v"], x["beta"], do))
    o, Sl, chk = K.delta_rule_fwd(tq, tk, tv, tb, dev(x["done"]))
    dq, dk, dv, db, dS0 = K.delta_rule_bwd(tq, tk, tv, tb, dev(x["done"]), chk, tdo)
    for g in (dq, dk, dv):
        assert np.isfinite(g.float().cpu().numpy()[0, :100]).all()
    assert np.isfinite(db.float().cpu().numpy()[0, :100]).all() and np.isfinite(dS0.cpu().numpy()).all()
    ref = G.delta_rule_grads(x["q"][:, :100], x["k"][:, :100], x["v"][:, :100], x["beta"][:, :100],
                             x["done"][:, :100], None, do[:, :100])
    assert relerr(dk[:, :100], ref["dk"]) <= TOL_BF16 and relerr(dq[:, :100], ref["dq"]) <= TOL_BF16


def test_bwd_config_shapes_small_batch():
    """Benchmark configurations 2 (fp32, elu+1) and 4 (bf16 delta rule) at reduced batch vs the C oracle."""
    from memorax_amd import kernels as K
    x = M.make_inputs(2, (4, 256, 4, 64))
    do = np.random.default_rng(0).standard_normal(x["v"].shape).astype(np.float32)
    tq, tk, tv, tdo = (dev(a) for a in (x["q"], x["k"], x["v"], do))
    o, Sl, chk = K.linear_attn_fwd(tq, tk, tv, dev(x["done"]), None, 1)
    got = K.linear_attn_bwd(tq, tk, tv, dev(x["done"]), chk, tdo, None, 1)
    ref = clib.linear_attn_bwd(x["q"], x["k"], x["v"], x["done"], None, do, None, 1)
    _check(got, dict(zip(("dq", "dk", "dv", "dS0"), ref)), TOL_F32, ("dq", "dk", "dv", "dS0"))

    x = M.make_inputs(4, (4, 1024, 8, 64))
    xb = {n: bf16_round(x[n]) for n in ("q", "k", "v", "beta")}
    do = bf16_round(np.random.default_rng(1).standard_normal(x["v"].shape).astype(np.float32))
    bf = torch.bfloat16
    tq, tk, tv, tb, tdo = (dev(a, bf) for a in (xb["q"], xb["k"], xb["v"], xb["beta"], do))
    o, Sl, chk = K.delta_rule_fwd(tq, tk, tv, tb, dev(x["done"]))
    got = K.delta_rule_bwd(tq, tk, tv, tb, dev(x["done"]), chk, tdo)
    ref = clib.delta_rule_bwd(xb["q"], xb["k"], xb["v"], xb["beta"], x["done"], None, do)
    _check(got, dict(zip(("dq", "dk", "dv", "dbeta", "dS0"), ref)), TOL_BF16, ("dq", "dk", "dv", "dbeta", "dS0"))


def test_autograd_functions():
    import memorax_amd as mx
    x = attn_inputs(2, 96, 2, p=0.03, seed=77, delta=True)
    for n in ("q", "k", "v", "beta"):
        x[n] = bf16_round(x[n])
    do = bf16_round(np.random.default_rng(4).standard_normal(x["v"].shape).astype(np.float32))
    bf = torch.bfloat16
    tq, tk, tv, tb = (dev(x[n], bf).requires_grad_() for n in ("q", "k", "v", "beta"))
    tS0 = dev(x["S0"]).requires_grad_()
    o, Sl = mx.delta_rule(tq, tk, tv, tb, dev(x["done"]), tS0)
    (o.float() * dev(do)).sum().backward()
    ref = G.delta_rule_grads(x["q"], x["k"], x["v"], x["beta"], x["done"], x["S0"], do)
    _check((tq.grad, tk.grad, tv.grad, tb.grad, tS0.grad), ref, TOL_BF16, ("dq", "dk", "dv", "dbeta", "dS0"))
    tq2, tk2, tv2 = (dev(x[n] / 8).requires_grad_() for n in ("q", "k", "v"))
    o2, _ = mx.linear_attention(tq2, tk2, tv2, dev(x["done"]), None, "elu1")
    (o2 * dev(do)).sum().backward()
    ref = G.linear_attention_grads(x["q"] / 8, x["k"] / 8, x["v"] / 8, x["done"], None, do, None, "elu1")
    _check((tq2.grad, tk2.grad, tv2.grad), ref, TOL_F32, ("dq", "dk", "dv"))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_linear_attention_state_walk_back_over_a_long_sequence(dtype):
    """The backward call recovers the state entering every chunk by undoing the chunks' updates from
    S_last in fp32.  With the elu+1 feature map the state grows with every step, so the first chunks
    hold a state hundreds of times smaller than the one the walk starts from: their dq (= dO S + ...)
    is where an error of the walk would show.  4096 steps, resets in the middle (one chunk with two of
    them), a non-zero initial state; dq is checked on the first chunks against their own scale."""
    from memorax_amd import kernels as K
    B, T, H = 2, 4096, 2
    rng = np.random.default_rng(77)
    q, k, v, do = ((rng.standard_normal((B, T, H, 64)) / 8).astype(np.float32) for _ in range(4))
    S0 = (rng.standard_normal((B, H, 64, 64)) * 0.1).astype(np.float32)
    done = np.zeros((B, T), bool)
    done[0, [1500, 1510, 3000]] = True
    done[1, 2047] = True
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    if dtype == "bf16":
        q, k, v, do = (bf16_round(a) for a in (q, k, v, do))
    print(f"case la walk-back dtype={dtype}", flush=True)
    tq, tk, tv, tdo = (dev(a, td) for a in (q, k, v, do))
    o, Sl, chk = K.linear_attn_fwd(tq, tk, tv, dev(done), dev(S0), 1, chunk_parallel=False)  # the sequential pair
    got = K.linear_attn_bwd(tq, tk, tv, dev(done), chk, tdo, None, 1)
    ref = clib.linear_attn_bwd(q, k, v, done, S0, do, None, 1)
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    for name, a, r in zip(("dq", "dk", "dv", "dS0"), got, ref):
        assert relerr(a, r) <= tol, name
    # the first 128 steps on their own scale (the state there is a thirtieth of the final one)
    for name, a, r in zip(("dq", "dk", "dv"), got, ref):
        assert relerr(a[:, :128], r[:, :128]) <= tol, name
    # and the steps right after each reset, where the state has just restarted from zero
    for b_, t_ in ((0, 1500), (0, 1510), (0, 3000), (1, 2047)):
        assert relerr(got[0][b_, t_:t_ + 32], ref[0][b_, t_:t_ + 32]) <= tol, (b_, t_)


@pytest.mark.parametrize("feature_map", [1, 0])
def test_linear_attention_walk_back_16k_steps_without_a_reset(feature_map):
    """The worst case for the walk: no reset in 16 384 steps and values with a positive mean, so that the
    state grows linearly to some five hundred times what the first chunk sees.  Undone chunk by chunk all
    the way from S_last, the rounding of the late state (about eps (T/C)^1.5 relative to the early one)
    would exceed 1e-4 in fp32; the walk starts afresh from the exact state the forward call leaves every
    32 chunks, and dq, dk of the first chunks -- on their own scale -- stay inside the tolerance."""
    from memorax_amd import kernels as K
    B, T, H = 1, 16384, 2
    rng = np.random.default_rng(91)
    q, k, do = ((rng.standard_normal((B, T, H, 64)) / 8).astype(np.float32) for _ in range(3))
    v = (rng.standard_normal((B, T, H, 64)) / 8 + 0.5).astype(np.float32)
    done = np.zeros((B, T), bool)
    print(f"case la walk-back 16k fmap={feature_map}", flush=True)
    tq, tk, tv, tdo = (dev(a) for a in (q, k, v, do))
    o, Sl, chk = K.linear_attn_fwd(tq, tk, tv, dev(done), None, feature_map, chunk_parallel=False)
    got = K.linear_attn_bwd(tq, tk, tv, dev(done), chk, tdo, None, feature_map)
    ref = clib.linear_attn_bwd(q, k, v, done, None, do, None, feature_map)
    for name, a, r in zip(("dq", "dk", "dv"), got, ref):
        assert relerr(a, r) <= TOL_F32, name
        for lo in (0, 32, 992, 1024, 4064):   # first chunks, and the chunks on either side of an anchor
            assert relerr(a[:, lo:lo + 32], r[:, lo:lo + 32]) <= TOL_F32, (name, lo)


def test_normalised_read_out_walks_across_an_anchor():
    """The normalised read-out's backward shares the walk and its anchors: 1 300 fp32 steps cross the
    anchor at chunk 32 (step 1 024) and end in a ragged chunk; gradients against torch-fp64 autograd.
    (Zero-mean values: with a common mean the normalised output hardly depends on the query and dq is
    what a cancellation leaves, in any implementation.)"""
    from memorax_amd import kernels as K
    B, T, H = 1, 1300, 1
    rng = np.random.default_rng(92)
    q, k, v, do = ((rng.standard_normal((B, T, H, 64)) / 8).astype(np.float32) for _ in range(4))
    done = np.zeros((B, T), bool)
    print("case la_norm walk-back across an anchor", flush=True)
    tq, tk, tv, tdo = (dev(a) for a in (q, k, v, do))
    on, den, Sl, zl, chkn = K.linear_attn_norm_fwd(tq, tk, tv, dev(done), None, None, 1)
    gn = K.linear_attn_norm_bwd(tq, tk, tv, dev(done), chkn, on, den, tdo, None, None, 1)
    rn = G.normalised_linear_attention_grads(q, k, v, done, None, None, do, None, None, "elu1")
    for name, a in zip(("dk", "dv"), gn[1:]):
        assert relerr(a, rn[name]) <= TOL_F32, name
        for lo in (0, 992, 1024):
            assert relerr(a[:, lo:lo + 32], rn[name][:, lo:lo + 32]) <= TOL_F32, (name, lo)
    # dq of a normalised read-out is what two terms leave that cancel -- the output does not depend on the
    # scale of the mapped query phi(q), and over a thousand steps S^T dnum and dden z are each a hundred times
    # their difference -- and each has the size of dk: that is the scale its error is judged on
    dq = gn[0].cpu().numpy()
    for lo, hi in ((0, T), (0, 32), (992, 1024), (1024, 1056)):
        scale = np.abs(rn["dk"][:, lo:hi]).max()
        assert np.abs(dq[:, lo:hi] - rn["dq"][:, lo:hi]).max() <= TOL_F32 * scale, (lo, hi)
