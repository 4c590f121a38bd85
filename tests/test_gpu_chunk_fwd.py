"""GPU parity of the chunked forward kernels (through the C ABI) against the oracle."""
import numpy as np
import pytest
import torch

from oracle import clib
from oracle import memoroid as M
from gpu_util import TOL_BF16, TOL_F32, attn_inputs, bf16_round, dev, relerr

pytestmark = pytest.mark.gpu

SHAPES = [(1, 64, 1), (2, 128, 2), (1, 1, 1), (2, 7, 1), (1, 65, 2), (2, 200, 3), (1, 33, 1)]


def _run_la(x, dtype, fmap, use_S0=True):
    from memorax_amd import kernels as K
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    S0 = dev(x["S0"]) if use_S0 else None
    return K.linear_attn_fwd(dev(x["q"], td), dev(x["k"], td), dev(x["v"], td), dev(x["done"]), S0, fmap)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.05])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("fmap", [0, 1])
def test_linear_attention_fwd(shape, p, dtype, fmap):
    B, T, H = shape
    x = attn_inputs(B, T, H, p=p, seed=B * 100 + T + H, scale=1.0 / 8)
    print(f"case la_fwd shape={shape} p={p} dtype={dtype} fmap={fmap}", flush=True)
    if dtype == "bf16":
        for n in ("q", "k", "v"):
            x[n] = bf16_round(x[n])
    o, Sl, chk = _run_la(x, dtype, fmap)
    ro, rSl = M.linear_attention(x["q"], x["k"], x["v"], x["done"], x["S0"], "elu1" if fmap else "none")
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    assert relerr(o, ro) <= tol, relerr(o, ro)
    assert relerr(Sl, rSl) <= tol, relerr(Sl, rSl)
    # The checkpoints are sparse (the backward call walks the state back from S_last through reset-free
    # chunks): a slot is written where its chunk contains a reset, with the state entering the chunk
    # = the state leaving the steps before it, in fp32.
    S_chk, S_last = chk
    assert S_last is Sl and S_chk.dtype == torch.float32
    C = 64 if dtype == "bf16" else 32
    for b in range(B):
        for c in range((T + C - 1) // C):
            if not x["done"][b, c * C:(c + 1) * C].any():
                continue
            t0 = c * C
            want = x["S0"][b:b + 1] if t0 == 0 else M.linear_attention(
                x["q"][b:b + 1, :t0], x["k"][b:b + 1, :t0], x["v"][b:b + 1, :t0], x["done"][b:b + 1, :t0],
                x["S0"][b:b + 1], "elu1" if fmap else "none")[1]
            assert relerr(S_chk[b:b + 1, :, c], want) <= tol, (b, c)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.05])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("save_chk", [True, False])
def test_delta_rule_fwd(shape, p, dtype, save_chk):
    """save_chk=True: the triangular factors come from the chunk-parallel kernel and the sequential
    kernel reads them; False (and no scratch for them): the sequential kernel inverts in place."""
    from memorax_amd import kernels as K
    B, T, H = shape
    x = attn_inputs(B, T, H, p=p, seed=B * 100 + T + H + 7, delta=True)
    print(f"case delta_fwd shape={shape} p={p} dtype={dtype} save_chk={save_chk}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    if dtype == "bf16":
        for n in ("q", "k", "v", "beta"):
            x[n] = bf16_round(x[n])
    o, Sl, chk = K.delta_rule_fwd(dev(x["q"], td), dev(x["k"], td), dev(x["v"], td), dev(x["beta"], td),
                                  dev(x["done"]), dev(x["S0"]), save_chk=save_chk, tm_scratch=False)
    assert (chk is not None) == save_chk
    ro, rSl = M.delta_rule(x["q"], x["k"], x["v"], x["beta"], x["done"], x["S0"])
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    assert relerr(o, ro) <= tol, relerr(o, ro)
    assert relerr(Sl, rSl) <= tol, relerr(Sl, rSl)


def test_reset_isolation_chunked():
    """Poison (NaN) before a reset must not reach the rows after it; done at t=0 ignores S0."""
    from memorax_amd import kernels as K
    B, T, H = 1, 192, 1
    x = attn_inputs(B, T, H, seed=3, delta=True)
    x["done"][:] = False
    x["done"][0, 100] = True
    x["v"][0, 70] = np.nan
    args = [dev(x[n]) for n in ("q", "k", "v", "beta")]
    o, Sl, _ = K.delta_rule_fwd(*args, dev(x["done"]), dev(x["S0"]))
    o = o.cpu().numpy()
    assert np.isfinite(o[0, 100:]).all() and np.isfinite(Sl.cpu().numpy()).all()
    ro, rSl = M.delta_rule(x["q"][:, 100:], x["k"][:, 100:], x["v"][:, 100:], x["beta"][:, 100:],
                           x["done"][:, 100:] & False)
    assert relerr(o[:, 100:], ro) <= TOL_F32 and relerr(Sl, rSl) <= TOL_F32
    o2, _, _ = K.linear_attn_fwd(args[0], args[1], args[2], dev(x["done"]), dev(x["S0"]), 0)
    assert np.isfinite(o2.cpu().numpy()[0, 100:]).all()


def test_config_shapes_small_batch():
    """Benchmark configurations 2 and 4 at a reduced batch, seeded as in the benchmark."""
    from memorax_amd import kernels as K
    x = M.make_inputs(2, (4, 256, 4, 64))
    o, Sl, _ = K.linear_attn_fwd(dev(x["q"]), dev(x["k"]), dev(x["v"]), dev(x["done"]), None, 1)
    ro, rSl = clib.linear_attn_fwd(x["q"], x["k"], x["v"], x["done"], None, 1)
    assert relerr(o, ro) <= TOL_F32 and relerr(Sl, rSl) <= TOL_F32
    x = M.make_inputs(4, (4, 1024, 8, 64))
    xb = {n: bf16_round(x[n]) for n in ("q", "k", "v", "beta")}
    bf = torch.bfloat16
    o, Sl, _ = K.delta_rule_fwd(dev(xb["q"], bf), dev(xb["k"], bf), dev(xb["v"], bf), dev(xb["beta"], bf),
                                dev(x["done"]))
    ro, rSl = clib.delta_rule_fwd(xb["q"], xb["k"], xb["v"], xb["beta"], x["done"])
    assert relerr(o, ro) <= TOL_BF16 and relerr(Sl, rSl) <= TOL_BF16


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("prologue", [False, True])
def test_delta_rule_factor_paths_agree(dtype, prologue):
    """The triangular factors of a chunk depend on its keys, gates and resets only.  Three ways to
    them: the chunk-parallel kernel (residuals asked, device not full), the sequential kernel with
    the factors stored (bf16: more than two sequences per compute unit) and without.  A batch large
    enough for the second way is cut into slices small enough for the first: same outputs and the
    same stored factors, up to rounding; and the backward call accepts either."""
    from memorax_amd import kernels as K
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    H, T = 8, 70
    B = 2 * cus // H + 3  # B*H just above two sequences per compute unit
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    g = torch.Generator(device="cuda").manual_seed(11)
    q, k, v, do = (torch.randn((B, T, H, 64), device="cuda", generator=g).to(td) for _ in range(4))
    if not prologue:
        k = torch.nn.functional.normalize(k.float(), dim=-1).to(td)
    beta = torch.randn((B, T, H), device="cuda", generator=g)
    beta = (beta if prologue else torch.sigmoid(beta)).to(td)
    done = torch.rand((B, T), device="cuda", generator=g) < 0.05
    print(f"case factor_paths dtype={dtype} prologue={prologue} B={B}", flush=True)
    # stored, in place (what the automatic rule picks for bf16 on a full device; float32 always takes the
    # chunk-parallel kernel when it has a buffer, so the path is named)
    o, Sl, chk = K.delta_rule_fwd(q, k, v, beta, done, prologue=prologue, factor_path="inline")
    o2, Sl2, _ = K.delta_rule_fwd(q, k, v, beta, done, save_chk=False, prologue=prologue, tm_scratch=False)
    assert torch.equal(o, o2) and torch.equal(Sl, Sl2)  # the same kernel with and without the stores
    grads = K.delta_rule_bwd(q, k, v, beta, done, chk, do, prologue=prologue)
    for lo in range(0, B, 32):
        sl = slice(lo, min(lo + 32, B))
        args = (q[sl].contiguous(), k[sl].contiguous(), v[sl].contiguous(), beta[sl].contiguous(), done[sl].contiguous())
        o3, Sl3, chk3 = K.delta_rule_fwd(*args, prologue=prologue)                   # chunk-parallel
        o4, Sl4, _ = K.delta_rule_fwd(*args, save_chk=False, prologue=prologue)      # the same through scratch
        assert torch.equal(o3, o4) and torch.equal(Sl3, Sl4)
        assert relerr(o3, o[sl].float().cpu().numpy()) <= tol and relerr(Sl3, Sl[sl].cpu().numpy()) <= tol
        assert relerr(chk3[1], chk[1][sl].float().cpu().numpy()) <= tol
        assert relerr(chk3[0], chk[0][sl].float().cpu().numpy()) <= tol
        g3 = K.delta_rule_bwd(*args, chk3, do[sl].contiguous(), prologue=prologue)
        for a, b_ in zip(g3, grads):
            assert relerr(a, b_[sl].float().cpu().numpy()) <= tol


def test_factor_path_argument():
    """factor_path = parallel takes the chunk-parallel factor kernel on a batch above the occupancy
    threshold, inline never does; same results as each other up to rounding, and the automatic
    choice above the threshold is the inline one bit for bit."""
    from memorax_amd import kernels as K
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    H, T = 8, 70
    B = 2 * cus // H + 3
    g = torch.Generator(device="cuda").manual_seed(5)
    q, k, v = (torch.randn((B, T, H, 64), device="cuda", generator=g).to(torch.bfloat16) for _ in range(3))
    k = torch.nn.functional.normalize(k.float(), dim=-1).to(torch.bfloat16)
    beta = torch.rand((B, T, H), device="cuda", generator=g).to(torch.bfloat16)
    done = torch.rand((B, T), device="cuda", generator=g) < 0.05
    out = {}
    for path in ("inline", "parallel", "auto"):
        print(f"case factor_path {path}", flush=True)
        o, Sl, chk = K.delta_rule_fwd(q, k, v, beta, done, factor_path=path)
        out[path] = dict(o=o.float().cpu().numpy(), Sl=Sl.cpu().numpy(), Tm=chk[1].float().cpu().numpy())
    a, b = out["inline"], out["parallel"]
    assert not np.array_equal(a["Tm"], b["Tm"])  # two different kernels made the factors
    for n in ("o", "Sl", "Tm"):
        assert relerr(torch.from_numpy(a[n]), b[n]) <= TOL_BF16, n
        assert np.array_equal(out["auto"][n], a[n]), n
    with pytest.raises(KeyError):
        K.delta_rule_fwd(q, k, v, beta, done, factor_path="sideways")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("tm_path", ["parallel", "inline"])
def test_delta_rule_correlated_keys(dtype, tm_path):
    """Keys that change slowly from step to step (AR(1), rho = 0.95, normalised) and gates near one make
    I + tril(diag(beta) K K^T) badly conditioned for repeated squaring: the powers of N grow and cancel.
    Both routes to the triangular factors must hold the tolerance there (forward and backward)."""
    from memorax_amd import kernels as K
    from oracle import grad as G
    B, T, H = 2, 96, 2
    rng = np.random.default_rng(42)
    z = rng.standard_normal((B, T, H, 64))
    for t in range(1, T):
        z[:, t] = 0.95 * z[:, t - 1] + np.sqrt(1 - 0.95 ** 2) * z[:, t]
    k = (z / np.linalg.norm(z, axis=-1, keepdims=True)).astype(np.float32)
    q = rng.standard_normal((B, T, H, 64)).astype(np.float32)
    v = rng.standard_normal((B, T, H, 64)).astype(np.float32)
    beta = rng.uniform(0.5, 1.0, (B, T, H)).astype(np.float32)
    do = rng.standard_normal((B, T, H, 64)).astype(np.float32)
    done = np.zeros((B, T), bool)
    done[1, 40] = True
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    if dtype == "bf16":
        q, k, v, beta, do = (bf16_round(a) for a in (q, k, v, beta, do))
    print(f"case correlated keys dtype={dtype} path={tm_path}", flush=True)
    tq, tk, tv, tb, tdo = (dev(a, td) for a in (q, k, v, beta, do))
    if tm_path == "parallel":
        o, Sl, chk = K.delta_rule_fwd(tq, tk, tv, tb, dev(done))
    else:
        o, Sl, _ = K.delta_rule_fwd(tq, tk, tv, tb, dev(done), save_chk=False, tm_scratch=False)
        chk = None
    ref = G.delta_rule_grads(q, k, v, beta, done, None, do)
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    assert relerr(o, ref["o"]) <= tol and relerr(Sl, ref["S_last"]) <= tol, (relerr(o, ref["o"]), relerr(Sl, ref["S_last"]))
    if chk is not None:
        got = K.delta_rule_bwd(tq, tk, tv, tb, dev(done), chk, tdo)
        errs = {n: relerr(g, ref[n]) for n, g in zip(("dq", "dk", "dv", "dbeta", "dS0"), got)}
        assert all(e <= tol for e in errs.values()), errs
