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
    # first checkpoint is the incoming state
    assert relerr(chk[:, :, 0], x["S0"]) <= (1e-2 if dtype == "bf16" else 1e-6)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.05])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_delta_rule_fwd(shape, p, dtype):
    from memorax_amd import kernels as K
    B, T, H = shape
    x = attn_inputs(B, T, H, p=p, seed=B * 100 + T + H + 7, delta=True)
    print(f"case delta_fwd shape={shape} p={p} dtype={dtype}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    if dtype == "bf16":
        for n in ("q", "k", "v", "beta"):
            x[n] = bf16_round(x[n])
    o, Sl, chk = K.delta_rule_fwd(dev(x["q"], td), dev(x["k"], td), dev(x["v"], td), dev(x["beta"], td),
                                  dev(x["done"]), dev(x["S0"]))
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
