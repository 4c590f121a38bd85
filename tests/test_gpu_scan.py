"""GPU parity of the diagonal scan (through the C ABI) against the fp64 oracle."""
import numpy as np
import pytest
import torch

from oracle import grad as G
from oracle import memoroid as M

pytestmark = pytest.mark.gpu
TOL = 1e-4  # fp32 max rel err (max|x-y| / max|y|)


def relerr(x, y):
    x = x.detach().cpu().numpy() if isinstance(x, torch.Tensor) else np.asarray(x)
    return float(np.abs(x - y).max() / max(np.abs(y).max(), 1e-30))


def dev(x):
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


SHAPES = [
    (32, 128, 256),   # benchmark configuration 1 (time split over waves)
    (1, 1, 1), (2, 1, 64), (3, 7, 5), (2, 9, 130), (5, 200, 64), (4, 300, 258),
    (64, 64, 1024),   # wide: vectorised, no time split (backward: two lanes per thread, eight waves)
    (32, 160, 1024),  # backward: two lanes per thread, time split over sixteen waves, ragged second super-step
    (2, 1000, 8),
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.05])
def test_scan_fwd_bwd_f32(shape, p):
    from memorax_amd import kernels as K
    B, T, D = shape
    rng = np.random.default_rng(B * 1000 + T * 10 + D)
    a = rng.uniform(0.9, 0.999, shape).astype(np.float32)
    b = rng.standard_normal(shape).astype(np.float32)
    h0 = rng.standard_normal((B, D)).astype(np.float32)
    P0 = rng.uniform(0.5, 1.0, (B, D)).astype(np.float32)
    done = rng.random((B, T)) < p
    print(f"case scan f32 shape={shape} p={p}", flush=True)
    h, hl, Pl = K.linear_scan_fwd(dev(a), dev(b), dev(done), dev(h0), dev(P0))
    rh, rhl, rPl = M.diag_scan(a, b, done, h0, P0)
    assert relerr(h, rh) <= TOL and relerr(hl, rhl) <= TOL and relerr(Pl, rPl) <= TOL
    g = rng.standard_normal(shape).astype(np.float32)
    gl = rng.standard_normal((B, D)).astype(np.float32)
    da, db, dh0 = K.linear_scan_bwd(dev(a), h, dev(done), dev(h0), dev(g), dev(gl))
    rda, rdb, rdh0 = M.diag_scan_bwd(a, rh, done, g, h0, gl)
    assert relerr(da, rda) <= TOL and relerr(db, rdb) <= TOL and relerr(dh0, rdh0) <= TOL


def test_scan_config1_seeded_and_null_optionals():
    from memorax_amd import kernels as K
    x = M.make_inputs(1)
    h, hl, Pl = K.linear_scan_fwd(dev(x["a"]), dev(x["b"]), dev(x["done"]))
    rh, rhl, rPl = M.diag_scan(x["a"], x["b"], x["done"])
    assert relerr(h, rh) <= TOL and relerr(hl, rhl) <= TOL and relerr(Pl, rPl) <= TOL
    g = np.ones_like(x["a"])
    da, db, dh0 = K.linear_scan_bwd(dev(x["a"]), h, dev(x["done"]), None, dev(g), None)
    rda, rdb, _ = M.diag_scan_bwd(x["a"], rh, x["done"], g)
    assert relerr(da, rda) <= TOL and relerr(db, rdb) <= TOL


@pytest.mark.parametrize("done_dtype", ["bool", "uint8", "float32"])
def test_scan_done_dtypes_and_reset_isolation(done_dtype):
    from memorax_amd import kernels as K
    B, T, D = 4, 96, 64
    rng = np.random.default_rng(5)
    a = rng.uniform(0.9, 0.999, (B, T, D)).astype(np.float32)
    b = rng.standard_normal((B, T, D)).astype(np.float32)
    done = np.zeros((B, T), bool)
    done[:, 40] = True
    done[1, 0] = True
    b[:, 13] = np.nan          # poison left of the reset
    a[:, 20] = np.inf
    dd = {"bool": done, "uint8": done.astype(np.uint8), "float32": done.astype(np.float32)}[done_dtype]
    h, hl, Pl = K.linear_scan_fwd(dev(a), dev(b), dev(dd))
    h = h.cpu().numpy()
    assert np.isfinite(h[:, 40:]).all() and np.isfinite(hl.cpu().numpy()).all()
    assert np.isfinite(Pl.cpu().numpy()).all()
    np.testing.assert_array_equal(h[:, 40], b[:, 40])   # reset step == its own element, exactly
    rh, _, _ = M.diag_scan(a[:, 40:], b[:, 40:], done[:, 40:] & False)
    assert relerr(h[:, 40:], rh) <= TOL


def test_scan_split_invariance_on_gpu():
    from memorax_amd import kernels as K
    B, T, D = 3, 160, 96
    rng = np.random.default_rng(9)
    a = rng.uniform(0.9, 0.999, (B, T, D)).astype(np.float32)
    b = rng.standard_normal((B, T, D)).astype(np.float32)
    done = rng.random((B, T)) < 0.03
    h, hl, Pl = K.linear_scan_fwd(dev(a), dev(b), dev(done))
    for s in (1, 63, 64, 100):
        h1, hl1, P1 = K.linear_scan_fwd(dev(a[:, :s]), dev(b[:, :s]), dev(done[:, :s]))
        h2, hl2, P2 = K.linear_scan_fwd(dev(a[:, s:]), dev(b[:, s:]), dev(done[:, s:]), hl1, P1)
        assert relerr(torch.cat([h1, h2], 1), h.cpu().numpy()) <= 1e-5
        assert relerr(hl2, hl.cpu().numpy()) <= 1e-5 and relerr(P2, Pl.cpu().numpy()) <= 1e-5


@pytest.mark.parametrize("ti", [False, True])
def test_scan_complex64(ti):
    from memorax_amd import kernels as K
    B, T, D = 3, 77, 48
    rng = np.random.default_rng(21)
    lam = (0.95 * np.exp(1j * rng.uniform(0, 3, (D,) if ti else (B, T, D)))).astype(np.complex64)
    b = (rng.standard_normal((B, T, D)) + 1j * rng.standard_normal((B, T, D))).astype(np.complex64)
    h0 = (rng.standard_normal((B, D)) + 1j * rng.standard_normal((B, D))).astype(np.complex64)
    g = (rng.standard_normal((B, T, D)) + 1j * rng.standard_normal((B, T, D))).astype(np.complex64)
    done = rng.random((B, T)) < 0.04
    h, hl, Pl = K.linear_scan_fwd(dev(lam), dev(b), dev(done), dev(h0))
    rh, rhl, rPl = M.diag_scan(lam, b, done, h0)
    assert relerr(h, rh) <= TOL and relerr(hl, rhl) <= TOL and relerr(Pl, rPl) <= TOL
    da, db, dh0 = K.linear_scan_bwd(dev(lam), h, dev(done), dev(h0), dev(g))
    ag = G.diag_scan_grads(np.broadcast_to(lam, (B, T, D)).copy(), b, done, h0, g)
    assert relerr(da, ag["da"]) <= TOL and relerr(db, ag["db"]) <= TOL and relerr(dh0, ag["dh0"]) <= TOL


@pytest.mark.parametrize("dtype", ["f32", "c64"])
@pytest.mark.parametrize("shape", [(3, 77, 48), (2, 1, 5), (64, 128, 256), (1024, 128, 64), (4, 300, 1024), (2, 1000, 130)])
def test_time_invariant_coefficient_gradient_summed_inside_the_kernel(dtype, shape):
    """a_time_invariant = 2: da comes back as (B,D), the per-step terms summed over the sequence by the kernel
    (both kernel families: the shapes cover the wave-split and the streaming plans) -- against the oracle's
    gradient of the broadcast coefficient and against the per-step array summed afterwards."""
    from memorax_amd import kernels as K
    B, T, D = shape
    rng = np.random.default_rng(B + T + D)
    cplx = dtype == "c64"
    rnd = (lambda *s: (rng.standard_normal(s) + 1j * rng.standard_normal(s)).astype(np.complex64)) if cplx \
        else (lambda *s: rng.standard_normal(s).astype(np.float32))
    lam = (rng.uniform(0.8, 0.999, D) * (np.exp(1j * rng.uniform(0, 3, D)) if cplx else 1.0)).astype(np.complex64 if cplx else np.float32)
    b, g, h0, gl = rnd(B, T, D), rnd(B, T, D), rnd(B, D), rnd(B, D)
    done = rng.random((B, T)) < 0.03
    print(f"case scan da summed dtype={dtype} shape={shape}", flush=True)
    h, _, _ = K.linear_scan_fwd(dev(lam), dev(b), dev(done), dev(h0))
    da_steps, db1, dh01 = K.linear_scan_bwd(dev(lam), h, dev(done), dev(h0), dev(g), dev(gl))
    da_sum, db2, dh02 = K.linear_scan_bwd(dev(lam), h, dev(done), dev(h0), dev(g), dev(gl), sum_da=True)
    assert da_sum.shape == (B, D) and torch.equal(db1, db2) and torch.equal(dh01, dh02)
    ref_steps = da_steps.cpu().numpy().astype(np.complex128 if cplx else np.float64).sum(1)
    assert relerr(da_sum, ref_steps) <= TOL
    if B * T * D <= 2_000_000:  # the oracle's autograd on the broadcast coefficient
        ag = G.diag_scan_grads(np.broadcast_to(lam, (B, T, D)).copy(), b, done, h0, g, gl)
        assert relerr(da_sum.sum(0), ag["da"].sum((0, 1))) <= TOL


def test_linear_scan_autograd_function():
    import memorax_amd as mx
    B, T, D = 4, 50, 32
    rng = np.random.default_rng(3)
    a = rng.uniform(0.9, 0.999, (B, T, D)).astype(np.float32)
    b = rng.standard_normal((B, T, D)).astype(np.float32)
    h0 = rng.standard_normal((B, D)).astype(np.float32)
    g = rng.standard_normal((B, T, D)).astype(np.float32)
    gl = rng.standard_normal((B, D)).astype(np.float32)
    done = rng.random((B, T)) < 0.05
    ta, tb, th0 = (dev(x).requires_grad_() for x in (a, b, h0))
    h, hl, _ = mx.linear_scan(ta, tb, dev(done), th0)
    ((h * dev(g)).sum() + (hl * dev(gl)).sum()).backward()
    ag = G.diag_scan_grads(a, b, done, h0, g, gl)
    assert relerr(ta.grad, ag["da"]) <= TOL and relerr(tb.grad, ag["db"]) <= TOL
    assert relerr(th0.grad, ag["dh0"]) <= TOL


@pytest.mark.parametrize("dtype", ["f32", "c64"])
@pytest.mark.parametrize("shape", [(2, 9, 3, (2, 2)), (3, 130, 16, (8,)), (1, 1, 4, ()), (2, 64, 5, (3,)), (4, 257, 32, (16, 4))])
def test_propagate_sensitivities(dtype, shape):
    """RTRL sensitivity update (memoroid.py:114-141) through mrx_linear_scan_last."""
    from memorax_amd.functional import propagate_sensitivities
    B, T, H, ps = shape
    rng = np.random.default_rng(B * 7 + T + H)
    cplx = dtype == "c64"
    rnd = (lambda *s: (rng.standard_normal(s) + 1j * rng.standard_normal(s)).astype(np.complex64)) if cplx \
        else (lambda *s: rng.standard_normal(s).astype(np.float32))
    decay = (rng.uniform(0.6, 1.0, (B, T, H)) * (np.exp(1j * rng.uniform(0, 6.28, (B, T, H))) if cplx else 1.0))
    decay = decay.astype(np.complex64 if cplx else np.float32)
    J = {"w": rnd(B, T, H, *ps), "u": rnd(B, T, H)}
    S = {"w": rnd(B, 1, H, *ps), "u": rnd(B, 1, H)}
    done = rng.random((B, T)) < 0.05
    print(f"case rtrl dtype={dtype} shape={shape}", flush=True)
    out = propagate_sensitivities(dev(decay), {k: dev(v) for k, v in J.items()}, {k: dev(v) for k, v in S.items()},
                                  dev(done))
    ref = M.propagate_sensitivities(decay, J, S, done)
    for name in J:
        assert out[name].shape == S[name].shape
        assert relerr(out[name], ref[name]) <= 1e-4, (name, relerr(out[name], ref[name]))


@pytest.mark.parametrize("shape", [(3, 77, 48), (2, 1, 5), (64, 128, 256), (4, 300, 1024), (512, 128, 64)])
@pytest.mark.parametrize("ti", [False, True])
def test_scan_bfloat16_arrays_float32_arithmetic(shape, ti):
    """a, b, h, g, da, db in bfloat16; arithmetic, carries and a summed da in float32."""
    from memorax_amd import kernels as K
    B, T, D = shape
    rng = np.random.default_rng(B + 3 * T + D)
    rb = lambda x: torch.from_numpy(x.astype(np.float32)).bfloat16().float().numpy()  # round to bfloat16
    a = rb(rng.uniform(0.8, 0.999, (D,) if ti else shape))
    b, g = rb(rng.standard_normal(shape)), rb(rng.standard_normal(shape))
    h0, gl = rng.standard_normal((B, D)).astype(np.float32), rng.standard_normal((B, D)).astype(np.float32)
    P0 = rng.uniform(0.5, 1.0, (B, D)).astype(np.float32)
    done = rng.random((B, T)) < 0.04
    print(f"case scan bf16 shape={shape} ti={ti}", flush=True)
    bf = torch.bfloat16
    h, hl, Pl = K.linear_scan_fwd(dev(a).to(bf), dev(b).to(bf), dev(done), dev(h0), dev(P0))
    assert h.dtype == bf and hl.dtype == torch.float32 and Pl.dtype == torch.float32
    rh, rhl, rPl = M.diag_scan(a, b, done, h0, P0)
    assert relerr(h.float(), rh) <= 2e-2 and relerr(hl, rhl) <= TOL and relerr(Pl, rPl) <= TOL
    da, db, dh0 = K.linear_scan_bwd(dev(a).to(bf), h, dev(done), dev(h0), dev(g).to(bf), dev(gl), sum_da=ti)
    ag = G.diag_scan_grads(np.broadcast_to(a, shape).copy(), b, done, h0, g, gl)
    assert db.dtype == bf and dh0.dtype == torch.float32 and da.dtype == (torch.float32 if ti else bf)
    assert relerr(db.float(), ag["db"]) <= 2e-2 and relerr(dh0, ag["dh0"]) <= 2e-2
    if ti:
        assert da.shape == (B, D) and relerr(da.sum(0), ag["da"].sum((0, 1))) <= 2e-2
    else:
        assert relerr(da.float(), ag["da"]) <= 2e-2
