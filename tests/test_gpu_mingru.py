"""GPU parity of the MinGRU scan with the gate arithmetic inside (mrx_mingru_scan_fwd / _bwd, through
the C ABI) against the oracle's log-space route (the reference's own formulation) and its gradients."""
import numpy as np
import pytest
import torch

from oracle import grad as G
from oracle import memoroid as M
from gpu_util import TOL_F32 as TOL, dev, relerr

pytestmark = pytest.mark.gpu

SHAPES = [
    (32, 128, 256),   # time split over waves
    (1, 1, 1), (2, 1, 64), (3, 7, 5), (2, 9, 130), (5, 200, 64), (4, 300, 258),
    (64, 64, 1024),   # streaming kernels, 16-byte vectors
    (40, 50, 516),    # D a multiple of 4 but not of 64: a partly filled last tile
    (2, 1000, 8),
    (1536, 131, 128),  # a call that moves over 600 MB: the streaming backward forms h again inside its groups of steps
]


def _ref(z, x, done, h0, P0):
    carry = None if h0 is None else (np.log(h0)[:, None], np.log(P0)[:, None])
    nxt, h = M.mingru_scan(z, x, done, carry)
    return h, np.exp(nxt[0][:, 0]), np.exp(nxt[1][:, 0])


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.05])
def test_mingru_scan_fwd_bwd(shape, p):
    from memorax_amd import kernels as K
    B, T, D = shape
    rng = np.random.default_rng(B * 1000 + T * 10 + D)
    z = (2 * rng.standard_normal(shape)).astype(np.float32)
    x = (2 * rng.standard_normal(shape)).astype(np.float32)
    h0 = np.exp(rng.standard_normal((B, D))).astype(np.float32)
    P0 = rng.uniform(0.5, 1.0, (B, D)).astype(np.float32)
    done = rng.random((B, T)) < p
    print(f"case mingru shape={shape} p={p}", flush=True)
    h, hl, Pl = K.mingru_scan_fwd(dev(z), dev(x), dev(done), dev(h0), dev(P0))
    rh, rhl, rPl = _ref(z, x, done, h0, P0)
    assert relerr(h, rh) <= TOL and relerr(hl, rhl) <= TOL and relerr(Pl, rPl) <= TOL
    g = rng.standard_normal(shape).astype(np.float32)
    gl = rng.standard_normal((B, D)).astype(np.float32)
    dz, dx, dh0 = K.mingru_scan_bwd(dev(z), dev(x), h, dev(done), dev(h0), dev(g), dev(gl))
    # reference gradients from the linear-space closed form (pinned against autograd through the
    # log-space restatement and finite differences on the CPU), in fp64 on the oracle's states
    a, b = M.mingru_linear_coeffs(z, x)
    hh, _, _ = M.diag_scan(a, b, done, h0)
    da, lam, rdh0 = M.diag_scan_bwd(a, hh, done, g, h0, gl)
    s = M.sigmoid(z.astype(np.float64))
    x64 = x.astype(np.float64)
    rdz = s * (1 - s) * (np.where(x64 >= 0, x64 + 0.5, M.sigmoid(x64)) * lam - da)
    rdx = lam * s * np.where(x64 >= 0, 1.0, M.sigmoid(x64) * (1 - M.sigmoid(x64)))
    assert relerr(dz, rdz) <= TOL and relerr(dx, rdx) <= TOL and relerr(dh0, rdh0) <= TOL
    if B * T * D > 1 << 24:   # the large call once more with float32 flags: the same kernel on the other flag type
        dz2, dx2, dh02 = K.mingru_scan_bwd(dev(z), dev(x), h, dev(done.astype(np.float32)), dev(h0), dev(g), dev(gl))
        assert torch.equal(dz2, dz) and torch.equal(dx2, dx) and torch.equal(dh02, dh0)


def test_mingru_autograd_function_against_the_log_space_autograd_oracle():
    import memorax_amd as mx
    B, T, D = 4, 50, 32
    rng = np.random.default_rng(3)
    z = (2 * rng.standard_normal((B, T, D))).astype(np.float32)
    x = (2 * rng.standard_normal((B, T, D))).astype(np.float32)
    h0 = np.exp(rng.standard_normal((B, D))).astype(np.float32)
    g = rng.standard_normal((B, T, D)).astype(np.float32)
    gl = rng.standard_normal((B, D)).astype(np.float32)
    done = rng.random((B, T)) < 0.05
    tz, tx, th0 = (dev(v).requires_grad_() for v in (z, x, h0))
    h, hl, _ = mx.functional.mingru_scan(tz, tx, dev(done), th0)
    ((h * dev(g)).sum() + (hl * dev(gl)).sum()).backward()
    ag = G.mingru_grads(z, x, done, h0, g, gl)
    assert relerr(tz.grad, ag["dz"]) <= TOL and relerr(tx.grad, ag["dh_tilde"]) <= TOL
    assert relerr(th0.grad, ag["dh0"]) <= TOL


@pytest.mark.parametrize("done_dtype", ["bool", "float32"])
def test_mingru_null_carry_extreme_gates_and_reset_isolation(done_dtype):
    """The cell's initial carry (h0 = 0: exp(-inf)), gates far in both tails (sigma(-z) must stay a
    relative-precision small number, not 1 - sigma(z)), and NaN before a reset staying there."""
    from memorax_amd import kernels as K
    B, T, D = 4, 96, 64
    rng = np.random.default_rng(5)
    z = (3 * rng.standard_normal((B, T, D))).astype(np.float32)
    x = (3 * rng.standard_normal((B, T, D))).astype(np.float32)
    z[:, 50] = 30.0     # sigma(-30) = 9.4e-14
    z[:, 60] = -40.0
    x[:, 70] = -100.0   # g = sigma(-100) = 0 in fp32
    done = np.zeros((B, T), bool)
    done[:, 40] = True
    done[1, 0] = True
    zp, xp = z.copy(), x.copy()
    zp[:, 13] = np.nan
    xp[:, 20] = np.inf
    dd = done if done_dtype == "bool" else done.astype(np.float32)
    h, hl, Pl = K.mingru_scan_fwd(dev(zp), dev(xp), dev(dd))
    hn = h.cpu().numpy()
    assert np.isfinite(hn[:, 40:]).all() and np.isfinite(hl.cpu().numpy()).all() and np.isfinite(Pl.cpu().numpy()).all()
    rh, rhl, rPl = _ref(z[:, 40:], x[:, 40:], done[:, 40:], None, None)
    assert relerr(hn[:, 40:], rh) <= TOL and relerr(hl, rhl) <= TOL
    # the cumulative decay spans 50 orders of magnitude: compare its logarithm where fp32 can hold
    # the product, and expect an underflow towards 0 where it cannot (a linear-space leaf)
    Pn = Pl.cpu().numpy().astype(np.float64)
    ok = rPl > 1e-30
    assert (Pn[~ok] <= 1e-29).all() and (not ok.any() or np.abs(np.log(Pn[ok]) - np.log(rPl[ok])).max() <= 1e-3)
    # steps 48..55 alone hold sigma(-30) among ordinary gates: a product fp32 can hold
    _, _, Ps = K.mingru_scan_fwd(dev(z[:, 48:56]), dev(x[:, 48:56]), dev(dd[:, 48:56]))
    _, _, rPs = _ref(z[:, 48:56], x[:, 48:56], done[:, 48:56], None, None)
    assert rPs.min() > 1e-30 and np.abs(np.log(Ps.cpu().numpy().astype(np.float64)) - np.log(rPs)).max() <= 1e-3
    g = rng.standard_normal((B, T, D)).astype(np.float32)
    dz, dx, _ = K.mingru_scan_bwd(dev(zp), dev(xp), h, dev(dd), None, dev(g))
    assert np.isfinite(dz.cpu().numpy()[:, 40:]).all() and np.isfinite(dx.cpu().numpy()[:, 40:]).all()
    ag = G.mingru_grads(z[:, 40:], x[:, 40:], done[:, 40:], None, g[:, 40:])
    assert relerr(dz[:, 40:], ag["dz"]) <= TOL and relerr(dx[:, 40:], ag["dh_tilde"]) <= TOL


def test_mingru_cell_fused_and_unfused_agree_and_match_the_reference_route():
    from memorax_amd import sequence_models as sm
    torch.manual_seed(1)
    B, T, Fe = 4, 90, 16
    cell = sm.MinGRUCell(Fe).cuda()
    model = sm.Memoroid(cell)
    x = torch.randn(B, T, Fe, device="cuda")
    done = torch.rand(B, T, device="cuda") < 0.04
    carry, y = model(x, done)
    y.sum().backward()
    gz, gh = cell.z.weight.grad.clone(), cell.h.weight.grad.clone()
    cell.zero_grad()
    cell.fused = False
    carry2, y2 = model(x, done)
    y2.sum().backward()
    assert relerr(y, y2.detach().cpu().numpy()) <= 1e-5
    assert relerr(carry[0], carry2[0].detach().cpu().numpy()) <= 1e-5 and relerr(carry[1], carry2[1].detach().cpu().numpy()) <= 1e-5
    assert relerr(gz, cell.z.weight.grad.cpu().numpy()) <= 1e-4 and relerr(gh, cell.h.weight.grad.cpu().numpy()) <= 1e-4
    nxt, rh = M.mingru_scan(cell.z(x).detach().cpu().numpy(), cell.h(x).detach().cpu().numpy(), done.float().cpu().numpy())
    assert relerr(y, rh) <= TOL and relerr(carry[0], nxt[0]) <= TOL and relerr(carry[1], nxt[1]) <= TOL


@pytest.mark.parametrize("shape", [(2, 1, 5), (3, 77, 48), (4, 300, 258), (64, 128, 256), (16, 1000, 130), (512, 128, 64),
                                   (3072, 131, 128)])   # the last: over 600 MB moved, h formed again in the backward
@pytest.mark.parametrize("p", [0.0, 0.05])
def test_bfloat16_arrays_float32_arithmetic(shape, p):
    """z, h~, h, g, dz, dh~ in bfloat16, arithmetic and carries in float32: against the oracle on the rounded
    inputs, within the bf16-in / fp32-accumulate tolerance (the backward walks the stored, rounded states, as
    the gradient of a function with a rounded output does)."""
    from memorax_amd import kernels as K
    from gpu_util import TOL_BF16, bf16_round
    B, T, D = shape
    rng = np.random.default_rng(B * 1000 + T * 10 + D + 1)
    z = bf16_round((2 * rng.standard_normal(shape)).astype(np.float32))
    x = bf16_round((2 * rng.standard_normal(shape)).astype(np.float32))
    g = bf16_round(rng.standard_normal(shape).astype(np.float32))
    h0 = np.exp(rng.standard_normal((B, D))).astype(np.float32)
    P0 = rng.uniform(0.5, 1.0, (B, D)).astype(np.float32)
    gl = rng.standard_normal((B, D)).astype(np.float32)
    done = rng.random((B, T)) < p
    print(f"case mingru bf16 shape={shape} p={p}", flush=True)
    bf = torch.bfloat16
    h, hl, Pl = K.mingru_scan_fwd(dev(z).to(bf), dev(x).to(bf), dev(done), dev(h0), dev(P0))
    assert h.dtype == bf and hl.dtype == torch.float32 and Pl.dtype == torch.float32
    rh, rhl, rPl = _ref(z, x, done, h0, P0)
    assert relerr(h.float(), rh) <= TOL_BF16 and relerr(hl, rhl) <= 1e-4 and relerr(Pl, rPl) <= 1e-4
    dz, dx, dh0 = K.mingru_scan_bwd(dev(z).to(bf), dev(x).to(bf), h, dev(done), dev(h0), dev(g).to(bf), dev(gl))
    assert dz.dtype == bf and dx.dtype == bf and dh0.dtype == torch.float32
    a, b = M.mingru_linear_coeffs(z, x)
    hh, _, _ = M.diag_scan(a, b, done, h0)
    da, lam, rdh0 = M.diag_scan_bwd(a, hh, done, g, h0, gl)
    s = M.sigmoid(z.astype(np.float64))
    x64 = x.astype(np.float64)
    rdz = s * (1 - s) * (np.where(x64 >= 0, x64 + 0.5, M.sigmoid(x64)) * lam - da)
    rdx = lam * s * np.where(x64 >= 0, 1.0, M.sigmoid(x64) * (1 - M.sigmoid(x64)))
    assert relerr(dz.float(), rdz) <= TOL_BF16 and relerr(dx.float(), rdx) <= TOL_BF16 and relerr(dh0, rdh0) <= TOL_BF16


def test_bfloat16_autograd_function_and_cell():
    """functional.mingru_scan on bfloat16 projections (what a bf16 torso hands over): states in bfloat16, carries
    and their gradients in float32, the projections' gradients in bfloat16."""
    import memorax_amd as mx
    from gpu_util import TOL_BF16
    B, T, D = 4, 90, 64
    rng = np.random.default_rng(11)
    z = torch.from_numpy((2 * rng.standard_normal((B, T, D))).astype(np.float32)).cuda().bfloat16().requires_grad_()
    x = torch.from_numpy((2 * rng.standard_normal((B, T, D))).astype(np.float32)).cuda().bfloat16().requires_grad_()
    h0 = torch.from_numpy(np.exp(rng.standard_normal((B, D))).astype(np.float32)).cuda().requires_grad_()
    done = torch.from_numpy(rng.random((B, T)) < 0.05).cuda()
    h, hl, Pl = mx.mingru_scan(z, x, done, h0)
    assert h.dtype == torch.bfloat16 and hl.dtype == torch.float32
    (h.float().sum() + hl.sum()).backward()
    assert z.grad.dtype == torch.bfloat16 and x.grad.dtype == torch.bfloat16 and h0.grad.dtype == torch.float32
    zf, xf, h0f = (t.detach().float().requires_grad_() for t in (z, x, h0))
    hf, hlf, _ = mx.mingru_scan(zf, xf, done, h0f)
    (hf.sum() + hlf.sum()).backward()
    assert relerr(h.float(), hf.detach().cpu().numpy()) <= TOL_BF16
    for a, b in ((z.grad, zf.grad), (x.grad, xf.grad), (h0.grad, h0f.grad)):
        assert relerr(a.float(), b.cpu().numpy()) <= TOL_BF16
