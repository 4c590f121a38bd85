"""The norm kernels (mrx_rms_norm_fwd / _bwd, mrx_layer_norm_fwd / _bwd, through the C ABI) against the oracle: y of
oracle.memoroid.rms_norm / layer_norm and the gradients of oracle.grad.rms_norm_grads / layer_norm_grads (torch-fp64
autograd, pinned by closed forms and finite differences in tests/test_oracle_grad.py).  Tolerances: float32 arrays 1e-5 of the
result's scale; bfloat16 arrays 2e-2 (one rounding of the stored result, 2^-9, and of the inputs read)."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import grad as G
from oracle import memoroid as M
from gpu_util import dev

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def _close(got, want, tol, what):
    got = got.float().cpu().numpy().astype(np.float64)
    scale = np.abs(want).max() + 1e-30
    err = np.abs(got - want).max() / scale
    assert err <= tol, f"{what}: {err:.3e} of scale {scale:.3e} (allowed {tol})"


def _as(a, dtype):
    """Array on the device in dtype, and the float64 values the kernel then reads."""
    t = dev(a.astype(np.float32)).to(dtype)
    return t, t.float().cpu().numpy().astype(np.float64)


@pytest.mark.parametrize("rows,D", [(1, 4), (7, 256), (1000, 260), (33, 512), (5, 1024), (3, 2048), (4099, 64), (16384, 256)])
@pytest.mark.parametrize("x_dtype,y_dtype", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16),
                                             (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32)])
def test_forward_and_backward(rows, D, x_dtype, y_dtype):
    from memorax_amd import kernels as K
    rng = np.random.default_rng(rows + D)
    print(f"case rms norm rows={rows} D={D} x={x_dtype} y={y_dtype}", flush=True)
    x, xr = _as(rng.standard_normal((rows, D)) * np.exp(rng.standard_normal((rows, 1))), x_dtype)   # row scales over a decade
    sc = (1.0 + 0.3 * rng.standard_normal(D)).astype(np.float32)
    dy, dyr = _as(rng.standard_normal((rows, D)), y_dtype)
    y = K.rms_norm_fwd(x, dev(sc), 1e-6, y_dtype)
    assert y.dtype == y_dtype and y.shape == x.shape
    _close(y, M.rms_norm(xr, sc, 1e-6), TOL[y_dtype], "y")
    dx, dscale = K.rms_norm_bwd(x, dev(sc), dy, 1e-6)
    rdx, rds = G.rms_norm_grads(xr, sc.astype(np.float64), dyr, 1e-6)
    assert dx.dtype == x_dtype and dscale.dtype == torch.float32
    # dx per row on the row's own scale (rows differ by a decade)
    got = dx.float().cpu().numpy().astype(np.float64)
    err = (np.abs(got - rdx).max(-1) / (np.abs(rdx).max(-1) + 1e-30)).max()
    assert err <= TOL[x_dtype], f"dx: {err:.3e}"
    _close(dscale, rds, 1e-5 * max(1.0, np.sqrt(rows) / 30), "dscale")   # a float32 sum over the rows
    # a gradient that reaches x by another way is added in the same pass
    add, addr = _as(rng.standard_normal((rows, D)), x_dtype)
    dx2, dscale2 = K.rms_norm_bwd(x, dev(sc), dy, 1e-6, dx_add=add)
    got = dx2.float().cpu().numpy().astype(np.float64)
    err = (np.abs(got - (rdx + addr)).max(-1) / (np.abs(rdx + addr).max(-1) + 1e-30)).max()
    assert err <= TOL[x_dtype], f"dx with dx_add: {err:.3e}"
    assert torch.equal(dscale2, dscale)
    # no scale: ones, and no gradient for it
    y1 = K.rms_norm_fwd(x, None, 1e-6, y_dtype)
    _close(y1, M.rms_norm(xr, None, 1e-6), TOL[y_dtype], "y without scale")
    dx1, none = K.rms_norm_bwd(x, None, dy, 1e-6, want_dscale=False)
    assert none is None
    rdx1, _ = G.rms_norm_grads(xr, None, dyr, 1e-6)
    err = (np.abs(dx1.float().cpu().numpy() - rdx1).max(-1) / (np.abs(rdx1).max(-1) + 1e-30)).max()
    assert err <= TOL[x_dtype], f"dx without scale: {err:.3e}"


def test_random_widths_and_row_counts():
    """Thirty drawn (rows, D): every width class of the kernels (one to eight 256-column groups per lane, widths that
    leave lanes and whole groups empty), row counts around the waves' strides."""
    from memorax_amd import kernels as K
    rng = np.random.default_rng(77)
    for case in range(30):
        D = 4 * int(rng.integers(1, 513))
        rows = int(rng.choice([1, 2, 3, 5, 17, 63, 257, 1025, 4097, 20001]))
        xd, yd = (torch.float32, torch.bfloat16)[int(rng.integers(2))], (torch.float32, torch.bfloat16)[int(rng.integers(2))]
        print(f"case rms norm random {case}: rows={rows} D={D} x={xd} y={yd}", flush=True)
        x, xr = _as(rng.standard_normal((rows, D)) * 2.0, xd)
        dy, dyr = _as(rng.standard_normal((rows, D)), yd)
        sc = (1.0 + 0.3 * rng.standard_normal(D)).astype(np.float32)
        _close(K.rms_norm_fwd(x, dev(sc), 1e-6, yd), M.rms_norm(xr, sc, 1e-6), TOL[yd], "y")
        dx, ds = K.rms_norm_bwd(x, dev(sc), dy, 1e-6)
        rdx, rds = G.rms_norm_grads(xr, sc.astype(np.float64), dyr, 1e-6)
        _close(dx, rdx, TOL[xd], "dx")
        _close(ds, rds, 1e-5 * max(1.0, np.sqrt(rows) / 30), "dscale")


def test_scale_gradient_does_not_depend_on_the_run():
    from memorax_amd import kernels as K
    rng = np.random.default_rng(3)
    x, dy = dev(rng.standard_normal((50000, 256)).astype(np.float32)), dev(rng.standard_normal((50000, 256)).astype(np.float32))
    sc = dev(np.ones(256, np.float32))
    a = K.rms_norm_bwd(x, sc, dy)[1]
    for _ in range(3):
        assert torch.equal(K.rms_norm_bwd(x, sc, dy)[1], a)


def test_large_eps_and_zero_rows():
    """A row of zeros normalises to zeros (rsqrt(eps) finite) and passes rsqrt(eps) * scale * dy back."""
    from memorax_amd import kernels as K
    x = torch.zeros((3, 8), device="cuda")
    sc = dev(np.arange(1, 9, dtype=np.float32))
    dy = dev(np.ones((3, 8), np.float32))
    assert torch.equal(K.rms_norm_fwd(x, sc, 0.25), torch.zeros_like(x))
    dx, ds = K.rms_norm_bwd(x, sc, dy, 0.25)
    np.testing.assert_allclose(dx.cpu().numpy(), 2.0 * np.arange(1, 9)[None] * np.ones((3, 1)), rtol=1e-6)
    assert torch.equal(ds, torch.zeros_like(ds))
    xe = torch.empty((0, 8), device="cuda")
    assert K.rms_norm_fwd(xe, sc).shape == (0, 8)
    dxe, dse = K.rms_norm_bwd(xe, sc, xe)
    assert dxe.shape == (0, 8) and torch.equal(dse, torch.zeros_like(dse))


def test_autograd_module_and_autocast():
    from memorax_amd import functional as Fn
    from memorax_amd import sequence_models as sm
    rng = np.random.default_rng(9)
    xn, dyn = rng.standard_normal((4, 9, 256)), rng.standard_normal((4, 9, 256))
    norm = sm.RMSNorm(256).cuda()
    with torch.no_grad():
        norm.scale.copy_(dev((1 + 0.1 * rng.standard_normal(256)).astype(np.float32)))
    sc = norm.scale.detach().cpu().numpy().astype(np.float64)
    x = dev(xn.astype(np.float32)).requires_grad_()
    y = norm(x)
    assert y.dtype == torch.float32
    y.backward(dev(dyn.astype(np.float32)))
    rdx, rds = G.rms_norm_grads(xn.astype(np.float32).astype(np.float64), sc, dyn.astype(np.float32).astype(np.float64))
    _close(y.detach(), M.rms_norm(xn.astype(np.float32), sc), 1e-5, "module y")
    _close(x.grad, rdx, 1e-5, "module dx")
    _close(norm.scale.grad, rds, 1e-5, "module dscale")
    # under autocast the result comes in the dtype the dense layers behind it compute in
    x2 = dev(xn.astype(np.float32)).requires_grad_()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y2 = norm(x2)
    assert y2.dtype == torch.bfloat16
    y2.float().backward(dev(dyn.astype(np.float32)))
    _close(y2.detach(), M.rms_norm(xn.astype(np.float32), sc), 2e-2, "autocast y")
    assert x2.grad.dtype == torch.float32
    _close(x2.grad, rdx, 2e-2, "autocast dx")
    # a float64 array is computed in float32 and its gradient comes back as float64; widths the kernel does not take go
    # to the array library
    x3 = dev(xn).requires_grad_()
    y3 = Fn.rms_norm(x3, norm.scale.detach())
    y3.sum().backward()
    assert x3.grad.dtype == torch.float64
    norm6 = sm.RMSNorm(6).cuda()
    x6 = torch.randn(5, 6, device="cuda")
    torch.testing.assert_close(norm6(x6), torch.nn.functional.rms_norm(x6, (6,), norm6.scale, 1e-6))


def test_residual_around_a_pre_norm_block_adds_both_gradients_in_the_norm_kernel():
    """Residual(PreNorm(f, RMSNorm)): x + f(norm(x)).  Values and gradients against the same block with the norm and
    the addition as separate array operations."""
    from memorax_amd import sequence_models as sm
    torch.manual_seed(0)
    inner = sm.Projection(256, 256).cuda()
    block = sm.Residual(sm.PreNorm(inner, 256, norm=sm.RMSNorm)).cuda()
    with torch.no_grad():
        block.module.norm.scale.copy_(1 + 0.1 * torch.randn(256, device="cuda"))
    x = torch.randn(6, 11, 256, device="cuda", requires_grad=True)
    x2 = x.detach().clone().requires_grad_()
    g = torch.randn(6, 11, 256, device="cuda")
    carry, y = block(x)
    assert carry is None
    y.backward(g)
    sc = block.module.norm.scale.detach().clone().requires_grad_()
    w, b = inner.proj.weight.detach().double(), inner.proj.bias.detach().double()
    xd, scd = x2.double(), sc.double()
    yr = xd + (xd * torch.rsqrt((xd * xd).mean(-1, keepdim=True) + 1e-6) * scd) @ w.T + b
    yr.backward(g.double())
    torch.testing.assert_close(y.detach().double(), yr.detach(), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(x.grad.double(), x2.grad.double(), rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(block.module.norm.scale.grad.double(), sc.grad.double(), rtol=1e-4, atol=1e-4)
    # an input that needs no gradient, and the norm's branch unused downstream of the fork
    _, y0 = block(x.detach())
    torch.testing.assert_close(y0, y.detach())
    from memorax_amd import functional as Fn
    x3 = x.detach().clone().requires_grad_()
    res, _unused = Fn.rms_norm_fork(x3, sc.detach())
    (res * g).sum().backward()
    torch.testing.assert_close(x3.grad, g)


@pytest.mark.parametrize("rows,D", [(1, 4), (7, 256), (1000, 260), (33, 512), (5, 1024), (3, 2048), (4099, 64), (16384, 256)])
@pytest.mark.parametrize("x_dtype,y_dtype", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16),
                                             (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32)])
def test_layer_norm_forward_and_backward(rows, D, x_dtype, y_dtype):
    from memorax_amd import kernels as K
    rng = np.random.default_rng(7 * rows + D)
    print(f"case layer norm rows={rows} D={D} x={x_dtype} y={y_dtype}", flush=True)
    # rows with means of the order of their spread, scales over a decade
    x, xr = _as((rng.standard_normal((rows, D)) + rng.standard_normal((rows, 1))) * np.exp(rng.standard_normal((rows, 1))), x_dtype)
    sc = (1.0 + 0.3 * rng.standard_normal(D)).astype(np.float32)
    bi = (0.2 * rng.standard_normal(D)).astype(np.float32)
    dy, dyr = _as(rng.standard_normal((rows, D)), y_dtype)
    add, addr = _as(rng.standard_normal((rows, D)), x_dtype)
    y = K.layer_norm_fwd(x, dev(sc), dev(bi), 1e-6, y_dtype)
    assert y.dtype == y_dtype and y.shape == x.shape
    _close(y, M.layer_norm(xr, sc, bi, 1e-6), TOL[y_dtype], "y")
    _close(K.layer_norm_fwd(x, None, None, 1e-6, y_dtype), M.layer_norm(xr, None, None, 1e-6), TOL[y_dtype], "y without parameters")
    dx, dscale, dbias = K.layer_norm_bwd(x, dev(sc), dy, 1e-6, dx_add=add)
    rdx, rds, rdb = G.layer_norm_grads(xr, sc.astype(np.float64), bi.astype(np.float64), dyr, 1e-6)
    got = dx.float().cpu().numpy().astype(np.float64)
    want = rdx + addr
    err = (np.abs(got - want).max(-1) / (np.abs(want).max(-1) + 1e-30)).max()
    # a bfloat16 row whose mean is several times its spread loses that factor in the centred values the kernel and the
    # oracle both start from (the same rounded inputs), so the bound stays the dtype's own
    assert err <= TOL[x_dtype], f"dx: {err:.3e}"
    tol_p = 1e-5 * max(1.0, np.sqrt(rows) / 30)
    _close(dscale, rds, tol_p, "dscale")
    _close(dbias, rdb, tol_p, "dbias")
    dx1, n1, n2 = K.layer_norm_bwd(x, dev(sc), dy, 1e-6, want_dparams=False)
    assert n1 is None and n2 is None
    err = (np.abs(dx1.float().cpu().numpy() - rdx).max(-1) / (np.abs(rdx).max(-1) + 1e-30)).max()
    assert err <= TOL[x_dtype], f"dx alone: {err:.3e}"


def test_layer_norm_module_pre_norm_residual_and_autocast():
    """sequence_models.LayerNorm keeps torch.nn.LayerNorm's parameters and values; Residual(PreNorm(f)) with it takes
    the forked route; values and gradients against torch's own layer norm in float64."""
    from memorax_amd import sequence_models as sm
    torch.manual_seed(1)
    inner = sm.Projection(256, 256).cuda()
    block = sm.Residual(sm.PreNorm(inner, 256)).cuda()      # the reference's default norm
    norm = block.module.norm
    assert isinstance(norm, torch.nn.LayerNorm) and sorted(n for n, _ in norm.named_parameters()) == ["bias", "weight"]
    with torch.no_grad():
        norm.weight.copy_(1 + 0.1 * torch.randn(256, device="cuda"))
        norm.bias.copy_(0.1 * torch.randn(256, device="cuda"))
    x = (torch.randn(6, 11, 256, device="cuda") + 0.5).requires_grad_()
    g = torch.randn(6, 11, 256, device="cuda")
    _, y = block(x)
    y.backward(g)
    xd = x.detach().double().requires_grad_()
    wd, bd = norm.weight.detach().double().requires_grad_(), norm.bias.detach().double().requires_grad_()
    yr = xd + torch.nn.functional.layer_norm(xd, (256,), wd, bd, 1e-6) @ inner.proj.weight.detach().double().T \
        + inner.proj.bias.detach().double()
    yr.backward(g.double())
    torch.testing.assert_close(y.detach().double(), yr.detach(), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(x.grad.double(), xd.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(norm.weight.grad.double(), wd.grad, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(norm.bias.grad.double(), bd.grad, rtol=1e-4, atol=1e-4)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        assert norm(x.detach()).dtype == torch.bfloat16
    # host arrays and widths the kernel does not take: torch's own layer norm
    n6 = sm.LayerNorm(6)
    x6 = torch.randn(5, 6)
    torch.testing.assert_close(n6(x6), torch.nn.functional.layer_norm(x6, (6,), n6.weight, n6.bias, 1e-6))
    torch.testing.assert_close(n6.cuda()(x6.cuda()).cpu(), n6.cpu()(x6), rtol=1e-5, atol=1e-6)


def test_refusals():
    from memorax_amd import _lib
    lib = _lib.load()
    x = torch.zeros((4, 256), device="cuda")
    y = torch.empty_like(x)
    sc = torch.ones(256, device="cuda")
    p = lambda t: ctypes.c_void_p(t.data_ptr())   # noqa: E731
    ok = lambda rows, D, xd=0, yd=0, eps=1e-6, xp=p(x), yp=p(y): lib.mrx_rms_norm_fwd(None, xp, p(sc), yp, rows, D, xd, yd, eps)   # noqa: E731
    assert ok(4, 256) == 0
    assert ok(4, 254) == -2          # rows are read four elements at a time
    assert ok(1, 4096) == -2
    assert ok(0, 256) == -1
    assert ok(4, 256, xd=2) == -1     # complex64 is no dtype of this call
    assert ok(4, 256, eps=-1.0) == -1
    assert ok(4, 256, xp=None) == -1
    assert ok(2, 256, xp=ctypes.c_void_p(x.data_ptr() + 4)) == -1
    dx, ds = torch.empty_like(x), torch.empty(256, device="cuda")
    bwd = lambda ws, dsp=p(ds): lib.mrx_rms_norm_bwd(None, p(x), p(sc), p(y), None, p(dx), dsp, ws, 4, 256, 0, 0, 1e-6)   # noqa: E731
    assert bwd(None) == -1             # the scale's gradient needs the workspace
    assert bwd(None, None) == 0
    db, ws = torch.empty(256, device="cuda"), torch.empty(2 * 1024 * 256, device="cuda")
    lbwd = lambda dsp, dbp: lib.mrx_layer_norm_bwd(None, p(x), p(sc), p(y), None, p(dx), dsp, dbp, p(ws), 4, 256, 0, 0, 1e-6)   # noqa: E731
    assert lbwd(p(ds), p(db)) == 0 and lbwd(None, None) == 0
    assert lbwd(p(ds), None) == -1 and lbwd(None, p(db)) == -1     # the layer norm's parameter gradients come as a pair
    assert lib.mrx_layer_norm_fwd(None, p(x), p(sc), None, p(y), 4, 256, 0, 0, 1e-6) == 0
    assert lib.mrx_layer_norm_fwd(None, p(x), p(sc), ctypes.c_void_p(sc.data_ptr() + 4), p(y), 4, 252, 0, 0, 1e-6) == -1
    torch.cuda.synchronize()
