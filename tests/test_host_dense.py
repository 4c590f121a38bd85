"""The dense layer of the host mirror: same values and gradients as torch.nn.Linear, with the
weight gradient as a sliced product."""
import pytest
import torch

from memorax_amd import dense as D


def test_dense_matches_linear_on_cpu():
    torch.manual_seed(0)
    lin = torch.nn.Linear(12, 7).double()
    den = D.Dense(12, 7).double()
    den.load_state_dict(lin.state_dict())
    x = torch.randn(3, 5, 12, dtype=torch.float64, requires_grad=True)
    x2 = x.detach().clone().requires_grad_()
    g = torch.randn(3, 5, 7, dtype=torch.float64)
    lin(x).backward(g)
    den(x2).backward(g)
    assert torch.equal(lin(x), den(x2))
    torch.testing.assert_close(x2.grad, x.grad, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(den.weight.grad, lin.weight.grad, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(den.bias.grad, lin.bias.grad, rtol=1e-12, atol=1e-12)
    assert torch.autograd.gradcheck(D.dense, (x, den.weight, den.bias))
    assert torch.autograd.gradcheck(lambda a, w: D.dense(a, w), (x, den.weight))


def test_slices_only_for_tall_products():
    assert D._slices(131072, 256, 256) == 64
    assert D._slices(131072, 4, 256) == 64
    assert D._slices(4096, 256, 256) == 1          # few rows
    assert D._slices(32768, 4096, 1024) == 1       # a result with tiles enough
    assert D._slices(3 * 8192, 64, 64) == 8        # odd multiples: as far as halving goes
    for rows in (8192, 100000, 131072, 1 << 20):
        s = D._slices(rows, 128, 128)
        assert rows % s == 0 and s <= D._MAX_SLICES


def test_weight_gradient_without_slices_is_the_plain_product():
    torch.manual_seed(1)
    dy, x = torch.randn(50, 3), torch.randn(50, 4)
    torch.testing.assert_close(D.weight_gradient(dy, x), dy.t() @ x)


@pytest.mark.gpu
@pytest.mark.parametrize("n_out,n_in,bias", [(256, 256, False), (4, 256, False), (256, 1024, True)])
@pytest.mark.parametrize("amp", [True, False])
def test_dense_sliced_weight_gradient_on_the_device(n_out, n_in, bias, amp):
    torch.manual_seed(2)
    B, T = 256, 128
    lin = torch.nn.Linear(n_in, n_out, bias=bias).cuda()
    den = D.Dense(n_in, n_out, bias=bias).cuda()
    den.load_state_dict(lin.state_dict())
    assert D._slices(B * T, n_out, n_in) > 1
    x = torch.randn(B, T, n_in, device="cuda", requires_grad=True)
    x2 = x.detach().clone().requires_grad_()
    g = torch.randn(B, T, n_out, device="cuda")
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=amp):
        y, y2 = lin(x), den(x2)
    assert y2.dtype == y.dtype
    y.backward(g.to(y.dtype))
    y2.backward(g.to(y.dtype))
    # the float64 product of the operands as the layers saw them
    xe = x.detach().bfloat16().double() if amp else x.detach().double()
    ge = g.bfloat16().double() if amp else g.double()
    dw = ge.reshape(-1, n_out).t() @ xe.reshape(-1, n_in)
    tol = dw.abs().max().item()
    assert (den.weight.grad.double() - dw).abs().max().item() <= (3e-5 if not amp else 1e-4) * tol
    assert (lin.weight.grad.double() - dw).abs().max().item() <= 2e-2 * tol
    torch.testing.assert_close(y2, y, rtol=0, atol=0)
    torch.testing.assert_close(x2.grad, x.grad, rtol=1e-2 if amp else 1e-5, atol=1e-2 if amp else 1e-5)
    if bias:
        db = ge.reshape(-1, n_out).sum(0)
        assert (den.bias.grad.double() - db).abs().max().item() <= 1e-4 * db.abs().max().item() + 1e-3


def test_dense_group_matches_separate_layers_on_cpu():
    torch.manual_seed(3)
    layers = [D.Dense(10, 6).double(), D.Dense(10, 3, bias=False).double(), D.Dense(10, 5).double()]
    x = torch.randn(4, 7, 10, dtype=torch.float64, requires_grad=True)
    x2 = x.detach().clone().requires_grad_()
    gs = [torch.randn(4, 7, m.out_features, dtype=torch.float64) for m in layers]
    ys = D.dense_group(x, layers)
    # the second output stays unused: its layer gets no gradient, the others are not disturbed
    (ys[0] * gs[0]).sum().add((ys[2] * gs[2]).sum()).backward()
    want = [torch.nn.functional.linear(x2, m.weight.detach().clone().requires_grad_(),
                                       None if m.bias is None else m.bias.detach().clone().requires_grad_()) for m in layers]
    for y, w in zip(ys, want):
        assert torch.equal(y, w)
    (want[0] * gs[0]).sum().add((want[2] * gs[2]).sum()).backward()
    torch.testing.assert_close(x.grad, x2.grad, rtol=1e-12, atol=1e-12)
    assert layers[1].weight.grad is None
    ref0 = gs[0].reshape(-1, 6).t() @ x.detach().reshape(-1, 10)
    torch.testing.assert_close(layers[0].weight.grad, ref0, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(layers[2].bias.grad, gs[2].reshape(-1, 5).sum(0), rtol=1e-12, atol=1e-12)
    params = [m.weight for m in layers] + [layers[0].bias, layers[2].bias]
    assert torch.autograd.gradcheck(lambda a, *p: D.dense_group(a, layers), (x, *params))


@pytest.mark.gpu
def test_dense_group_on_the_device_under_autocast():
    torch.manual_seed(4)
    B, T, n_in = 128, 128, 256
    layers = [D.Dense(n_in, 256, bias=False).cuda(), D.Dense(n_in, 256, bias=False).cuda(), D.Dense(n_in, 4, bias=True).cuda()]
    x = torch.randn(B, T, n_in, device="cuda", requires_grad=True)
    x2 = x.detach().clone().requires_grad_()
    gs = [torch.randn(B, T, m.out_features, device="cuda") for m in layers]
    with torch.autocast("cuda", dtype=torch.bfloat16):
        ys = D.dense_group(x, layers)
        want = [torch.nn.functional.linear(x2, m.weight.detach(), None if m.bias is None else m.bias.detach()) for m in layers]
    for y, w in zip(ys, want):
        assert y.dtype == torch.bfloat16 and torch.equal(y, w)
    sum((y.float() * g).sum() for y, g in zip(ys, gs)).backward()
    sum((y.float() * g).sum() for y, g in zip(want, gs)).backward()
    assert x.grad.dtype == torch.float32
    torch.testing.assert_close(x.grad, x2.grad, rtol=2e-2, atol=2e-2 * x2.grad.abs().max().item())
    xe = x.detach().bfloat16().double().reshape(-1, n_in)
    for m, g in zip(layers, gs):
        dw = g.bfloat16().double().reshape(-1, m.out_features).t() @ xe
        assert (m.weight.grad.double() - dw).abs().max().item() <= 1e-4 * dw.abs().max().item()
