"""Dense layers of the host-side mirror (flax.linen.Dense in the reference's cells and blocks,
e.g. linear_attention.py:62-80, min_gru.py:49-62, blocks/ffn.py:11-123).

The products stay the array library's; what this module changes is their shape.  A rollout batch
has a hundred thousand rows and a few hundred features, so the weight gradient ``dy^T x`` is a
product with a tiny result and an enormous inner dimension, which the library's GEMM runs on as
many workgroups as the result has tiles (sixteen for 256 x 256: 330 us where the forward product
of the same operands takes 32 us).  ``dense`` cuts the rows into slices, multiplies them as one
batched product with float32 partial results and sums those (41 us); ``dense_group`` runs the
layers that share an input on one cast of it and lets their products add up the input gradient.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

_SLICE_ROWS = 2048   # rows per slice of the weight-gradient product
_MAX_SLICES = 128
_HALVES = (torch.bfloat16, torch.float16)


def _wide(dtype):
    return torch.float32 if dtype in _HALVES else dtype


def autocast_dtype(x):
    """The dtype the array library's autocast would run a product on ``x`` in, or None."""
    if x.is_cuda and x.is_floating_point() and torch.is_autocast_enabled("cuda"):
        return torch.get_autocast_dtype("cuda")
    return None


def _slices(rows, n_out, n_in):
    """Into how many slices the rows of a weight-gradient product are cut: none while the result
    has tiles enough to fill the device or the rows are few."""
    if rows < 4 * _SLICE_ROWS or rows < 32 * max(n_out, n_in):
        return 1
    s = 1
    while s < _MAX_SLICES and rows % (2 * s) == 0 and rows // (2 * s) >= _SLICE_ROWS:
        s *= 2
    return s


def weight_gradient(dy, x):
    """dy^T x for dy (rows, n_out), x (rows, n_in); float32 from 16-bit operands."""
    rows, n_out = dy.shape
    n_in = x.shape[1]
    s = _slices(rows, n_out, n_in) if dy.is_cuda else 1
    if s == 1:
        return (dy.t() @ x).to(_wide(dy.dtype))
    a, b = dy.reshape(s, rows // s, n_out).transpose(1, 2), x.reshape(s, rows // s, n_in)
    if dy.dtype in _HALVES:
        return torch.bmm(a, b, out_dtype=torch.float32).sum(0)
    return torch.bmm(a, b).sum(0)


class _Dense(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias):
        dt = autocast_dtype(x)
        xc, wc = (x, weight) if dt is None else (x.to(dt), weight.to(dt))
        bc = bias if bias is None or dt is None else bias.to(dt)
        ctx.save_for_backward(xc, wc)
        ctx.x_dtype, ctx.has_bias = x.dtype, bias is not None
        return F.linear(xc, wc, bc)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dy):
        xc, wc = ctx.saved_tensors
        dy = dy.to(xc.dtype)
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            dx = (dy @ wc).to(ctx.x_dtype)
        dy2 = dy.reshape(-1, dy.shape[-1])
        if ctx.needs_input_grad[1]:
            dw = weight_gradient(dy2, xc.reshape(-1, xc.shape[-1]))
        if ctx.has_bias and ctx.needs_input_grad[2]:
            db = dy2.sum(0, dtype=_wide(dy2.dtype))
        return dx, dw, db


class _DenseGroup(torch.autograd.Function):
    """Several dense layers on one input.  Their gradients with respect to the input are accumulated by the
    products themselves (each adds onto the sum so far) instead of by a pass per layer."""

    @staticmethod
    def forward(ctx, x, n, *params):
        weights, biases = params[:n], params[n:]
        dt = autocast_dtype(x)
        xc = x if dt is None else x.to(dt)
        wcs = [w if dt is None else w.to(dt) for w in weights]
        ctx.save_for_backward(xc, *wcs)
        ctx.set_materialize_grads(False)   # an output nobody used costs no products
        ctx.x_dtype, ctx.n, ctx.has_bias = x.dtype, n, [b is not None for b in biases]
        return tuple(F.linear(xc, w, b if b is None or dt is None else b.to(dt)) for w, b in zip(wcs, biases))

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, *dys):
        xc, *wcs = ctx.saved_tensors
        n = ctx.n
        x2 = xc.reshape(-1, xc.shape[-1])
        dx, dws, dbs = None, [None] * n, [None] * n
        for i, (dy, w) in enumerate(zip(dys, wcs)):
            if dy is None:
                continue
            dy2 = dy.to(xc.dtype).reshape(-1, dy.shape[-1])
            if ctx.needs_input_grad[0]:
                dx = dy2 @ w if dx is None else dx.addmm_(dy2, w)
            if ctx.needs_input_grad[2 + i]:
                dws[i] = weight_gradient(dy2, x2)
            if ctx.has_bias[i] and ctx.needs_input_grad[2 + n + i]:
                dbs[i] = dy2.sum(0, dtype=_wide(dy2.dtype))
        if dx is not None:
            dx = dx.view(xc.shape).to(ctx.x_dtype)
        return (dx, None, *dws, *dbs)


def dense_group(x, layers):
    """The outputs of several Dense / torch.nn.Linear layers that read the same input, as a tuple.
    The layers lend their parameters; their own ``forward`` (and hooks registered on it) does not run."""
    return _DenseGroup.apply(x, len(layers), *[m.weight for m in layers], *[m.bias for m in layers])


def dense(x, weight, bias=None):
    """x W^T + b like torch.nn.functional.linear (autocast included), with the weight gradient as a
    sliced product (module docstring).  Gradients of weight and bias are formed in float32 when the
    operands are 16-bit and cast to the parameters' dtype by the array library."""
    return _Dense.apply(x, weight, bias)


class Dense(nn.Linear):
    """torch.nn.Linear (same parameters, same state dict) on ``dense``."""

    def forward(self, x):
        return dense(x, self.weight, self.bias)
