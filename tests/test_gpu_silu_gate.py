"""The gating product kernels (mrx_silu_gate_fwd / _bwd, through the C ABI) against the oracle:
oracle.memoroid.silu_gate and oracle.grad.silu_gate_grads (pinned by closed forms and finite differences in
tests/test_oracle_grad.py).  Tolerances: float32 1e-5 of the result's scale, bfloat16 2e-2 (one rounding of a
stored result)."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import grad as G
from oracle import memoroid as M
from gpu_util import dev

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def _err(got, want):
    return np.abs(got.float().cpu().numpy() - want).max() / (np.abs(want).max() + 1e-30)


@pytest.mark.parametrize("shape", [(1,), (7,), (8,), (3, 5, 9), (64, 128, 256), (1000003,)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_forward_and_backward(shape, dtype):
    from memorax_amd import kernels as K
    rng = np.random.default_rng(len(shape) + shape[0])
    print(f"case silu gate shape={shape} dtype={dtype}", flush=True)
    h, g, dy = (dev((rng.standard_normal(shape) * s).astype(np.float32)).to(dtype) for s in (1.0, 3.0, 1.0))
    hr, gr, dyr = (t.float().cpu().numpy().astype(np.float64) for t in (h, g, dy))
    y = K.silu_gate_fwd(h, g)
    assert y.dtype == dtype and y.shape == h.shape
    assert _err(y, M.silu_gate(hr, gr)) <= TOL[dtype]
    dh, dg = K.silu_gate_bwd(h, g, dy)
    rh, rg = G.silu_gate_grads(hr, gr, dyr)
    assert _err(dh, rh) <= TOL[dtype] and _err(dg, rg) <= TOL[dtype]


def test_autograd_mixed_dtypes_and_the_recurrence_block():
    from memorax_amd import functional as Fn
    rng = np.random.default_rng(2)
    hn, gn, dyn = (rng.standard_normal((5, 6, 8)).astype(np.float32) for _ in range(3))
    h, g = dev(hn).requires_grad_(), dev(gn).bfloat16().requires_grad_()   # promoted to float32 for the kernel
    y = Fn.silu_gate(h, g)
    assert y.dtype == torch.float32
    y.backward(dev(dyn))
    rh, rg = G.silu_gate_grads(hn, g.detach().float().cpu().numpy(), dyn)
    assert h.grad.dtype == torch.float32 and g.grad.dtype == torch.bfloat16
    assert _err(h.grad, rh) <= 1e-5 and _err(g.grad, rg) <= 2e-2
    assert Fn.silu_gate(h[:0], g[:0].float()).shape == (0, 6, 8)


def test_refusals():
    from memorax_amd import _lib
    lib = _lib.load()
    a = torch.zeros(64, device="cuda")
    p = lambda t, off=0: ctypes.c_void_p(t.data_ptr() + off)   # noqa: E731
    assert lib.mrx_silu_gate_fwd(None, p(a), p(a), p(a), 64, 0) == 0
    assert lib.mrx_silu_gate_fwd(None, p(a), p(a), p(a), 0, 0) == -1
    assert lib.mrx_silu_gate_fwd(None, p(a), p(a), p(a), 64, 2) == -1        # complex64 is no dtype of this call
    assert lib.mrx_silu_gate_fwd(None, p(a), None, p(a), 64, 0) == -1
    assert lib.mrx_silu_gate_fwd(None, p(a), p(a, 4), p(a), 32, 0) == -1     # sixteen bytes at a time
    assert lib.mrx_silu_gate_bwd(None, p(a), p(a), p(a), p(a), None, 64, 0) == -1
    torch.cuda.synchronize()
