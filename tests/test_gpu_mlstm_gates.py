"""The mLSTM cell's stabiliser kernels (mrx_mlstm_gates_fwd / _bwd, through the C ABI) against the oracle:
m, g, w of oracle.memoroid.mlstm_gates (itself pinned against the stabilised scan of mlstm.py:190-206) and
the gradients of oracle.grad.mlstm_gates_grads (torch-fp64 autograd, pinned by finite differences)."""
import numpy as np
import pytest
import torch

from oracle import grad as G
from oracle import memoroid as M
from gpu_util import dev

pytestmark = pytest.mark.gpu


def _inputs(B, T, H, seed, p, drift=0.0):
    rng = np.random.default_rng(seed)
    li = (rng.standard_normal((B, T, H)) * 2 + drift * np.arange(T)[None, :, None]).astype(np.float32)
    lf = (-np.abs(rng.standard_normal((B, T, H)))).astype(np.float32)
    done = rng.random((B, T)) < p
    m0 = rng.standard_normal((B, H)).astype(np.float32)
    return li, lf, done, m0


@pytest.mark.parametrize("B,T,H,p", [(2, 1, 1, 0.0), (3, 7, 2, 0.3), (5, 64, 4, 0.05), (4, 131, 3, 0.02), (1, 1000, 8, 0.01),
                                      (70, 9, 1, 0.2)])
@pytest.mark.parametrize("carried", [True, False])
def test_gates_forward_and_backward(B, T, H, p, carried):
    from memorax_amd import kernels as K
    li, lf, done, m0 = _inputs(B, T, H, 100 + T, p)
    if T > 2:
        done[0, 0] = True          # the carried m is dropped for this row
        lf[-1, T // 2] = -200.0     # a step whose g sits on the floor
    m0_ = m0 if carried else None
    print(f"case mlstm gates B={B} T={T} H={H} carried={carried}", flush=True)
    for done_t in (dev(done), dev(done.astype(np.float32))):
        m, g, w = K.mlstm_gates_fwd(dev(li), dev(lf), done_t, None if m0_ is None else dev(m0_))
        rm, rg, rw = M.mlstm_gates(li, lf, done, m0_)
        np.testing.assert_allclose(m.cpu().numpy(), rm, rtol=1e-6, atol=1e-5)
        np.testing.assert_allclose(g.cpu().numpy(), rg, rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(w.cpu().numpy(), rw, rtol=1e-5, atol=1e-6)
    rng = np.random.default_rng(5)
    dm, dg, dw = (rng.standard_normal((B, T, H)).astype(np.float32) for _ in range(3))
    # the branch the maximum took is decided on float32 values in the kernel and on float64 ones in the oracle: keep the
    # two branches apart by more than float32 rounding (a tie has no gradient to compare)
    mp = np.concatenate([(m0_ if carried else np.full((B, H), -1e9))[:, None], rm[:, :-1]], 1)
    assert (np.abs(mp + lf - li) > 1e-4).all()
    dli, dlf, dm0 = K.mlstm_gates_bwd(dev(li), dev(lf), dev(done), None if m0_ is None else dev(m0_), m, dev(dm), dev(dg), dev(dw),
                                      want_dm0=carried)
    ri, rf, r0 = G.mlstm_gates_grads(li, lf, done, m0_, dm, dg, dw)
    np.testing.assert_allclose(dli.cpu().numpy(), ri, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(dlf.cpu().numpy(), rf, rtol=1e-4, atol=1e-4)
    if carried:
        np.testing.assert_allclose(dm0.cpu().numpy(), r0, rtol=1e-4, atol=1e-4)
    # absent gradients count as zeros
    dli2, dlf2, _ = K.mlstm_gates_bwd(dev(li), dev(lf), dev(done), None if m0_ is None else dev(m0_), m, None, dev(dg), None,
                                      want_dm0=False)
    ri2, rf2, _ = G.mlstm_gates_grads(li, lf, done, m0_, np.zeros_like(dm), dg, np.zeros_like(dw))
    np.testing.assert_allclose(dli2.cpu().numpy(), ri2, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(dlf2.cpu().numpy(), rf2, rtol=1e-4, atol=1e-4)


def test_gates_drifting_by_hundreds_of_nats_stay_finite():
    """Input gates that climb by 3 nats a step for 400 steps: exp(log_i) leaves the float32 range, m follows it and
    every g and w stays in (−60, 0] and (0, 1]."""
    from memorax_amd import kernels as K
    li, lf, done, m0 = _inputs(2, 400, 2, 7, 0.01, drift=3.0)
    m, g, w = K.mlstm_gates_fwd(dev(li), dev(lf), dev(done), dev(m0))
    rm, rg, rw = M.mlstm_gates(li, lf, done, m0)
    assert torch.isfinite(m).all() and torch.isfinite(g).all() and torch.isfinite(w).all()
    np.testing.assert_allclose(m.cpu().numpy(), rm, rtol=1e-6, atol=1e-4)
    np.testing.assert_allclose(w.cpu().numpy(), rw, rtol=1e-4, atol=1e-6)
    assert (g.cpu().numpy() >= -60).all() and (g.cpu().numpy() <= 0).all() and (w.cpu().numpy() <= 1 + 1e-6).all()


def test_gates_through_autograd_and_refusals():
    import ctypes
    import memorax_amd.functional as F
    from memorax_amd import _lib
    li, lf, done, m0 = _inputs(3, 40, 2, 11, 0.1)
    tli, tlf, tm0 = (dev(a).requires_grad_() for a in (li, lf, m0))
    m, g, w = F.mlstm_gates(tli, tlf, dev(done), tm0)
    rng = np.random.default_rng(3)
    dm, dg, dw = (rng.standard_normal(li.shape).astype(np.float32) for _ in range(3))
    ((m * dev(dm)).sum() + (g * dev(dg)).sum() + (w * dev(dw)).sum()).backward()
    ri, rf, r0 = G.mlstm_gates_grads(li, lf, done, m0, dm, dg, dw)
    np.testing.assert_allclose(tli.grad.cpu().numpy(), ri, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(tlf.grad.cpu().numpy(), rf, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(tm0.grad.cpu().numpy(), r0, rtol=1e-4, atol=1e-4)
    lib = _lib.load()
    a = dev(li)
    p = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    dn = dev(done)
    out = [torch.empty_like(a) for _ in range(3)]
    st = torch.cuda.current_stream().cuda_stream
    assert lib.mrx_mlstm_gates_fwd(st, None, p(a), p(dn), None, p(out[0]), p(out[1]), p(out[2]), 3, 40, 2, 0, -60.0) == -1
    assert lib.mrx_mlstm_gates_fwd(st, p(a), p(a), p(dn), None, p(out[0]), p(out[1]), p(out[2]), 3, 0, 2, 0, -60.0) == -1
    assert lib.mrx_mlstm_gates_fwd(st, p(a), p(a), p(dn), None, p(out[0]), p(out[1]), p(out[2]), 3, 40, 2, 7, -60.0) == -1
    assert lib.mrx_mlstm_gates_fwd(st, p(a), p(a), p(dn), None, p(out[0]), p(out[1]), p(out[2]), 3, 40, 2, 0, 1.0) == -1
    assert lib.mrx_mlstm_gates_bwd(st, p(a), p(a), p(dn), None, None, None, None, None, p(out[0]), p(out[1]), None, 3, 40, 2, 0, -60.0) == -1
