"""The default ``MemoroidCellBase.scan`` (memoroid.py:60-91 for a cell that only defines
``binary_operator``): array operations only, so it runs on the CPU here, against the oracle's two
association orders of the same scan."""
import numpy as np
import pytest
import torch

from memorax_amd import sequence_models as sm
from oracle import memoroid as M


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a))


class _FFMStyleCell(sm.MemoroidCellBase):
    """Position-relative decay, the algebra of ffm.py:109-115: (S_i gamma(t_j - t_i) + S_j, t_j) with
    gamma(dt) = exp((alpha + i omega) dt); S (B,T,M,C) complex, t (B,T)."""

    def __init__(self, M_, C_):
        super().__init__()
        g = torch.Generator().manual_seed(5)
        self.alpha = -torch.rand(M_, generator=g, dtype=torch.float64) - 0.01
        self.omega = torch.rand(C_, generator=g, dtype=torch.float64) * 3.0

    def gamma(self, dt, xp):
        a = self.alpha.numpy() if xp is np else self.alpha
        w = self.omega.numpy() if xp is np else self.omega
        rate = a.reshape(1, -1, 1) + 1j * w.reshape(1, 1, -1)
        return xp.exp(rate * dt[..., None, None])

    def binary_operator(self, a, b):
        S_i, t_i = a
        S_j, t_j = b
        xp = np if isinstance(S_i, np.ndarray) else torch
        return (S_i * self.gamma(t_j - t_i, xp) + S_j, t_j)


class _MLSTMStyleCell(sm.MemoroidCellBase):
    """The max-stabilised gated sum of mlstm.py:188-203 on (C, log_f, n, m)."""

    def binary_operator(self, a, b):
        C_a, lf_a, n_a, m_a = a
        C_b, lf_b, n_b, m_b = b
        xp = np if isinstance(C_a, np.ndarray) else torch
        md = m_a + lf_b
        mc = xp.maximum(md, m_b)
        sa, sb = xp.exp(md - mc), xp.exp(m_b - mc)
        return (sa * C_a + sb * C_b, lf_a + lf_b, sa * n_a + sb * n_b, mc)


def _done(rng, B, T, p):
    d = rng.random((B, T)) < p
    return d


@pytest.mark.parametrize("T", [1, 2, 7, 16, 33])
@pytest.mark.parametrize("p", [0.0, 0.3])
def test_ffm_style_cell_against_both_oracle_orders(T, p):
    rng = np.random.default_rng(100 + T)
    B, Mm, Cc = 3, 4, 5
    cell = _FFMStyleCell(Mm, Cc)
    S = rng.standard_normal((B, T, Mm, Cc)) + 1j * rng.standard_normal((B, T, Mm, Cc))
    t = np.broadcast_to(np.arange(T, dtype=np.float64), (B, T)).copy()
    S0 = rng.standard_normal((B, 1, Mm, Cc)) + 0j
    t0 = np.full((B, 1), -1.0)
    done = _done(rng, B, T, p)
    want_h, want_c = M.scan_fn_sequential((S, t), (S0, t0), done, cell.binary_operator)
    tree_h, tree_c = M.scan_fn_tree((S, t), (S0, t0), done, cell.binary_operator)
    (h, ht), (c, ct) = cell.scan((_t(S), _t(t)), (_t(S0), _t(t0)), _t(done))
    assert h.shape == (B, T, Mm, Cc) and c.shape == (B, 1, Mm, Cc) and ct.shape == (B, 1)
    for got, a, b in ((h, want_h[0], tree_h[0]), (ht, want_h[1], tree_h[1]), (c, want_c[0], tree_c[0]),
                      (ct, want_c[1], tree_c[1])):
        np.testing.assert_allclose(got.numpy(), a, rtol=1e-10, atol=1e-10)
        np.testing.assert_allclose(got.numpy(), b, rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("done_dtype", [torch.bool, torch.float32])
def test_mlstm_style_cell_named_tuple_carry_and_reset_isolation(done_dtype):
    from collections import namedtuple
    Carry = namedtuple("Carry", "C log_f n m")
    rng = np.random.default_rng(7)
    B, T, H, d = 2, 19, 2, 3   # leaves shaped as mlstm.py:163-188 makes them
    z = (rng.standard_normal((B, T, H, d, d)), -np.abs(rng.standard_normal((B, T, H, 1, 1))) * 40.0,
         rng.standard_normal((B, T, H, d, 1)), rng.standard_normal((B, T, H, 1, 1)) * 30.0)
    c0 = (np.zeros((B, 1, H, d, d)), np.zeros((B, 1, H, 1, 1)), np.zeros((B, 1, H, d, 1)), np.full((B, 1, H, 1, 1), -1e9))
    done = _done(rng, B, T, 0.2)
    done[0, 11] = True
    zp = tuple(a.copy() for a in z)
    zp[0][0, 5] = np.nan       # poison before the reset at step 11 of row 0
    zp[2][0, 5] = np.inf
    cell = _MLSTMStyleCell()
    want_h, want_c = M.scan_fn_tree(z, c0, done, M.mlstm_operator)
    h, c = cell.scan(Carry(*map(_t, zp)), Carry(*map(_t, c0)), _t(done).to(done_dtype))
    assert isinstance(h, Carry) and isinstance(c, Carry)
    first_reset_after = 5 + 1 + int(np.argmax(done[0, 6:]))
    for got, want in zip(h, want_h):
        g = got.numpy()
        assert np.isfinite(g[0, first_reset_after:]).all()       # the reset is a select: nothing leaks past it
        np.testing.assert_allclose(g[0, first_reset_after:], want[0, first_reset_after:], rtol=1e-9, atol=1e-9)
        np.testing.assert_allclose(g[0, :5], want[0, :5], rtol=1e-9, atol=1e-9)
        np.testing.assert_allclose(g[1], want[1], rtol=1e-9, atol=1e-9)
    for got, want in zip(c, want_c):
        np.testing.assert_allclose(got.numpy(), want, rtol=1e-9, atol=1e-9)


def test_memoroid_runs_a_user_cell_and_autograd_flows_through_the_scan():
    class Cell(sm.MemoroidCellBase):     # a diagonal recurrence written by a user, no kernel hook
        def __init__(self):
            super().__init__()
            self.w = torch.nn.Parameter(torch.tensor([0.3, -0.2, 0.5], dtype=torch.float64))

        def forward(self, x, **kw):
            return {"state": x * self.w, "decay": torch.sigmoid(x)}

        def binary_operator(self, a, b):
            return {"state": b["decay"] * a["state"] + b["state"], "decay": b["decay"] * a["decay"]}

        def read(self, h, x, **kw):
            return h["state"]

        def initialize_carry(self, key, input_shape):
            B, Fe = input_shape
            return {"state": torch.zeros(B, 1, Fe, dtype=torch.float64), "decay": torch.ones(B, 1, Fe, dtype=torch.float64)}

    rng = np.random.default_rng(3)
    B, T, Fe = 2, 12, 3
    x = _t(rng.standard_normal((B, T, Fe))).requires_grad_(True)
    done = _t(rng.random((B, T)) < 0.2)
    model = sm.Memoroid(Cell())
    carry, y = model(x, done)
    a = torch.sigmoid(x).detach().numpy()
    b = (x * model.cell.w).detach().numpy()
    want, want_last, want_P = M.diag_scan(a, b, done.numpy())
    np.testing.assert_allclose(y.detach().numpy(), want, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(carry["state"][:, 0].detach().numpy(), want_last, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(carry["decay"][:, 0].detach().numpy(), want_P, rtol=1e-12, atol=1e-12)
    # split invariance through the carry
    s = 5
    c1, y1 = model(x[:, :s], done[:, :s])
    c2, y2 = model(x[:, s:], done[:, s:], initial_carry=c1)
    np.testing.assert_allclose(torch.cat([y1, y2], 1).detach().numpy(), want, rtol=1e-12, atol=1e-12)
    # gradients: the analytic reverse scan of the oracle
    g = _t(rng.standard_normal((B, T, Fe)))
    (y * g).sum().backward()
    da, db, _ = M.diag_scan_bwd(a, want, done.numpy(), g.numpy())[:3]
    sig = a
    want_dx = da * sig * (1 - sig) + db * model.cell.w.detach().numpy()
    np.testing.assert_allclose(x.grad.numpy(), want_dx, rtol=1e-10, atol=1e-10)
