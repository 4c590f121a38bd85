"""Pins the gradient oracle: torch-fp64 autograd vs central finite differences on
the NumPy forward, and vs the analytic reverse-scan formulas."""
import numpy as np
import pytest

from oracle import grad as G
from oracle import memoroid as M

RNG = np.random.default_rng(11)


def rnd(*s):
    return RNG.standard_normal(s)


def fd(f, x, eps=1e-6):
    """Central finite-difference gradient of scalar f at x."""
    g = np.zeros_like(x)
    it = np.nditer(x, flags=["multi_index"])
    for _ in it:
        i = it.multi_index
        old = x[i]
        x[i] = old + eps
        fp = f()
        x[i] = old - eps
        fm = f()
        x[i] = old
        g[i] = (fp - fm) / (2 * eps)
    return g


def test_diag_grads_fd_and_analytic():
    B, T, D = 2, 9, 2
    a, b, h0 = RNG.uniform(0.5, 1, (B, T, D)), rnd(B, T, D), rnd(B, D)
    g, gl = rnd(B, T, D), rnd(B, D)
    d = np.zeros((B, T), bool)
    d[0, 4] = True
    d[1, 0] = True

    def L():
        h, hl, _ = M.diag_scan(a, b, d, h0)
        return (h * g).sum() + (hl * gl).sum()

    ag = G.diag_scan_grads(a, b, d, h0, g, gl)
    np.testing.assert_allclose(ag["da"], fd(L, a), rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(ag["db"], fd(L, b), rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(ag["dh0"], fd(L, h0), rtol=1e-6, atol=1e-8)
    h, _, _ = M.diag_scan(a, b, d, h0)
    da, db, dh0 = M.diag_scan_bwd(a, h, d, g, h0, gl)
    np.testing.assert_allclose(da, ag["da"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(db, ag["db"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(dh0, ag["dh0"], rtol=1e-12, atol=1e-13)


def test_mingru_grads_fd_and_the_linear_space_formulas():
    """Autograd through the log-space restatement vs finite differences of the NumPy log-space scan,
    and vs the closed form the fused kernel uses: with (lam, da) the reverse scan of the linear-space
    coefficients, dz = s (1 - s) (g(h~) lam - da), dh~ = lam s g'(h~), s = sigma(z)."""
    B, T, F = 2, 9, 3
    z, x = 2 * rnd(B, T, F), 2 * rnd(B, T, F)
    x[0, 3, 0], x[1, 5, 2] = 0.7, -0.4   # both branches of g near the kink stay on their side under fd
    h0 = np.exp(rnd(B, F))
    g, gl = rnd(B, T, F), rnd(B, F)
    d = np.zeros((B, T), bool)
    d[0, 4] = True
    d[1, 0] = True

    def L():
        nxt, h = M.mingru_scan(z, x, d, (np.log(h0)[:, None], np.zeros((B, 1, F))))
        return (h * g).sum() + (np.exp(nxt[0][:, 0]) * gl).sum()

    ag = G.mingru_grads(z, x, d, h0, g, gl)
    np.testing.assert_allclose(ag["dz"], fd(L, z), rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(ag["dh_tilde"], fd(L, x), rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(ag["dh0"], fd(L, h0), rtol=1e-6, atol=1e-8)
    a, b = M.mingru_linear_coeffs(z, x)
    h, _, _ = M.diag_scan(a, b, d, h0)
    da, lam, dh0 = M.diag_scan_bwd(a, h, d, g, h0, gl)
    s = M.sigmoid(z)
    gx = np.where(x >= 0, x + 0.5, M.sigmoid(x))
    dgx = np.where(x >= 0, 1.0, M.sigmoid(x) * (1 - M.sigmoid(x)))
    np.testing.assert_allclose(s * (1 - s) * (gx * lam - da), ag["dz"], rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(lam * s * dgx, ag["dh_tilde"], rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(dh0, ag["dh0"], rtol=1e-10, atol=1e-12)
    # the cell's initial carry (-inf, 0): the first step is b_1 whatever z says about the decay
    ag0 = G.mingru_grads(z, x, d, None, g)
    h00, _, _ = M.diag_scan(a, b, d)
    da0, lam0, _ = M.diag_scan_bwd(a, h00, d, g)
    np.testing.assert_allclose(s * (1 - s) * (gx * lam0 - da0), ag0["dz"], rtol=1e-10, atol=1e-12)


def test_diag_grads_complex_analytic_matches_autograd():
    B, T, D = 2, 8, 3
    a = 0.9 * np.exp(1j * RNG.uniform(0, 3, (B, T, D)))
    b, h0 = rnd(B, T, D) + 1j * rnd(B, T, D), rnd(B, D) + 1j * rnd(B, D)
    g = rnd(B, T, D) + 1j * rnd(B, T, D)
    d = RNG.random((B, T)) < 0.2
    ag = G.diag_scan_grads(a, b, d, h0, g)
    h, _, _ = M.diag_scan(a, b, d, h0)
    da, db, dh0 = M.diag_scan_bwd(a, h, d, g, h0)
    np.testing.assert_allclose(da, ag["da"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(db, ag["db"], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(dh0, ag["dh0"], rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("fmap", ["none", "elu1"])
def test_linear_attention_grads_fd(fmap):
    B, T, H, dk, dv = 1, 7, 1, 3, 2
    q, k, v, S0 = rnd(B, T, H, dk), rnd(B, T, H, dk), rnd(B, T, H, dv), rnd(B, H, dv, dk)
    do, dSl = rnd(B, T, H, dv), rnd(B, H, dv, dk)
    d = np.zeros((B, T), bool)
    d[0, 3] = True

    def L():
        o, Sl = M.linear_attention(q, k, v, d, S0, fmap)
        return (o * do).sum() + (Sl * dSl).sum()

    ag = G.linear_attention_grads(q, k, v, d, S0, do, dSl, fmap)
    for name, x in (("dq", q), ("dk", k), ("dv", v), ("dS0", S0)):
        np.testing.assert_allclose(ag[name], fd(L, x), rtol=1e-6, atol=1e-8, err_msg=name)
    o, Sl = M.linear_attention(q, k, v, d, S0, fmap)
    np.testing.assert_allclose(ag["o"], o, rtol=1e-12)
    np.testing.assert_allclose(ag["S_last"], Sl, rtol=1e-12)


@pytest.mark.parametrize("eps", [1e-6, 7.0])
def test_normalised_linear_attention_grads_fd(eps):
    """eps = 7 puts two of the seven rows under the clamp (no gradient through the denominator)."""
    B, T, H, dk, dv = 1, 7, 1, 3, 2
    r = np.random.default_rng(2)   # own stream: which rows the clamp catches must not depend on test order
    rnd = lambda *s: r.standard_normal(s)  # noqa: E731
    q, k, v, S0 = rnd(B, T, H, dk), rnd(B, T, H, dk), rnd(B, T, H, dv), rnd(B, H, dv, dk)
    z0 = np.abs(rnd(B, H, dk))
    do, dSl, dzl = rnd(B, T, H, dv), rnd(B, H, dv, dk), rnd(B, H, dk)
    d = np.zeros((B, T), bool)
    d[0, 3] = True

    def L():
        o, den, Sl, zl = M.normalised_linear_attention(q, k, v, d, S0, z0, "elu1", eps)
        return (o * do).sum() + (Sl * dSl).sum() + (zl * dzl).sum()

    _, den, _, _ = M.normalised_linear_attention(q, k, v, d, S0, z0, "elu1", eps)
    if eps > 1:
        assert (den == eps).any() and (den > eps).any()
        assert np.abs(den[den > eps] - eps).min() > 1.0    # no row sits near the kink
    ag = G.normalised_linear_attention_grads(q, k, v, d, S0, z0, do, dSl, dzl, "elu1", eps)
    for name, x in (("dq", q), ("dk", k), ("dv", v), ("dS0", S0), ("dz0", z0)):
        np.testing.assert_allclose(ag[name], fd(L, x), rtol=1e-5, atol=1e-7, err_msg=name)


def test_deltanet_prologue_grads_fd_scale_invariance_and_orthogonality():
    """The fused prologue (k / |k|, sigmoid(beta_raw)) in front of the delta rule: finite
    differences; the output does not change when a key is rescaled, hence (Euler, degree 0)
    every key's gradient is orthogonal to the key."""
    r = np.random.default_rng(5)
    B, T, H, dk, dv = 1, 7, 2, 3, 2
    q, k, v = r.standard_normal((B, T, H, dk)), r.standard_normal((B, T, H, dk)) * 3, r.standard_normal((B, T, H, dv))
    braw, S0 = r.standard_normal((B, T, H)), r.standard_normal((B, H, dv, dk))
    do, dSl = r.standard_normal((B, T, H, dv)), r.standard_normal((B, H, dv, dk))
    d = np.zeros((B, T), bool)
    d[0, 4] = True

    def L():
        o, Sl = M.deltanet(q, k, v, braw, d, S0)
        return (o * do).sum() + (Sl * dSl).sum()

    ag = G.deltanet_grads(q, k, v, braw, d, S0, do, dSl)
    for name, x in (("dq", q), ("dk", k), ("dv", v), ("dbeta", braw), ("dS0", S0)):
        np.testing.assert_allclose(ag[name], fd(L, x), rtol=1e-5, atol=1e-7, err_msg=name)
    o, Sl = M.deltanet(q, k, v, braw, d, S0)
    np.testing.assert_allclose(ag["o"], o, rtol=1e-12)
    scale = np.exp(r.standard_normal((B, T, H, 1)))
    o2, Sl2 = M.deltanet(q, k * scale, v, braw, d, S0)
    np.testing.assert_allclose(o2, o, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(Sl2, Sl, rtol=1e-10, atol=1e-12)
    assert np.abs((ag["dk"] * k).sum(-1)).max() <= 1e-10 * np.abs(ag["dk"]).max() * np.abs(k).max()
    # on unit keys and gates given as logits it is the plain delta rule
    kn = k / np.linalg.norm(k, axis=-1, keepdims=True)
    o3, Sl3 = M.delta_rule(q, kn, v, M.sigmoid(braw), d, S0)
    np.testing.assert_allclose(o3, o, rtol=1e-12, atol=1e-12)


def test_delta_rule_grads_fd():
    B, T, H, dk, dv = 1, 7, 1, 3, 2
    q, k, v, S0 = rnd(B, T, H, dk), rnd(B, T, H, dk), rnd(B, T, H, dv), rnd(B, H, dv, dk)
    beta = M.sigmoid(rnd(B, T, H))
    do, dSl = rnd(B, T, H, dv), rnd(B, H, dv, dk)
    d = np.zeros((B, T), bool)
    d[0, 4] = True

    def L():
        o, Sl = M.delta_rule(q, k, v, beta, d, S0)
        return (o * do).sum() + (Sl * dSl).sum()

    ag = G.delta_rule_grads(q, k, v, beta, d, S0, do, dSl)
    for name, x in (("dq", q), ("dk", k), ("dv", v), ("dbeta", beta), ("dS0", S0)):
        np.testing.assert_allclose(ag[name], fd(L, x), rtol=1e-6, atol=1e-8, err_msg=name)


def test_gated_linear_attention_grads_finite_differences_and_rowdot_identity():
    """dg equals, inside each episode, the suffix sum of q_t . dq_t - k_t . dk_t (what the kernels
    use); all gradients agree with central finite differences."""
    from oracle import grad as G
    rng = np.random.default_rng(4)
    B, T, H, d = 1, 7, 2, 3
    q, k, v = (rng.standard_normal((B, T, H, d)) for _ in range(3))
    g = -np.abs(rng.standard_normal((B, T, H))) * 0.4
    done = np.zeros((B, T), bool)
    done[0, 3] = True
    S0 = rng.standard_normal((B, H, d, d))
    do = rng.standard_normal((B, T, H, d))
    dSl = rng.standard_normal((B, H, d, d))
    r = G.gated_linear_attention_grads(q, k, v, g, done, S0, do, dSl)

    def loss(q_, k_, v_, g_, S0_):
        o, S = M.gated_linear_attention(q_, k_, v_, g_, done, S0_)
        return (o * do).sum() + (S * dSl).sum()

    eps = 1e-6
    for name, arr in (("dq", q), ("dk", k), ("dv", v), ("dg", g), ("dS0", S0)):
        idx = tuple(rng.integers(0, s) for s in arr.shape)
        args = dict(q_=q, k_=k, v_=v, g_=g, S0_=S0)
        key = {"dq": "q_", "dk": "k_", "dv": "v_", "dg": "g_", "dS0": "S0_"}[name]
        up, dn = arr.copy(), arr.copy()
        up[idx] += eps
        dn[idx] -= eps
        fd = (loss(**{**args, key: up}) - loss(**{**args, key: dn})) / (2 * eps)
        assert abs(fd - r[name][idx]) <= 1e-6 * max(1.0, abs(fd)), (name, fd, r[name][idx])
    e = (q * r["dq"]).sum(-1) - (k * r["dk"]).sum(-1)      # (B,T,H)
    # the final state's own dependence on g enters through dS_last: include it
    _, S_last = M.gated_linear_attention(q, k, v, g, done, S0)
    tail = (S_last * dSl).sum((-1, -2))                    # d/dG_last of <S_last, dS_last>
    ref = np.zeros_like(g)
    acc = tail.copy()
    for t in range(T - 1, -1, -1):
        acc = acc + e[:, t]
        ref[:, t] = np.where(done[:, t][:, None], 0.0, acc)
        acc = np.where(done[:, t][:, None], 0.0, acc)
    np.testing.assert_allclose(r["dg"], ref, rtol=1e-9, atol=1e-9)


def test_torso_parts_of_the_gradient_oracle():
    """rms_norm_t against the closed form; gated_linear_recurrence_t: values against the NumPy
    log-space MinGRU (oracle.memoroid.mingru_scan) composed with the gating by hand, carry against
    the cumulative product of decays since the last reset, and split invariance through the carry;
    deltanet_cell_t against the NumPy composition."""
    import torch
    from oracle import grad as G
    from oracle import memoroid as M
    rng = np.random.default_rng(77)
    B, T, Fe, H, d = 2, 23, 6, 2, 4
    x = rng.standard_normal((B, T, Fe))
    done = rng.random((B, T)) < 0.15
    done[0, 0] = False
    scale = rng.uniform(0.5, 1.5, Fe)
    xn = x / np.sqrt((x ** 2).mean(-1, keepdims=True) + 1e-6) * scale
    assert np.allclose(G.rms_norm_t(torch.from_numpy(x), torch.from_numpy(scale)).numpy(), xn, atol=1e-13)
    Wz, Wh, Wg, Wo = (rng.standard_normal((Fe, Fe)) * 0.7 for _ in range(4))
    t = torch.from_numpy
    carry, y = G.gated_linear_recurrence_t(t(x), t(done), t(Wz), t(Wh), t(Wg), t(Wo))
    z, ht, gt = x @ Wz.T, x @ Wh.T, x @ Wg.T
    nxt, h = M.mingru_scan(z, ht, done.astype(np.float64))
    want = (h * (gt / (1 + np.exp(-gt)))) @ Wo.T
    assert np.allclose(y.numpy(), want, atol=1e-12)
    assert np.allclose(carry[0].numpy(), nxt[0], atol=1e-12) and np.allclose(carry[1].numpy(), nxt[1], atol=1e-12)
    a = 1 / (1 + np.exp(z))   # sigma(-z); cumulative product since the last reset, by brute force
    for b in range(B):
        last = max([i for i in range(T) if done[b, i]] + [0])
        assert np.allclose(np.exp(carry[1].numpy()[b, 0]), a[b, last:].prod(0), atol=1e-13)
    for s in (1, 9, 22):
        c1, y1 = G.gated_linear_recurrence_t(t(x[:, :s]), t(done[:, :s]), t(Wz), t(Wh), t(Wg), t(Wo))
        c2, y2 = G.gated_linear_recurrence_t(t(x[:, s:]), t(done[:, s:]), t(Wz), t(Wh), t(Wg), t(Wo), c1)
        assert np.allclose(np.concatenate([y1.numpy(), y2.numpy()], 1), want, atol=1e-11)
        assert np.allclose(c2[0].numpy(), nxt[0], atol=1e-11) and np.allclose(c2[1].numpy(), nxt[1], atol=1e-11)
    Wq, Wk, Wv = (rng.standard_normal((H * d, Fe)) for _ in range(3))
    Wb, ns = rng.standard_normal((H, Fe)), rng.uniform(0.5, 1.5, H * d)
    Wout, bout = rng.standard_normal((Fe, H * d)), rng.standard_normal(Fe)
    (S,), yd = G.deltanet_cell_t(t(x), t(done), t(Wq), t(Wk), t(Wv), t(Wb), t(ns), t(Wout), t(bout), H)
    hv = lambda w: (x @ w.T).reshape(B, T, H, d)  # noqa: E731
    o, Sl = M.deltanet(hv(Wq), hv(Wk), hv(Wv), x @ Wb.T, done.astype(np.float64))
    o = o.reshape(B, T, H * d)
    o = o / np.sqrt((o ** 2).mean(-1, keepdims=True) + 1e-6) * ns
    assert np.allclose(yd.numpy(), o @ Wout.T + bout, atol=1e-11) and np.allclose(S.numpy()[:, 0], Sl, atol=1e-12)


def test_sum_of_squares_gradient_stored_quotient_and_g_side_options():
    """The three options the GPU comparisons use.  d_ss: the term <d_ss, |o|^2> of the loss, by finite
    differences.  o_stored: with the exact outputs it changes nothing; with perturbed ones only the
    denominator's share of the gradients moves, by -(g . delta o) / den.  side: equal to the default
    when it is the sign of h_tilde; an element within 1e-3 of the kink forced to the other branch moves
    the values by at most 3/4 |x| and is differentiated with that branch's slope."""
    import torch
    B, T, H, dk, dv = 1, 6, 2, 3, 2
    r = np.random.default_rng(4)
    rnd = lambda *s: r.standard_normal(s)  # noqa: E731
    q, k, v, S0 = rnd(B, T, H, dk), rnd(B, T, H, dk), rnd(B, T, H, dv), rnd(B, H, dv, dk)
    z0 = np.abs(rnd(B, H, dk))
    do, d_ss = rnd(B, T, H, dv), rnd(B, T, H)
    d = np.zeros((B, T), bool)
    d[0, 2] = True

    def L():
        o, den, Sl, zl = M.normalised_linear_attention(q, k, v, d, S0, z0, "elu1", 1e-6)
        return (o * do).sum() + ((o * o).sum(-1) * d_ss).sum()

    ag = G.normalised_linear_attention_grads(q, k, v, d, S0, z0, do, None, None, "elu1", 1e-6, d_ss=d_ss)
    for name, x in (("dq", q), ("dk", k), ("dv", v), ("dS0", S0), ("dz0", z0)):
        np.testing.assert_allclose(ag[name], fd(L, x), rtol=1e-5, atol=1e-7, err_msg=name)
    same = G.normalised_linear_attention_grads(q, k, v, d, S0, z0, do, None, None, "elu1", 1e-6, d_ss=d_ss, o_stored=ag["o"])
    for name in ("dq", "dk", "dv", "dS0", "dz0"):
        np.testing.assert_allclose(same[name], ag[name], rtol=1e-12, atol=1e-13, err_msg=name)
    base = G.normalised_linear_attention_grads(q, k, v, d, S0, z0, do)
    off = G.normalised_linear_attention_grads(q, k, v, d, S0, z0, do, o_stored=base["o"] + 0.01)
    np.testing.assert_allclose(off["dv"], base["dv"], rtol=1e-12, atol=1e-13)   # values never see the denominator
    assert np.abs(off["dq"] - base["dq"]).max() > 1e-4                           # queries do

    z, ht = rnd(2, 7, 3), rnd(2, 7, 3)
    ht[0, 3, 1], ht[1, 5, 0] = 4e-4, -7e-4
    done = np.zeros((2, 7), bool)
    t = lambda a: torch.from_numpy(a)  # noqa: E731
    h_def, _ = G.mingru_scan_t(t(z), t(ht), t(done))
    h_same, _ = G.mingru_scan_t(t(z), t(ht), t(done), side=t(ht >= 0))
    assert torch.equal(h_def, h_same)
    side = ht >= 0
    side[0, 3, 1], side[1, 5, 0] = False, True
    htt = t(ht).requires_grad_()
    h_flip, _ = G.mingru_scan_t(t(z), htt, t(done), side=t(side))
    assert (h_flip - h_def).abs().max() <= 0.75 * 7e-4
    h_flip[:, -1].sum().backward()
    htd = t(ht).requires_grad_()
    G.mingru_scan_t(t(z), htd, t(done))[0][:, -1].sum().backward()
    ratio = (htt.grad / htd.grad).numpy()
    assert abs(ratio[0, 3, 1] - 0.25) < 2e-3 and abs(ratio[1, 5, 0] - 4.0) < 2e-2   # slope 1/4 <-> 1
    mask = np.ones_like(ratio, bool)
    mask[0, 3, 1] = mask[1, 5, 0] = False
    np.testing.assert_allclose(ratio[mask], 1.0, rtol=2e-3)


def test_linear_attention_cell_of_the_gradient_oracle():
    """linear_attention_cell_t against the NumPy composition: the reference's materialise-and-scan
    route for numerator and denominator (linear_attention.py:62-110), RMS norm over the heads, projection."""
    import torch
    rng = np.random.default_rng(78)
    B, T, Fe, H, d = 2, 17, 5, 2, 3
    x = rng.standard_normal((B, T, Fe))
    done = rng.random((B, T)) < 0.15
    Wq, Wk, Wv = (rng.standard_normal((H * d, Fe)) for _ in range(3))
    ns, Wout, bout = rng.uniform(0.5, 1.5, H * d), rng.standard_normal((Fe, H * d)), rng.standard_normal(Fe)
    t = torch.from_numpy
    (S, z), y = G.linear_attention_cell_t(t(x), t(done), t(Wq), t(Wk), t(Wv), t(ns), t(Wout), t(bout), H)
    hv = lambda w: (x @ w.T).reshape(B, T, H, d)  # noqa: E731
    nxt, num, den = M.linear_attention_memoroid(hv(Wq), hv(Wk), hv(Wv), done.astype(np.float64), None, "elu1")
    out = (num / np.maximum(den, 1e-6)[..., None]).reshape(B, T, H * d)
    out = out / np.sqrt((out ** 2).mean(-1, keepdims=True) + 1e-6) * ns
    assert np.allclose(y.numpy(), out @ Wout.T + bout, atol=1e-11)
    assert np.allclose(S.numpy(), nxt[0], atol=1e-12) and np.allclose(z.numpy(), nxt[1], atol=1e-12)
    s = 6
    c1, y1 = G.linear_attention_cell_t(t(x[:, :s]), t(done[:, :s]), t(Wq), t(Wk), t(Wv), t(ns), t(Wout), t(bout), H)
    c2, y2 = G.linear_attention_cell_t(t(x[:, s:]), t(done[:, s:]), t(Wq), t(Wk), t(Wv), t(ns), t(Wout), t(bout), H, c1)
    assert np.allclose(np.concatenate([y1.numpy(), y2.numpy()], 1), y.numpy(), atol=1e-11)


def test_mlstm_gates_grads_fd():
    """torch autograd through the gates' restatement against central differences on the NumPy forward:
    a carried m, resets (first step, mid-sequence), one step whose g sits on the floor."""
    B, T, H = 2, 7, 2
    li, lf = rnd(B, T, H) * 2, -np.abs(rnd(B, T, H))
    m0 = rnd(B, H)
    lf[0, 3] = -100.0                 # g_3 is clamped for batch row 0: no gradient through it
    d = np.zeros((B, T), bool)
    d[0, 5] = True
    d[1, 0] = True
    dm, dg, dw = rnd(B, T, H), rnd(B, T, H), rnd(B, T, H)

    def L():
        m, g, w = M.mlstm_gates(li, lf, d, m0)
        return (m * dm).sum() + (g * dg).sum() + (w * dw).sum()
    gi, gf, g0 = G.mlstm_gates_grads(li, lf, d, m0, dm, dg, dw)
    np.testing.assert_allclose(gi, fd(L, li), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(gf, fd(L, lf), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(g0, fd(L, m0), rtol=1e-6, atol=1e-7)
    assert g0[1].tolist() == [0.0, 0.0]   # batch row 1 resets at its first step: the carried m is dropped


def test_rms_norm_closed_forms_and_grads_fd():
    """The norm's restatement against what fixes it: unit mean square and invariance under x -> c x without
    eps, the closed form of a constant row with it; its gradients against central differences, and dx
    orthogonal to x (what the invariance implies) with the analytic formula dx = r g - x r^3 (g . x) / D."""
    x, sc, dy = rnd(3, 5, 8), rnd(8), rnd(3, 5, 8)
    y = M.rms_norm(x, None, eps=0.0)
    np.testing.assert_allclose((y * y).mean(-1), 1.0, rtol=1e-12)
    np.testing.assert_allclose(M.rms_norm(3.7 * x, sc, eps=0.0), M.rms_norm(x, sc, eps=0.0), rtol=1e-12)
    np.testing.assert_allclose(M.rms_norm(np.full((2, 8), 0.5), sc, eps=0.75), 0.5 * sc[None] * np.ones((2, 1)), rtol=1e-12)
    for eps in (0.0, 1e-6, 0.3):
        dx, ds = G.rms_norm_grads(x, sc, dy, eps)
        np.testing.assert_allclose(dx, fd(lambda: (M.rms_norm(x, sc, eps) * dy).sum(), x), rtol=1e-6, atol=1e-8)
        np.testing.assert_allclose(ds, fd(lambda: (M.rms_norm(x, sc, eps) * dy).sum(), sc), rtol=1e-6, atol=1e-8)
        r = 1.0 / np.sqrt((x * x).mean(-1, keepdims=True) + eps)
        g = dy * sc
        np.testing.assert_allclose(dx, r * g - x * r ** 3 * (g * x).sum(-1, keepdims=True) / 8, rtol=1e-10, atol=1e-12)
        np.testing.assert_allclose(ds, (dy * x * r).sum((0, 1)), rtol=1e-10)
    dx0, none = G.rms_norm_grads(x, None, dy, 0.0)
    assert none is None
    np.testing.assert_allclose((dx0 * x).sum(-1), 0.0, atol=1e-12)


def test_silu_gate_closed_forms_and_grads_fd():
    """h * silu(g): silu(0) = 0, silu(g) - silu(-g) = g, silu(g) -> g for large g; gradients against central
    differences and the closed form d silu = s (1 + g (1 - s)), s = sigmoid(g)."""
    h, g, dy = rnd(4, 6), rnd(4, 6) * 3, rnd(4, 6)
    one = np.ones_like(g)
    np.testing.assert_allclose(M.silu_gate(h, np.zeros_like(g)), 0.0)
    np.testing.assert_allclose(M.silu_gate(one, g) - M.silu_gate(one, -g), g, rtol=1e-12)
    np.testing.assert_allclose(M.silu_gate(h, np.full_like(g, 50.0)), 50.0 * h, rtol=1e-12)
    dh, dg = G.silu_gate_grads(h, g, dy)
    np.testing.assert_allclose(dh, fd(lambda: (M.silu_gate(h, g) * dy).sum(), h), rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(dg, fd(lambda: (M.silu_gate(h, g) * dy).sum(), g), rtol=1e-6, atol=1e-8)
    s = 1 / (1 + np.exp(-g))
    np.testing.assert_allclose(dg, dy * h * s * (1 + g * (1 - s)), rtol=1e-10)


def test_layer_norm_closed_forms_and_grads_fd():
    """The layer norm's restatement: zero mean and unit mean square of every row without eps, invariance under
    x -> a x + b (a > 0), agreement with the RMS norm on rows of zero mean, scipy's z-score; gradients against
    central differences, dx orthogonal to the constant row and to x - mean (what the two invariances imply)."""
    from scipy import stats
    x, sc, bi, dy = rnd(3, 5, 8), rnd(8), rnd(8), rnd(3, 5, 8)
    y = M.layer_norm(x, None, None, eps=0.0)
    np.testing.assert_allclose(y.mean(-1), 0.0, atol=1e-14)
    np.testing.assert_allclose((y * y).mean(-1), 1.0, rtol=1e-12)
    np.testing.assert_allclose(y, stats.zscore(x, axis=-1), rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(M.layer_norm(2.5 * x - 7.0, sc, bi, eps=0.0), M.layer_norm(x, sc, bi, eps=0.0), rtol=1e-10, atol=1e-12)
    xz = x - x.mean(-1, keepdims=True)
    np.testing.assert_allclose(M.layer_norm(xz, sc, None, 1e-6), M.rms_norm(xz, sc, 1e-6), rtol=1e-12, atol=1e-14)
    for eps in (0.0, 1e-6, 0.3):
        dx, ds, db = G.layer_norm_grads(x, sc, bi, dy, eps)
        L = lambda: (M.layer_norm(x, sc, bi, eps) * dy).sum()   # noqa: E731
        np.testing.assert_allclose(dx, fd(L, x), rtol=1e-6, atol=1e-8)
        np.testing.assert_allclose(ds, fd(L, sc), rtol=1e-6, atol=1e-8)
        np.testing.assert_allclose(db, fd(L, bi), rtol=1e-6, atol=1e-8)
        np.testing.assert_allclose(db, dy.sum((0, 1)), rtol=1e-12)
        np.testing.assert_allclose(dx.sum(-1), 0.0, atol=1e-12)
    dx0, _, _ = G.layer_norm_grads(x, sc, bi, dy, 0.0)
    np.testing.assert_allclose((dx0 * xz).sum(-1), 0.0, atol=1e-12)
