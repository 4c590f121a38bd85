"""Pins the NumPy oracle by mathematics: independent formulations, closed forms,
brute force and invariants (the reference ships no vectors for this path)."""
import numpy as np
import pytest
import scipy.signal

from oracle import memoroid as M

RNG = np.random.default_rng(7)


def rnd(*s):
    return RNG.standard_normal(s)


def dones(B, T, p):
    return RNG.random((B, T)) < p


# ---------------------------------------------------------------- scan_fn
def _carry_diag(B, D, rng=True):
    return (rnd(B, 1, D), RNG.uniform(0.5, 1.0, (B, 1, D))) if rng else (
        np.zeros((B, 1, D)), np.ones((B, 1, D)))


@pytest.mark.parametrize("T", [1, 2, 7, 9, 33])
@pytest.mark.parametrize("p", [0.0, 0.3, 1.0])
def test_scan_sequential_equals_tree_diag(T, p):
    B, D = 2, 3
    z = (rnd(B, T, D), RNG.uniform(0.5, 1.0, (B, T, D)))
    c = _carry_diag(B, D)
    d = dones(B, T, p)
    hs, cs = M.scan_fn_sequential(z, c, d, M.diag_operator)
    ht, ct = M.scan_fn_tree(z, c, d, M.diag_operator)
    for x, y in zip(hs + cs, ht + ct):
        np.testing.assert_allclose(x, y, rtol=1e-12, atol=1e-13)


def test_scan_brute_force_tiny():
    """Every prefix computed by folding the augmented operator from scratch."""
    B, T, D = 1, 6, 2
    z = (rnd(B, T, D), RNG.uniform(0.5, 1.0, (B, T, D)))
    c = _carry_diag(B, D)
    d = np.array([[0, 1, 0, 0, 1, 0]])
    hs, _ = M.scan_fn_sequential(z, c, d, M.diag_operator)
    aug = M._augmented(M.diag_operator)
    zz, reset = M._prepend(z, c, d)
    for t in range(1, T + 1):
        acc = (tuple(x[:, 0:1] for x in zz), reset[:, 0:1])
        for j in range(1, t + 1):
            acc = aug(acc, (tuple(x[:, j:j + 1] for x in zz), reset[:, j:j + 1]))
        np.testing.assert_allclose(acc[0][0][:, 0], hs[0][:, t - 1], rtol=1e-13)
        np.testing.assert_allclose(acc[0][1][:, 0], hs[1][:, t - 1], rtol=1e-13)


@pytest.mark.parametrize("op,mk", [
    (M.diag_operator, lambda: (rnd(2, 1, 3), rnd(2, 1, 3))),
    (M.additive_operator, lambda: (rnd(2, 1, 3, 3), rnd(2, 1, 3))),
    (M.mingru_operator, lambda: (rnd(2, 1, 3), -np.abs(rnd(2, 1, 3)))),
    (M.delta_operator, lambda: (rnd(2, 1, 3, 3), rnd(2, 1, 3, 3))),
])
def test_augmented_operator_associative(op, mk):
    aug = M._augmented(op)
    for bits in range(8):
        x, y, z = [(mk(), np.full((2, 1, 1), float((bits >> i) & 1))) for i in range(3)]
        l = aug(aug(x, y), z)
        r = aug(x, aug(y, z))
        for a, b in zip(l[0], r[0]):
            np.testing.assert_allclose(a, b, rtol=1e-12, atol=1e-12)
        np.testing.assert_array_equal(l[1], r[1])


def test_diag_scan_matches_scan_fn():
    B, T, D = 3, 40, 5
    a, b = RNG.uniform(0.5, 1.0, (B, T, D)), rnd(B, T, D)
    h0, P0 = rnd(B, D), RNG.uniform(0.5, 1, (B, D))
    d = dones(B, T, 0.1)
    h, hl, Pl = M.diag_scan(a, b, d, h0, P0)
    (hs, Ps), (ch, cP) = M.scan_fn_tree((b, a), (h0[:, None], P0[:, None]), d, M.diag_operator)
    np.testing.assert_allclose(h, hs, rtol=1e-12)
    np.testing.assert_allclose(hl, ch[:, 0], rtol=1e-12)
    np.testing.assert_allclose(Pl, cP[:, 0], rtol=1e-12)


def test_diag_closed_forms():
    B, T, D = 2, 50, 4
    b = rnd(B, T, D)
    nd = np.zeros((B, T), bool)
    # a == 1 -> cumsum
    h, _, _ = M.diag_scan(np.ones((B, T, D)), b, nd)
    np.testing.assert_allclose(h, np.cumsum(b, 1), rtol=1e-12, atol=1e-12)
    # constant a -> IIR filter / geometric series
    a = 0.9
    h, hl, Pl = M.diag_scan(np.full((B, T, D), a), b, nd)
    np.testing.assert_allclose(h, scipy.signal.lfilter([1.0], [1.0, -a], b, axis=1), rtol=1e-11)
    geo = sum(a ** (T - 1 - s) * b[:, s] for s in range(T))
    np.testing.assert_allclose(hl, geo, rtol=1e-11)
    np.testing.assert_allclose(Pl, a ** T, rtol=1e-12)
    # P_T = product of a since the last reset (inclusive)
    av = RNG.uniform(0.5, 1.0, (B, T, D))
    d = np.zeros((B, T), bool)
    d[0, 17] = True
    d[1, 0] = True
    _, _, Pl = M.diag_scan(av, b, d)
    np.testing.assert_allclose(Pl[0], np.prod(av[0, 17:], 0), rtol=1e-12)
    np.testing.assert_allclose(Pl[1], np.prod(av[1, 0:], 0), rtol=1e-12)


def test_diag_complex_time_invariant():
    B, T, D = 2, 20, 3
    lam = 0.9 * np.exp(1j * RNG.uniform(0, 3, D))
    b = rnd(B, T, D) + 1j * rnd(B, T, D)
    h, hl, _ = M.diag_scan(lam, b, np.zeros((B, T), bool))
    ref = sum(lam ** (T - 1 - s) * b[:, s] for s in range(T))
    np.testing.assert_allclose(hl, ref, rtol=1e-11)


def test_split_invariance_and_done_first():
    B, T, D = 2, 24, 3
    a, b = RNG.uniform(0.5, 1, (B, T, D)), rnd(B, T, D)
    h0 = rnd(B, D)
    d = dones(B, T, 0.2)
    d[0, 8] = True
    full = M.diag_scan(a, b, d, h0)
    for s in range(1, T):
        h1, hl1, P1 = M.diag_scan(a[:, :s], b[:, :s], d[:, :s], h0)
        h2, hl2, P2 = M.diag_scan(a[:, s:], b[:, s:], d[:, s:], hl1, P1)
        np.testing.assert_allclose(np.concatenate([h1, h2], 1), full[0], rtol=1e-12)
        np.testing.assert_allclose(hl2, full[1], rtol=1e-12)
        np.testing.assert_allclose(P2, full[2], rtol=1e-12)
    d2 = d.copy()
    d2[:, 0] = True
    x = M.diag_scan(a, b, d2, h0)
    y = M.diag_scan(a, b, d2, h0 * 0 + 123.0)
    np.testing.assert_array_equal(x[0], y[0])


def test_reset_isolation_poison():
    B, T, D = 1, 12, 2
    a, b = RNG.uniform(0.5, 1, (B, T, D)), rnd(B, T, D)
    b[0, 3] = np.nan
    a[0, 4] = np.inf
    d = np.zeros((B, T), bool)
    d[0, 6] = True
    h, hl, Pl = M.diag_scan(a, b, d)
    assert np.isfinite(h[0, 6:]).all() and np.isfinite(hl).all() and np.isfinite(Pl).all()
    np.testing.assert_array_equal(h[0, 6], b[0, 6])
    (hs, _), _ = M.scan_fn_tree((b, a), (np.zeros((B, 1, D)), np.ones((B, 1, D))), d, M.diag_operator)
    assert np.isfinite(hs[0, 6:]).all()
    np.testing.assert_allclose(hs[0, 6:], h[0, 6:], rtol=1e-12)


# ---------------------------------------------------------------- MinGRU
def test_mingru_log_space_equals_linear_space():
    B, T, F = 2, 30, 4
    z, ht = 2 * rnd(B, T, F), 2 * rnd(B, T, F)
    d = dones(B, T, 0.1)
    nxt, h = M.mingru_scan(z, ht, d)
    a, b = M.mingru_linear_coeffs(z, ht)
    h2, hl, Pl = M.diag_scan(a, b, d)
    np.testing.assert_allclose(h, h2, rtol=1e-10)
    np.testing.assert_allclose(np.exp(nxt[0][:, 0]), hl, rtol=1e-10)
    np.testing.assert_allclose(nxt[1][:, 0], np.log(Pl), rtol=1e-10)
    np.testing.assert_allclose(h[:, 0], b[:, 0], rtol=1e-12)   # (-inf, 0) carry
    assert (h > 0).all()


# ---------------------------------------------------------------- linear attention
@pytest.mark.parametrize("fmap", ["none", "elu1"])
@pytest.mark.parametrize("p", [0.0, 0.15])
def test_linear_attention_formulations(fmap, p):
    B, T, H, dk, dv = 2, 37, 2, 5, 4
    q, k, v = rnd(B, T, H, dk), rnd(B, T, H, dk), rnd(B, T, H, dv)
    S0 = rnd(B, H, dv, dk)
    d = dones(B, T, p)
    o, Sl = M.linear_attention(q, k, v, d, S0, fmap)
    oq = M.linear_attention_quadratic(q, k, v, d, S0, fmap)
    np.testing.assert_allclose(o, oq, rtol=1e-10, atol=1e-10)
    for C in (1, 16, 64, T):
        oc, Sc = M.linear_attention_chunked(q, k, v, d, S0, fmap, chunk=C)
        np.testing.assert_allclose(o, oc, rtol=1e-10, atol=1e-10)
        np.testing.assert_allclose(Sl, Sc, rtol=1e-10, atol=1e-10)
    kf = M._fmap(k, fmap)
    z0 = rnd(B, H, dk)
    nxt, num, den = M.linear_attention_memoroid(q, k, v, d, (S0[:, None], z0[:, None]), fmap)
    np.testing.assert_allclose(num, o, rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(nxt[0][:, 0], Sl, rtol=1e-10, atol=1e-10)
    # denominator: diagonal scan with a == 1 on z = phi(k), dotted with phi(q)
    zc, _, _ = M.diag_scan(np.ones((B, T, H * dk)), kf.reshape(B, T, -1), d, z0.reshape(B, -1))
    den2 = np.einsum("bthd,bthd->bth", M._fmap(q, fmap), zc.reshape(B, T, H, dk))
    np.testing.assert_allclose(den, den2, rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("p", [0.0, 0.15])
def test_normalised_linear_attention_against_the_materialised_route_and_convexity(p):
    B, T, H, dk, dv = 2, 29, 2, 5, 4
    q, k, v = rnd(B, T, H, dk), rnd(B, T, H, dk), rnd(B, T, H, dv)
    S0, z0 = rnd(B, H, dv, dk), np.abs(rnd(B, H, dk))
    d = dones(B, T, p)
    o, den, Sl, zl = M.normalised_linear_attention(q, k, v, d, S0, z0, "elu1", 1e-6)
    # the reference's route: materialised outer products, additive tree scan, read-out
    nxt, num, den2 = M.linear_attention_memoroid(q, k, v, d, (S0[:, None], z0[:, None]), "elu1")
    np.testing.assert_allclose(den, np.maximum(den2, 1e-6), rtol=1e-10)
    np.testing.assert_allclose(o, num / np.maximum(den2, 1e-6)[..., None], rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(Sl, nxt[0][:, 0], rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(zl, nxt[1][:, 0], rtol=1e-10, atol=1e-12)
    # without carry the read-out is a convex combination of the episode's values:
    # constant values come back unchanged, and every output lies within the values' range
    c = rnd(dv)
    oc, _, _, _ = M.normalised_linear_attention(q, k, np.broadcast_to(c, v.shape), d, None, None, "elu1", 1e-6)
    np.testing.assert_allclose(oc, np.broadcast_to(c, v.shape), rtol=1e-10, atol=1e-12)
    on, _, _, _ = M.normalised_linear_attention(q, k, v, d, None, None, "elu1", 1e-6)
    assert on.max() <= v.max() + 1e-12 and on.min() >= v.min() - 1e-12
    # the clamp: a denominator below eps is replaced by eps
    ob, denb, _, _ = M.normalised_linear_attention(q, k, v, d, None, None, "elu1", 1e3)
    assert (denb == 1e3).all()
    num0, _ = M.linear_attention(q, k, v, d, None, "elu1")
    np.testing.assert_allclose(ob, num0 / 1e3, rtol=1e-12)


def test_linear_attention_cumsum_special_case():
    B, T, H, d = 1, 20, 1, 3
    e1 = np.zeros((B, T, H, d))
    e1[..., 0] = 1.0
    v = rnd(B, T, H, d)
    o, _ = M.linear_attention(e1, e1, v, np.zeros((B, T), bool))
    np.testing.assert_allclose(o, np.cumsum(v, 1), rtol=1e-12, atol=1e-12)


def test_elu1_values():
    np.testing.assert_allclose(M.elu1(np.array([-1.0, 0.0, 2.0])), [np.exp(-1.0), 1.0, 3.0])


# ---------------------------------------------------------------- delta rule
@pytest.mark.parametrize("p", [0.0, 0.1])
def test_delta_rule_formulations(p):
    B, T, H, dk, dv = 2, 45, 2, 6, 5
    q, k, v = rnd(B, T, H, dk), rnd(B, T, H, dk), rnd(B, T, H, dv)
    k /= np.linalg.norm(k, axis=-1, keepdims=True)
    beta = M.sigmoid(rnd(B, T, H))
    S0 = rnd(B, H, dv, dk)
    d = dones(B, T, p)
    o, Sl = M.delta_rule(q, k, v, beta, d, S0)
    o2, S2 = M.delta_rule_explicit(q, k, v, beta, d, S0)
    np.testing.assert_allclose(o, o2, rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(Sl, S2, rtol=1e-10, atol=1e-11)
    o3, S3 = M.delta_rule_memoroid(q, k, v, beta, d, S0)
    np.testing.assert_allclose(o, o3, rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(Sl, S3, rtol=1e-9, atol=1e-10)
    for C in (1, 8, 16, 64):
        oc, Sc = M.delta_rule_chunked(q, k, v, beta, d, S0, chunk=C)
        np.testing.assert_allclose(o, oc, rtol=1e-9, atol=1e-10)
        np.testing.assert_allclose(Sl, Sc, rtol=1e-9, atol=1e-10)


def test_delta_rule_special_cases():
    B, T, H, d = 1, 6, 1, 6
    q = rnd(B, T, H, d)
    S0 = rnd(B, H, d, d)
    nd = np.zeros((B, T), bool)
    # beta = 0: state never changes
    k, v = rnd(B, T, H, d), rnd(B, T, H, d)
    o, Sl = M.delta_rule(q, k, v, np.zeros((B, T, H)), nd, S0)
    np.testing.assert_allclose(Sl, S0)
    np.testing.assert_allclose(o, np.einsum("bhij,bthj->bthi", S0, q))
    # beta = 1, orthonormal keys: exact overwrite, earlier pairs retained
    Qm, _ = np.linalg.qr(rnd(d, d))
    k = Qm[None, :, None, :]
    o, Sl = M.delta_rule(q, k, v, np.ones((B, T, H)), nd, S0)
    for t in range(T):
        np.testing.assert_allclose(Sl[0, 0] @ k[0, t, 0], v[0, t, 0], rtol=1e-10, atol=1e-12)
    # unit keys, beta in (0,1): transition eigenvalues within [0,1]
    kk = rnd(d)
    kk /= np.linalg.norm(kk)
    ev = np.linalg.eigvalsh(np.eye(d) - 0.7 * np.outer(kk, kk))
    assert ev.min() >= -1e-12 and ev.max() <= 1 + 1e-12


def test_delta_rule_split_invariance_with_resets():
    B, T, H, d = 2, 20, 1, 4
    q, k, v = rnd(B, T, H, d), rnd(B, T, H, d), rnd(B, T, H, d)
    beta = M.sigmoid(rnd(B, T, H))
    dn = dones(B, T, 0.2)
    dn[0, 9] = True
    o, Sl = M.delta_rule(q, k, v, beta, dn)
    for s in (1, 9, 10, 19):
        o1, S1 = M.delta_rule(q[:, :s], k[:, :s], v[:, :s], beta[:, :s], dn[:, :s])
        o2, S2 = M.delta_rule(q[:, s:], k[:, s:], v[:, s:], beta[:, s:], dn[:, s:], S1)
        np.testing.assert_allclose(np.concatenate([o1, o2], 1), o, rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(S2, Sl, rtol=1e-12, atol=1e-12)


def test_make_inputs_shapes_and_determinism():
    x = M.make_inputs(4, (2, 16, 2, 8))
    y = M.make_inputs(4, (2, 16, 2, 8))
    for key in x:
        np.testing.assert_array_equal(x[key], y[key])
    np.testing.assert_allclose(np.linalg.norm(x["k"], axis=-1), 1.0, rtol=1e-5)
    assert M.make_inputs(1)["a"].shape == (32, 128, 256)


# ---- gated linear attention (the Mamba cell's algebra) -------------------------------------
def _gla_inputs(B=2, T=13, H=2, d=4, p=0.2, seed=0):
    rng = np.random.default_rng(seed)
    q, k, v = (rng.standard_normal((B, T, H, d)) for _ in range(3))
    g = -np.abs(rng.standard_normal((B, T, H))) * 0.5
    done = rng.random((B, T)) < p
    S0 = rng.standard_normal((B, H, d, d))
    return q, k, v, g, done, S0


def test_gated_linear_attention_forms_agree():
    q, k, v, g, done, S0 = _gla_inputs()
    o, S = M.gated_linear_attention(q, k, v, g, done, S0)
    oq = M.gated_linear_attention_quadratic(q, k, v, g, done, S0)
    np.testing.assert_allclose(o, oq, rtol=1e-11, atol=1e-11)
    carry = (S0[:, None], np.ones((2, 1, 2, 1, 1)))
    nxt, om = M.gated_linear_attention_memoroid(q, k, v, g, done, carry)
    np.testing.assert_allclose(o, om, rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(S, nxt[0][:, 0], rtol=1e-11, atol=1e-11)


def test_gated_linear_attention_special_cases():
    q, k, v, g, done, S0 = _gla_inputs(seed=1)
    # zero log-decay is plain linear attention
    o0, S0l = M.gated_linear_attention(q, k, v, 0 * g, done, S0)
    o1, S1l = M.linear_attention(q, k, v, done, S0)
    np.testing.assert_allclose(o0, o1, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(S0l, S1l, rtol=1e-12, atol=1e-12)
    # constant decay, k = q = e_1, no resets: o[..., i] is a first-order IIR filter of v[..., i]
    from scipy.signal import lfilter
    B, T, H, d = q.shape
    e1 = np.zeros_like(q)
    e1[..., 0] = 1.0
    a = 0.8
    o, _ = M.gated_linear_attention(e1, e1, v, np.full_like(g, np.log(a)), np.zeros((B, T), bool))
    ref = lfilter([1.0], [1.0, -a], v, axis=1)
    np.testing.assert_allclose(o, ref, rtol=1e-11, atol=1e-11)
    # the decay of an episode's first step has no effect
    g2 = g.copy()
    g2[done] = -7.0
    oa, Sa = M.gated_linear_attention(q, k, v, g, done, None)
    ob, Sb = M.gated_linear_attention(q, k, v, g2, done, None)
    bt0 = np.cumsum(done, 1) > 0    # steps whose history does not reach the carry
    np.testing.assert_allclose(oa[bt0], ob[bt0], rtol=1e-12, atol=1e-12)


def test_gated_linear_attention_split_invariance():
    q, k, v, g, done, S0 = _gla_inputs(T=11, seed=2)
    o, S = M.gated_linear_attention(q, k, v, g, done, S0)
    for s in range(1, 11):
        o1, S1 = M.gated_linear_attention(q[:, :s], k[:, :s], v[:, :s], g[:, :s], done[:, :s], S0)
        o2, S2 = M.gated_linear_attention(q[:, s:], k[:, s:], v[:, s:], g[:, s:], done[:, s:], S1)
        np.testing.assert_allclose(np.concatenate([o1, o2], 1), o, rtol=1e-11, atol=1e-11)
        np.testing.assert_allclose(S2, S, rtol=1e-11, atol=1e-11)


def test_propagate_sensitivities_is_the_diagonal_scan_with_repeated_decay():
    rng = np.random.default_rng(8)
    B, T, H, ps = 2, 9, 3, (2, 2)
    decay = rng.uniform(0.5, 1.0, (B, T, H))
    J = {"w": rng.standard_normal((B, T, H, *ps)), "b": rng.standard_normal((B, T, H))}
    S = {"w": rng.standard_normal((B, 1, H, *ps)), "b": rng.standard_normal((B, 1, H))}
    done = rng.random((B, T)) < 0.25
    out = M.propagate_sensitivities(decay, J, S, done)
    for name, n in (("w", 4), ("b", 1)):
        a = np.repeat(decay, n, axis=-1)
        h, h_last, _ = M.diag_scan(a, J[name].reshape(B, T, H * n), done, S[name].reshape(B, H * n))
        np.testing.assert_allclose(out[name].reshape(B, H * n), h_last, rtol=1e-12, atol=1e-12)
    # no resets, constant decay: closed form sum_s a^(T-s) J_s + a^T S
    a0 = 0.9
    o2 = M.propagate_sensitivities(np.full((B, T, H), a0), {"b": J["b"]}, {"b": S["b"]}, np.zeros((B, T), bool))
    w = a0 ** np.arange(T - 1, -1, -1)
    ref = (J["b"] * w[None, :, None]).sum(1) + a0 ** T * S["b"][:, 0]
    np.testing.assert_allclose(o2["b"][:, 0], ref, rtol=1e-12, atol=1e-12)


# ---- mLSTM (stabilised gated linear attention) -------------------------------------------------
def _mlstm_inputs(B=2, T=12, H=2, d=3, p=0.2, seed=0):
    rng = np.random.default_rng(seed)
    q, k, v = (rng.standard_normal((B, T, H, d)) for _ in range(3))
    ig = rng.standard_normal((B, T, H)) * 2.0
    fg = rng.standard_normal((B, T, H)) * 2.0 + 2.0
    done = rng.random((B, T)) < p
    return q, k, v, ig, fg, done


def test_mlstm_operator_is_associative_and_orders_agree():
    rng = np.random.default_rng(3)
    def el():
        return (rng.standard_normal((2, 1, 2, 3, 3)), -np.abs(rng.standard_normal((2, 1, 2, 1, 1))),
                rng.standard_normal((2, 1, 2, 3, 1)), rng.standard_normal((2, 1, 2, 1, 1)) * 3)
    a, b, c = el(), el(), el()
    l = M.mlstm_operator(M.mlstm_operator(a, b), c)
    r = M.mlstm_operator(a, M.mlstm_operator(b, c))
    for x, y in zip(l, r):
        np.testing.assert_allclose(x, y, rtol=1e-12, atol=1e-12)
    q, k, v, ig, fg, done = _mlstm_inputs()
    n1, h1 = M.mlstm(q, k, v, ig, fg, done, tree=True)
    n2, h2 = M.mlstm(q, k, v, ig, fg, done, tree=False)
    np.testing.assert_allclose(h1, h2, rtol=1e-10, atol=1e-12)
    for x, y in zip(n1, n2):
        np.testing.assert_allclose(x, y, rtol=1e-10, atol=1e-12)


def test_mlstm_stabilised_scan_equals_plain_recurrence():
    q, k, v, ig, fg, done = _mlstm_inputs(seed=4)
    _, h = M.mlstm(q, k, v, ig, fg, done)
    np.testing.assert_allclose(h, M.mlstm_unstabilised(q, k, v, ig, fg, done), rtol=1e-9, atol=1e-12)
    # split invariance through the carry
    nxt, ha = M.mlstm(q[:, :5], k[:, :5], v[:, :5], ig[:, :5], fg[:, :5], done[:, :5])
    _, hb = M.mlstm(q[:, 5:], k[:, 5:], v[:, 5:], ig[:, 5:], fg[:, 5:], done[:, 5:], nxt)
    np.testing.assert_allclose(np.concatenate([ha, hb], 1), h, rtol=1e-9, atol=1e-12)


def test_mlstm_gates_are_the_stabilised_scan_unrolled():
    """oracle.memoroid.mlstm_gates against the cell's own route: m is the m leaf of the stabilised scan
    (mlstm_operator under the select-reset scan), and a plain gated recurrence driven by its g and w
    reproduces the scan's C and n leaves step by step -- with a carried state, resets at the first step and
    in runs, and through a split."""
    q, k, v, ig, fg, done = _mlstm_inputs(seed=9, p=0.2)
    done[0, 0] = True
    done[1, 3:5] = True
    B, T, H, d = q.shape
    rng = np.random.default_rng(10)
    carry = (rng.standard_normal((B, 1, H, d, d)), -np.abs(rng.standard_normal((B, 1, H, 1, 1))),
             rng.standard_normal((B, 1, H, d, 1)), rng.standard_normal((B, 1, H, 1, 1)))
    z = M.mlstm_elements(q, k, v, ig, fg)
    h, nxt = M.scan_fn_sequential(z, carry, done, M.mlstm_operator)
    log_f = -M.softplus(-fg)
    m, g, w = M.mlstm_gates(ig, log_f, done, carry[3][:, 0, :, 0, 0], g_floor=-1e30)
    np.testing.assert_allclose(m, h[3][..., 0, 0], rtol=1e-12, atol=1e-12)
    assert (g <= 1e-12).all() and (w <= 1 + 1e-12).all()
    C, n = carry[0][:, 0].copy(), carry[2][:, 0, ..., 0].copy()
    ks = k / np.sqrt(d)
    for t in range(T):
        r = (done[:, t] != 0)[:, None]
        dec = np.where(r, 0.0, np.exp(g[:, t]))          # a reset drops the state; its g is 0 by convention
        C = dec[..., None, None] * C + w[:, t][..., None, None] * np.einsum("bhi,bhj->bhij", ks[:, t], v[:, t])
        n = dec[..., None] * n + w[:, t][..., None] * ks[:, t]
        np.testing.assert_allclose(C, h[0][:, t], rtol=1e-9, atol=1e-12)
        np.testing.assert_allclose(n, h[2][:, t, ..., 0], rtol=1e-9, atol=1e-12)
    # the floor only ever raises a decay that multiplies a state e^60 times smaller than the new term
    _, g60, _ = M.mlstm_gates(ig, log_f, done, carry[3][:, 0, :, 0, 0])
    assert (g60 >= -60).all() and np.array_equal(g60[g > -60], g[g > -60])
    # split through the carried m
    ma, ga, wa = M.mlstm_gates(ig[:, :5], log_f[:, :5], done[:, :5], carry[3][:, 0, :, 0, 0])
    mb, gb, wb = M.mlstm_gates(ig[:, 5:], log_f[:, 5:], done[:, 5:], ma[:, -1])
    for whole, a_, b_ in ((m, ma, mb), (g60, ga, gb), (w, wa, wb)):
        np.testing.assert_array_equal(np.concatenate([a_, b_], 1), whole)
    # no carried state = the cell's initial -1e9
    m_n, _, _ = M.mlstm_gates(ig, log_f, done)
    np.testing.assert_allclose(m_n, M.mlstm_gates(ig, log_f, done, np.full((B, H), -1e9))[0])
