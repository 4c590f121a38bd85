"""Property tests of the oracle over drawn shapes, reset patterns and split points (hypothesis):
the formulations that the seeded tests compare on a few fixed shapes must agree on any."""
import numpy as np
from hypothesis import given, settings, strategies as st

from oracle import memoroid as M

CFG = dict(max_examples=30, deadline=None)


@st.composite
def case(draw, max_t=14):
    B, T = draw(st.integers(1, 3)), draw(st.integers(1, max_t))
    seed = draw(st.integers(0, 2**31 - 1))
    done = np.array(draw(st.lists(st.booleans(), min_size=B * T, max_size=B * T))).reshape(B, T)
    return B, T, np.random.default_rng(seed), done


@settings(**CFG)
@given(case(), st.integers(1, 4))
def test_diagonal_scan_orders_splits_and_poison(c, D):
    B, T, rng, done = c
    a, b = rng.uniform(0.3, 1.2, (B, T, D)), rng.standard_normal((B, T, D))
    h0, P0 = rng.standard_normal((B, D)), rng.uniform(0.5, 1.0, (B, D))
    h, hl, Pl = M.diag_scan(a, b, done, h0, P0)
    for scan in (M.scan_fn_sequential, M.scan_fn_tree):
        (hs, Ps), (nh, nP) = scan((b, a), (h0[:, None], P0[:, None]), done, M.diag_operator)
        np.testing.assert_allclose(hs, h, rtol=1e-10, atol=1e-12)
        np.testing.assert_allclose(nh[:, 0], hl, rtol=1e-10, atol=1e-12)
        np.testing.assert_allclose(nP[:, 0], Pl, rtol=1e-10, atol=1e-12)
    s = int(rng.integers(0, T + 1))
    if 0 < s < T:
        h1, hl1, P1 = M.diag_scan(a[:, :s], b[:, :s], done[:, :s], h0, P0)
        h2, hl2, P2 = M.diag_scan(a[:, s:], b[:, s:], done[:, s:], hl1, P1)
        np.testing.assert_allclose(np.concatenate([h1, h2], 1), h, rtol=1e-12, atol=1e-14)
        np.testing.assert_allclose(hl2, hl, rtol=1e-12, atol=1e-14)
        np.testing.assert_allclose(P2, Pl, rtol=1e-12, atol=1e-14)
    # poison: whatever precedes a reset never reaches what follows it
    for bi in range(B):
        idx = np.flatnonzero(done[bi])
        if len(idx) and idx[-1] > 0:
            r = idx[-1]
            bp, ap = b.copy(), a.copy()
            bp[bi, :r], ap[bi, :r] = np.nan, np.inf
            hp, hlp, Plp = M.diag_scan(ap, bp, done, h0, P0)
            np.testing.assert_array_equal(hp[bi, r:], h[bi, r:])
            np.testing.assert_array_equal(hlp[bi], hl[bi])
            np.testing.assert_array_equal(Plp[bi], Pl[bi])


@settings(**CFG)
@given(case(), st.integers(1, 3), st.integers(1, 4), st.sampled_from(["none", "elu1"]), st.integers(1, 9))
def test_linear_attention_recurrent_quadratic_chunked(c, H, d, fmap, chunk):
    B, T, rng, done = c
    q, k, v = (rng.standard_normal((B, T, H, d)) for _ in range(3))
    S0 = rng.standard_normal((B, H, d, d))
    o, Sl = M.linear_attention(q, k, v, done, S0, fmap)
    np.testing.assert_allclose(M.linear_attention_quadratic(q, k, v, done, S0, fmap), o, rtol=1e-9, atol=1e-10)
    oc, Sc = M.linear_attention_chunked(q, k, v, done, S0, fmap, chunk=chunk)
    np.testing.assert_allclose(oc, o, rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(Sc, Sl, rtol=1e-9, atol=1e-10)


@settings(**CFG)
@given(case(max_t=12), st.integers(1, 2), st.integers(2, 4), st.integers(1, 8))
def test_delta_rule_sequential_explicit_chunked(c, H, d, chunk):
    B, T, rng, done = c
    q, v = rng.standard_normal((B, T, H, d)), rng.standard_normal((B, T, H, d))
    k = rng.standard_normal((B, T, H, d))
    k /= np.linalg.norm(k, axis=-1, keepdims=True)
    beta = rng.uniform(0.0, 1.0, (B, T, H))
    S0 = rng.standard_normal((B, H, d, d))
    o, Sl = M.delta_rule(q, k, v, beta, done, S0)
    oe, Se = M.delta_rule_explicit(q, k, v, beta, done, S0)
    oc, Sc = M.delta_rule_chunked(q, k, v, beta, done, S0, chunk=chunk)
    for x, y in ((oe, o), (Se, Sl), (oc, o), (Sc, Sl)):
        np.testing.assert_allclose(x, y, rtol=1e-9, atol=1e-10)


@settings(**CFG)
@given(case(), st.integers(1, 4))
def test_mingru_log_space_equals_linear_space(c, F):
    B, T, rng, done = c
    z, x = 3 * rng.standard_normal((B, T, F)), 3 * rng.standard_normal((B, T, F))
    nxt, h = M.mingru_scan(z, x, done)
    a, b = M.mingru_linear_coeffs(z, x)
    h2, hl, _ = M.diag_scan(a, b, done)
    np.testing.assert_allclose(h, h2, rtol=1e-9, atol=1e-300)
    np.testing.assert_allclose(np.exp(nxt[0][:, 0]), hl, rtol=1e-9, atol=1e-300)
