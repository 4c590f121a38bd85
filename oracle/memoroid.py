"""NumPy fp64 restatement of the reference's sequence-model hot path.

TEST INFRASTRUCTURE: imported only by tests, smoke() and bench.py's cpu_baseline.

Reference anchors (paths relative to the reference tree):

* reset-aware associative scan ........ memorax/networks/sequence_models/memoroid.py:60-91
* reset broadcasting / slicing ......... memorax/utils/axes.py:19-32,64-77
* diagonal algebra ..................... lru.py:92-95, s5.py:133-136, mamba.py:119-122
* MinGRU log-space algebra ............. min_gru.py:49-78
* linear attention (phi = elu+1) ....... linear_attention.py:58-117
* DeltaNet delta rule .................. not in the reference; specified by
  S_t = S_{t-1}(I - beta_t k_t k_t^T) + beta_t v_t k_t^T, o_t = S_t q_t.

Conventions: arrays are (B, T, ...) with time on axis 1; carries have a size-1
time axis (B, 1, ...) like the reference's ``initialize_carry``; ``done`` is
(B, T), nonzero meaning "step t starts a new episode: clear the carry before
step t consumes its input".  The matrix state is d_v x d_k (``S[i, j] = v_i k_j``,
linear_attention.py:78).
"""
from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------
# axes helpers (memorax/utils/axes.py:19-32,64-67)
# --------------------------------------------------------------------------


def tail(x):
    return x[:, 1:]


def last(x):
    return x[:, -1:]


def broadcast_done(done, carry):
    """axes.py:64-67: append feature axes to ``done`` until ranks match."""
    while done.ndim != carry.ndim:
        done = done[..., None] if done.ndim < carry.ndim else done[..., 0]
    return done


# --------------------------------------------------------------------------
# cell algebras: binary_operator(a=left/earlier, b=right/later)
# --------------------------------------------------------------------------


def diag_operator(a, b):
    """lru.py:92-95 / s5.py:133-136 / mamba.py:119-122."""
    state_i, decay_i = a
    state_j, decay_j = b
    return (decay_j * state_i + state_j, decay_j * decay_i)


def mingru_operator(a, b):
    """min_gru.py:67-74 (log space)."""
    ls_i, d_i = a
    ls_j, d_j = b
    return (np.logaddexp(d_j + ls_i, ls_j), d_i + d_j)


def additive_operator(a, b):
    """linear_attention.py:82-86."""
    return tuple(x + y for x, y in zip(a, b))


def delta_operator(a, b):
    """Affine-map composition for the delta rule written in the reference's
    idiom: element (Bm, Am) stands for S -> S @ Am + Bm."""
    B_i, A_i = a
    B_j, A_j = b
    return (B_i @ A_j + B_j, A_i @ A_j)


def mlstm_operator(a, b):
    """mlstm.py:190-206: max-stabilised gated sum of (C, log_f, n, m)."""
    C_a, log_f_a, n_a, m_a = a
    C_b, log_f_b, n_b, m_b = b
    log_f = log_f_a + log_f_b
    m_a_decayed = m_a + log_f_b
    m_combined = np.maximum(m_a_decayed, m_b)
    scale_a = np.exp(m_a_decayed - m_combined)
    scale_b = np.exp(m_b - m_combined)
    return (scale_a * C_a + scale_b * C_b, log_f, scale_a * n_a + scale_b * n_b, m_combined)


# --------------------------------------------------------------------------
# Memoroid.scan_fn, two independent formulations
# --------------------------------------------------------------------------


def _augmented(op):
    """memoroid.py:72-85: ((carry, reset) x (carry, reset)) -> (carry, reset);
    the right element wins by *select* when its reset flag is set."""

    def aug(lhs, rhs):
        lc, lr = lhs
        rc, rr = rhs
        comb = op(lc, rc)
        out = tuple(
            np.where(broadcast_done(rr, r) != 0, r, c) for r, c in zip(rc, comb)
        )
        return out, np.maximum(lr, rr)

    return aug


def _prepend(z, initial_carry, done):
    """memoroid.py:61-68: carry becomes slot 0 with reset flag 0."""
    zz = tuple(np.concatenate([c, e], axis=1) for c, e in zip(initial_carry, z))
    done = np.asarray(done, dtype=np.float64)
    reset = np.concatenate([np.zeros((done.shape[0], 1)), done], axis=1)[..., None]
    return zz, reset


def scan_fn_sequential(z, initial_carry, done, op):
    """Left fold with select-style reset: h_j = reset_j ? z_j : op(h_{j-1}, z_j).

    Returns (h, next_carry) like memoroid.py:87-91 (h has the carry slot removed).
    """
    zz, reset = _prepend(z, initial_carry, done)
    n = reset.shape[1]
    cur = tuple(x[:, 0:1] for x in zz)
    outs = [cur]
    for j in range(1, n):
        nxt = tuple(x[:, j : j + 1] for x in zz)
        with np.errstate(all="ignore"):
            comb = op(cur, nxt)
        r = reset[:, j : j + 1]
        cur = tuple(
            np.where(broadcast_done(r, e) != 0, e, c) for e, c in zip(nxt, comb)
        )
        outs.append(cur)
    h = tuple(np.concatenate([o[i] for o in outs], axis=1) for i in range(len(zz)))
    return tuple(tail(x) for x in h), tuple(last(x) for x in h)


def scan_fn_tree(z, initial_carry, done, op):
    """Inclusive scan with the augmented operator applied in Hillis-Steele
    (doubling) order: a different association order from the sequential fold,
    as jax.lax.associative_scan's is (memoroid.py:87)."""
    zz, reset = _prepend(z, initial_carry, done)
    aug = _augmented(op)
    n = reset.shape[1]
    cur, cur_r = zz, reset
    shift = 1
    while shift < n:
        left = (tuple(x[:, :-shift] for x in cur), cur_r[:, :-shift])
        right = (tuple(x[:, shift:] for x in cur), cur_r[:, shift:])
        with np.errstate(all="ignore"):
            comb, comb_r = aug(left, right)
        cur = tuple(
            np.concatenate([x[:, :shift], c], axis=1) for x, c in zip(cur, comb)
        )
        cur_r = np.concatenate([cur_r[:, :shift], comb_r], axis=1)
        shift *= 2
    return tuple(tail(x) for x in cur), tuple(last(x) for x in cur)


# --------------------------------------------------------------------------
# diagonal linear recurrence  h_t = a_t * h_{t-1} + b_t   (config 1)
# --------------------------------------------------------------------------


def diag_scan(a, b, done, h0=None, P0=None):
    """Direct sequential definition (formulation independent of scan_fn_*).

    h_t = done_t ? b_t : a_t h_{t-1} + b_t ;  P_t = done_t ? a_t : a_t P_{t-1}.
    ``a`` may be (B,T,D) or broadcastable ((D,) time-invariant, lru.py:86).
    Returns (h (B,T,D), h_last (B,D), P_last (B,D)).
    """
    b = np.asarray(b)
    B, T, D = b.shape
    dt = np.result_type(np.asarray(a).dtype, b.dtype, np.float64)
    a = np.broadcast_to(np.asarray(a, dtype=dt), (B, T, D))
    b = b.astype(dt)
    h = np.zeros((B, D), dt) if h0 is None else np.asarray(h0, dtype=dt).copy()
    P = np.ones((B, D), dt) if P0 is None else np.asarray(P0, dtype=dt).copy()
    done = np.asarray(done) != 0
    out = np.empty((B, T, D), dt)
    for t in range(T):
        r = done[:, t][:, None]
        with np.errstate(all="ignore"):
            hn = a[:, t] * h + b[:, t]
            Pn = a[:, t] * P
        h = np.where(r, b[:, t], hn)
        P = np.where(r, a[:, t], Pn)
        out[:, t] = h
    return out, h, P


def diag_scan_bwd(a, h, done, g, h0=None, g_last=None):
    """Analytic reverse scan for the real diagonal recurrence.

    lam_t = g_t + abar_{t+1} lam_{t+1},  abar_t = done_t ? 0 : a_t,
    db_t = lam_t,  da_t = done_t ? 0 : lam_t h_{t-1},  dh0 = abar_1 lam_1.
    For complex inputs the conjugate convention of torch.autograd is used
    (lam_t = g_t + conj(abar_{t+1}) lam_{t+1}, da_t = lam_t conj(h_{t-1})).
    Returns (da, db, dh0).
    """
    g = np.asarray(g)
    B, T, D = g.shape
    dt = np.result_type(np.asarray(a).dtype, g.dtype, np.float64)
    a = np.broadcast_to(np.asarray(a, dtype=dt), (B, T, D))
    h = np.asarray(h, dtype=dt)
    hprev0 = np.zeros((B, D), dt) if h0 is None else np.asarray(h0, dtype=dt)
    done = np.asarray(done) != 0
    lam = np.zeros((B, D), dt) if g_last is None else np.asarray(g_last, dtype=dt).copy()
    da = np.empty((B, T, D), dt)
    db = np.empty((B, T, D), dt)
    abar_next = np.zeros((B, D), dt)
    first = True
    for t in range(T - 1, -1, -1):
        if first:
            lam = g[:, t] + lam
            first = False
        else:
            lam = g[:, t] + np.conj(abar_next) * lam
        r = done[:, t][:, None]
        hp = h[:, t - 1] if t > 0 else hprev0
        db[:, t] = lam
        da[:, t] = np.where(r, 0, lam * np.conj(hp))
        abar_next = np.where(r, 0, a[:, t])
    dh0 = np.conj(abar_next) * lam
    return da, db, dh0


# --------------------------------------------------------------------------
# MinGRU (min_gru.py:49-78)
# --------------------------------------------------------------------------


def propagate_sensitivities(decay, jacobians, sensitivity, done):
    """Memoroid._propagate_sensitivities (memoroid.py:114-141), restated step by step: per name the
    Jacobians (B,T,H,*param_shape) are flattened to H*param_size channels, the decay is repeated
    param_size times and zeroed where done, the carried sensitivity is prepended with decay 1, the
    diagonal operator is scanned and the last state kept."""
    decay = np.asarray(decay)
    B, T, H = decay.shape
    d = (np.asarray(done) != 0)[..., None]
    out = {}
    for name in sorted(jacobians.keys()):
        J = np.asarray(jacobians[name])
        param_shape = J.shape[3:]
        ps = int(np.prod(param_shape)) if param_shape else 1
        ct = np.complex128 if np.iscomplexobj(J) or np.iscomplexobj(decay) else np.float64
        Jf = J.reshape(B, T, H * ps).astype(ct)
        S = np.asarray(sensitivity[name]).reshape(B, 1, H * ps).astype(ct)
        a = np.where(d, 0, np.repeat(decay, ps, axis=-1)).astype(ct)
        state = np.concatenate([S, Jf], axis=1)
        a = np.concatenate([np.ones_like(S), a], axis=1)
        s_acc, a_acc = state[:, 0], a[:, 0]
        for t in range(1, T + 1):  # left fold of (decay_j * state_i + state_j, decay_j * decay_i)
            s_acc, a_acc = a[:, t] * s_acc + state[:, t], a[:, t] * a_acc
        out[name] = s_acc.reshape(B, 1, H, *param_shape)
    return out


def softplus(x):
    return np.logaddexp(0.0, x)


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def mingru_elements(z, h_tilde):
    """min_gru.py:52-65: per-step (log_state, decay) from the two projections."""
    z = np.asarray(z, dtype=np.float64)
    h_tilde = np.asarray(h_tilde, dtype=np.float64)
    log_z = -softplus(-z)
    with np.errstate(all="ignore"):
        log_h = np.where(
            h_tilde >= 0, np.log(np.maximum(h_tilde, 0) + 0.5), -softplus(-h_tilde)
        )
    return (log_z + log_h, -softplus(z))


def mingru_linear_coeffs(z, h_tilde):
    """Linear-space equivalent: h_t = sigma(-z) h_{t-1} + sigma(z) g(h~)."""
    z = np.asarray(z, dtype=np.float64)
    h_tilde = np.asarray(h_tilde, dtype=np.float64)
    gfun = np.where(h_tilde >= 0, np.maximum(h_tilde, 0) + 0.5, sigmoid(h_tilde))
    return sigmoid(-z), sigmoid(z) * gfun


def mingru_scan(z, h_tilde, done, carry=None):
    """MinGRU through the reference's own route: log-space elements + scan_fn
    + read (exp).  carry = (log_state (B,1,F), decay (B,1,F)); default is the
    reference's (-inf, 0) (min_gru.py:80-90).  Returns (next_carry, h)."""
    el = mingru_elements(z, h_tilde)
    B, T, F = el[0].shape
    if carry is None:
        carry = (np.full((B, 1, F), -np.inf), np.zeros((B, 1, F)))
    hs, nxt = scan_fn_sequential(el, carry, done, mingru_operator)
    return nxt, np.exp(hs[0])


# --------------------------------------------------------------------------
# linear attention (linear_attention.py:58-117)
# --------------------------------------------------------------------------


def elu1(x):
    """linear_attention.py:58-60."""
    x = np.asarray(x, dtype=np.float64)
    return np.where(x > 0, x + 1.0, np.exp(np.minimum(x, 0)))


def _fmap(x, feature_map):
    if feature_map in (None, "none", 0):
        return np.asarray(x, dtype=np.float64)
    if feature_map in ("elu1", 1):
        return elu1(x)
    raise ValueError(feature_map)


def linear_attention(q, k, v, done, S0=None, feature_map="none"):
    """Recurrent form.  S_t = r_t S_{t-1} + v_t k_t^T ; o_t = S_t q_t.

    q,k: (B,T,H,dk), v: (B,T,H,dv), S0: (B,H,dv,dk).  Unnormalised numerator
    (linear_attention.py:105).  Returns (o (B,T,H,dv), S_last (B,H,dv,dk)).
    """
    q = _fmap(q, feature_map)
    k = _fmap(k, feature_map)
    v = np.asarray(v, dtype=np.float64)
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    S = np.zeros((B, H, dv, dk)) if S0 is None else np.asarray(S0, np.float64).copy()
    done = np.asarray(done) != 0
    o = np.empty((B, T, H, dv))
    for t in range(T):
        r = done[:, t][:, None, None, None]
        S = np.where(r, 0.0, S)
        S = S + np.einsum("bhi,bhj->bhij", v[:, t], k[:, t])
        o[:, t] = np.einsum("bhij,bhj->bhi", S, q[:, t])
    return o, S


def linear_attention_memoroid(q, k, v, done, carry=None, feature_map="none"):
    """The reference's own route (linear_attention.py:62-117 + memoroid.py:60-91):
    materialise per-step outer products, scan (S, z) additively, read
    numerator and denominator.  Returns (next_carry, numerator, denominator)."""
    q = _fmap(q, feature_map)
    k = _fmap(k, feature_map)
    v = np.asarray(v, dtype=np.float64)
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    S = np.einsum("bthi,bthj->bthij", v, k)
    if carry is None:
        carry = (np.zeros((B, 1, H, dv, dk)), np.zeros((B, 1, H, dk)))
    (Sc, zc), nxt = scan_fn_tree((S, k), carry, done, additive_operator)
    num = np.einsum("bthij,bthj->bthi", Sc, q)
    den = np.einsum("bthi,bthi->bth", q, zc)
    return nxt, num, den


def deltanet(q, k, v, beta_raw, done, S0=None):
    """DeltaNet cell on raw projections: delta_rule on k / max(|k|, 1e-12) and sigmoid(beta_raw)
    (the prologue a cell in the idiom of memoroid.py:20-33 runs before it emits its elements)."""
    k = np.asarray(k, dtype=np.float64)
    kn = k / np.maximum(np.linalg.norm(k, axis=-1, keepdims=True), 1e-12)
    return delta_rule(q, kn, v, sigmoid(np.asarray(beta_raw, dtype=np.float64)), done, S0)


def normalised_linear_attention(q, k, v, done, S0=None, z0=None, feature_map="elu1", eps=1e-6):
    """Recurrent form of the cell with its read-out (linear_attention.py:62-86 for the
    elements, :93-110 for the read-out, scanned by memoroid.py:60-91):
        S_t = r_t S_{t-1} + v_t k_t^T ;  z_t = r_t z_{t-1} + k_t ;
        o_t = S_t q_t / max(q_t . z_t, eps)          (q, k after the feature map).
    Returns (o (B,T,H,dv), den (B,T,H) clamped, S_last (B,H,dv,dk), z_last (B,H,dk))."""
    q = _fmap(q, feature_map)
    k = _fmap(k, feature_map)
    v = np.asarray(v, dtype=np.float64)
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    S = np.zeros((B, H, dv, dk)) if S0 is None else np.asarray(S0, np.float64).copy()
    z = np.zeros((B, H, dk)) if z0 is None else np.asarray(z0, np.float64).copy()
    done = np.asarray(done) != 0
    o = np.empty((B, T, H, dv))
    den = np.empty((B, T, H))
    for t in range(T):
        r = done[:, t]
        S = np.where(r[:, None, None, None], 0.0, S) + np.einsum("bhi,bhj->bhij", v[:, t], k[:, t])
        z = np.where(r[:, None, None], 0.0, z) + k[:, t]
        den[:, t] = np.maximum(np.einsum("bhd,bhd->bh", q[:, t], z), eps)
        o[:, t] = np.einsum("bhij,bhj->bhi", S, q[:, t]) / den[:, t][..., None]
    return o, den, S, z


def gated_linear_attention(q, k, v, g, done, S0=None, feature_map="none"):
    """Recurrent form with a scalar log-decay per step and head:
        S_t = r_t exp(g_t) S_{t-1} + v_t k_t^T ;  o_t = S_t q_t.
    This is the Mamba cell's algebra (mamba.py:109-122: elements (h = (B dt) (x) x,
    decay = exp(dt A)), binary_operator (decay_j h_i + h_j, decay_j decay_i)) with
    k = B dt, v = x, q = C and the state stored as (d_v, d_k); g = log decay (B,T,H)."""
    q = _fmap(q, feature_map)
    k = _fmap(k, feature_map)
    v = np.asarray(v, dtype=np.float64)
    g = np.asarray(g, dtype=np.float64)
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    S = np.zeros((B, H, dv, dk)) if S0 is None else np.asarray(S0, np.float64).copy()
    done = np.asarray(done) != 0
    o = np.empty((B, T, H, dv))
    for t in range(T):
        r = done[:, t][:, None, None, None]
        S = np.where(r, 0.0, np.exp(g[:, t])[:, :, None, None] * S)
        S = S + np.einsum("bhi,bhj->bhij", v[:, t], k[:, t])
        o[:, t] = np.einsum("bhij,bhj->bhi", S, q[:, t])
    return o, S


def gated_linear_attention_memoroid(q, k, v, g, done, carry=None):
    """The reference's own route for the Mamba cell: materialise h_t = v_t k_t^T and the decay leaf
    and scan them with the diagonal operator (mamba.py:109-122 under memoroid.py:60-91).
    Returns (next_carry, o) with carry = (S (B,1,H,dv,dk), decay (B,1,H,1,1))."""
    q, k, v, g = (np.asarray(x, np.float64) for x in (q, k, v, g))
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    h = np.einsum("bthi,bthj->bthij", v, k)
    decay = np.exp(g)[..., None, None]
    if carry is None:
        carry = (np.zeros((B, 1, H, dv, dk)), np.ones((B, 1, H, 1, 1)))
    (Sc, _), nxt = scan_fn_tree((h, np.broadcast_to(decay, h.shape).copy()), (carry[0], np.broadcast_to(carry[1], carry[0].shape).copy()), done, diag_operator)
    o = np.einsum("bthij,bthj->bthi", Sc, q)
    return nxt, o


def gated_linear_attention_quadratic(q, k, v, g, done, S0=None, feature_map="none"):
    """Masked-matmul form: o_i = sum_{j<=i, same episode} exp(G_i - G_j) (q_i . k_j) v_j
    + [episode 0] exp(G_i) S0 q_i, with G the cumulative sum of g inside the episode (the
    decay of an episode's first step multiplies a zero state and drops out)."""
    q = _fmap(q, feature_map)
    k = _fmap(k, feature_map)
    v = np.asarray(v, dtype=np.float64)
    g = np.asarray(g, dtype=np.float64)
    B, T, H, dk = q.shape
    seg = segment_ids(done)
    Gc = np.cumsum(g, axis=1)                                 # (B,T,H) global cumulative sum
    M = (seg[:, :, None] == seg[:, None, :]) & np.tril(np.ones((T, T), bool))[None]
    D = np.exp(np.where(M[:, None], (Gc.transpose(0, 2, 1)[:, :, :, None] - Gc.transpose(0, 2, 1)[:, :, None, :]), -np.inf))
    A = np.einsum("bihd,bjhd->bhij", q, k) * D
    o = np.einsum("bhij,bjhe->bihe", A, v)
    if S0 is not None:
        m = (seg == 0)[:, :, None, None]
        o = o + m * np.exp(Gc)[..., None] * np.einsum("bihd,bhed->bihe", q, np.asarray(S0, np.float64))
    return o


def mlstm_elements(q, k, v, i_gate, f_gate):
    """mlstm.py:163-188: elements (C = k (x) v, log_f, n = k, m = log_i) with k pre-scaled by
    1/sqrt(head_dim); q,k,v: (B,T,H,d), gates (B,T,H)."""
    k = np.asarray(k, np.float64) / np.sqrt(k.shape[-1])
    v = np.asarray(v, np.float64)
    log_f = -softplus(-np.asarray(f_gate, np.float64))
    log_i = np.asarray(i_gate, np.float64)
    C = np.einsum("...i,...j->...ij", k, v)
    return (C, log_f[..., None, None], k[..., None], log_i[..., None, None])


def mlstm_read(h, q):
    """mlstm.py:208-221 up to the division: h_tilde = q C / (max(|q . n|, exp(-m)) + 1e-6)."""
    C, _, n, m = h
    q = np.asarray(q, np.float64)
    den = np.maximum(np.abs(np.einsum("...i,...i->...", q, n[..., 0])), np.exp(-m[..., 0, 0]))[..., None]
    return np.einsum("...j,...jk->...k", q, C) / (den + 1e-6)


def mlstm(q, k, v, i_gate, f_gate, done, carry=None, tree=True):
    """The reference's route: scan the elements with the stabilised operator (memoroid.py:60-91),
    read.  Returns (next_carry, h_tilde (B,T,H,d))."""
    z = mlstm_elements(q, k, v, i_gate, f_gate)
    B, T, H, d = np.asarray(q).shape
    if carry is None:
        carry = (np.zeros((B, 1, H, d, d)), np.zeros((B, 1, H, 1, 1)), np.zeros((B, 1, H, d, 1)),
                 np.full((B, 1, H, 1, 1), -1e9))
    scan = scan_fn_tree if tree else scan_fn_sequential
    h, nxt = scan(z, carry, done, mlstm_operator)
    return nxt, mlstm_read(h, q)


def silu_gate(h, g):
    """activation(gate) * value of the GLU block (blocks/ffn.py:108-121) with silu: h * g * sigmoid(g)."""
    h, g = np.asarray(h, np.float64), np.asarray(g, np.float64)
    return h * g / (1.0 + np.exp(-g))


def rms_norm(x, scale=None, eps=1e-6):
    """flax.linen.RMSNorm with its defaults over the last axis (the norm of LinearAttentionCell.read,
    linear_attention.py:109-115, and of PreNorm blocks built with it, blocks/normalization.py:10-35):
    x * rsqrt(mean(x^2) + eps) * scale."""
    x = np.asarray(x, np.float64)
    y = x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)
    return y if scale is None else y * np.asarray(scale, np.float64)


def layer_norm(x, scale=None, bias=None, eps=1e-6):
    """flax.linen.LayerNorm with its defaults over the last axis (the default norm of PreNorm / PostNorm,
    blocks/normalization.py:10-65): (x - mean) * rsqrt(var + eps) * scale + bias, var the mean squared deviation."""
    x = np.asarray(x, np.float64)
    xc = x - x.mean(-1, keepdims=True)
    y = xc / np.sqrt((xc * xc).mean(-1, keepdims=True) + eps)
    if scale is not None:
        y = y * np.asarray(scale, np.float64)
    return y if bias is None else y + np.asarray(bias, np.float64)


def mlstm_gates(log_i, log_f, done, m0=None, g_floor=-60.0):
    """The stabiliser of mlstm.py:190-206 unrolled over time, resets as memoroid.py:72-85 (the element wins by
    select): m_t = done_t ? log_i_t : max(m_{t-1} + log_f_t, log_i_t), and with it the log-decay and the key
    weight of the gated recurrence the stabilised C and n follow: g_t = done_t ? 0 : max(log_f_t + m_{t-1} - m_t,
    g_floor), w_t = exp(log_i_t - m_t).  log_i, log_f: (B,T,H); m0: (B,H) or None (the cell's initial -1e9).
    Returns (m, g, w)."""
    log_i, log_f = np.asarray(log_i, np.float64), np.asarray(log_f, np.float64)
    B, T, H = log_i.shape
    done = np.asarray(done) != 0
    mp = np.full((B, H), -1e9) if m0 is None else np.asarray(m0, np.float64)
    m, g, w = np.empty((B, T, H)), np.empty((B, T, H)), np.empty((B, T, H))
    for t in range(T):
        r = done[:, t][:, None]
        mt = np.where(r, log_i[:, t], np.maximum(mp + log_f[:, t], log_i[:, t]))
        g[:, t] = np.where(r, 0.0, np.maximum(log_f[:, t] + mp - mt, g_floor))
        w[:, t] = np.exp(log_i[:, t] - mt)
        m[:, t] = mp = mt
    return m, g, w


def mlstm_unstabilised(q, k, v, i_gate, f_gate, done):
    """The recurrence the docstring of mlstm.py:8-11 states, without the stabiliser:
    C~_t = f_t C~_{t-1} + i_t k_t v_t^T, n~_t = f_t n~_{t-1} + i_t k_t (zero carry),
    h = q C~ / (max(|q . n~|, 1) + 1e-6 exp(m_t)), m_t = max(m_{t-1} + log f_t, log i_t)."""
    q, v = np.asarray(q, np.float64), np.asarray(v, np.float64)
    k = np.asarray(k, np.float64) / np.sqrt(q.shape[-1])
    log_f = -softplus(-np.asarray(f_gate, np.float64))
    log_i = np.asarray(i_gate, np.float64)
    B, T, H, d = q.shape
    done = np.asarray(done) != 0
    C = np.zeros((B, H, d, d)); n = np.zeros((B, H, d)); m = np.full((B, H), -1e9)
    out = np.empty((B, T, H, d))
    for t in range(T):
        r = done[:, t]
        f = np.where(r[:, None], 0.0, np.exp(log_f[:, t]))
        i = np.exp(log_i[:, t])
        C = f[..., None, None] * C + i[..., None, None] * np.einsum("bhi,bhj->bhij", k[:, t], v[:, t])
        n = f[..., None] * n + i[..., None] * k[:, t]
        m = np.where(r[:, None], log_i[:, t], np.maximum(m + log_f[:, t], log_i[:, t]))
        den = np.maximum(np.abs((q[:, t] * n).sum(-1)), 1.0) + 1e-6 * np.exp(m)
        out[:, t] = np.einsum("bhj,bhjk->bhk", q[:, t], C) / den[..., None]
    return out


def segment_ids(done):
    """Inclusive cumsum of done along time: rows with equal id share an episode."""
    return np.cumsum(np.asarray(done) != 0, axis=1)


def linear_attention_quadratic(q, k, v, done, S0=None, feature_map="none"):
    """Textbook masked-matmul form: o = ((Q K^T) * tril * M) V + m * (Q S0^T)."""
    q = _fmap(q, feature_map)
    k = _fmap(k, feature_map)
    v = np.asarray(v, dtype=np.float64)
    B, T, H, dk = q.shape
    seg = segment_ids(done)
    M = (seg[:, :, None] == seg[:, None, :]) & np.tril(np.ones((T, T), bool))[None]
    A = np.einsum("bihd,bjhd->bhij", q, k) * M[:, None]
    o = np.einsum("bhij,bjhe->bihe", A, v)
    if S0 is not None:
        m = (seg == 0)[:, :, None, None]
        o = o + m * np.einsum("bihd,bhed->bihe", q, np.asarray(S0, np.float64))
    return o


def linear_attention_chunked(q, k, v, done, S0=None, feature_map="none", chunk=64):
    """Chunk form with per-chunk masks M, m, l, e computed from the cumsum of
    done *within* the chunk: O = diag(m) Q S^T + (tril(QK^T)*M) V ;
    S <- l S + (diag(e) V)^T K."""
    q = _fmap(q, feature_map)
    k = _fmap(k, feature_map)
    v = np.asarray(v, dtype=np.float64)
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    S = np.zeros((B, H, dv, dk)) if S0 is None else np.asarray(S0, np.float64).copy()
    done = np.asarray(done) != 0
    o = np.empty((B, T, H, dv))
    for c0 in range(0, T, chunk):
        c1 = min(T, c0 + chunk)
        C = c1 - c0
        seg = np.cumsum(done[:, c0:c1], axis=1)
        M = (seg[:, :, None] == seg[:, None, :]) & np.tril(np.ones((C, C), bool))[None]
        m = (seg == 0).astype(np.float64)
        e = (seg == seg[:, -1:]).astype(np.float64)
        l = (seg[:, -1] == 0).astype(np.float64)
        Q, K, V = q[:, c0:c1], k[:, c0:c1], v[:, c0:c1]
        A = np.einsum("bihd,bjhd->bhij", Q, K) * M[:, None]
        O = np.einsum("bhij,bjhe->bihe", A, V)
        O = O + m[:, :, None, None] * np.einsum("bihd,bhed->bihe", Q, S)
        o[:, c0:c1] = O
        S = l[:, None, None, None] * S + np.einsum(
            "bjhe,bjhd->bhed", V * e[:, :, None, None], K
        )
    return o, S


# --------------------------------------------------------------------------
# DeltaNet delta rule (config 4)
# --------------------------------------------------------------------------


def delta_rule(q, k, v, beta, done, S0=None):
    """Sequential u-form.  S' = r_t S_{t-1}; u_t = beta_t (v_t - S' k_t);
    S_t = S' + u_t k_t^T ; o_t = S_t q_t.   beta: (B,T,H)."""
    q = np.asarray(q, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    beta = np.asarray(beta, np.float64)
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    S = np.zeros((B, H, dv, dk)) if S0 is None else np.asarray(S0, np.float64).copy()
    done = np.asarray(done) != 0
    o = np.empty((B, T, H, dv))
    for t in range(T):
        r = done[:, t][:, None, None, None]
        S = np.where(r, 0.0, S)
        u = beta[:, t][..., None] * (v[:, t] - np.einsum("bhij,bhj->bhi", S, k[:, t]))
        S = S + np.einsum("bhi,bhj->bhij", u, k[:, t])
        o[:, t] = np.einsum("bhij,bhj->bhi", S, q[:, t])
    return o, S


def delta_rule_explicit(q, k, v, beta, done, S0=None):
    """Literal S_t = S_{t-1}(I - beta k k^T) + beta v k^T with select reset."""
    q = np.asarray(q, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    beta = np.asarray(beta, np.float64)
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    S = np.zeros((B, H, dv, dk)) if S0 is None else np.asarray(S0, np.float64).copy()
    done = np.asarray(done) != 0
    eye = np.eye(dk)
    o = np.empty((B, T, H, dv))
    for t in range(T):
        bt = beta[:, t][..., None, None]
        A = eye - bt * np.einsum("bhi,bhj->bhij", k[:, t], k[:, t])
        Bm = bt * np.einsum("bhi,bhj->bhij", v[:, t], k[:, t])
        Sn = S @ A + Bm
        S = np.where(done[:, t][:, None, None, None], Bm, Sn)
        o[:, t] = np.einsum("bhij,bhj->bhi", S, q[:, t])
    return o, S


def delta_rule_memoroid(q, k, v, beta, done, S0=None):
    """The delta rule pushed through the reference's scan_fn with the affine
    pair algebra (element (B_t, A_t)); O(T d^2) memory, tiny shapes only."""
    q = np.asarray(q, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    beta = np.asarray(beta, np.float64)[..., None, None]
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    Am = np.eye(dk) - beta * np.einsum("bthi,bthj->bthij", k, k)
    Bm = beta * np.einsum("bthi,bthj->bthij", v, k)
    S0 = np.zeros((B, H, dv, dk)) if S0 is None else np.asarray(S0, np.float64)
    carry = (S0[:, None], np.broadcast_to(np.eye(dk), (B, 1, H, dk, dk)).copy())
    (Sc, _), nxt = scan_fn_tree((Bm, Am), carry, done, delta_operator)
    o = np.einsum("bthij,bthj->bthi", Sc, q)
    return o, nxt[0][:, 0]


def delta_rule_chunked(q, k, v, beta, done, S0=None, chunk=64):
    """WY / UT-transform chunk form with resets:
    A = tril(diag(beta)(K K^T * M), -1);  Tm = (I + A)^-1 diag(beta);
    W = Tm K; U = Tm V; U' = U - diag(m) W S^T;
    O = diag(m) Q S^T + (tril(Q K^T) * M) U';  S <- l S + (diag(e) U')^T K."""
    q = np.asarray(q, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    beta = np.asarray(beta, np.float64)
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    S = np.zeros((B, H, dv, dk)) if S0 is None else np.asarray(S0, np.float64).copy()
    done = np.asarray(done) != 0
    o = np.empty((B, T, H, dv))
    for c0 in range(0, T, chunk):
        c1 = min(T, c0 + chunk)
        C = c1 - c0
        seg = np.cumsum(done[:, c0:c1], axis=1)
        tril = np.tril(np.ones((C, C), bool))
        M = (seg[:, :, None] == seg[:, None, :]) & tril[None]
        m = (seg == 0).astype(np.float64)
        e = (seg == seg[:, -1:]).astype(np.float64)
        l = (seg[:, -1] == 0).astype(np.float64)
        Q, K, V, bt = q[:, c0:c1], k[:, c0:c1], v[:, c0:c1], beta[:, c0:c1]
        KK = np.einsum("bihd,bjhd->bhij", K, K) * M[:, None]
        A = np.tril(np.einsum("bih,bhij->bhij", bt, KK), -1)
        Tm = np.linalg.inv(np.eye(C) + A) * np.transpose(bt, (0, 2, 1))[:, :, None, :]
        W = np.einsum("bhij,bjhd->bihd", Tm, K)
        U = np.einsum("bhij,bjhe->bihe", Tm, V)
        Up = U - m[:, :, None, None] * np.einsum("bihd,bhed->bihe", W, S)
        Aqk = np.einsum("bihd,bjhd->bhij", Q, K) * M[:, None]
        O = m[:, :, None, None] * np.einsum("bihd,bhed->bihe", Q, S)
        O = O + np.einsum("bhij,bjhe->bihe", Aqk, Up)
        o[:, c0:c1] = O
        S = l[:, None, None, None] * S + np.einsum(
            "bjhe,bjhd->bhed", Up * e[:, :, None, None], K
        )
    return o, S


# --------------------------------------------------------------------------
# seeded synthetic inputs for the benchmark configurations
# --------------------------------------------------------------------------


def make_inputs(cfg, shape=None, seed=None):
    """Seeded fp32 inputs for configuration ``cfg`` (1..4); ``shape`` overrides
    the default sizes.  done = rng.random((B,T)) < p."""
    rng = np.random.default_rng(1000 + cfg if seed is None else seed)
    if cfg == 1:
        B, T, D = shape or (32, 128, 256)
        a = rng.uniform(0.9, 0.999, (B, T, D)).astype(np.float32)
        b = rng.standard_normal((B, T, D)).astype(np.float32)
        done = rng.random((B, T)) < 0.01
        return dict(a=a, b=b, done=done)
    if cfg in (2, 3):
        B, T, H, d = shape or ((64, 256, 4, 64) if cfg == 2 else (256, 4096, 8, 64))
        q, k, v = (
            (rng.standard_normal((B, T, H, d)) / np.sqrt(64)).astype(np.float32)
            for _ in range(3)
        )
        p = 0.005 if cfg == 2 else 0.0
        done = rng.random((B, T)) < p
        return dict(q=q, k=k, v=v, done=done)
    if cfg == 4:
        B, T, H, d = shape or (64, 1024, 8, 64)
        q = rng.standard_normal((B, T, H, d)).astype(np.float32)
        k = rng.standard_normal((B, T, H, d)).astype(np.float32)
        k /= np.linalg.norm(k, axis=-1, keepdims=True)
        v = rng.standard_normal((B, T, H, d)).astype(np.float32)
        beta = (1.0 / (1.0 + np.exp(-rng.standard_normal((B, T, H))))).astype(np.float32)
        done = rng.random((B, T)) < 0.002
        return dict(q=q, k=k, v=v, beta=beta, done=done)
    raise ValueError(cfg)
