"""Gradient oracle: torch-fp64 autograd through sequential restatements.

TEST INFRASTRUCTURE: imported only by tests, smoke() and bench.py's cpu_baseline.

Each function re-states the forward recurrence of ``oracle.memoroid`` with
torch ops (select-style resets through ``torch.where``, as memoroid.py:79-83
does with ``jnp.where``) so that ``torch.autograd`` yields reference gradients.
Autograd keeps every per-step state alive, so these are for shapes up to a few
thousand (b, h, t) triples; full-size gradients are checked against the C
oracle, which is itself checked against these.
"""
from __future__ import annotations

import numpy as np
import torch

F64 = torch.float64


def _t(x, requires_grad=False, dtype=None):
    if isinstance(x, torch.Tensor):
        t = x.detach().clone()
    else:
        t = torch.from_numpy(np.ascontiguousarray(np.asarray(x)))
    if dtype is None:
        dtype = torch.complex128 if t.is_complex() else F64
    t = t.to(dtype)
    t.requires_grad_(requires_grad)
    return t


def _done(done):
    return torch.from_numpy(np.ascontiguousarray(np.asarray(done) != 0))


def diag_scan_t(a, b, done, h0, P0=None):
    """torch restatement of oracle.memoroid.diag_scan (differentiable)."""
    B, T, D = b.shape
    a = a.expand(B, T, D)
    h = h0
    P = torch.ones_like(h0) if P0 is None else P0
    hs = []
    for t in range(T):
        r = done[:, t][:, None]
        h = torch.where(r, b[:, t], a[:, t] * h + b[:, t])
        P = torch.where(r, a[:, t], a[:, t] * P)
        hs.append(h)
    return torch.stack(hs, 1), h, P


def mingru_scan_t(z, h_tilde, done, h0=None, side=None):
    """MinGRU in the reference's log space (elements min_gru.py:52-65, operator :67-74, read :76-78),
    folded sequentially with select resets (memoroid.py:79-83).  h0: linear-space carry (B,F) > 0,
    or None for the cell's initial (-inf, 0).  Returns (h (B,T,F), h_last).
    side (bool, optional): which branch of g(x) = x + 0.5 (x >= 0) | sigmoid(x) each element takes,
    when it is not to be decided by the sign of this evaluation's own h_tilde: a test that compares
    gradients with a lower-precision evaluation passes the sides that evaluation saw, so that an
    element within rounding of the kink (slope 1/4 against 1) is differentiated on the same branch
    on both sides of the comparison.  The value moves by at most 3/4 |x| there."""
    sp = torch.nn.functional.softplus
    if side is None:
        log_g = torch.where(h_tilde >= 0, torch.log(torch.relu(h_tilde) + 0.5), -sp(-h_tilde))
    else:
        log_g = torch.where(side, torch.log(torch.where(side, h_tilde, torch.zeros_like(h_tilde)) + 0.5), -sp(-h_tilde))
    log_b = -sp(-z) + log_g
    log_a = -sp(z)
    B, T, F = z.shape
    ls = torch.full((B, F), -float("inf"), dtype=z.dtype) if h0 is None else torch.log(h0)
    out = []
    for t in range(T):
        r = done[:, t][:, None]
        ls = torch.where(r, log_b[:, t], torch.logaddexp(log_a[:, t] + ls, log_b[:, t]))
        out.append(ls)
    return torch.exp(torch.stack(out, 1)), torch.exp(ls)


def mlstm_gates_t(log_i, log_f, done, m0=None, g_floor=-60.0):
    """torch restatement of oracle.memoroid.mlstm_gates (differentiable)."""
    B, T, H = log_i.shape
    mp = torch.full((B, H), -1e9, dtype=log_i.dtype) if m0 is None else m0
    ms, gs, ws = [], [], []
    for t in range(T):
        r = done[:, t][:, None]
        mt = torch.where(r, log_i[:, t], torch.maximum(mp + log_f[:, t], log_i[:, t]))
        gs.append(torch.where(r, torch.zeros_like(mt), torch.clamp(log_f[:, t] + mp - mt, min=g_floor)))
        ws.append(torch.exp(log_i[:, t] - mt))
        ms.append(mt)
        mp = mt
    return torch.stack(ms, 1), torch.stack(gs, 1), torch.stack(ws, 1)


def mlstm_gates_grads(log_i, log_f, done, m0, dm, dg, dw, g_floor=-60.0):
    """(dlog_i, dlog_f, dm0) of L = sum(dm * m) + sum(dg * g) + sum(dw * w)."""
    li, lf = _t(log_i, True), _t(log_f, True)
    m0_ = None if m0 is None else _t(m0, True)
    m, g, w = mlstm_gates_t(li, lf, _done(done), m0_, g_floor)
    L = (m * _t(dm)).sum() + (g * _t(dg)).sum() + (w * _t(dw)).sum()
    L.backward()
    return _np(li.grad), _np(lf.grad), (None if m0 is None else _np(m0_.grad))


def silu_gate_grads(h, g, dy):
    """(dh, dg) of L = sum(dy * h * silu(g))."""
    h_, g_ = _t(h, True), _t(g, True)
    (h_ * torch.nn.functional.silu(g_) * _t(dy)).sum().backward()
    return _np(h_.grad), _np(g_.grad)


def layer_norm_grads(x, scale, bias, dy, eps=1e-6):
    """(dx, dscale, dbias) of L = sum(dy * layer_norm(x, scale, bias))."""
    x_, s_, b_ = _t(x, True), _t(scale, True), _t(bias, True)
    xc = x_ - x_.mean(-1, keepdim=True)
    y = xc * torch.rsqrt((xc * xc).mean(-1, keepdim=True) + eps) * s_ + b_
    (y * _t(dy)).sum().backward()
    return _np(x_.grad), _np(s_.grad), _np(b_.grad)


def rms_norm_grads(x, scale, dy, eps=1e-6):
    """(dx, dscale) of L = sum(dy * rms_norm(x, scale)); scale None: (dx, None)."""
    x_ = _t(x, True)
    s_ = None if scale is None else _t(scale, True)
    y = x_ * torch.rsqrt((x_ * x_).mean(-1, keepdim=True) + eps)
    if s_ is not None:
        y = y * s_
    (y * _t(dy)).sum().backward()
    return _np(x_.grad), (None if s_ is None else _np(s_.grad))


def elu1_t(x):
    return torch.where(x > 0, x + 1.0, torch.exp(torch.clamp(x, max=0.0)))


def linear_attention_t(q, k, v, done, S0, feature_map="none"):
    if feature_map in ("elu1", 1):
        q, k = elu1_t(q), elu1_t(k)
    B, T, H, dk = q.shape
    S = S0
    os_ = []
    for t in range(T):
        r = done[:, t][:, None, None, None]
        S = torch.where(r, torch.zeros_like(S), S)
        S = S + torch.einsum("bhi,bhj->bhij", v[:, t], k[:, t])
        os_.append(torch.einsum("bhij,bhj->bhi", S, q[:, t]))
    return torch.stack(os_, 1), S


class _DivideKeepingStoredQuotient(torch.autograd.Function):
    """num / den whose backward takes the quotient from a given array instead of recomputing it:
    d num = g / den, d den = -(g . o_stored) / den.  With o_stored the outputs as a lower-precision
    implementation stored them (and reads them back in its backward), the gradients are those of that
    implementation's own formula on the same information, so that a comparison is not charged with the
    rounding of o, which cancellation in g . o can amplify."""

    @staticmethod
    def forward(ctx, num, den, o_stored):
        ctx.save_for_backward(den, o_stored)
        return num / den[..., None]

    @staticmethod
    def backward(ctx, g):
        den, o = ctx.saved_tensors
        return g / den[..., None], -(g * o).sum(-1) / den, None


def normalised_linear_attention_t(q, k, v, done, S0, z0, feature_map="elu1", eps=1e-6, o_stored=None):
    if feature_map in ("elu1", 1):
        q, k = elu1_t(q), elu1_t(k)
    B, T, H, dk = q.shape
    S, z = S0, z0
    os_ = []
    for t in range(T):
        r = done[:, t]
        S = torch.where(r[:, None, None, None], torch.zeros_like(S), S) + torch.einsum("bhi,bhj->bhij", v[:, t], k[:, t])
        z = torch.where(r[:, None, None], torch.zeros_like(z), z) + k[:, t]
        den = torch.clamp((q[:, t] * z).sum(-1), min=eps)
        num = torch.einsum("bhij,bhj->bhi", S, q[:, t])
        os_.append(num / den[..., None] if o_stored is None else _DivideKeepingStoredQuotient.apply(num, den, o_stored[:, t]))
    return torch.stack(os_, 1), S, z


def gated_linear_attention_t(q, k, v, g, done, S0, feature_map="none"):
    if feature_map in ("elu1", 1):
        q, k = elu1_t(q), elu1_t(k)
    B, T, H, dk = q.shape
    S = S0
    os_ = []
    for t in range(T):
        r = done[:, t][:, None, None, None]
        S = torch.where(r, torch.zeros_like(S), torch.exp(g[:, t])[:, :, None, None] * S)
        S = S + torch.einsum("bhi,bhj->bhij", v[:, t], k[:, t])
        os_.append(torch.einsum("bhij,bhj->bhi", S, q[:, t]))
    return torch.stack(os_, 1), S


def delta_rule_t(q, k, v, beta, done, S0):
    B, T, H, dk = q.shape
    S = S0
    os_ = []
    for t in range(T):
        r = done[:, t][:, None, None, None]
        S = torch.where(r, torch.zeros_like(S), S)
        u = beta[:, t][..., None] * (v[:, t] - torch.einsum("bhij,bhj->bhi", S, k[:, t]))
        S = S + torch.einsum("bhi,bhj->bhij", u, k[:, t])
        os_.append(torch.einsum("bhij,bhj->bhi", S, q[:, t]))
    return torch.stack(os_, 1), S


def _np(x):
    return None if x is None else x.detach().numpy()


def diag_scan_grads(a, b, done, h0, g, g_last=None):
    """Returns dict(da, db, dh0) for L = sum(g*h) + sum(g_last*h_last) (real
    part for complex inputs, torch's conjugate-cotangent convention)."""
    a_, b_, h0_ = _t(a, True), _t(b, True), _t(h0, True)
    h, hl, _ = diag_scan_t(a_, b_, _done(done), h0_)
    L = (h * _t(g).conj()).sum().real if h.is_complex() else (h * _t(g)).sum()
    if g_last is not None:
        L = L + ((hl * _t(g_last).conj()).sum().real if hl.is_complex() else (hl * _t(g_last)).sum())
    L.backward()
    return dict(da=_np(a_.grad), db=_np(b_.grad), dh0=_np(h0_.grad))


def mingru_grads(z, h_tilde, done, h0, g, g_last=None):
    """Returns dict(dz, dh_tilde, dh0) for L = sum(g*h) + sum(g_last*h_last); h0 linear space or None."""
    z_, x_ = _t(z, True), _t(h_tilde, True)
    h0_ = None if h0 is None else _t(h0, True)
    h, hl = mingru_scan_t(z_, x_, _done(done), h0_)
    L = (h * _t(g)).sum()
    if g_last is not None:
        L = L + (hl * _t(g_last)).sum()
    L.backward()
    return dict(dz=_np(z_.grad), dh_tilde=_np(x_.grad), dh0=None if h0_ is None else _np(h0_.grad))


def linear_attention_grads(q, k, v, done, S0, do, dS_last=None, feature_map="none"):
    """Returns dict(o, S_last, dq, dk, dv, dS0) for L = sum(do*o) + sum(dS_last*S_last)."""
    q_, k_, v_ = _t(q, True), _t(k, True), _t(v, True)
    B, T, H, dk = q_.shape
    S0_ = _t(np.zeros((B, H, v_.shape[-1], dk)) if S0 is None else S0, True)
    o, Sl = linear_attention_t(q_, k_, v_, _done(done), S0_, feature_map)
    L = (o * _t(do)).sum()
    if dS_last is not None:
        L = L + (Sl * _t(dS_last)).sum()
    L.backward()
    return dict(o=_np(o), S_last=_np(Sl), dq=_np(q_.grad), dk=_np(k_.grad),
                dv=_np(v_.grad), dS0=_np(S0_.grad))


def normalised_linear_attention_grads(q, k, v, done, S0, z0, do, dS_last=None, dz_last=None,
                                      feature_map="elu1", eps=1e-6, d_ss=None, o_stored=None):
    """Returns dict(o, S_last, z_last, dq, dk, dv, dS0, dz0) for
    L = sum(do*o) + sum(dS_last*S_last) + sum(dz_last*z_last) + sum(d_ss * ss), ss[b,t,h] = |o[b,t,h]|^2
    (d_ss (B,T,H): the per-head sums of squares an RMS norm over the heads is built from).
    o_stored (B,T,H,dv): see _DivideKeepingStoredQuotient."""
    q_, k_, v_ = _t(q, True), _t(k, True), _t(v, True)
    B, T, H, dk = q_.shape
    S0_ = _t(np.zeros((B, H, v_.shape[-1], dk)) if S0 is None else S0, True)
    z0_ = _t(np.zeros((B, H, dk)) if z0 is None else z0, True)
    o, Sl, zl = normalised_linear_attention_t(q_, k_, v_, _done(done), S0_, z0_, feature_map, eps,
                                              None if o_stored is None else _t(o_stored))
    L = (o * _t(do)).sum()
    if dS_last is not None:
        L = L + (Sl * _t(dS_last)).sum()
    if dz_last is not None:
        L = L + (zl * _t(dz_last)).sum()
    if d_ss is not None:
        L = L + ((o * o).sum(-1) * _t(d_ss)).sum()
    L.backward()
    return dict(o=_np(o), S_last=_np(Sl), z_last=_np(zl), dq=_np(q_.grad), dk=_np(k_.grad),
                dv=_np(v_.grad), dS0=_np(S0_.grad), dz0=_np(z0_.grad))


def delta_rule_grads(q, k, v, beta, done, S0, do, dS_last=None):
    """Returns dict(o, S_last, dq, dk, dv, dbeta, dS0)."""
    q_, k_, v_, b_ = _t(q, True), _t(k, True), _t(v, True), _t(beta, True)
    B, T, H, dk = q_.shape
    S0_ = _t(np.zeros((B, H, v_.shape[-1], dk)) if S0 is None else S0, True)
    o, Sl = delta_rule_t(q_, k_, v_, b_, _done(done), S0_)
    L = (o * _t(do)).sum()
    if dS_last is not None:
        L = L + (Sl * _t(dS_last)).sum()
    L.backward()
    return dict(o=_np(o), S_last=_np(Sl), dq=_np(q_.grad), dk=_np(k_.grad),
                dv=_np(v_.grad), dbeta=_np(b_.grad), dS0=_np(S0_.grad))


def deltanet_grads(q, k, v, beta_raw, done, S0, do, dS_last=None):
    """Returns dict(o, S_last, dq, dk, dv, dbeta, dS0) w.r.t. the raw k and beta_raw."""
    q_, k_, v_, b_ = _t(q, True), _t(k, True), _t(v, True), _t(beta_raw, True)
    B, T, H, dk = q_.shape
    S0_ = _t(np.zeros((B, H, v_.shape[-1], dk)) if S0 is None else S0, True)
    kn = k_ / torch.clamp(k_.norm(dim=-1, keepdim=True), min=1e-12)
    o, Sl = delta_rule_t(q_, kn, v_, torch.sigmoid(b_), _done(done), S0_)
    L = (o * _t(do)).sum()
    if dS_last is not None:
        L = L + (Sl * _t(dS_last)).sum()
    L.backward()
    return dict(o=_np(o), S_last=_np(Sl), dq=_np(q_.grad), dk=_np(k_.grad), dv=_np(v_.grad),
                dbeta=_np(b_.grad), dS0=_np(S0_.grad))


def gated_linear_attention_grads(q, k, v, g, done, S0, do, dS_last=None, feature_map="none"):
    """Returns dict(o, S_last, dq, dk, dv, dg, dS0) for L = sum(do*o) + sum(dS_last*S_last)."""
    q_, k_, v_, g_ = _t(q, True), _t(k, True), _t(v, True), _t(g, True)
    B, T, H, dk = q_.shape
    S0_ = _t(np.zeros((B, H, v_.shape[-1], dk)) if S0 is None else S0, True)
    o, Sl = gated_linear_attention_t(q_, k_, v_, g_, _done(done), S0_, feature_map)
    L = (o * _t(do)).sum()
    if dS_last is not None:
        L = L + (Sl * _t(dS_last)).sum()
    L.backward()
    return dict(o=_np(o), S_last=_np(Sl), dq=_np(q_.grad), dk=_np(k_.grad), dv=_np(v_.grad),
                dg=_np(g_.grad), dS0=_np(S0_.grad))


# --------------------------------------------------------------------------
# The torso block of configuration 5, composed from the reference's parts:
# PreNorm (blocks/normalization.py:30-31) with RMSNorm, Residual (blocks/residual.py:23-26),
# Stack (blocks/stack.py:40-51), a DeltaNet cell in the Memoroid idiom (memoroid.py:93-109) and a
# MinGRU recurrence (min_gru.py:49-78) inside the gating pattern of GLU (blocks/ffn.py:82-123).
# Dense algebra around recurrences that are pinned on their own (delta_rule_t, mingru_scan_t).
# --------------------------------------------------------------------------
def rms_norm_t(x, scale, eps=1e-6):
    """flax.linen.RMSNorm defaults: x * rsqrt(mean(x^2) + eps) * scale."""
    return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * scale


def gated_linear_recurrence_t(x, done, Wz, Wh, Wg, Wo, carry=None, side=None):
    """y = Wo( mingru(Wz x, Wh x) * silu(Wg x) ); carry = (log h_T, log of the cumulative decay since
    the last reset), both (B,1,F) as MinGRUCell.initialize_carry gives them (-inf, 0).
    Returns ((log_state, log_decay), y)."""
    z, ht = x @ Wz.T, x @ Wh.T
    B, T, F = z.shape
    if carry is None:
        h0, ld = None, torch.zeros(B, F, dtype=x.dtype)
    else:
        h0, ld = torch.exp(carry[0][:, 0]), carry[1][:, 0]
        if bool(torch.isinf(carry[0]).all()):
            h0 = None
    h, h_last = mingru_scan_t(z, ht, done, h0, side)
    log_a = -torch.nn.functional.softplus(z)
    for t in range(T):
        ld = torch.where(done[:, t][:, None], log_a[:, t], ld + log_a[:, t])
    y = (h * torch.nn.functional.silu(x @ Wg.T)) @ Wo.T
    return (torch.log(h_last)[:, None], ld[:, None]), y


def linear_attention_cell_t(x, done, Wq, Wk, Wv, norm_scale, Wout, bout, H, carry=None, eps=1e-6):
    """LinearAttentionCell (linear_attention.py:58-117): projections, phi = elu + 1 on keys and queries,
    the additive recurrence with the key sum, read-out num / max(q . z, eps), RMSNorm over the heads'
    concatenated outputs, output projection.  Returns ((S (B,1,H,d,d), z (B,1,H,d)), y)."""
    B, T, _ = x.shape
    heads = lambda t: t.reshape(B, T, H, -1)  # noqa: E731
    q, k, v = heads(x @ Wq.T), heads(x @ Wk.T), heads(x @ Wv.T)
    d = q.shape[-1]
    S0 = torch.zeros(B, H, d, d, dtype=x.dtype) if carry is None else carry[0][:, 0]
    z0 = torch.zeros(B, H, d, dtype=x.dtype) if carry is None else carry[1][:, 0]
    o, S, z = normalised_linear_attention_t(q, k, v, done, S0, z0, "elu1", eps)
    y = rms_norm_t(o.reshape(B, T, H * d), norm_scale) @ Wout.T + bout
    return (S[:, None], z[:, None]), y


def deltanet_cell_t(x, done, Wq, Wk, Wv, Wb, norm_scale, Wout, bout, H, S0=None):
    """DeltaNet cell: projections, L2-normalised keys, beta = sigmoid, delta rule, RMSNorm over the
    heads' concatenated outputs, output projection.  Returns ((S (B,1,H,d,d),), y)."""
    B, T, _ = x.shape
    heads = lambda t: t.reshape(B, T, H, -1)  # noqa: E731
    q, k, v = heads(x @ Wq.T), heads(x @ Wk.T), heads(x @ Wv.T)
    d = q.shape[-1]
    kn = k / torch.clamp(k.norm(dim=-1, keepdim=True), min=1e-12)
    S0 = torch.zeros(B, H, d, d, dtype=x.dtype) if S0 is None else S0[:, 0]
    o, S = delta_rule_t(q, kn, v, torch.sigmoid(x @ Wb.T), done, S0)
    y = rms_norm_t(o.reshape(B, T, H * d), norm_scale) @ Wout.T + bout
    return (S[:, None],), y
