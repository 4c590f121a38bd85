"""Differentiable entry points over the HIP kernels (torch.autograd.Function plays
the role jax.custom_vjp would in a JAX host).

    linear_scan(a, b, done, h0=None, P0=None)            -> (h, h_last, P_last)
    mingru_scan(z, h_tilde, done, h0=None, P0=None)      -> (h, h_last, P_last)  (gates fused)
    linear_attention(q, k, v, done, S0=None, feature_map) -> (o, S_last)
    delta_rule(q, k, v, beta, done, S0=None)             -> (o, S_last)
    deltanet(q, k, v, beta_raw, done, S0=None)           -> (o, S_last)   (key L2-norm and sigmoid fused)
    rms_norm(x, scale, eps, out_dtype)                   -> y      (layer_norm likewise, with a bias)
    silu_gate(h, g)                                      -> h * silu(g)

Layouts follow the reference: (B,T,D) / (B,T,H,d), state (B,H,d_v,d_k), done (B,T)
bool or float where nonzero clears the carry before step t (memoroid.py:60-91).
"""
from __future__ import annotations

import contextlib
import functools

import torch

from . import kernels as K

_step_in_place = False


@contextlib.contextmanager
def step_in_place():
    """Inside this context the acting paths (one time step, no gradients) update the carried state where it
    lies instead of writing a new array: the state handed in is overwritten and handed back.  For a caller that
    owns the carry's buffers (rollout.GraphedStep); elsewhere the carry a caller passes stays untouched."""
    global _step_in_place
    before, _step_in_place = _step_in_place, True
    try:
        yield
    finally:
        _step_in_place = before


def _own(given, used):
    """inplace for a step kernel: only on the caller's own array (a converted copy is a new array already)."""
    return _step_in_place and given is not None and used is given


_FMAP = {None: 0, "none": 0, 0: 0, "elu1": 1, 1: 1}
_FMAP_NAME = {0: "none", 1: "elu1"}
_HD = 64  # widest head dim of the kernels (d_k = d_v = 64 or 32)


def _batched(core_rank, ref):
    """Extra leading axes on the arguments (what jax.vmap over seeds or agents adds around the
    reference's calls, examples/ppo_popjym.py:84-85, mappo.py:21-27) are folded into the batch axis
    for the kernel call and restored on the results.  ``ref``: index of the argument whose rank tells
    (its rank without extra axes is ``core_rank``); arguments that do not carry the leading axes
    (a time-invariant decay, scalars) pass through."""
    def deco(fn):
        @functools.wraps(fn)
        def wrapper(*args, **kwargs):
            extra = args[ref].dim() - core_rank
            if extra <= 0:
                return fn(*args, **kwargs)
            lead = tuple(args[ref].shape[:extra + 1])

            def fold(x):
                if torch.is_tensor(x) and x.dim() > extra and tuple(x.shape[:extra + 1]) == lead:
                    return x.reshape(-1, *x.shape[extra + 1:])
                return x

            def unfold(y):
                return y.reshape(*lead, *y.shape[1:]) if torch.is_tensor(y) else y

            out = fn(*[fold(a) for a in args], **{k: fold(v) for k, v in kwargs.items()})
            return tuple(unfold(y) for y in out) if isinstance(out, tuple) else unfold(out)
        return wrapper
    return deco


def _no_steps(x):
    """No sequences or no time steps: the reference's scan then hands the carry back unchanged
    (memoroid.py:60-91 scans the carry prepended to T = 0 elements) and there is nothing to launch."""
    return x.shape[0] == 0 or x.shape[1] == 0


def _scan_without_steps(b, h0, P0):
    B, _, D = b.shape
    ct = torch.float32 if b.dtype == torch.bfloat16 else b.dtype   # bf16 arrays carry float32 state, as the kernels do
    h_last = b.new_zeros((B, D), dtype=ct) if h0 is None else h0.to(ct) + 0
    P_last = b.new_ones((B, D), dtype=ct) if P0 is None else P0.detach().to(ct).clone()
    return b.new_zeros(b.shape), h_last, P_last


def _attention_without_steps(q, v, S0):
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    S_last = q.new_zeros((B, H, dv, dk), dtype=torch.float32) if S0 is None else S0.float() + 0
    return v.new_zeros((B, T, H, dv)), S_last


class _Heads:
    """Maps other head dims onto what the kernels take (the reference's cells take any head_dim; its
    guides use 16).  The 32-wide kernels serve d_k <= 32, the 64-wide ones the rest.  The kernels of the
    linear-attention family (`narrow`) take any d_k, d_v up to their build's width that is a whole
    number of 16-byte segments as it is; everything else goes through padding: d_k below the kernel's
    width is zero-padded -- after the feature map, since phi(0) = 1 would otherwise count -- and d_v is
    zero-padded to a multiple of the value width and split into blocks that run as extra heads sharing
    q and k (rows of the state are independent recurrences).  Where the output is linear in the state
    (`split_k`: plain and gated linear attention), d_k > 64 is split the same way into key blocks
    whose outputs add up (o = sum over blocks of S[:, block] q[block]); the delta rule and the
    normalised read-out couple the key features and stay at d_k <= 64.
    Padding, blocks, sums and slices are ordinary differentiable array ops around the kernel call."""

    def __init__(self, q, v, fmap=0, narrow=False, split_k=False):
        self.B, self.T, self.H, self.dk = q.shape
        self.dv = v.shape[-1]
        if self.dk > _HD and not split_k:
            raise ValueError(f"d_k = {self.dk} > {_HD} is not supported by this operator (d_v may be any size)")
        self.hd = 32 if self.dk <= 32 else _HD
        seg = 16 // q.element_size()                    # elements per 16 bytes
        self.kw = self.dk if narrow and self.dk <= self.hd and self.dk % seg == 0 else self.hd   # key width the kernel sees
        self.vw = self.dv if narrow and self.dv <= self.hd and self.dv % seg == 0 else self.hd   # value width per block
        self.nkb = (self.dk + self.kw - 1) // self.kw   # key blocks (1 unless d_k > 64)
        self.nb = (self.dv + self.vw - 1) // self.vw    # value blocks
        self.native = self.dk == self.kw and self.dv == self.vw
        self.pre = fmap if self.dk != self.nkb * self.kw else 0    # feature map applied here, before the padding
        self.fmap = 0 if self.pre else fmap                        # feature map left to the kernel

    # the kernel's head axis is (H, nkb, nb) flattened
    def qk(self, x):  # (B,T,H,dk) -> (B,T,H*nkb*nb,kw), every value block a copy
        if self.native:
            return x
        if self.pre:
            xf = x if x.dtype in (torch.float32, torch.float64) else x.float()
            x = (torch.nn.functional.elu(xf) + 1).to(x.dtype)
        x = torch.nn.functional.pad(x, (0, self.nkb * self.kw - self.dk))
        if self.nkb * self.nb == 1:
            return x
        x = x.reshape(self.B, self.T, self.H, self.nkb, 1, self.kw).expand(self.B, self.T, self.H, self.nkb, self.nb, self.kw)
        return x.reshape(self.B, self.T, self.H * self.nkb * self.nb, self.kw)

    def v(self, x):  # (B,T,H,dv) -> (B,T,H*nkb*nb,vw), every key block a copy
        if self.native:
            return x
        x = torch.nn.functional.pad(x, (0, self.nb * self.vw - self.dv))
        x = x.reshape(self.B, self.T, self.H, 1, self.nb, self.vw).expand(self.B, self.T, self.H, self.nkb, self.nb, self.vw)
        return x.reshape(self.B, self.T, self.H * self.nkb * self.nb, self.vw)

    def per_head(self, x):  # (B,T,H) -> (B,T,H*nkb*nb)
        return x if self.nkb * self.nb == 1 else x.repeat_interleave(self.nkb * self.nb, dim=2)

    def state_in(self, S):  # (B,H,dv,dk) -> (B,H*nkb*nb,vw,kw)
        if S is None or self.native:
            return S
        S = torch.nn.functional.pad(S, (0, self.nkb * self.kw - self.dk, 0, self.nb * self.vw - self.dv))
        S = S.reshape(self.B, self.H, self.nb, self.vw, self.nkb, self.kw).permute(0, 1, 4, 2, 3, 5)
        return S.reshape(self.B, self.H * self.nkb * self.nb, self.vw, self.kw)

    def z_in(self, z):  # (B,H,dk) -> (B,H*nb,kw)   (normalised read-out: one key block)
        if z is None or self.native:
            return z
        z = torch.nn.functional.pad(z, (0, self.kw - self.dk))
        return z if self.nb == 1 else z.repeat_interleave(self.nb, dim=1)

    def out(self, o):  # (B,T,H*nkb*nb,vw) -> (B,T,H,dv): the key blocks' outputs add up
        if self.native:
            return o
        o = o.reshape(self.B, o.shape[1], self.H, self.nkb, self.nb * self.vw)
        if self.nkb > 1:
            o = (o if o.dtype in (torch.float32, torch.float64) else o.float()).sum(3).to(o.dtype)
        else:
            o = o[:, :, :, 0]
        return o[..., :self.dv]

    def state_out(self, S):
        if self.native:
            return S
        S = S.reshape(self.B, self.H, self.nkb, self.nb, self.vw, self.kw).permute(0, 1, 3, 4, 2, 5)
        return S.reshape(self.B, self.H, self.nb * self.vw, self.nkb * self.kw)[:, :, :self.dv, :self.dk]

    def z_out(self, z):
        return z if self.native else z.reshape(self.B, self.H, self.nb, self.kw)[:, :, 0, :self.dk]


class _LinearScan(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, b, done, h0, P0):
        a_, b_ = a.contiguous(), b.contiguous()
        carry = (lambda x: x.float()) if b.dtype == torch.bfloat16 else (lambda x: x)  # bfloat16 arrays: float32 carries
        h0_ = None if h0 is None else carry(h0).contiguous()
        P0_ = None if P0 is None else carry(P0).contiguous()
        h, h_last, P_last = K.linear_scan_fwd(a_, b_, done, h0_, P0_)
        ctx.save_for_backward(a_, h, h0_ if h0_ is not None else torch.empty(0, device=b.device))
        ctx.done = done
        ctx.has_h0 = h0 is not None
        ctx.h0_dtype = None if h0 is None else h0.dtype
        ctx.mark_non_differentiable(P_last)
        return h, h_last, P_last

    @staticmethod
    def backward(ctx, g, g_last, _gP):
        a, h, h0 = ctx.saved_tensors
        h0 = h0 if ctx.has_h0 else None
        g = torch.zeros_like(h) if g is None else g.contiguous()
        g_last = None if g_last is None else g_last.contiguous()
        ti = a.dim() == 1  # a broadcast coefficient: the kernel sums its gradient over time, the rest is (B,D)
        da, db, dh0 = K.linear_scan_bwd(a, h, ctx.done, h0, g, g_last, sum_da=ti)
        if ti:
            da = da.sum(dim=0).to(a.dtype)
        return (da if ctx.needs_input_grad[0] else None,
                db if ctx.needs_input_grad[1] else None,
                None,
                dh0.to(ctx.h0_dtype) if (ctx.has_h0 and ctx.needs_input_grad[3]) else None,
                None)


@_batched(3, 1)
def linear_scan(a, b, done, h0=None, P0=None):
    """Reset-aware diagonal recurrence h_t = a_t h_{t-1} + b_t (lru.py:92-95 scanned
    by memoroid.py:60-91).  a: (B,T,D) or (D,); b: (B,T,D); h0,P0: (B,D).
    P_last (the cumulative-decay leaf of the carry) is not differentiable."""
    if _no_steps(b):
        return _scan_without_steps(b, h0, P0)
    return _LinearScan.apply(a, b, done, h0, P0)


class _MinGRUScan(torch.autograd.Function):
    @staticmethod
    def forward(ctx, z, h_tilde, done, h0, P0):
        z_, x_ = z.contiguous(), h_tilde.contiguous().to(z.dtype)
        h0_ = None if h0 is None else h0.float().contiguous()   # the carries are float32 whatever the arrays are
        P0_ = None if P0 is None else P0.float().contiguous()
        h, h_last, P_last = K.mingru_scan_fwd(z_, x_, done, h0_, P0_)
        ctx.save_for_backward(z_, x_, h, h0_ if h0_ is not None else torch.empty(0, device=z.device))
        ctx.done = done
        ctx.has_h0 = h0 is not None
        ctx.h0_dtype = None if h0 is None else h0.dtype
        ctx.mark_non_differentiable(P_last)
        return h, h_last, P_last

    @staticmethod
    def backward(ctx, g, g_last, _gP):
        z, x, h, h0 = ctx.saved_tensors
        h0 = h0 if ctx.has_h0 else None
        g = torch.zeros_like(h) if g is None else g.contiguous()
        g_last = None if g_last is None else g_last.contiguous()
        dz, dx, dh0 = K.mingru_scan_bwd(z, x, h, ctx.done, h0, g, g_last)
        return (dz if ctx.needs_input_grad[0] else None,
                dx if ctx.needs_input_grad[1] else None,
                None,
                dh0.to(ctx.h0_dtype) if (ctx.has_h0 and ctx.needs_input_grad[3]) else None,
                None)


@_batched(3, 0)
def mingru_scan(z, h_tilde, done, h0=None, P0=None):
    """MinGRU from its two projections (min_gru.py:49-78 scanned by memoroid.py:60-91), linear space:
    h_t = sigmoid(-z_t) h_{t-1} + sigmoid(z_t) g(h~_t), g(x) = x + 0.5 (x >= 0) | sigmoid(x), with the
    gate arithmetic inside the scan kernels.  z, h_tilde: (B,T,D) float32 or bfloat16 (the arithmetic and the
    carries are float32 either way); h0, P0: (B,D).
    Returns (h, h_last, P_last); P_last is not differentiable."""
    if _no_steps(z):
        return _scan_without_steps(z, h0, P0)
    return _MinGRUScan.apply(z, h_tilde, done, h0, P0)


class _LinearAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, done, S0, fmap):
        q_, k_, v_ = q.contiguous(), k.contiguous(), v.contiguous()
        S0_ = None if S0 is None else S0.contiguous().float()
        need = any(ctx.needs_input_grad)
        if q_.shape[1] == 1 and not need:  # acting: one step, no residuals (memoroid.py:93-109 with T = 1)
            o, S_last, _ = K.linear_attn_step(q_[:, 0], k_[:, 0], v_[:, 0], done[:, 0], S0_,
                                              feature_map=_FMAP_NAME[fmap], inplace=_own(S0, S0_))
            ctx.done, ctx.fmap, ctx.has_S0 = done, fmap, S0 is not None
            return o[:, None], S_last
        o, S_last, chk = K.linear_attn_fwd(q_, k_, v_, done, S0_, fmap, save_chk=need)
        if need:  # chk[1] (S_last) is None when the chunk-parallel pair of kernels ran
            ctx.save_for_backward(q_, k_, v_, *(t for t in chk if t is not None))
        ctx.done, ctx.fmap, ctx.has_S0 = done, fmap, S0 is not None
        return o, S_last

    @staticmethod
    def backward(ctx, do, dS_last):
        q, k, v, S_chk, *rest = ctx.saved_tensors
        do = torch.zeros_like(v) if do is None else do.contiguous()
        dS_last = None if dS_last is None else dS_last.contiguous().float()
        dq, dk, dv, dS0 = K.linear_attn_bwd(q, k, v, ctx.done, (S_chk, rest[0] if rest else None), do, dS_last,
                                            ctx.fmap, want_dS0=ctx.has_S0)
        return dq, dk, dv, None, (dS0 if ctx.has_S0 else None), None


@_batched(4, 0)
def linear_attention(q, k, v, done, S0=None, feature_map="none"):
    """Causal unnormalised linear attention, chunked: S_t = r_t S_{t-1} + v_t phi(k_t)^T,
    o_t = S_t phi(q_t) (linear_attention.py:62-86,105).  Returns (o, S_last)."""
    if _no_steps(q):
        return _attention_without_steps(q, v, S0)
    hd = _Heads(q, v, _FMAP[feature_map], narrow=True, split_k=True)
    o, S_last = _LinearAttention.apply(hd.qk(q), hd.qk(k), hd.v(v), done, hd.state_in(S0), hd.fmap)
    return hd.out(o), hd.state_out(S_last)


class _NormalisedLinearAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, done, S0, z0, fmap, eps, want_ss):
        q_, k_, v_ = q.contiguous(), k.contiguous(), v.contiguous()
        S0_ = None if S0 is None else S0.contiguous().float()
        z0_ = None if z0 is None else z0.contiguous().float()
        need = any(ctx.needs_input_grad)
        ctx.done, ctx.fmap, ctx.eps, ctx.has_0 = done, fmap, eps, (S0 is not None, z0 is not None)
        if q_.shape[1] == 1 and not need:  # acting: one fused step
            o, S_last, z_last = K.linear_attn_step(q_[:, 0], k_[:, 0], v_[:, 0], done[:, 0], S0_, z0_,
                                                   feature_map=_FMAP_NAME[fmap], normalise=True, eps=eps,
                                                   inplace=_own(S0, S0_) and _own(z0, z0_))
            ss = o.float().square().sum(-1)[..., None] if want_ss else None   # (B,H,1)
            return o[:, None], S_last, z_last, ss
        o, den, S_last, z_last, chk, ss = K.linear_attn_norm_fwd(q_, k_, v_, done, S0_, z0_, fmap, eps, save_chk=need,
                                                                 want_ss=True) if want_ss else \
            (*K.linear_attn_norm_fwd(q_, k_, v_, done, S0_, z0_, fmap, eps, save_chk=need), None)
        if need:
            ctx.save_for_backward(q_, k_, v_, o, den, *chk)
        return o, S_last, z_last, ss

    @staticmethod
    def backward(ctx, do, dS_last, dz_last, d_ss):
        q, k, v, o, den, S_chk, z_chk, S_last = ctx.saved_tensors
        do = torch.zeros_like(v) if do is None else do.contiguous()
        dS_last = None if dS_last is None else dS_last.contiguous().float()
        dz_last = None if dz_last is None else dz_last.contiguous().float()
        d_ss = None if d_ss is None else d_ss.contiguous().float()
        dq, dk, dv, dS0, dz0 = K.linear_attn_norm_bwd(q, k, v, ctx.done, (S_chk, z_chk, S_last), o, den, do, dS_last,
                                                      dz_last, ctx.fmap, ctx.eps, want_d0=any(ctx.has_0), d_ss=d_ss)
        return dq, dk, dv, None, (dS0 if ctx.has_0[0] else None), (dz0 if ctx.has_0[1] else None), None, None, None


@_batched(4, 0)
def normalised_linear_attention(q, k, v, done, S0=None, z0=None, feature_map="elu1", eps=1e-6, return_ss=False):
    """Causal linear attention with the normalised read-out of LinearAttentionCell.read
    (linear_attention.py:93-110) in the same kernel: z_t = r_t z_{t-1} + phi(k_t),
    o_t = S_t phi(q_t) / max(phi(q_t) . z_t, eps).  Returns (o, S_last, z_last), and with return_ss a
    fourth result ss (B,T,H) float32, ss[b,t,h] = sum_d o[b,t,h,d]^2 from the kernel's output tile
    (differentiable): what the RMS norm over all heads that follows (linear_attention.py:114) needs
    from each head, so that its caller does one rescale of o and no reduction over it."""
    if _no_steps(q):
        B, T, H, dk = q.shape
        z_last = q.new_zeros((B, H, dk), dtype=torch.float32) if z0 is None else z0.float() + 0
        out = (*_attention_without_steps(q, v, S0), z_last)
        return (*out, q.new_zeros((B, T, H), dtype=torch.float32)) if return_ss else out
    hd = _Heads(q, v, _FMAP[feature_map], narrow=True)
    o, S_last, z_last, ss = _NormalisedLinearAttention.apply(hd.qk(q), hd.qk(k), hd.v(v), done, hd.state_in(S0),
                                                             hd.z_in(z0), hd.fmap, float(eps), bool(return_ss))
    out = (hd.out(o), hd.state_out(S_last), hd.z_out(z_last))
    if not return_ss:
        return out
    B, Hk, T = ss.shape   # kernel heads = (H, value blocks): a head's sum of squares is the sum over its blocks
    return (*out, ss.view(B, hd.H, Hk // hd.H, T).sum(2).transpose(1, 2))


class _GatedLinearAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, g, done, S0, fmap):
        q_, k_, v_ = q.contiguous(), k.contiguous(), v.contiguous()
        g_ = g.contiguous().float()
        S0_ = None if S0 is None else S0.contiguous().float()
        need = any(ctx.needs_input_grad)
        if q_.shape[1] == 1 and not need:  # acting: one step, no residuals (memoroid.py:93-109 with T = 1)
            o, S_last = K.gated_linear_attn_step(q_[:, 0], k_[:, 0], v_[:, 0], g_[:, 0], done[:, 0], S0_,
                                                 feature_map=_FMAP_NAME[fmap], inplace=_own(S0, S0_))
            ctx.done, ctx.fmap, ctx.has_S0 = done, fmap, S0 is not None
            return o[:, None], S_last
        o, S_last, S_chk = K.gated_linear_attn_fwd(q_, k_, v_, g_, done, S0_, fmap, save_chk=need)
        if need:
            ctx.save_for_backward(q_, k_, v_, g_, S_chk, S_last)
        ctx.done, ctx.fmap, ctx.has_S0 = done, fmap, S0 is not None
        return o, S_last

    @staticmethod
    def backward(ctx, do, dS_last):
        q, k, v, g, S_chk, S_last = ctx.saved_tensors
        do = torch.zeros_like(v) if do is None else do.contiguous()
        dS_last = None if dS_last is None else dS_last.contiguous().float()
        dq, dk, dv, dg, dS0 = K.gated_linear_attn_bwd(q, k, v, g, ctx.done, S_chk, do, dS_last, ctx.fmap,
                                                      want_dS0=ctx.has_S0, S_last=S_last)
        return dq, dk, dv, dg, None, (dS0 if ctx.has_S0 else None), None


@_batched(4, 0)
def gated_linear_attention(q, k, v, g, done, S0=None, feature_map="none"):
    """Linear attention with a scalar log-decay g:(B,T,H) per step and head:
    S_t = r_t exp(g_t) S_{t-1} + v_t phi(k_t)^T, o_t = S_t phi(q_t) -- the Mamba cell's algebra
    (mamba.py:109-122) in chunked form.  Returns (o, S_last)."""
    if _no_steps(q):
        return _attention_without_steps(q, v, S0)
    hd = _Heads(q, v, _FMAP[feature_map], narrow=True, split_k=True)
    o, S_last = _GatedLinearAttention.apply(hd.qk(q), hd.qk(k), hd.v(v), hd.per_head(g), done, hd.state_in(S0),
                                            hd.fmap)
    return hd.out(o), hd.state_out(S_last)


class _DeltaRule(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, beta, done, S0, prologue=False, resets=None):
        q_, k_, v_, b_ = q.contiguous(), k.contiguous(), v.contiguous(), beta.contiguous()
        S0_ = None if S0 is None else S0.contiguous().float()
        need = any(ctx.needs_input_grad)
        ctx.done, ctx.has_S0, ctx.prologue, ctx.resets = done, S0 is not None, prologue, resets
        if q_.shape[1] == 1 and not need:  # acting: one step, no residuals
            k1, b1 = k_[:, 0], b_[:, 0]
            if prologue:  # a (B,H,d) array: the prologue as array ops costs nothing here
                k1 = torch.nn.functional.normalize(k1.float(), dim=-1).to(k_.dtype)
                b1 = torch.sigmoid(b1.float()).to(b_.dtype)
            o, S_last = K.delta_rule_step(q_[:, 0], k1, v_[:, 0], b1, done[:, 0], S0_, inplace=_own(S0, S0_))
            return o[:, None], S_last
        o, S_last, chk = K.delta_rule_fwd(q_, k_, v_, b_, done, S0_, save_chk=need, prologue=prologue, reset_path=resets)
        if need:
            ctx.save_for_backward(q_, k_, v_, b_, *chk)
        return o, S_last

    @staticmethod
    def backward(ctx, do, dS_last):
        q, k, v, beta, S_chk, Tm_chk = ctx.saved_tensors
        do = torch.zeros_like(v) if do is None else do.contiguous()
        dS_last = None if dS_last is None else dS_last.contiguous().float()
        dq, dk, dv, db, dS0 = K.delta_rule_bwd(q, k, v, beta, ctx.done, (S_chk, Tm_chk), do, dS_last,
                                               want_dS0=ctx.has_S0, prologue=ctx.prologue, reset_path=ctx.resets)
        return dq, dk, dv, db, None, (dS0 if ctx.has_S0 else None), None, None


@_batched(4, 0)
def delta_rule(q, k, v, beta, done, S0=None, resets=None):
    """DeltaNet recurrence S_t = r_t S_{t-1}(I - beta_t k_t k_t^T) + beta_t v_t k_t^T,
    o_t = S_t q_t, in chunked WY form.  Returns (o, S_last).
    resets: None / "passes" / "merged" -- how the kernels treat a chunk that holds resets
    (mrx_reset_path; "merged" for callers whose episodes end every hundred steps or so)."""
    if _no_steps(q):
        return _attention_without_steps(q, v, S0)
    hd = _Heads(q, v, narrow=True)
    o, S_last = _DeltaRule.apply(hd.qk(q), hd.qk(k), hd.v(v), hd.per_head(beta), done, hd.state_in(S0), False, resets)
    return hd.out(o), hd.state_out(S_last)


@_batched(4, 0)
def deltanet(q, k, v, beta_raw, done, S0=None, resets=None):
    """The DeltaNet cell's recurrence on its raw projections: delta_rule with
    k / max(|k|, 1e-12) and sigmoid(beta_raw) formed inside the kernels (the normalised keys and
    the gates never reach memory; gradients come back w.r.t. the raw arrays).  Returns (o, S_last)."""
    if _no_steps(q):
        return _attention_without_steps(q, v, S0)
    hd = _Heads(q, v, narrow=True)   # where keys are padded: zeros leave their norm unchanged
    o, S_last = _DeltaRule.apply(hd.qk(q), hd.qk(k), hd.v(v), hd.per_head(beta_raw), done, hd.state_in(S0), True, resets)
    return hd.out(o), hd.state_out(S_last)


class _MlstmGates(torch.autograd.Function):
    @staticmethod
    def forward(ctx, log_i, log_f, done, m0, g_floor):
        li, lf = log_i.contiguous().float(), log_f.contiguous().float()
        m0_ = None if m0 is None else m0.contiguous().float()
        m, g, w = K.mlstm_gates_fwd(li, lf, done, m0_, g_floor)
        ctx.done, ctx.g_floor, ctx.has_m0 = done, g_floor, m0 is not None
        ctx.save_for_backward(li, lf, m, *([m0_] if m0 is not None else []))
        return m, g, w

    @staticmethod
    def backward(ctx, dm, dg, dw):
        li, lf, m, *rest = ctx.saved_tensors
        m0 = rest[0] if rest else None
        c = lambda t: None if t is None else t.contiguous().float()  # noqa: E731
        dli, dlf, dm0 = K.mlstm_gates_bwd(li, lf, ctx.done, m0, m, c(dm), c(dg), c(dw), ctx.g_floor, want_dm0=ctx.has_m0)
        return dli, dlf, None, dm0, None


def mlstm_gates(log_i, log_f, done, m0=None, g_floor=-60.0):
    """The stabiliser of the mLSTM cell's gates (mlstm.py:190-206 unrolled over time, resets as memoroid.py:72-85):
    m_t = done_t ? log_i_t : max(m_{t-1} + log_f_t, log_i_t); returns (m, g, w), each (B,T,H), with
    g_t = log_f_t + m_{t-1} - m_t (0 at a reset, not below g_floor) and w_t = exp(log_i_t - m_t) -- the log-decay
    and the key weight of the gated linear recurrence that carries the cell's C and n.  m0: (B,H) or None."""
    return _MlstmGates.apply(log_i, log_f, done, m0, g_floor)


class _SiluGate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, h, g):
        dt = torch.promote_types(h.dtype, g.dtype)
        if dt not in (torch.float32, torch.bfloat16):
            dt = torch.float32
        hc, gc = h.to(dt).contiguous(), g.to(dt).contiguous()
        ctx.save_for_backward(hc, gc)
        ctx.dtypes = (h.dtype, g.dtype)
        return K.silu_gate_fwd(hc, gc)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, dy):
        hc, gc = ctx.saved_tensors
        dh, dg = K.silu_gate_bwd(hc, gc, dy.to(hc.dtype).contiguous())
        return dh.to(ctx.dtypes[0]), dg.to(ctx.dtypes[1])


def silu_gate(h, g):
    """h * silu(g) -- activation(gate) * value of the reference's GLU block (blocks/ffn.py:108-121) with silu --
    in one kernel each way.  h, g of one shape; float32 or bfloat16 (anything else is computed in float32)."""
    return _SiluGate.apply(h, g)


def _norm_operand(t):
    t = t.contiguous()
    return t if t.dtype in (torch.float32, torch.bfloat16) else t.float()


class _Norm(torch.autograd.Function):
    """RMS norm (center False) or layer norm of x; fork: the input is handed on beside its norm -- (x, norm(x)) -- so
    that the gradients of both meet in the norm's backward kernel instead of in a pass of their own."""

    @staticmethod
    def forward(ctx, x, scale, bias, eps, out_dtype, center, fork):
        xc = _norm_operand(x)
        sc = None if scale is None else scale.contiguous().float()
        bi = None if bias is None else bias.contiguous().float()
        ctx.save_for_backward(xc, *([sc] if sc is not None else []))
        ctx.eps, ctx.x_dtype, ctx.center, ctx.fork = eps, x.dtype, center, fork
        ctx.has_scale, ctx.has_bias = sc is not None, bi is not None
        y = K.layer_norm_fwd(xc, sc, bi, eps, out_dtype, center)
        if fork:
            ctx.set_materialize_grads(False)
            return xc.view_as(xc).to(x.dtype), y
        return y

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, *grads):
        xc, *rest = ctx.saved_tensors
        sc = rest[0] if rest else None
        dres, dy = grads if ctx.fork else (None, grads[0])
        if dy is None:   # the norm's branch was not used
            return dres, None, None, None, None, None, None
        want = (ctx.has_scale and ctx.needs_input_grad[1]) or (ctx.has_bias and ctx.needs_input_grad[2])
        add = None if dres is None else dres.contiguous().to(xc.dtype)
        dx, dscale, dbias = K.layer_norm_bwd(xc, sc, _norm_operand(dy), ctx.eps, want, add, ctx.center)
        return (dx.to(ctx.x_dtype), dscale if ctx.has_scale else None, dbias if ctx.has_bias else None, None, None, None, None)


def rms_norm(x, scale=None, eps=1e-6, out_dtype=None):
    """flax.linen.RMSNorm with its defaults over the last axis (linear_attention.py:109-115; the norm of the
    torso's PreNorm blocks): x * rsqrt(mean(x^2) + eps) * scale, one kernel each way.  x (..., D) float32 or
    bfloat16 with D a multiple of 4 up to 2048, scale (D) or None; the result in out_dtype (default x's)."""
    return _Norm.apply(x, scale, None, eps, out_dtype, False, False)


def rms_norm_fork(x, scale=None, eps=1e-6, out_dtype=None):
    """(x, rms_norm(x, scale, eps, out_dtype)) for the residual branch around a pre-norm block
    (blocks/residual.py:23-26 around normalization.py:30-31): use the first result where x itself would be
    used.  The backward adds the gradient of that branch inside the norm's kernel."""
    return _Norm.apply(x, scale, None, eps, out_dtype, False, True)


def layer_norm(x, scale=None, bias=None, eps=1e-6, out_dtype=None):
    """flax.linen.LayerNorm with its defaults over the last axis (the default norm of PreNorm / PostNorm,
    blocks/normalization.py:10-65): (x - mean(x)) * rsqrt(var(x) + eps) * scale + bias, one kernel each way.
    Shapes and dtypes as rms_norm."""
    return _Norm.apply(x, scale, bias, eps, out_dtype, True, False)


def layer_norm_fork(x, scale=None, bias=None, eps=1e-6, out_dtype=None):
    """(x, layer_norm(x, ...)): rms_norm_fork for the layer norm."""
    return _Norm.apply(x, scale, bias, eps, out_dtype, True, True)


def propagate_sensitivities(decay, jacobians, sensitivity, done):
    """Real-time recurrent learning: carry the parameter sensitivities of a diagonal recurrence
    over a (B,T) block of steps -- Memoroid._propagate_sensitivities (memoroid.py:114-141).
    decay: (B,T,H); jacobians[name]: (B,T,H,*param_shape) local Jacobians; sensitivity[name]:
    (B,1,H,*param_shape).  Returns the sensitivities after the last step, same shapes.  The
    reference repeats the decay param_size times and scans the concatenated (B,T+1,H*param_size)
    array; the kernel reads the Jacobians once and writes only the final state."""
    import math
    B, T, H = decay.shape
    if B == 0 or T == 0:  # nothing to propagate through
        return {name: sensitivity[name] for name in sorted(jacobians.keys())}
    decay = decay.contiguous()
    out = {}
    for name in sorted(jacobians.keys()):
        J, S = jacobians[name], sensitivity[name]
        param_shape = tuple(J.shape[3:])
        ps = math.prod(param_shape)
        last = K.linear_scan_last(decay.to(J.dtype), J.reshape(B, T, H * ps).contiguous(), done,
                                  S.reshape(B, H * ps).to(J.dtype).contiguous())
        out[name] = last.reshape(B, 1, H, *param_shape)
    return out
