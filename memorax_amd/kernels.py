"""Thin, allocation-explicit wrappers: torch device tensors in, C-ABI call, tensors out.

torch is used for device memory and the current HIP stream only.  Every function
validates device / dtype / contiguity, allocates the outputs and forwards raw
pointers to the library; there is no alternative code path.
"""
from __future__ import annotations

import torch

from . import _lib

_DT = {torch.float32: _lib.MRX_F32, torch.bfloat16: _lib.MRX_BF16, torch.complex64: _lib.MRX_C64}


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current device's current stream as a raw handle (the short way where torch has it: building
    a torch.cuda.Stream object per call costs several microseconds of a 15-microsecond call)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


def _chk(t, name, dtype=None, shape=None):
    if t is None:
        return
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (memorax_amd has no CPU path)")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise ValueError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")


def _done(done, B, T):
    """Accept bool / uint8 / float32 (B,T); returns (tensor, done_dtype enum)."""
    if tuple(done.shape) != (B, T):
        raise ValueError(f"done must have shape {(B, T)}, got {tuple(done.shape)}")
    if done.dtype == torch.bool:
        done = done.contiguous().view(torch.uint8)
    elif done.dtype == torch.uint8:
        done = done.contiguous()
    elif done.dtype == torch.float32:
        done = done.contiguous()
        _chk(done, "done")
        return done, _lib.MRX_DONE_F32
    else:
        done = (done != 0).contiguous().view(torch.uint8)
    _chk(done, "done")
    return done, _lib.MRX_DONE_U8


_chunk_sizes = {}


def chunk_size(dtype, delta=False) -> int:
    """Chunk length of the (gated) linear-attention kernels, or of the delta-rule kernels."""
    c = _chunk_sizes.get((dtype, delta))
    if c is None:
        lib = _lib.load()
        c = _chunk_sizes[(dtype, delta)] = int((lib.mrx_delta_chunk_size if delta else lib.mrx_chunk_size)(_DT[dtype]))
    return c


# ----------------------------------------------------------------- diagonal scan
def linear_scan_fwd(a, b, done, h0=None, P0=None, want_P=True):
    """h_t = done ? b_t : a_t h_{t-1} + b_t.  a: (B,T,D) or (D,) time-invariant.  float32, complex64, or
    bfloat16 arrays with float32 arithmetic and float32 carries (h0, P0, h_last, P_last).
    Returns (h, h_last, P_last)."""
    lib = _lib.load()
    B, T, D = b.shape
    dt = b.dtype
    if dt not in (torch.float32, torch.complex64, torch.bfloat16):
        raise ValueError("linear_scan supports float32, complex64 and bfloat16")
    ct = torch.float32 if dt == torch.bfloat16 else dt  # the carries' type
    ti = a.dim() == 1
    _chk(a, "a", dt, (D,) if ti else (B, T, D))
    _chk(b, "b", dt)
    _chk(h0, "h0", ct, (B, D))
    _chk(P0, "P0", ct, (B, D))
    done, dd = _done(done, B, T)
    h = torch.empty_like(b)
    h_last = torch.empty((B, D), dtype=ct, device=b.device)
    P_last = torch.empty((B, D), dtype=ct, device=b.device) if want_P else None
    st = lib.mrx_linear_scan_fwd(_stream(), _ptr(a), _ptr(b), _ptr(done), _ptr(h0), _ptr(P0),
                                 _ptr(h), _ptr(h_last), _ptr(P_last), B, T, D, _DT[dt], dd, int(ti))
    _lib.check(st, "mrx_linear_scan_fwd")
    return h, h_last, P_last


def mlstm_gates_fwd(log_i, log_f, done, m0=None, g_floor=-60.0):
    """The mLSTM cell's stabiliser in one pass (mrx_mlstm_gates_fwd): log_i, log_f (B,T,H) float32, m0 (B,H) or
    None (the cell's initial -1e9).  Returns (m, g, w), each (B,T,H): the running maximum, the log-decay
    g_t = log_f_t + m_{t-1} - m_t (0 at a reset, not below g_floor) and the key weight exp(log_i_t - m_t)."""
    lib = _lib.load()
    B, T, H = log_i.shape
    _chk(log_i, "log_i", torch.float32)
    _chk(log_f, "log_f", torch.float32, (B, T, H))
    _chk(m0, "m0", torch.float32, (B, H))
    done, dd = _done(done, B, T)
    m, g, w = (torch.empty_like(log_i) for _ in range(3))
    st = lib.mrx_mlstm_gates_fwd(_stream(), _ptr(log_i), _ptr(log_f), _ptr(done), _ptr(m0), _ptr(m), _ptr(g), _ptr(w),
                                 B, T, H, dd, float(g_floor))
    _lib.check(st, "mrx_mlstm_gates_fwd")
    return m, g, w


def mlstm_gates_bwd(log_i, log_f, done, m0, m, dm, dg, dw, g_floor=-60.0, want_dm0=True):
    """Gradients of mlstm_gates_fwd: dm, dg, dw (each (B,T,H) or None) in, (dlog_i, dlog_f, dm0) out."""
    lib = _lib.load()
    B, T, H = log_i.shape
    for t, n in ((log_i, "log_i"), (log_f, "log_f"), (m, "m"), (dm, "dm"), (dg, "dg"), (dw, "dw")):
        _chk(t, n, torch.float32, (B, T, H))
    _chk(m0, "m0", torch.float32, (B, H))
    done, dd = _done(done, B, T)
    dli, dlf = torch.empty_like(log_i), torch.empty_like(log_f)
    dm0 = torch.empty((B, H), dtype=torch.float32, device=log_i.device) if want_dm0 else None
    st = lib.mrx_mlstm_gates_bwd(_stream(), _ptr(log_i), _ptr(log_f), _ptr(done), _ptr(m0), _ptr(m), _ptr(dm), _ptr(dg),
                                 _ptr(dw), _ptr(dli), _ptr(dlf), _ptr(dm0), B, T, H, dd, float(g_floor))
    _lib.check(st, "mrx_mlstm_gates_bwd")
    return dli, dlf, dm0


RMS_NORM_PARTS = 1024   # MRX_RMS_NORM_PARTS: rows of the backward's workspace
RMS_NORM_MAX_D = 2048


def _norm_dtypes(*ts):
    for t in ts:
        if t not in (torch.float32, torch.bfloat16):
            raise ValueError("the norm kernels take float32 or bfloat16 arrays")


def rms_norm_fwd(x, scale, eps=1e-6, out_dtype=None):
    """y = x * rsqrt(mean(x^2) + eps) * scale over the last axis (mrx_rms_norm_fwd): x (..., D) float32 or
    bfloat16, scale (D) float32 or None (ones); y in out_dtype (default: x's)."""
    return layer_norm_fwd(x, scale, None, eps, out_dtype, center=False)


def rms_norm_bwd(x, scale, dy, eps=1e-6, want_dscale=True, dx_add=None):
    """Gradients of rms_norm_fwd: dy (..., D) float32 or bfloat16 in; (dx in x's dtype, dscale (D) float32 or
    None) out.  The statistics are recomputed from x.  dx_add (like x, or None): added to dx."""
    dx, dscale, _ = layer_norm_bwd(x, scale, dy, eps, want_dscale, dx_add, center=False)
    return dx, dscale


def layer_norm_fwd(x, scale, bias, eps=1e-6, out_dtype=None, center=True):
    """y = (x - mean(x)) * rsqrt(var(x) + eps) * scale + bias over the last axis (mrx_layer_norm_fwd); center=False:
    the RMS norm (no mean, no bias).  x (..., D) float32 or bfloat16; scale, bias (D) float32 or None."""
    lib = _lib.load()
    D = x.shape[-1]
    out_dtype = x.dtype if out_dtype is None else out_dtype
    _norm_dtypes(x.dtype, out_dtype)
    _chk(x, "x")
    _chk(scale, "scale", torch.float32, (D,))
    _chk(bias, "bias", torch.float32, (D,))
    y = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    if x.numel() == 0:
        return y
    rows = x.numel() // D
    if center:
        st = lib.mrx_layer_norm_fwd(_stream(), _ptr(x), _ptr(scale), _ptr(bias), _ptr(y), rows, D, _DT[x.dtype], _DT[out_dtype],
                                    float(eps))
    else:
        st = lib.mrx_rms_norm_fwd(_stream(), _ptr(x), _ptr(scale), _ptr(y), rows, D, _DT[x.dtype], _DT[out_dtype], float(eps))
    _lib.check(st, "mrx_layer_norm_fwd" if center else "mrx_rms_norm_fwd")
    return y


def layer_norm_bwd(x, scale, dy, eps=1e-6, want_dparams=True, dx_add=None, center=True):
    """Gradients of layer_norm_fwd: (dx in x's dtype, dscale, dbias) -- the parameters' gradients (D) float32, or
    None when not wanted (dbias also None for the RMS norm).  dx_add (like x, or None): added to dx."""
    lib = _lib.load()
    D = x.shape[-1]
    _norm_dtypes(x.dtype, dy.dtype)
    _chk(x, "x")
    _chk(dy, "dy", None, x.shape)
    _chk(dx_add, "dx_add", x.dtype, x.shape)
    _chk(scale, "scale", torch.float32, (D,))
    dx = torch.empty_like(x)
    dscale = dbias = work = None
    if want_dparams:
        dscale = torch.empty((D,), dtype=torch.float32, device=x.device)
        dbias = torch.empty_like(dscale) if center else None
        work = torch.empty(((2 if center else 1) * RMS_NORM_PARTS, D), dtype=torch.float32, device=x.device)
    if x.numel() == 0:   # dx (and dx_add) are empty
        return dx, (None if dscale is None else dscale.zero_()), (None if dbias is None else dbias.zero_())
    rows = x.numel() // D
    if center:
        st = lib.mrx_layer_norm_bwd(_stream(), _ptr(x), _ptr(scale), _ptr(dy), _ptr(dx_add), _ptr(dx), _ptr(dscale), _ptr(dbias),
                                    _ptr(work), rows, D, _DT[x.dtype], _DT[dy.dtype], float(eps))
    else:
        st = lib.mrx_rms_norm_bwd(_stream(), _ptr(x), _ptr(scale), _ptr(dy), _ptr(dx_add), _ptr(dx), _ptr(dscale), _ptr(work),
                                  rows, D, _DT[x.dtype], _DT[dy.dtype], float(eps))
    _lib.check(st, "mrx_layer_norm_bwd" if center else "mrx_rms_norm_bwd")
    return dx, dscale, dbias


def silu_gate_fwd(h, g):
    """y = h * silu(g) (mrx_silu_gate_fwd): h, g of one shape and dtype, float32 or bfloat16."""
    lib = _lib.load()
    if h.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("silu_gate takes float32 or bfloat16 arrays")
    _chk(h, "h")
    _chk(g, "g", h.dtype, h.shape)
    y = torch.empty_like(h)
    if h.numel():
        _lib.check(lib.mrx_silu_gate_fwd(_stream(), _ptr(h), _ptr(g), _ptr(y), h.numel(), _DT[h.dtype]), "mrx_silu_gate_fwd")
    return y


def silu_gate_bwd(h, g, dy):
    """(dh, dg) of y = h * silu(g) for the gradient dy of y."""
    lib = _lib.load()
    if h.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("silu_gate takes float32 or bfloat16 arrays")
    _chk(h, "h")
    _chk(g, "g", h.dtype, h.shape)
    _chk(dy, "dy", h.dtype, h.shape)
    dh, dg = torch.empty_like(h), torch.empty_like(h)
    if h.numel():
        _lib.check(lib.mrx_silu_gate_bwd(_stream(), _ptr(h), _ptr(g), _ptr(dy), _ptr(dh), _ptr(dg), h.numel(), _DT[h.dtype]),
                   "mrx_silu_gate_bwd")
    return dh, dg


def linear_scan_last(a, b, done, h0=None):
    """Final state of h_t = done ? b_t : a_t h_{t-1} + b_t with one decay per group of channels:
    a: (B,T,D/group), b: (B,T,D), h0: (B,D) or None.  Returns h_last (B,D)."""
    lib = _lib.load()
    B, T, D = b.shape
    dt = b.dtype
    if dt not in (torch.float32, torch.complex64):
        raise ValueError("linear_scan_last supports float32 and complex64")
    if a.dim() != 3 or a.shape[:2] != (B, T) or D % a.shape[2] != 0:
        raise ValueError(f"a must be (B,T,D/group), got {tuple(a.shape)} for b {tuple(b.shape)}")
    _chk(a, "a", dt)
    _chk(b, "b", dt)
    _chk(h0, "h0", dt, (B, D))
    done, dd = _done(done, B, T)
    h_last = torch.empty((B, D), dtype=dt, device=b.device)
    st = lib.mrx_linear_scan_last(_stream(), _ptr(a), _ptr(b), _ptr(done), _ptr(h0), _ptr(h_last), B, T, D,
                                  D // a.shape[2], _DT[dt], dd)
    _lib.check(st, "mrx_linear_scan_last")
    return h_last


def linear_scan_bwd(a, h, done, h0, g, g_last=None, sum_da=False):
    """Returns (da (B,T,D) per step, db, dh0).  sum_da (time-invariant a only): da is (B,D), the per-step
    terms summed over the sequence inside the kernel."""
    lib = _lib.load()
    B, T, D = g.shape
    dt = g.dtype
    ct = torch.float32 if dt == torch.bfloat16 else dt  # the carries' type (and a summed da's)
    ti = a.dim() == 1
    _chk(a, "a", dt, (D,) if ti else (B, T, D))
    _chk(h, "h", dt, (B, T, D))
    _chk(g, "g", dt)
    _chk(h0, "h0", ct, (B, D))
    _chk(g_last, "g_last", ct, (B, D))
    done, dd = _done(done, B, T)
    if sum_da and not ti:
        raise ValueError("sum_da belongs to a time-invariant a")
    da = torch.empty((B, D), dtype=ct, device=g.device) if sum_da else torch.empty_like(g)
    db = torch.empty_like(g)
    dh0 = torch.empty((B, D), dtype=ct, device=g.device)
    st = lib.mrx_linear_scan_bwd(_stream(), _ptr(a), _ptr(h), _ptr(done), _ptr(h0), _ptr(g),
                                 _ptr(g_last), _ptr(da), _ptr(db), _ptr(dh0), B, T, D, _DT[dt],
                                 dd, _lib.MRX_A_TIME_INVARIANT_SUM_DA if sum_da else int(ti))
    _lib.check(st, "mrx_linear_scan_bwd")
    return da, db, dh0


def mingru_scan_fwd(z, h_tilde, done, h0=None, P0=None, want_P=True):
    """MinGRU recurrence from its two projections (min_gru.py:49-78, in linear space):
    h_t = done ? b_t : a_t h_{t-1} + b_t with a = sigmoid(-z), b = sigmoid(z) g(h~) formed inside
    the kernel.  z, h_tilde: (B,T,D) float32 or bfloat16 (float32 arithmetic); h0, P0: (B,D) float32,
    linear space.  Returns (h in the dtype of z, h_last, P_last)."""
    lib = _lib.load()
    B, T, D = z.shape
    if z.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("mingru_scan supports float32 and bfloat16")
    _chk(z, "z", z.dtype)
    _chk(h_tilde, "h_tilde", z.dtype, (B, T, D))
    _chk(h0, "h0", torch.float32, (B, D))
    _chk(P0, "P0", torch.float32, (B, D))
    done, dd = _done(done, B, T)
    h = torch.empty_like(z)
    h_last = torch.empty((B, D), dtype=torch.float32, device=z.device)
    P_last = torch.empty((B, D), dtype=torch.float32, device=z.device) if want_P else None
    st = lib.mrx_mingru_scan_fwd(_stream(), _ptr(z), _ptr(h_tilde), _ptr(done), _ptr(h0), _ptr(P0), _ptr(h),
                                 _ptr(h_last), _ptr(P_last), B, T, D, _DT[z.dtype], dd)
    _lib.check(st, "mrx_mingru_scan_fwd")
    return h, h_last, P_last


def mingru_scan_bwd(z, h_tilde, h, done, h0, g, g_last=None):
    """Returns (dz, dh_tilde, dh0) for the states h of mingru_scan_fwd and their gradients g."""
    lib = _lib.load()
    B, T, D = g.shape
    if g.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("mingru_scan supports float32 and bfloat16")
    for t_, n_ in ((z, "z"), (h_tilde, "h_tilde"), (h, "h"), (g, "g")):
        _chk(t_, n_, g.dtype, (B, T, D))
    _chk(h0, "h0", torch.float32, (B, D))
    _chk(g_last, "g_last", torch.float32, (B, D))
    done, dd = _done(done, B, T)
    dz, dx = torch.empty_like(g), torch.empty_like(g)
    dh0 = torch.empty((B, D), dtype=torch.float32, device=g.device)
    st = lib.mrx_mingru_scan_bwd(_stream(), _ptr(z), _ptr(h_tilde), _ptr(h), _ptr(done), _ptr(h0), _ptr(g),
                                 _ptr(g_last), _ptr(dz), _ptr(dx), _ptr(dh0), B, T, D, _DT[g.dtype], dd)
    _lib.check(st, "mrx_mingru_scan_bwd")
    return dz, dx, dh0


# ----------------------------------------------------------------- chunked attention
def _attn_shapes(q, k, v):
    B, T, H, dk = q.shape
    dv = v.shape[-1]
    dt = q.dtype
    if dt not in (torch.float32, torch.bfloat16):
        raise ValueError("chunked kernels support float32 and bfloat16")
    _chk(q, "q", dt)
    _chk(k, "k", dt, (B, T, H, dk))
    _chk(v, "v", dt, (B, T, H, dv))
    return B, T, H, dk, dv, dt


def _n_chunks(T, dt, delta=False):
    C = chunk_size(dt, delta)
    return (T + C - 1) // C


def linear_attn_chunk_parallel_pays(B, T, H, dtype):
    """The library's rule: cut the work along time (one workgroup per chunk) instead of along sequences."""
    return bool(_lib.load().mrx_linear_attn_chunk_parallel_pays(B, T, H, _DT[dtype]))


def linear_attn_fwd(q, k, v, done, S0=None, feature_map=0, save_chk=True, chunk_parallel=None):
    """Returns (o, S_last fp32, chk) with chk = (S_chk, S_last), what the backward call needs, or None.
    Sequential form (one workgroup per sequence): S_chk is float32 and sparse -- the library writes only
    the slots of chunks that contain a reset (the backward call walks the state back from S_last through
    the others).  Chunk-parallel form (chunk_parallel=True, or None and the library's rule prefers it:
    few sequences, several chunks each): S_chk is dense and chk = (S_chk, None); linear_attn_bwd takes
    either."""
    lib = _lib.load()
    B, T, H, dk, dv, dt = _attn_shapes(q, k, v)
    _chk(S0, "S0", torch.float32, (B, H, dv, dk))
    done, dd = _done(done, B, T)
    if chunk_parallel is None:
        chunk_parallel = linear_attn_chunk_parallel_pays(B, T, H, dt)
    o = torch.empty_like(v)
    S_last = torch.empty((B, H, dv, dk), dtype=torch.float32, device=q.device)
    S_chk = (torch.empty((B, H, _n_chunks(T, dt), dv, dk), dtype=torch.float32, device=q.device)
             if save_chk or chunk_parallel else None)
    if chunk_parallel:
        st = lib.mrx_linear_attn_fwd_chunk_parallel(_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(done), _ptr(S0),
                                                    _ptr(o), _ptr(S_last), _ptr(S_chk), B, T, H, dk, dv, _DT[dt],
                                                    dd, int(feature_map))
        _lib.check(st, "mrx_linear_attn_fwd_chunk_parallel")
        return o, S_last, ((S_chk, None) if save_chk else None)
    st = lib.mrx_linear_attn_fwd(_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(done), _ptr(S0),
                                 _ptr(o), _ptr(S_last), _ptr(S_chk), B, T, H, dk, dv, _DT[dt], dd,
                                 int(feature_map))
    _lib.check(st, "mrx_linear_attn_fwd")
    return o, S_last, ((S_chk, S_last) if save_chk else None)


def linear_attn_bwd(q, k, v, done, chk, do, dS_last=None, feature_map=0, want_dS0=True):
    """chk = (S_chk, S_last) from linear_attn_fwd (S_last None: the chunk-parallel pair).
    Returns (dq, dk, dv, dS0)."""
    lib = _lib.load()
    B, T, H, dk, dv, dt = _attn_shapes(q, k, v)
    S_chk, S_last = chk
    _chk(do, "do", dt, (B, T, H, dv))
    _chk(S_chk, "S_chk", torch.float32, (B, H, _n_chunks(T, dt), dv, dk))
    _chk(S_last, "S_last", torch.float32, (B, H, dv, dk))
    _chk(dS_last, "dS_last", torch.float32, (B, H, dv, dk))
    done, dd = _done(done, B, T)
    dq, dk_, dv_ = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dS0 = (torch.empty((B, H, dv, dk), dtype=torch.float32, device=q.device)
           if want_dS0 else None)
    if S_last is None:
        ws = torch.empty_like(S_chk)
        st = lib.mrx_linear_attn_bwd_chunk_parallel(_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(done), _ptr(S_chk),
                                                    _ptr(do), _ptr(dS_last), _ptr(dq), _ptr(dk_), _ptr(dv_),
                                                    _ptr(dS0), _ptr(ws), B, T, H, dk, dv, _DT[dt], dd,
                                                    int(feature_map))
        _lib.check(st, "mrx_linear_attn_bwd_chunk_parallel")
        return dq, dk_, dv_, dS0
    st = lib.mrx_linear_attn_bwd(_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(done), _ptr(S_chk), _ptr(S_last),
                                 _ptr(do), _ptr(dS_last), _ptr(dq), _ptr(dk_), _ptr(dv_),
                                 _ptr(dS0), B, T, H, dk, dv, _DT[dt], dd, int(feature_map))
    _lib.check(st, "mrx_linear_attn_bwd")
    return dq, dk_, dv_, dS0


def linear_attn_norm_fwd(q, k, v, done, S0=None, z0=None, feature_map=0, eps=1e-6, save_chk=True, want_ss=False):
    """Linear attention with the normalised read-out fused.
    Returns (o, den fp32 (B,H,T), S_last fp32, z_last fp32, (S_chk, z_chk, S_last) or None); S_chk as for
    linear_attn_fwd.  want_ss: a sixth result, ss fp32 (B,H,T), the per-head sums of squares of the
    outputs (what an RMS norm over the heads needs from each of them)."""
    lib = _lib.load()
    B, T, H, dk, dv, dt = _attn_shapes(q, k, v)
    _chk(S0, "S0", torch.float32, (B, H, dv, dk))
    _chk(z0, "z0", torch.float32, (B, H, dk))
    done, dd = _done(done, B, T)
    o = torch.empty_like(v)
    den = torch.empty((B, H, T), dtype=torch.float32, device=q.device)
    S_last = torch.empty((B, H, dv, dk), dtype=torch.float32, device=q.device)
    z_last = torch.empty((B, H, dk), dtype=torch.float32, device=q.device)
    nc = _n_chunks(T, dt)
    S_chk = torch.empty((B, H, nc, dv, dk), dtype=torch.float32, device=q.device) if save_chk else None
    z_chk = torch.empty((B, H, nc, dk), dtype=torch.float32, device=q.device) if save_chk else None
    ss = torch.empty((B, H, T), dtype=torch.float32, device=q.device) if want_ss else None
    st = lib.mrx_linear_attn_norm_fwd(_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(done), _ptr(S0), _ptr(z0),
                                      _ptr(o), _ptr(den), _ptr(ss), _ptr(S_last), _ptr(z_last), _ptr(S_chk), _ptr(z_chk),
                                      B, T, H, dk, dv, _DT[dt], dd, int(feature_map), float(eps))
    _lib.check(st, "mrx_linear_attn_norm_fwd")
    chk = (S_chk, z_chk, S_last) if save_chk else None
    return (o, den, S_last, z_last, chk, ss) if want_ss else (o, den, S_last, z_last, chk)


def linear_attn_norm_bwd(q, k, v, done, chk, o, den, do, dS_last=None, dz_last=None, feature_map=0, eps=1e-6,
                         want_d0=True, d_ss=None):
    """Returns (dq, dk, dv, dS0, dz0).  d_ss: gradient of the forward call's ss, fp32 (B,H,T)."""
    lib = _lib.load()
    B, T, H, dk, dv, dt = _attn_shapes(q, k, v)
    S_chk, z_chk, S_last = chk
    nc = _n_chunks(T, dt)
    _chk(S_last, "S_last", torch.float32, (B, H, dv, dk))
    _chk(do, "do", dt, (B, T, H, dv))
    _chk(o, "o", dt, (B, T, H, dv))
    _chk(den, "den", torch.float32, (B, H, T))
    _chk(S_chk, "S_chk", torch.float32, (B, H, nc, dv, dk))
    _chk(z_chk, "z_chk", torch.float32, (B, H, nc, dk))
    _chk(dS_last, "dS_last", torch.float32, (B, H, dv, dk))
    _chk(dz_last, "dz_last", torch.float32, (B, H, dk))
    _chk(d_ss, "d_ss", torch.float32, (B, H, T))
    done, dd = _done(done, B, T)
    dq, dk_, dv_ = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dS0 = torch.empty((B, H, dv, dk), dtype=torch.float32, device=q.device) if want_d0 else None
    dz0 = torch.empty((B, H, dk), dtype=torch.float32, device=q.device) if want_d0 else None
    st = lib.mrx_linear_attn_norm_bwd(_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(done), _ptr(S_chk), _ptr(S_last), _ptr(z_chk),
                                      _ptr(o), _ptr(den), _ptr(do), _ptr(d_ss), _ptr(dS_last), _ptr(dz_last), _ptr(dq),
                                      _ptr(dk_), _ptr(dv_), _ptr(dS0), _ptr(dz0), B, T, H, dk, dv, _DT[dt], dd,
                                      int(feature_map), float(eps))
    _lib.check(st, "mrx_linear_attn_norm_bwd")
    return dq, dk_, dv_, dS0, dz0


_FACTORS = {None: _lib.MRX_FACTORS_AUTO, "auto": _lib.MRX_FACTORS_AUTO, "parallel": _lib.MRX_FACTORS_PARALLEL,
            "inline": _lib.MRX_FACTORS_INLINE}
_RESETS = {None: _lib.MRX_RESETS_AUTO, "auto": _lib.MRX_RESETS_AUTO, "passes": _lib.MRX_RESETS_PASSES,
           "merged": _lib.MRX_RESETS_MERGED}


def init(device=None):
    """Per-device set-up of the library (mrx_init): optional, the first launch on a device does
    the same, but it must precede a HIP-graph capture that holds the first call on that device."""
    lib = _lib.load()
    dev = torch.cuda.current_device() if device is None else int(device)
    _lib.check(lib.mrx_init(dev), "mrx_init")


def delta_rule_fwd_noalloc(q, k, v, beta, done, S0=None, out=None):
    """mrx_delta_rule_fwd_noalloc: forward without residuals, the triangular factors in the
    library's static scratch array (nothing is allocated by the library; this wrapper allocates
    o and S_last unless out = (o, S_last) is given).  Returns (o, S_last)."""
    lib = _lib.load()
    B, T, H, dk, dv, dt = _attn_shapes(q, k, v)
    _chk(beta, "beta", dt, (B, T, H))
    _chk(S0, "S0", torch.float32, (B, H, dv, dk))
    done, dd = _done(done, B, T)
    if out is not None:
        o, S_last = out
        _chk(o, "out o", dt, (B, T, H, dv))
        _chk(S_last, "out S_last", torch.float32, (B, H, dv, dk))
    else:
        o = torch.empty_like(v)
        S_last = torch.empty((B, H, dv, dk), dtype=torch.float32, device=q.device)
    st = lib.mrx_delta_rule_fwd_noalloc(_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(beta), _ptr(done), _ptr(S0),
                                        _ptr(o), _ptr(S_last), B, T, H, dk, dv, _DT[dt], dd)
    _lib.check(st, "mrx_delta_rule_fwd_noalloc")
    return o, S_last


def delta_rule_fwd(q, k, v, beta, done, S0=None, save_chk=True, out=None, prologue=False, tm_scratch=None,
                   factor_path=None, reset_path=None):
    """Returns (o, S_last fp32, chk) where chk = (S_chk, Tm_chk) are the residuals the
    backward call needs, or None.  out = (o, S_last, S_chk, Tm_chk) reuses buffers of an earlier
    call with the same shapes instead of allocating.  prologue=True: k is L2-normalised and
    beta = sigmoid(beta) inside the kernel (mrx_deltanet_fwd).
    tm_scratch (only without residuals): give the library a buffer for the triangular factors
    anyway, which lets it compute them chunk-parallel.  None: when the library would use it (float32;
    bf16 with B*H at most two sequences per compute unit).
    factor_path: None / "auto" (by occupancy), "parallel" or "inline" (mrx_factor_path).
    reset_path: None / "auto", "passes" (one unit of work per episode of a chunk) or "merged" (one per chunk
    behind a screen of its inputs: mrx_reset_path); the backward call takes the same argument."""
    lib = _lib.load()
    B, T, H, dk, dv, dt = _attn_shapes(q, k, v)
    _chk(beta, "beta", dt, (B, T, H))
    _chk(S0, "S0", torch.float32, (B, H, dv, dk))
    done, dd = _done(done, B, T)
    if out is not None:
        o, S_last, S_chk, Tm_chk = out
        C, NC = chunk_size(dt, True), _n_chunks(T, dt, True)
        _chk(o, "out o", dt, (B, T, H, dv))
        _chk(S_last, "out S_last", torch.float32, (B, H, dv, dk))
        _chk(S_chk, "out S_chk", dt, (B, H, NC, dv, dk))
        _chk(Tm_chk, "out Tm_chk", dt, (B, H, NC, C, C))
        save_chk = S_chk is not None
    else:
        o = torch.empty_like(v)
        S_last = torch.empty((B, H, dv, dk), dtype=torch.float32, device=q.device)
        S_chk = Tm_chk = None
        if save_chk:
            C, NC = chunk_size(dt, True), _n_chunks(T, dt, True)
            S_chk = torch.empty((B, H, NC, dv, dk), dtype=dt, device=q.device)
            Tm_chk = torch.empty((B, H, NC, C, C), dtype=dt, device=q.device)
        else:
            if tm_scratch is None:
                tm_scratch = (dt == torch.float32 or
                              B * H <= 2 * torch.cuda.get_device_properties(q.device).multi_processor_count)
            if tm_scratch:
                C, NC = chunk_size(dt, True), _n_chunks(T, dt, True)
                Tm_chk = torch.empty((B, H, NC, C, C), dtype=dt, device=q.device)
    name = "mrx_deltanet_fwd" if prologue else "mrx_delta_rule_fwd"
    st = getattr(lib, name)(_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(beta), _ptr(done),
                            _ptr(S0), _ptr(o), _ptr(S_last), _ptr(S_chk), _ptr(Tm_chk), B, T, H,
                            dk, dv, _DT[dt], dd, _FACTORS[factor_path], _RESETS[reset_path])
    _lib.check(st, name)
    return o, S_last, ((S_chk, Tm_chk) if save_chk else None)


def delta_rule_bwd(q, k, v, beta, done, chk, do, dS_last=None, want_dS0=True, out=None, prologue=False,
                   reset_path=None):
    """chk = (S_chk, Tm_chk) from delta_rule_fwd.  Returns (dq, dk, dv, dbeta, dS0).
    out = (dq, dk, dv, dbeta, dS0) reuses buffers instead of allocating.  prologue=True pairs with
    delta_rule_fwd(prologue=True): k and beta are the raw projections and so are dk and dbeta."""
    lib = _lib.load()
    B, T, H, dk, dv, dt = _attn_shapes(q, k, v)
    S_chk, Tm_chk = chk
    C = chunk_size(dt, True)
    _chk(Tm_chk, "Tm_chk", dt, (B, H, _n_chunks(T, dt, True), C, C))
    _chk(beta, "beta", dt, (B, T, H))
    _chk(do, "do", dt, (B, T, H, dv))
    _chk(S_chk, "S_chk", dt, (B, H, _n_chunks(T, dt, True), dv, dk))
    _chk(dS_last, "dS_last", torch.float32, (B, H, dv, dk))
    done, dd = _done(done, B, T)
    if out is not None:
        dq, dk_, dv_, dbeta, dS0 = out
        for t_, n_, ref in ((dq, "out dq", q), (dk_, "out dk", k), (dv_, "out dv", v), (dbeta, "out dbeta", beta)):
            _chk(t_, n_, dt, tuple(ref.shape))
        _chk(dS0, "out dS0", torch.float32, (B, H, dv, dk))
    else:
        dq, dk_, dv_ = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        dbeta = torch.empty_like(beta)
        dS0 = (torch.empty((B, H, dv, dk), dtype=torch.float32, device=q.device)
               if want_dS0 else None)
    name = "mrx_deltanet_bwd" if prologue else "mrx_delta_rule_bwd"
    st = getattr(lib, name)(_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(beta), _ptr(done),
                            _ptr(S_chk), _ptr(Tm_chk), _ptr(do), _ptr(dS_last), _ptr(dq), _ptr(dk_),
                            _ptr(dv_), _ptr(dbeta), _ptr(dS0), B, T, H, dk, dv, _DT[dt], dd, _RESETS[reset_path])
    _lib.check(st, name)
    return dq, dk_, dv_, dbeta, dS0


# ---------------------------------------------------- gated linear attention
def gated_linear_attn_fwd(q, k, v, g, done, S0=None, feature_map=0, save_chk=True):
    """g: (B,T,H) float32 log-decay.  Returns (o, S_last fp32, S_chk or None)."""
    lib = _lib.load()
    B, T, H, dk, dv, dt = _attn_shapes(q, k, v)
    _chk(g, "g", torch.float32, (B, T, H))
    _chk(S0, "S0", torch.float32, (B, H, dv, dk))
    done, dd = _done(done, B, T)
    o = torch.empty_like(v)
    S_last = torch.empty((B, H, dv, dk), dtype=torch.float32, device=q.device)
    S_chk = (torch.empty((B, H, _n_chunks(T, dt), dv, dk), dtype=dt, device=q.device)
             if save_chk else None)
    st = lib.mrx_gated_linear_attn_fwd(_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(g), _ptr(done), _ptr(S0),
                                       _ptr(o), _ptr(S_last), _ptr(S_chk), B, T, H, dk, dv, _DT[dt], dd,
                                       int(feature_map))
    _lib.check(st, "mrx_gated_linear_attn_fwd")
    return o, S_last, S_chk


def gated_linear_attn_bwd(q, k, v, g, done, S_chk, do, dS_last=None, feature_map=0, want_dS0=True,
                          S_last=None):
    """Returns (dq, dk, dv, dg, dS0).  S_last (the forward call's) is needed when dS_last is given: its
    inner product with dS_last enters dg at the last step."""
    lib = _lib.load()
    B, T, H, dk, dv, dt = _attn_shapes(q, k, v)
    _chk(g, "g", torch.float32, (B, T, H))
    _chk(do, "do", dt, (B, T, H, dv))
    _chk(S_chk, "S_chk", dt, (B, H, _n_chunks(T, dt), dv, dk))
    _chk(dS_last, "dS_last", torch.float32, (B, H, dv, dk))
    _chk(S_last, "S_last", torch.float32, (B, H, dv, dk))
    if dS_last is not None and S_last is None:
        raise ValueError("S_last is required with dS_last")
    done_u, dd = _done(done, B, T)
    dq, dk_, dv_ = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dg = torch.empty((B, T, H), dtype=torch.float32, device=q.device)
    dS0 = (torch.empty((B, H, dv, dk), dtype=torch.float32, device=q.device) if want_dS0 else None)
    st = lib.mrx_gated_linear_attn_bwd(_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(g), _ptr(done_u), _ptr(S_chk),
                                       _ptr(S_last), _ptr(do), _ptr(dS_last), _ptr(dq), _ptr(dk_), _ptr(dv_),
                                       _ptr(dg), _ptr(dS0), B, T, H, dk, dv, _DT[dt], dd, int(feature_map))
    _lib.check(st, "mrx_gated_linear_attn_bwd")
    return dq, dk_, dv_, dg, dS0


# ------------------------------------------------------------- single time step
def _step_shapes(q, k, v):
    if q.dim() != 3:
        raise ValueError(f"q must be (B,H,d), got {tuple(q.shape)}")
    B, H, dk = q.shape
    dv = v.shape[-1]
    dt = q.dtype
    if dt not in (torch.float32, torch.bfloat16):
        raise ValueError(f"unsupported dtype {dt}")
    _chk(q, "q", dt, (B, H, dk))
    _chk(k, "k", dt, (B, H, dk))
    _chk(v, "v", dt, (B, H, dv))
    return B, H, dk, dv, dt


def linear_attn_step(q, k, v, done, S=None, z=None, feature_map="none", normalise=False, eps=1e-6,
                     inplace=False):
    """One time step.  q,k,v: (B,H,d); done: (B,); S: (B,H,dv,dk) fp32 or None; z: (B,H,dk) fp32 or
    None.  Returns (o, S_new, z_new) (z_new None unless normalise).  inplace updates S and z."""
    lib = _lib.load()
    B, H, dk, dv, dt = _step_shapes(q, k, v)
    _chk(S, "S", torch.float32, (B, H, dv, dk))
    _chk(z, "z", torch.float32, (B, H, dk))
    done, dd = _done(done.reshape(B, 1), B, 1)
    o = torch.empty_like(v)
    S_new = S if (inplace and S is not None) else torch.empty((B, H, dv, dk), dtype=torch.float32, device=q.device)
    z_new = None
    if normalise:
        z_new = z if (inplace and z is not None) else torch.empty((B, H, dk), dtype=torch.float32, device=q.device)
    fm = {"none": _lib.MRX_FMAP_NONE, "elu1": _lib.MRX_FMAP_ELU1}[feature_map]
    st = lib.mrx_linear_attn_step(_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(done), _ptr(S),
                                  _ptr(z) if normalise else None, _ptr(o), _ptr(S_new), _ptr(z_new),
                                  B, H, dk, dv, _DT[dt], dd, fm, float(eps))
    _lib.check(st, "mrx_linear_attn_step")
    return o, S_new, z_new


def gated_linear_attn_step(q, k, v, g, done, S=None, feature_map="none", inplace=False):
    """One time step of gated linear attention.  q,k: (B,H,dk); v: (B,H,dv); g: (B,H) fp32 log-decay;
    done: (B,); S: (B,H,dv,dk) fp32 or None.  Returns (o, S_new).  inplace updates S."""
    lib = _lib.load()
    B, H, dk, dv, dt = _step_shapes(q, k, v)
    _chk(g, "g", torch.float32, (B, H))
    _chk(S, "S", torch.float32, (B, H, dv, dk))
    done, dd = _done(done.reshape(B, 1), B, 1)
    o = torch.empty_like(v)
    S_new = S if (inplace and S is not None) else torch.empty((B, H, dv, dk), dtype=torch.float32, device=q.device)
    fm = {"none": _lib.MRX_FMAP_NONE, "elu1": _lib.MRX_FMAP_ELU1}[feature_map]
    st = lib.mrx_gated_linear_attn_step(_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(g), _ptr(done), _ptr(S), _ptr(o),
                                        _ptr(S_new), B, H, dk, dv, _DT[dt], dd, fm)
    _lib.check(st, "mrx_gated_linear_attn_step")
    return o, S_new


def delta_rule_step(q, k, v, beta, done, S=None, inplace=False):
    """One time step of the delta rule.  beta: (B,H).  Returns (o, S_new)."""
    lib = _lib.load()
    B, H, dk, dv, dt = _step_shapes(q, k, v)
    _chk(beta, "beta", dt, (B, H))
    _chk(S, "S", torch.float32, (B, H, dv, dk))
    done, dd = _done(done.reshape(B, 1), B, 1)
    o = torch.empty_like(v)
    S_new = S if (inplace and S is not None) else torch.empty((B, H, dv, dk), dtype=torch.float32, device=q.device)
    st = lib.mrx_delta_rule_step(_stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(beta), _ptr(done), _ptr(S),
                                 _ptr(o), _ptr(S_new), B, H, dk, dv, _DT[dt], dd)
    _lib.check(st, "mrx_delta_rule_step")
    return o, S_new
