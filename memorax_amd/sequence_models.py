"""Host-side mirror of memorax's sequence-model interface, on top of the HIP kernels.

Same contract as the reference (memorax/networks/sequence_models):

    SequenceModel.__call__(inputs (B,T,F), done (B,T), initial_carry=None) -> (next_carry, y)
    SequenceModel.initialize_carry(key, input_shape=(B,F)) -> carry          sequence_model.py:8-19
    MemoroidCellBase: __call__(x) -> elements, binary_operator(a, b), read(h, x),
                      initialize_carry(key, input_shape)                      memoroid.py:20-33
    Memoroid(cell)(inputs, done, initial_carry) = read(scan(cell(inputs)))    memoroid.py:93-109

Carries keep the reference's pytree shapes (leaves with a size-1 time axis, (B,1,...)),
so Stack-style per-block carry tuples and checkpointing keep working.

What differs: the reference scans *any* cell algebra with jax.lax.associative_scan
(memoroid.py:60-91).  Here each cell also implements ``scan(elements, carry, done)``,
which hands its algebra to the matching fused kernel (diagonal scan, chunked linear
attention, chunked delta rule) instead of materialising per-step states;
``binary_operator`` remains the definition of the algebra (and is what the tests fold
to check ``scan``).  Modules are torch.nn.Modules: torch plays the role of the array
library / autodiff host here, the arithmetic of the recurrences runs in the kernels.
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from typing import NamedTuple

from .dense import Dense, autocast_dtype, dense_group
from .functional import (deltanet, gated_linear_attention, linear_attention, linear_scan, mingru_scan, mlstm_gates,
                         normalised_linear_attention, layer_norm, layer_norm_fork, rms_norm, rms_norm_fork, silu_gate)
from .kernels import RMS_NORM_MAX_D as _RMS_NORM_MAX_D


# ----------------------------------------------------------------------------------
# axes helpers (memorax/utils/axes.py:19-32,46-49)
# ----------------------------------------------------------------------------------
def add_time_axis(x):
    return x[:, None]


def remove_time_axis(x):
    return x.squeeze(1)


def get_input_shape(inputs):
    """(B, T, F) -> (B, F)."""
    return inputs.shape[:1] + inputs.shape[2:]


class SequenceModel(nn.Module):
    """sequence_model.py:8-19."""

    def forward(self, inputs, done, initial_carry=None, **kwargs):  # pragma: no cover
        raise NotImplementedError

    def initialize_carry(self, key, input_shape):  # pragma: no cover
        raise NotImplementedError


class MemoroidCellBase(nn.Module):
    """memoroid.py:20-33 plus the kernel hook ``scan``."""

    def forward(self, x, **kwargs):  # elements
        raise NotImplementedError

    def binary_operator(self, a, b):
        raise NotImplementedError

    def read(self, h, x, **kwargs):
        raise NotImplementedError

    def initialize_carry(self, key, input_shape):
        raise NotImplementedError

    def scan(self, z, initial_carry, done):
        """Reset-aware inclusive scan of the cell's algebra over time, carry-in
        prepended (memoroid.py:60-91).  Returns (h, next_carry).

        The cells of this module override it with a fused kernel.  This default serves any other
        cell that only defines ``binary_operator``: the same scan with array operations, on whatever
        device the elements live on (``generic_scan``)."""
        return generic_scan(self.binary_operator, z, initial_carry, done)


def _tree_map(fn, tree, *rest):
    """fn over the leaves of nested tuples / lists / dicts (named tuples keep their type)."""
    if isinstance(tree, dict):
        return {k: _tree_map(fn, v, *(r[k] for r in rest)) for k, v in tree.items()}
    if isinstance(tree, (tuple, list)):
        out = [_tree_map(fn, v, *(r[i] for r in rest)) for i, v in enumerate(tree)]
        return type(tree)(*out) if hasattr(tree, "_fields") else type(tree)(out)
    return fn(tree, *rest)


def broadcast_done(done, carry):
    """utils/axes.py:64-68: trailing axes added to (or dropped from) done until its rank is the leaf's."""
    while done.dim() != carry.dim():
        done = done[..., None] if done.dim() < carry.dim() else done[..., 0]
    return done


def generic_scan(binary_operator, z, initial_carry, done):
    """Memoroid.scan_fn (memoroid.py:60-91) for an arbitrary pytree algebra.

    The carry becomes slot 0 of every leaf with reset flag 0; slots are combined with the augmented
    operator ``(where(reset_b, b, a (+) b), max(reset_a, reset_b))`` -- the right element wins by
    *select* when its reset flag is set -- and the result is split into the T prefixes and the last
    one (time axis of size 1).  Instead of jax.lax.associative_scan's odd/even recursion the slots
    are combined by doubling: ceil(log2(T + 1)) rounds, each one call of ``binary_operator`` on leaves
    of shape (B, n, ...) (n slots at once; the reference maps the operator over B, so it sees
    (n, ...)); there is no host loop over time steps, and autograd differentiates through it.
    Leaves are (B, T, ...); ``done`` is (B, T), bool or float."""
    zz = _tree_map(lambda c, e: torch.cat([c, e], dim=1), initial_carry, z)
    first = zz
    while isinstance(first, (tuple, list, dict)):
        first = next(iter(first.values())) if isinstance(first, dict) else first[0]
    reset = torch.cat([done.new_zeros((done.shape[0], 1), dtype=torch.bool), done != 0], dim=1)[..., None]
    n, shift = first.shape[1], 1
    while shift < n:
        left = _tree_map(lambda x: x[:, :-shift], zz)
        right = _tree_map(lambda x: x[:, shift:], zz)
        rr = reset[:, shift:]
        comb = binary_operator(left, right)
        comb = _tree_map(lambda r, c: torch.where(broadcast_done(rr, r), r, c), right, comb)
        zz = _tree_map(lambda x, c: torch.cat([x[:, :shift], c], dim=1), zz, comb)
        reset = torch.cat([reset[:, :shift], reset[:, :-shift] | rr], dim=1)
        shift *= 2
    return _tree_map(lambda x: x[:, 1:], zz), _tree_map(lambda x: x[:, -1:], zz)


class Memoroid(SequenceModel):
    """memoroid.py:57-112 (without the RTRL hooks).  The cells of this module scan with their fused
    kernels: the matrix-state cells (linear attention, Mamba, mLSTM) put the query among their elements,
    because their kernels fuse the read-out contraction into the scan, so that ``scan`` returns the
    carry like any other cell's.  Any other MemoroidCellBase -- a user's cell that defines only
    ``binary_operator`` -- is scanned by the base class's generic ``scan``, as the reference scans
    every cell."""

    def __init__(self, cell: MemoroidCellBase):
        super().__init__()
        self.cell = cell

    def forward(self, inputs, done, initial_carry=None, **kwargs):
        if initial_carry is None:
            initial_carry = self.cell.initialize_carry(None, get_input_shape(inputs))
        z = self.cell(inputs, **kwargs)
        h, next_carry = self.cell.scan(z, initial_carry, done)
        y = self.cell.read(h, inputs, **kwargs)
        return next_carry, y

    def initialize_carry(self, key, input_shape):
        return self.cell.initialize_carry(key, input_shape)


# ----------------------------------------------------------------------------------
# diagonal algebra cells
# ----------------------------------------------------------------------------------
class _DiagonalCell(MemoroidCellBase):
    """Cells whose elements are (state, decay) with
    binary_operator(a, b) = (decay_b * state_a + state_b, decay_b * decay_a)
    (lru.py:92-95, s5.py:133-136).  ``scan`` returns h = (states (B,T,N), None): the
    per-step cumulative decay is never materialised, only its last value (the carry)."""

    def binary_operator(self, a, b):
        state_i, decay_i = a
        state_j, decay_j = b
        return (decay_j * state_i + state_j, decay_j * decay_i)

    def scan(self, z, initial_carry, done):
        state, decay = z            # decay: (B,T,N) or time-invariant (N,)
        h0, P0 = initial_carry      # (B,1,N)
        h, h_last, P_last = linear_scan(decay, state, done, h0[:, 0].contiguous(), P0[:, 0].contiguous())
        return (h, None), (h_last[:, None], P_last[:, None])


class LRUCell(_DiagonalCell):
    """Linear Recurrent Unit, complex diagonal recurrence (lru.py:32-108).  The decay
    lambda is time-invariant and is passed to the kernel as an (N,) vector instead of
    being broadcast to (B,T,N) (lru.py:86)."""

    def __init__(self, features, hidden_dim, r_min=0.0, r_max=1.0, max_phase=6.28):
        super().__init__()
        self.features, self.hidden_dim = features, hidden_dim
        u1, u2 = torch.rand(hidden_dim), torch.rand(hidden_dim)
        nu_log = torch.log(-0.5 * torch.log(u1 * (r_max**2 - r_min**2) + r_min**2))   # lru.py:12-14
        theta_log = torch.log(max_phase * u2)                                          # lru.py:17-19
        lam = torch.exp(-torch.exp(nu_log) + 1j * torch.exp(theta_log))
        self.nu_log = nn.Parameter(nu_log)
        self.theta_log = nn.Parameter(theta_log)
        self.gamma_log = nn.Parameter(torch.log(torch.sqrt(1 - torch.abs(lam) ** 2)))  # lru.py:22-25
        self.B_real = nn.Parameter(torch.randn(hidden_dim, features) / math.sqrt(2 * features))
        self.B_imag = nn.Parameter(torch.randn(hidden_dim, features) / math.sqrt(2 * features))
        self.C_real = nn.Parameter(torch.randn(features, hidden_dim) / math.sqrt(hidden_dim))
        self.C_imag = nn.Parameter(torch.randn(features, hidden_dim) / math.sqrt(hidden_dim))
        self.D = nn.Parameter(torch.randn(features))

    def forward(self, x, **kwargs):
        lam = torch.exp(torch.complex(-torch.exp(self.nu_log), torch.exp(self.theta_log)))
        B_norm = torch.complex(self.B_real, self.B_imag) * torch.exp(self.gamma_log)[:, None]
        state = x.to(torch.complex64) @ B_norm.T
        return (state.contiguous(), lam.to(torch.complex64))

    def read(self, h, x, **kwargs):
        state, _ = h
        C = torch.complex(self.C_real, self.C_imag)
        return (state @ C.T).real + self.D * x

    def initialize_carry(self, key, input_shape):
        *batch, _ = input_shape
        dev = self.nu_log.device
        return (torch.zeros(*batch, 1, self.hidden_dim, dtype=torch.complex64, device=dev),
                torch.ones(*batch, 1, self.hidden_dim, dtype=torch.complex64, device=dev))


def _dplr_hippo(n):
    """Eigenvalues and eigenvectors of the normal part of the HiPPO-LegS matrix
    (networks/hippo.py:6-37), in float64 NumPy."""
    import numpy as np
    p = np.sqrt(1.0 + 2.0 * np.arange(n))
    a = -(np.tril(p[:, None] * p[None, :]) - np.diag(np.arange(n)))
    pl = np.sqrt(np.arange(n) + 0.5)
    sm = a + pl[:, None] * pl[None, :]
    lam_real = np.full(n, np.mean(np.diag(sm)))
    lam_imag, v = np.linalg.eigh(sm * (-1j))
    return lam_real + 1j * lam_imag, v


class S5Cell(_DiagonalCell):
    """S5: diagonal state space model with HiPPO-N initialised eigenvalues, discretised with a
    learned per-state step (s5.py:28-149).  As for the LRU the discretised decay is time-invariant
    and goes to the kernel as an (N,) vector instead of being broadcast (s5.py:127)."""

    def __init__(self, features, state_size, discretization="zoh", dt_min=0.001, dt_max=0.1,
                 clip_eigens=False, step_rescale=1.0):
        super().__init__()
        import numpy as np
        self.features, self.state_size = features, state_size
        self.discretization, self.clip_eigens, self.step_rescale = discretization, clip_eigens, step_rescale
        lam, v = _dplr_hippo(state_size)
        v_inv = torch.from_numpy(v.conj().T.copy())
        vt = torch.from_numpy(v.copy())
        self.lambda_real = nn.Parameter(torch.from_numpy(lam.real.copy()).float())
        self.lambda_imag = nn.Parameter(torch.from_numpy(lam.imag.copy()).float())
        b = (v_inv @ (torch.randn(state_size, features, dtype=torch.float64) / math.sqrt(features)).to(v_inv.dtype))
        c = (torch.randn(features, state_size, dtype=torch.float64).clamp(-2, 2).to(vt.dtype) @ vt)
        self.B = nn.Parameter(torch.stack([b.real, b.imag], -1).float())     # (N, F, 2)
        self.C = nn.Parameter(torch.stack([c.real, c.imag], -1).float())     # (F, N, 2)
        self.d = nn.Parameter(torch.randn(features))
        self.log_step = nn.Parameter(torch.rand(state_size, 1) * (math.log(dt_max) - math.log(dt_min)) + math.log(dt_min))

    def _discretized_params(self):
        lr = torch.clamp(self.lambda_real, max=-1e-4) if self.clip_eigens else self.lambda_real
        lam = torch.complex(lr, self.lambda_imag)
        b_tilde = torch.complex(self.B[..., 0], self.B[..., 1])
        c_tilde = torch.complex(self.C[..., 0], self.C[..., 1])
        step = (self.step_rescale * torch.exp(self.log_step[:, 0])).to(torch.complex64)
        if self.discretization == "zoh":          # hippo.py:51-57
            lambda_bar = torch.exp(lam * step)
            b_bar = ((lambda_bar - 1.0) / lam)[:, None] * b_tilde
        elif self.discretization == "bilinear":   # hippo.py:40-48
            bl = 1.0 / (1.0 - (step / 2.0) * lam)
            lambda_bar = bl * (1.0 + (step / 2.0) * lam)
            b_bar = (bl * step)[:, None] * b_tilde
        else:
            raise ValueError(f"Invalid discretization: {self.discretization}")
        return lambda_bar, b_bar, c_tilde

    def forward(self, x, **kwargs):
        lambda_bar, b_bar, _ = self._discretized_params()
        state = x.to(torch.complex64) @ b_bar.T
        return (state.contiguous(), lambda_bar.to(torch.complex64))

    def read(self, h, x, **kwargs):
        _, _, c_tilde = self._discretized_params()
        state, _ = h
        return (state @ c_tilde.T).real + self.d * x

    def initialize_carry(self, key, input_shape):
        *batch, _ = input_shape
        dev = self.d.device
        return (torch.zeros(*batch, 1, self.state_size, dtype=torch.complex64, device=dev),
                torch.ones(*batch, 1, self.state_size, dtype=torch.complex64, device=dev))


class _SownValues(dict):
    """What the reference records with flax's ``sow`` (min_gru.py:63): the value is formed when it is read,
    not when it is recorded -- a mean over a (B,T,F) array is a pass over memory that a training step never
    looks at.  Until then the entry holds on to the array it will be formed from."""

    def sow(self, name, thunk):
        dict.__setitem__(self, name, thunk)

    def __getitem__(self, name):
        value = dict.__getitem__(self, name)
        if callable(value):
            value = value()
            dict.__setitem__(self, name, value)
        return value


def _gated(value, gate):
    """value * silu(gate) (blocks/ffn.py:108-121 with silu): the library's kernel on the device."""
    return silu_gate(value, gate) if gate.is_cuda else value * F.silu(gate)


class MinGRUProjections(NamedTuple):
    """MinGRU's elements before the element map: the step's two projections.  ``MinGRUCell.scan``
    hands them to the kernel that applies the map (a = sigma(-z), b = sigma(z) g(h~)) itself."""
    z: torch.Tensor
    h_tilde: torch.Tensor


class MinGRUCell(_DiagonalCell):
    """MinGRU (min_gru.py:14-90).  The reference scans (log_state, log_decay) with
    logaddexp; the same recurrence in linear space is h_t = sigma(-z) h_{t-1} +
    sigma(z) g(h~), g(x) = x + 0.5 (x >= 0) | sigma(x), which is what the kernel scans.
    The carry keeps the reference's log-space leaves: (log h_T, sum of log decays).
    fused (default): the cell returns the projections and the scan kernel forms the coefficients,
    so neither they nor the half dozen elementwise intermediates behind them exist in memory;
    fused=False returns the linear-space elements (b, a) for the generic diagonal scan."""

    def __init__(self, features, in_features=None, fused=True):
        super().__init__()
        self.features, self.fused = features, fused
        in_features = features if in_features is None else in_features
        self.z = Dense(in_features, features, bias=False)
        self.h = Dense(in_features, features, bias=False)
        self.intermediates = _SownValues()

    def forward(self, x, **kwargs):
        return self.elements(*dense_group(x, [self.z, self.h]))

    def elements(self, z, h_tilde):
        """The cell's elements from its two projections."""
        self.intermediates.sow("gate", lambda z=z.detach(): z.float().mean())   # min_gru.py:63 sows the mean gate
        if self.fused:   # the recurrence runs in fp32 whatever the projections' dtype (autocast): the kernels
            # read bfloat16 projections as they are (and write bfloat16 states); anything else goes in as float32
            if z.dtype == torch.bfloat16 and h_tilde.dtype == torch.bfloat16:
                return MinGRUProjections(z, h_tilde)
            return MinGRUProjections(z.float(), h_tilde.float())
        z, h_tilde = z.float(), h_tilde.float()
        a = torch.sigmoid(-z)
        g = torch.where(h_tilde >= 0, torch.relu(h_tilde) + 0.5, torch.sigmoid(h_tilde))
        return ((torch.sigmoid(z) * g).contiguous(), a.contiguous())

    def scan(self, z, initial_carry, done):
        log_state, log_decay = initial_carry
        h0, P0 = torch.exp(log_state), torch.exp(log_decay)
        if isinstance(z, MinGRUProjections):
            h, h_last, P_last = mingru_scan(z.z, z.h_tilde, done, h0[:, 0].contiguous(), P0[:, 0].contiguous())
            h_last, P_last = h_last[:, None], P_last[:, None]
        else:
            (h, _), (h_last, P_last) = super().scan(z, (h0, P0), done)
        return (h, None), (torch.log(h_last), torch.log(P_last))

    def read(self, h, x, **kwargs):
        return h[0]

    def initialize_carry(self, key, input_shape):
        *batch, _ = input_shape
        dev = self.z.weight.device
        return (torch.full((*batch, 1, self.features), -math.inf, device=dev),
                torch.zeros(*batch, 1, self.features, device=dev))


class GatedLinearRecurrence(SequenceModel):
    """Gated MLP whose hidden activation is a MinGRU-style diagonal recurrence:
    y = W_o( scan(a = sigma(-W_z x), b = sigma(W_z x) g(W_h x)) * silu(W_g x) ),
    i.e. the recurrence of min_gru.py:49-78 inside the gating pattern of the reference's GLU
    block (blocks/ffn.py:82-123).  Carry = MinGRUCell's (log_state, log_decay)."""

    def __init__(self, features, hidden=None):
        super().__init__()
        hidden = features if hidden is None else hidden
        self.cell = MinGRUCell(hidden, in_features=features)
        self.gate = Dense(features, hidden, bias=False)
        self.out = Dense(hidden, features, bias=False)

    def forward(self, inputs, done, initial_carry=None, **kwargs):
        if initial_carry is None:
            initial_carry = self.cell.initialize_carry(None, get_input_shape(inputs))
        z, h_tilde, gate = dense_group(inputs, [self.cell.z, self.cell.h, self.gate])
        h, next_carry = self.cell.scan(self.cell.elements(z, h_tilde), initial_carry, done)
        return next_carry, self.out(_gated(h[0], gate))

    def initialize_carry(self, key, input_shape):
        return self.cell.initialize_carry(key, input_shape)


# ----------------------------------------------------------------------------------
# matrix-state cells
# ----------------------------------------------------------------------------------
def _norm_on_kernel(x):
    """Rows the library's norm kernels take: on the device, a multiple of four features, at most 2048."""
    return x.is_cuda and x.shape[-1] % 4 == 0 and x.shape[-1] <= _RMS_NORM_MAX_D


class _RMSNorm(nn.Module):
    """y = x * rsqrt(mean(x^2) + eps) * scale (flax.linen.RMSNorm defaults, eps = 1e-6)."""

    def __init__(self, dim, eps=1e-6):
        super().__init__()
        self.scale = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x):
        """Statistics in float32.  On the device: the library's kernel, one pass each way, with the result in
        the dtype its readers compute in (under autocast the dense layers behind a norm would each cast it
        again); rows it does not take (wider than 2048 features, a width that is no multiple of 4) and host
        arrays go to the array library."""
        if _norm_on_kernel(x):
            return rms_norm(x, self.scale, self.eps, autocast_dtype(x) or x.dtype)
        return F.rms_norm(x.float(), (x.shape[-1],), self.scale.float(), self.eps).to(x.dtype)

    def fork(self, x):
        """(x, norm(x)) for a residual branch around this norm: with the first result used in place of x, the
        gradients of the two branches are added inside the norm's backward kernel."""
        if _norm_on_kernel(x) and x.dtype in (torch.float32, torch.bfloat16):
            return rms_norm_fork(x, self.scale, self.eps, autocast_dtype(x) or x.dtype)
        return x, self(x)


class LinearAttentionCell(MemoroidCellBase):
    """Causal linear attention with phi = elu + 1 (linear_attention.py:14-124).
    Elements are (v phi(k)^T, phi(k)) combined by addition; the reference materialises
    S (B,T,H,d,d); here the recurrence, the key sum z and the normalised read-out run in one
    chunked kernel per direction."""

    def __init__(self, features, head_dim, num_heads, in_features=None, eps=1e-6):
        super().__init__()
        in_features = features if in_features is None else in_features
        self.features, self.head_dim, self.num_heads, self.eps = features, head_dim, num_heads, eps
        hidden = head_dim * num_heads
        self.key = Dense(in_features, hidden, bias=False)
        self.value = Dense(in_features, hidden, bias=False)
        self.query = Dense(in_features, hidden, bias=False)
        self.norm = _RMSNorm(hidden)
        self.output_projection = Dense(hidden, features)

    def _heads(self, x):
        return x.view(*x.shape[:2], self.num_heads, self.head_dim)

    def forward(self, x, **kwargs):
        """Elements in kernel form: (v, k, q), keys and queries before the feature map (phi is applied
        inside the kernel).  The reference's elements are (v phi(k)^T, phi(k)); the query joins them here
        because the kernel contracts the state with it as it goes."""
        v, k, q = dense_group(x, [self.value, self.key, self.query])
        return (self._heads(v), self._heads(k), self._heads(q))

    def binary_operator(self, a, b):
        return tuple(x + y for x, y in zip(a, b))

    def scan(self, z, initial_carry, done):
        """The recurrence, the running key sum and the normalised read-out in one kernel per direction
        (the single-step kernel when T = 1 and no gradient is asked for).  Returns h = the normalised
        numerator (B,T,H,dv) and the carry (S (B,1,H,dv,dk), z (B,1,H,dk))."""
        v, k_raw, q = z
        S0, z0 = initial_carry
        out, S_last, z_last = normalised_linear_attention(q, k_raw, v, done, S0[:, 0].float(), z0[:, 0].float(),
                                                          "elu1", self.eps)
        return out, (S_last[:, None], z_last[:, None])

    def read(self, h, x, **kwargs):
        """linear_attention.py:109-117: RMS norm over the heads' concatenated outputs, then the output
        projection.  The norm is the library's kernel, one pass over the outputs each way.  (The attention
        kernels can also leave each head's sum of squares beside its outputs -- ``return_ss`` -- for a host
        that folds the rescale out * rsqrt(sum_h ss / (H d) + eps) * scale into its next operation; as array
        operations here that rescale and its gradient cost more passes than the norm kernel, which gets the
        row's statistic from the row it reads anyway: 1.72 -> 1.20 ms for this cell's forward and backward at
        1024 x 128 x 4 x 64.)"""
        return self.output_projection(self.norm(h.reshape(*x.shape[:2], -1)).to(x.dtype))

    def initialize_carry(self, key, input_shape):
        *batch, _ = input_shape
        dev = self.key.weight.device
        return (torch.zeros(*batch, 1, self.num_heads, self.head_dim, self.head_dim, device=dev),
                torch.zeros(*batch, 1, self.num_heads, self.head_dim, device=dev))


class LinearAttention(Memoroid):
    """Memoroid(LinearAttentionCell) under its own name."""

    def __init__(self, cell: LinearAttentionCell):
        super().__init__(cell)


class DeltaNetCell(MemoroidCellBase):
    """DeltaNet: S_t = S_{t-1}(I - beta_t k_t k_t^T) + beta_t v_t k_t^T, o_t = S_t q_t with
    L2-normalised keys and beta = sigmoid(.) (both formed inside the kernels).  Not in the reference; written in its cell
    idiom the elements are the affine maps (beta v k^T, I - beta k k^T) with
    binary_operator(a, b) = (B_a A_b + B_b, A_a A_b).  The carry is (S (B,1,H,d,d),)."""

    def __init__(self, features, head_dim, num_heads, in_features=None, dtype=torch.bfloat16, resets=None):
        super().__init__()
        in_features = features if in_features is None else in_features
        self.features, self.head_dim, self.num_heads, self.dtype = features, head_dim, num_heads, dtype
        self.resets = resets   # None / "passes" / "merged": mrx_reset_path, for rollouts whose episodes end often
        hidden = head_dim * num_heads
        self.query = Dense(in_features, hidden, bias=False)
        self.key = Dense(in_features, hidden, bias=False)
        self.value = Dense(in_features, hidden, bias=False)
        self.beta = Dense(in_features, num_heads, bias=False)
        self.norm = _RMSNorm(hidden)
        self.output_projection = Dense(hidden, features)

    def _heads(self, x):
        return x.view(*x.shape[:2], self.num_heads, self.head_dim)

    def forward(self, x, **kwargs):
        """The raw projections (q, k, v, beta logits): the key normalisation and the sigmoid run
        inside the kernels."""
        dt = self.dtype
        q, k, v, beta = dense_group(x, [self.query, self.key, self.value, self.beta])
        return (self._heads(q).to(dt), self._heads(k).to(dt), self._heads(v).to(dt), beta.to(dt))

    def binary_operator(self, a, b):
        B_i, A_i = a
        B_j, A_j = b
        return (B_i @ A_j + B_j, A_i @ A_j)

    def scan(self, z, initial_carry, done):
        q, k, v, beta_raw = z
        (S0,) = initial_carry
        o, S_last = deltanet(q, k, v, beta_raw, done, S0[:, 0].float(), resets=self.resets)
        return o, (S_last[:, None],)

    def read(self, h, x, **kwargs):
        out = h.reshape(*x.shape[:2], -1)
        return self.output_projection(self.norm(out).to(x.dtype))

    def initialize_carry(self, key, input_shape):
        *batch, _ = input_shape
        dev = self.key.weight.device
        return (torch.zeros(*batch, 1, self.num_heads, self.head_dim, self.head_dim, device=dev),)


class MambaCell(MemoroidCellBase):
    """Mamba-2 style selective state space cell (mamba.py:33-144).  Elements are
    (h_t = (B_t dt_t) (x) x_t : (H,N,P), decay_t = exp(dt_t A) : (H,1,1)) combined by the diagonal
    operator; read is y_t = C_t . h_t + D x_t, gated by silu(z) after RMSNorm.  The reference
    materialises h (B,T,H,N,P); here the scan and the C-contraction run in the gated chunked
    kernel with k = B dt, v = x, q = C and log-decay g = dt A (native at state_dim = head_dim = 64 or
    32; other sizes are padded by the op, state_dim up to 64).
    Carry: (h (B,1,H,N,P), decay (B,1,H,1,1)), the reference's shapes."""

    def __init__(self, features, num_heads=8, head_dim=64, state_dim=64, conv_dim=4, in_features=None):
        super().__init__()
        in_features = features if in_features is None else in_features
        self.features, self.num_heads, self.head_dim = features, num_heads, head_dim
        self.state_dim, self.conv_dim = state_dim, conv_dim
        hidden, sp = num_heads * head_dim, num_heads * state_dim
        conv_channels = hidden + 2 * sp
        self.A_log = nn.Parameter(torch.empty(num_heads).uniform_(math.log(1.0), math.log(16.0)))
        self.D = nn.Parameter(torch.ones(num_heads))
        dt = torch.exp(torch.rand(num_heads) * (math.log(0.1) - math.log(0.001)) + math.log(0.001))
        self.dt_bias = nn.Parameter(dt + torch.log(-torch.expm1(-dt)))
        self.input_projection = Dense(in_features, hidden * 2, bias=False)
        self.B = Dense(in_features, sp, bias=False)
        self.C = Dense(in_features, sp, bias=False)
        self.dt = Dense(in_features, num_heads, bias=False)
        self.conv = nn.Conv1d(conv_channels, conv_channels, conv_dim, groups=conv_channels)
        self.norm = _RMSNorm(hidden)
        self.output_projection = Dense(hidden, features)

    def _project(self, x):
        Bn, T, _ = x.shape
        H, P, N = self.num_heads, self.head_dim, self.state_dim
        up, B_in, C_in, dt_in = dense_group(x, [self.input_projection, self.B, self.C, self.dt])
        hidden, z = up.chunk(2, dim=-1)
        ci = torch.cat([hidden, B_in, C_in], dim=-1).transpose(1, 2)      # (B, channels, T)
        ci = F.silu(self.conv(F.pad(ci, (self.conv_dim - 1, 0)))).transpose(1, 2)   # causal, per call
        hidden = ci[..., :H * P].reshape(Bn, T, H, P)
        B_proj = ci[..., H * P:H * P + H * N].reshape(Bn, T, H, N)
        C_proj = ci[..., H * P + H * N:].reshape(Bn, T, H, N)
        dt = F.softplus(dt_in + self.dt_bias)
        return hidden, B_proj, C_proj, z, dt

    def forward(self, x, **kwargs):
        """Elements in kernel form: (k = B dt, v = x, log-decay g = dt A, q = C); the reference's
        (h, decay) are v (x) k and exp(g), and the C projection joins them because the kernel fuses the
        contraction y_t = C_t . h_t into the scan."""
        hidden, B_proj, C_proj, _, dt = self._project(x)
        g = dt * (-torch.exp(self.A_log))[None, None, :]
        return (B_proj * dt[..., None], hidden, g, C_proj)

    def binary_operator(self, a, b):
        h_i, decay_i = a
        h_j, decay_j = b
        return (decay_j * h_i + h_j, decay_j * decay_i)

    def scan(self, z, initial_carry, done):
        k, v, g, q = z
        h0, decay0 = initial_carry                      # (B,1,H,N,P), (B,1,H,1,1)
        S0 = h0[:, 0].transpose(-1, -2).float().contiguous()   # kernel state is (P, N) = (d_v, d_k)
        o, S_last = gated_linear_attention(q.contiguous(), k.contiguous(), v.contiguous(), g.float(), done, S0)
        Bn, T, H = g.shape
        ones = torch.ones(H, device=g.device)
        _, G_last, _ = linear_scan(ones, g.float().contiguous(), done,
                                   torch.log(decay0[:, 0, :, 0, 0].float()).contiguous())
        carry = (S_last.transpose(-1, -2)[:, None], torch.exp(G_last)[:, None, :, None, None])
        return o, carry

    def read(self, o, x, **kwargs):
        Bn, T, _ = x.shape
        hidden, _, _, z, _ = self._project(x)
        y = o.float() + self.D[None, None, :, None] * hidden
        y = y.reshape(Bn, T, self.num_heads * self.head_dim)
        return self.output_projection(_gated(self.norm(y), z).to(x.dtype))

    def initialize_carry(self, key, input_shape):
        *batch, _ = input_shape
        dev = self.A_log.device
        return (torch.zeros(*batch, 1, self.num_heads, self.state_dim, self.head_dim, device=dev),
                torch.ones(*batch, 1, self.num_heads, 1, 1, device=dev))


class Mamba(Memoroid):
    """Memoroid(MambaCell) under its own name."""

    def __init__(self, cell: MambaCell):
        super().__init__(cell)


class _BlockDiagonalDense(nn.Module):
    """One dense map per head (layers/block_diagonal_dense.py:10-50), no bias."""

    def __init__(self, features, num_heads):
        super().__init__()
        bs = features // num_heads
        self.num_heads = num_heads
        self.kernel = nn.Parameter(torch.randn(num_heads, bs, bs) * math.sqrt(2.0 / (5.0 * bs)))

    def forward(self, x):
        *batch, f = x.shape
        y = torch.einsum("...hd,hod->...ho", x.reshape(*batch, self.num_heads, -1), self.kernel)
        return y.reshape(*batch, f)


class mLSTMCell(MemoroidCellBase):
    """Matrix LSTM (mlstm.py:31-240).  Elements (C = k (x) v, log_f, n = k, m = log_i) combine by the
    max-stabilised gated sum of mlstm.py:190-206; read divides q C by max(|q . n|, exp(-m)) + 1e-6.
    Unrolled, that operator is the recurrence
        m_t = max(m_{t-1} + log f_t, log i_t)
        C_t = exp(log f_t + m_{t-1} - m_t) C_{t-1} + exp(log i_t - m_t) k_t v_t^T      (n_t alike),
    a gated linear recurrence whose log-decay g_t = log f_t + m_{t-1} - m_t and key weight
    exp(log i_t - m_t) are both <= 1 whatever the gates do: m, g and the weights come from one pass per
    (b, h) in the library (functional.mlstm_gates), q C runs in the gated chunked kernel and n in the
    diagonal scan.  State, normaliser and m come out in the reference's stabilised
    units, step by step, so gates may drift by any amount inside an episode.
    Carry: (C (B,1,H,d,d), log_f (B,1,H,1,1), n (B,1,H,d,1), m (B,1,H,1,1)) as in the reference."""

    def __init__(self, features, hidden_dim, num_heads=4, conv_kernel_size=4, in_features=None):
        super().__init__()
        if hidden_dim % num_heads != 0:
            raise ValueError(f"hidden_dim ({hidden_dim}) must be divisible by num_heads ({num_heads}).")
        in_features = features if in_features is None else in_features
        self.features, self.hidden_dim, self.num_heads = features, hidden_dim, num_heads
        self.conv_kernel_size = conv_kernel_size
        self.up_projection = Dense(in_features, 2 * hidden_dim, bias=False)
        self.causal_conv = nn.Conv1d(hidden_dim, hidden_dim, conv_kernel_size, groups=hidden_dim)
        self.query = _BlockDiagonalDense(hidden_dim, num_heads)
        self.key = _BlockDiagonalDense(hidden_dim, num_heads)
        self.value = _BlockDiagonalDense(hidden_dim, num_heads)
        self.i_gate = Dense(3 * hidden_dim, num_heads)
        self.f_gate = Dense(3 * hidden_dim, num_heads)
        with torch.no_grad():
            self.i_gate.weight.zero_()
            self.i_gate.bias.normal_(std=0.1)
            self.f_gate.weight.zero_()
            self.f_gate.bias.copy_(torch.linspace(3.0, 6.0, num_heads))
        self.learnable_skip = nn.Parameter(torch.ones(hidden_dim))
        self.norm_weight = nn.Parameter(torch.zeros(num_heads, hidden_dim // num_heads))
        self.output_projection = Dense(hidden_dim, features, bias=False)

    def _project(self, x):
        Bn, T, _ = x.shape
        d = self.hidden_dim // self.num_heads
        x_mlstm, z = self.up_projection(x).chunk(2, dim=-1)
        u = F.silu(self.causal_conv(F.pad(x_mlstm.transpose(1, 2), (self.conv_kernel_size - 1, 0))).transpose(1, 2))
        heads = lambda t: t.reshape(Bn, T, self.num_heads, d)  # noqa: E731
        return heads(self.query(u)), heads(self.key(u)), heads(self.value(x_mlstm)), z, u

    def forward(self, x, **kwargs):
        """Elements in kernel form: (k / sqrt(d), v, log_i, log_f, q)."""
        Bn, T, _ = x.shape
        q, k, v, _, _ = self._project(x)
        gate_input = torch.cat([q, k, v], dim=-1).reshape(Bn, T, -1)
        i_pre, f_pre = dense_group(gate_input, [self.i_gate, self.f_gate])
        log_i = i_pre.float()
        log_f = -F.softplus(-f_pre.float())
        return (k / math.sqrt(k.shape[-1]), v, log_i, log_f, q)

    def binary_operator(self, a, b):
        C_a, log_f_a, n_a, m_a = a
        C_b, log_f_b, n_b, m_b = b
        m_a_decayed = m_a + log_f_b
        m = torch.maximum(m_a_decayed, m_b)
        sa, sb = torch.exp(m_a_decayed - m), torch.exp(m_b - m)
        return (sa * C_a + sb * C_b, log_f_a + log_f_b, sa * n_a + sb * n_b, m)

    # A log-decay below this is a state multiplied by exp(-60) < 1e-26 next to a new term of weight one:
    # clamping keeps the in-chunk prefix sums of the kernel small (no cancellation between them).
    _G_FLOOR = -60.0

    def scan(self, z, initial_carry, done):
        k, v, log_i, log_f, q = z
        C0, lf0, n0, m0 = initial_carry
        Bn, T, H, d = k.shape
        ones = torch.ones(H, device=k.device)
        m0_ = m0[:, 0, :, 0, 0].float()                                          # (B,H)
        # m_t = max(m_{t-1} + log f_t, log i_t), restarted at resets; g_t = log f_t + m_{t-1} - m_t (0 at a reset:
        # it zeroes the state anyway) and the key weights exp(log i_t - m_t) <= 1: one pass per (b, h) in the library
        m, g, wk = mlstm_gates(log_i, log_f, done, m0_, self._G_FLOOR)            # each (B,T,H)
        k_in = k.float() * wk[..., None]
        S0 = C0[:, 0].float().transpose(-1, -2).contiguous()
        num, S_last = gated_linear_attention(q.float().contiguous(), k_in.contiguous(), v.float().contiguous(),
                                             g.contiguous(), done, S0)
        a = torch.exp(g)[..., None].expand(Bn, T, H, d).reshape(Bn, T, H * d).contiguous()
        nvec, n_last, _ = linear_scan(a, k_in.reshape(Bn, T, H * d).contiguous(), done,
                                      n0[:, 0, :, :, 0].float().reshape(Bn, H * d).contiguous())
        qn = (q.float() * nvec.view(Bn, T, H, d)).sum(-1)                         # (B,T,H)
        den = torch.maximum(qn.abs(), torch.exp(-m)) + 1e-6
        h_tilde = num / den[..., None]
        _, lf_last, _ = linear_scan(ones, log_f.contiguous(), done, lf0[:, 0, :, 0, 0].float().contiguous())
        carry = (S_last.transpose(-1, -2)[:, None],
                 lf_last[:, None, :, None, None],
                 n_last.view(Bn, H, d)[:, None, :, :, None],
                 m[:, -1][:, None, :, None, None])
        return h_tilde, carry

    def read(self, h_tilde, x, **kwargs):
        Bn, T, _ = x.shape
        _, _, _, z, u = self._project(x)
        y = F.layer_norm(h_tilde, (h_tilde.shape[-1],), eps=1e-5) * (1.0 + self.norm_weight)[None, None]
        y = y.reshape(Bn, T, self.hidden_dim) + self.learnable_skip * u
        return self.output_projection(_gated(y, z).to(x.dtype))

    def initialize_carry(self, key, input_shape):
        *batch, _ = input_shape
        H, d = self.num_heads, self.hidden_dim // self.num_heads
        dev = self.learnable_skip.device
        return (torch.zeros(*batch, 1, H, d, d, device=dev), torch.zeros(*batch, 1, H, 1, 1, device=dev),
                torch.zeros(*batch, 1, H, d, 1, device=dev), torch.full((*batch, 1, H, 1, 1), -1e9, device=dev))


class mLSTM(Memoroid):
    """Memoroid(mLSTMCell) under its own name."""

    def __init__(self, cell: mLSTMCell):
        super().__init__(cell)


# ----------------------------------------------------------------------------------
# block composition used by the torso configuration (blocks/{stack,residual,normalization,ffn}.py)
# ----------------------------------------------------------------------------------
class _LayerNorm(nn.LayerNorm):
    """torch.nn.LayerNorm (same parameters, same state dict) on the library's kernel where the rows fit it."""

    def forward(self, x):
        if _norm_on_kernel(x) and self.elementwise_affine:
            return layer_norm(x, self.weight, self.bias, self.eps, autocast_dtype(x) or x.dtype)
        return super().forward(x)

    def fork(self, x):
        """(x, norm(x)) for a residual branch around this norm (see _RMSNorm.fork)."""
        if _norm_on_kernel(x) and self.elementwise_affine and x.dtype in (torch.float32, torch.bfloat16):
            return layer_norm_fork(x, self.weight, self.bias, self.eps, autocast_dtype(x) or x.dtype)
        return x, self(x)


def LayerNorm(dim):
    """flax.linen.LayerNorm with its defaults: mean and variance over the last axis, eps = 1e-6,
    learned scale and bias -- the default norm of the reference's PreNorm / PostNorm."""
    return _LayerNorm(dim, eps=1e-6)


RMSNorm = _RMSNorm


class PreNorm(nn.Module):
    """normalization.py:10-35: norm, then the wrapped sequence model.  ``norm`` is a constructor taking
    the feature width (the reference's flax modules infer it); default LayerNorm as in the reference,
    ``norm=RMSNorm`` for the torso configuration."""

    def __init__(self, module, dim, norm=LayerNorm):
        super().__init__()
        self.module, self.norm = module, norm(dim)

    def forward(self, inputs, done=None, initial_carry=None, **kwargs):
        return self.module(self.norm(inputs), done, initial_carry, **kwargs)

    def initialize_carry(self, key, input_shape):
        return self.module.initialize_carry(key, input_shape)


class PostNorm(nn.Module):
    """normalization.py:38-65: the wrapped sequence model, then norm."""

    def __init__(self, module, dim, norm=LayerNorm):
        super().__init__()
        self.module, self.norm = module, norm(dim)

    def forward(self, inputs, done=None, initial_carry=None, **kwargs):
        carry, y = self.module(inputs, done, initial_carry, **kwargs)
        return carry, self.norm(y)

    def initialize_carry(self, key, input_shape):
        return self.module.initialize_carry(key, input_shape)


class Residual(nn.Module):
    """residual.py:10-30: x + module(x)."""

    def __init__(self, module):
        super().__init__()
        self.module = module

    def forward(self, inputs, done=None, initial_carry=None, **kwargs):
        inner = self.module
        if isinstance(inner, PreNorm) and hasattr(inner.norm, "fork"):   # x + f(norm(x)): one kernel takes both gradients of x
            inputs, normed = inner.norm.fork(inputs)
            carry, y = inner.module(normed, done, initial_carry, **kwargs)
        else:
            carry, y = inner(inputs, done, initial_carry, **kwargs)
        return carry, inputs + y

    def initialize_carry(self, key, input_shape):
        return self.module.initialize_carry(key, input_shape)


class GatedResidual(nn.Module):
    """residual.py:33-63: x + gate(Dense(x)) * module(x), the gate a dense layer of the block's width
    (with bias) on the block's input."""

    def __init__(self, module, dim, gate=torch.sigmoid):
        super().__init__()
        self.module, self.gate, self.gate_fn = module, Dense(dim, dim), gate

    def forward(self, inputs, done=None, initial_carry=None, **kwargs):
        carry, y = self.module(inputs, done, initial_carry, **kwargs)
        return carry, inputs + self.gate_fn(self.gate(inputs)) * y

    def initialize_carry(self, key, input_shape):
        return self.module.initialize_carry(key, input_shape)


def gelu(x):
    """flax.linen.gelu as the reference's blocks call it (blocks/ffn.py:16,86): the tanh approximation, which is
    jax.nn.gelu's default -- not the error-function form that is the array library's."""
    return F.gelu(x, approximate="tanh")


class _Stateless(nn.Module):
    """Blocks without a recurrence (blocks/base.py:6-21): the carry is None on the way in and out."""

    def initialize_carry(self, key, input_shape):
        return None


class FFN(_Stateless):
    """ffn.py:11-50: Dense -> activation -> dropout -> Dense, hidden width features * expansion_factor."""

    def __init__(self, features, expansion_factor=4, activation=gelu, dropout_rate=0.0):
        super().__init__()
        self.up = Dense(features, features * expansion_factor)
        self.down = Dense(features * expansion_factor, features)
        self.activation, self.dropout = activation, nn.Dropout(dropout_rate)

    def forward(self, inputs, done=None, initial_carry=None, **kwargs):
        return None, self.down(self.dropout(self.activation(self.up(inputs))))


class Projection(_Stateless):
    """ffn.py:53-79: a single dense layer."""

    def __init__(self, in_features, features, use_bias=True):
        super().__init__()
        self.proj = Dense(in_features, features, bias=use_bias)

    def forward(self, inputs, done=None, initial_carry=None, **kwargs):
        return None, self.proj(inputs)


class GLU(_Stateless):
    """ffn.py:82-123: up_proj to 2 * hidden, split into (gate, value) in that order,
    activation(gate) * value, dropout, down_proj; no biases by default."""

    def __init__(self, features, expansion_factor=4, activation=gelu, dropout_rate=0.0, use_bias=False):
        super().__init__()
        hidden = features * expansion_factor
        self.up_proj = Dense(features, 2 * hidden, bias=use_bias)
        self.down_proj = Dense(hidden, features, bias=use_bias)
        self.activation, self.dropout = activation, nn.Dropout(dropout_rate)

    def forward(self, inputs, done=None, initial_carry=None, **kwargs):
        gate, value = self.up_proj(inputs).chunk(2, dim=-1)
        return None, self.down_proj(self.dropout(self.activation(gate) * value))


class Stack(nn.Module):
    """stack.py:10-60: one carry per block, threaded as a tuple."""

    def __init__(self, blocks):
        super().__init__()
        self.blocks = nn.ModuleList(blocks)

    def forward(self, inputs, done=None, initial_carry=None, **kwargs):
        if initial_carry is None:
            initial_carry = tuple(None for _ in self.blocks)
        x, carries = inputs, []
        for block, c in zip(self.blocks, initial_carry):
            carry, x = block(x, done=done, initial_carry=c, **kwargs)
            carries.append(carry)
        return tuple(carries), x

    def initialize_carry(self, key, input_shape):
        return tuple(b.initialize_carry(key, input_shape) if hasattr(b, "initialize_carry") else None
                     for b in self.blocks)
