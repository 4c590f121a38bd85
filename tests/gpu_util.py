"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

TOL_F32 = 1e-4   # fp32: max|x-y| / max|y|
TOL_BF16 = 2e-2  # bf16 inputs, fp32 state/accumulate


def relerr(x, y):
    if isinstance(x, torch.Tensor):
        x = x.detach().float().cpu().numpy() if not x.is_complex() else x.detach().cpu().numpy()
    x = np.asarray(x)
    return float(np.abs(x - y).max() / max(np.abs(y).max(), 1e-30))


def dev(x, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(x)).cuda()
    return t if dtype is None else t.to(dtype)


def bf16_round(x):
    """fp32 array rounded to bf16 and back (what the kernel actually receives)."""
    return torch.from_numpy(np.ascontiguousarray(x)).to(torch.bfloat16).float().numpy()


def attn_inputs(B, T, H, d=64, p=0.0, seed=0, delta=False, scale=None):
    rng = np.random.default_rng(seed)
    s = 1.0 / np.sqrt(d) if scale is None else scale
    q = (rng.standard_normal((B, T, H, d)) * s).astype(np.float32)
    k = (rng.standard_normal((B, T, H, d)) * s).astype(np.float32)
    v = (rng.standard_normal((B, T, H, d)) * s).astype(np.float32)
    out = dict(q=q, k=k, v=v)
    if delta:
        out["q"] = rng.standard_normal((B, T, H, d)).astype(np.float32)
        out["v"] = rng.standard_normal((B, T, H, d)).astype(np.float32)
        kk = rng.standard_normal((B, T, H, d)).astype(np.float32)
        out["k"] = kk / np.linalg.norm(kk, axis=-1, keepdims=True)
        out["beta"] = (1 / (1 + np.exp(-rng.standard_normal((B, T, H))))).astype(np.float32)
    out["done"] = rng.random((B, T)) < p
    out["S0"] = (rng.standard_normal((B, H, d, d)) * 0.1).astype(np.float32)
    return out
