"""Seeded random sweep of the chunked kernels against the oracle: shapes, head dims (64, 32 and narrow heads
with d_k != d_v), dtypes, reset rates, feature maps, optional initial
state and state gradient, every factor path of the delta rule -- combinations the hand-written case lists
do not enumerate.  Every case is drawn from a fixed seed, so a failure names its case."""
import numpy as np
import pytest
import torch

from oracle import grad as G
from gpu_util import TOL_BF16, TOL_F32, bf16_round, dev, relerr

pytestmark = pytest.mark.gpu

LENGTHS = [1, 2, 31, 32, 33, 63, 64, 65, 96, 127, 130, 257, 300]
CASES_PER_SEED = 16


def _case(rng):
    op = str(rng.choice(["la", "lapar", "gated", "norm", "delta", "deltanet"]))
    dtype = str(rng.choice(["f32", "bf16"]))
    seg = 8 if dtype == "bf16" else 4
    kind = int(rng.integers(0, 4))
    if kind == 0:
        dk = dv = 64
    elif kind == 1:
        dk = dv = 32
    else:  # narrow heads: whole 16-byte segments, widths independent of one another, up to 32 or up to 64
        dk, dv = (int(rng.integers(1, (32 if kind == 2 else 64) // seg + 1)) * seg for _ in range(2))
    return dict(op=op, dtype=dtype, dk=dk, dv=dv, B=int(rng.integers(1, 4)), H=int(rng.integers(1, 4)),
                T=int(rng.choice(LENGTHS)), p=float(rng.choice([0.0, 0.01, 0.1, 0.5])), fm=int(rng.integers(0, 2)),
                S0=bool(rng.integers(0, 2)), dSl=bool(rng.integers(0, 2)),
                path=str(rng.choice(["auto", "parallel", "inline"])))


@pytest.mark.parametrize("seed", range(12))
def test_random_cases(seed):
    from memorax_amd import kernels as K
    rng = np.random.default_rng(1000 + seed)
    failures = []
    for it in range(CASES_PER_SEED):
        c = _case(rng)
        op, dtype, dk, dv, B, T, H, fm = (c[n] for n in ("op", "dtype", "dk", "dv", "B", "T", "H", "fm"))
        desc = f"seed={seed} it={it} " + " ".join(f"{k}={v}" for k, v in c.items())
        print("case", desc, flush=True)
        td = torch.bfloat16 if dtype == "bf16" else torch.float32
        tol = TOL_BF16 if dtype == "bf16" else TOL_F32
        r = lambda *s: rng.standard_normal(s).astype(np.float32)
        q, k, v, do = r(B, T, H, dk) / 6, r(B, T, H, dk) / 6, r(B, T, H, dv), r(B, T, H, dv)
        S0 = r(B, H, dv, dk) * 0.1 if c["S0"] else None
        dSl = r(B, H, dv, dk) * 0.1 if c["dSl"] else None
        done = rng.random((B, T)) < c["p"]
        g, beta, z0 = -np.abs(r(B, T, H)) * 0.3, r(B, T, H) * 1.5, np.abs(r(B, H, dk))
        if op in ("delta", "deltanet"):
            q, k = r(B, T, H, dk), r(B, T, H, dk)
            if op == "delta":  # unit keys and gates in (0, 1); deltanet forms both inside the kernels
                k, beta = k / np.linalg.norm(k, axis=-1, keepdims=True), 1 / (1 + np.exp(-beta))
        if dtype == "bf16":
            q, k, v, do, beta = (bf16_round(a) for a in (q, k, v, do, beta))
        tq, tk, tv, tdo = (dev(a, td) for a in (q, k, v, do))
        dn = dev(done)
        tS0, tdSl = (None if a is None else dev(a) for a in (S0, dSl))
        name = "elu1" if fm else "none"
        if op in ("la", "lapar"):
            o, Sl, chk = K.linear_attn_fwd(tq, tk, tv, dn, tS0, fm, chunk_parallel=(op == "lapar"))
            got = K.linear_attn_bwd(tq, tk, tv, dn, chk, tdo, tdSl, fm)
            ref = G.linear_attention_grads(q, k, v, done, S0, do, dSl, name)
            names = ("dq", "dk", "dv", "dS0")
        elif op == "gated":
            o, Sl, chk = K.gated_linear_attn_fwd(tq, tk, tv, dev(g), dn, tS0, fm)
            got = K.gated_linear_attn_bwd(tq, tk, tv, dev(g), dn, chk, tdo, tdSl, fm, S_last=Sl)
            ref = G.gated_linear_attention_grads(q, k, v, g, done, S0, do, dSl, name)
            names = ("dq", "dk", "dv", "dg", "dS0")
        elif op == "norm":
            o, den, Sl, zl, chk = K.linear_attn_norm_fwd(tq, tk, tv, dn, tS0, dev(z0), 1, 1e-6)
            got = K.linear_attn_norm_bwd(tq, tk, tv, dn, chk, o, den, tdo, tdSl, None, 1, 1e-6)
            # The backward call reads the quotient o back as the forward call stored it (bf16) and forms
            # dden = -(dout . o) / den from it, a sum that can cancel; the oracle differentiates the divide on
            # the same stored o (values are still compared with its own exact quotient), so that the
            # tolerance is not charged with the rounding of a residual.
            o_st = o.float().cpu().numpy().astype(np.float64) if dtype == "bf16" else None
            ref = G.normalised_linear_attention_grads(q, k, v, done, S0, z0, do, dSl, None, "elu1", 1e-6, o_stored=o_st)
            names = ("dq", "dk", "dv", "dS0", "dz0")
        else:
            pro = op == "deltanet"
            tb = dev(beta, td)
            # every second case with all episodes of a chunk in one unit (taken from the drawn sizes, so that
            # the cases themselves stay what they were)
            resets = "merged" if (B + T + H) % 2 else None
            o, Sl, chk = K.delta_rule_fwd(tq, tk, tv, tb, dn, tS0, prologue=pro, factor_path=c["path"], reset_path=resets)
            got = K.delta_rule_bwd(tq, tk, tv, tb, dn, chk, tdo, tdSl, prologue=pro, reset_path=resets)
            ref = (G.deltanet_grads if pro else G.delta_rule_grads)(q, k, v, beta, done, S0, do, dSl)
            names = ("dq", "dk", "dv", "dbeta", "dS0")
        torch.cuda.synchronize()
        errs = {"o": relerr(o, ref["o"]), "S_last": relerr(Sl, ref["S_last"])}
        for n, a in zip(names, got):
            if a is None or (B * T * H < 4 and n in ("dbeta", "dg")):  # a lone scalar has no scale to be judged against
                continue
            an, top = a.float().cpu().numpy(), np.abs(ref[n]).max()
            # a gradient that is zero in exact arithmetic (dg of a one-step sequence without an initial state; dq of
            # a normalised read-out whose only step follows a reset: the quotient does not depend on q) comes out of
            # the oracle as exactly zero or as float64 rounding noise, and has no scale of its own: what the kernel
            # returns must be rounding noise of the products behind it, bounded absolutely by their operands:
            # eps(dtype) |dout|_max |q|_max |k|_max d
            bound = (2.0 ** -8 if dtype == "bf16" else 2.0 ** -23) * np.abs(do).max() * max(np.abs(q).max(), 1.0) * \
                max(np.abs(k).max(), 1.0) * q.shape[-1]
            if top <= 1e-9 * bound:
                errs[n] = 0.0 if np.abs(an).max() <= bound else float("inf")
            else:
                errs[n] = float(np.abs(an - ref[n]).max() / top)
        bad = {n: e for n, e in errs.items() if not e <= tol}
        if bad:
            failures.append((desc, bad))
    assert not failures, failures
