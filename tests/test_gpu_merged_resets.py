"""The delta-rule kernels with all episodes of a chunk in one unit (MRX_RESETS_MERGED, through the C ABI):
same results as one unit per episode -- against the oracle and against that path itself -- for every reset
pattern; a chunk whose inputs fail the screen (a NaN, an Inf, magnitudes beyond the bounds) falls back to
the units per episode, so that nothing of one episode ever reaches another."""
import numpy as np
import pytest
import torch

from oracle import clib
from oracle import grad as G
from gpu_util import TOL_BF16, TOL_F32, attn_inputs, bf16_round, dev, relerr

pytestmark = pytest.mark.gpu


def _case(B, T, H, seed, dtype, done):
    x = attn_inputs(B, T, H, seed=seed, delta=True)
    x["done"] = done
    rng = np.random.default_rng(seed + 7)
    x["do"] = rng.standard_normal((B, T, H, 64)).astype(np.float32)
    x["dSl"] = (rng.standard_normal((B, H, 64, 64)) * 0.1).astype(np.float32)
    if dtype == "bf16":
        for n in ("q", "k", "v", "beta", "do"):
            x[n] = bf16_round(x[n])
    return x


def _run(K, x, dtype, resets, prologue=False, S0=True, dSl=True):
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    tq, tk, tv, tb, tdo = (dev(x[n], td) for n in ("q", "k", "v", "beta", "do"))
    dn = dev(x["done"])
    o, Sl, chk = K.delta_rule_fwd(tq, tk, tv, tb, dn, dev(x["S0"]) if S0 else None, prologue=prologue, reset_path=resets,
                                  factor_path="parallel")
    g = K.delta_rule_bwd(tq, tk, tv, tb, dn, chk, tdo, dev(x["dSl"]) if dSl else None, prologue=prologue,
                         reset_path=resets, want_dS0=True)
    torch.cuda.synchronize()
    return dict(o=o, S_last=Sl, dq=g[0], dk=g[1], dv=g[2], dbeta=g[3], dS0=g[4], S_chk=chk[0], Tm_chk=chk[1])


def _patterns(B, T, rng):
    """Reset masks that put every position of an episode boundary inside a 32-row chunk to the test."""
    out = {}
    out["bernoulli_0.02"] = rng.random((B, T)) < 0.02
    out["bernoulli_0.2"] = rng.random((B, T)) < 0.2
    d = np.zeros((B, T), bool)
    d[:, ::32] = True               # first row of every chunk (the entering episode is empty)
    out["chunk_starts"] = d
    d = np.zeros((B, T), bool)
    d[:, 31::32] = True             # last row of every chunk (the leaving episode is one row)
    out["chunk_ends"] = d
    d = np.zeros((B, T), bool)
    d[0, [t for t in (5, 6, 7, 40, 41, 70) if t < T]] = True   # runs of consecutive resets, several per chunk
    d[-1, [t for t in (0, 16, 17, 63, 64) if t < T]] = True
    out["runs"] = d
    out["every_step"] = np.ones((B, T), bool)
    out["none"] = np.zeros((B, T), bool)
    return out


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("T", [100, 32, 9])
def test_merged_equals_units_per_episode_and_the_oracle(dtype, T):
    from memorax_amd import kernels as K
    B, H = 2, 2
    rng = np.random.default_rng(40 + T)
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    for name, done in _patterns(B, T, rng).items():
        x = _case(B, T, H, 11, dtype, done)
        print(f"case merged dtype={dtype} T={T} pattern={name}", flush=True)
        a = _run(K, x, dtype, "merged")
        b = _run(K, x, dtype, "passes")
        ro, rS = clib.delta_rule_fwd(x["q"], x["k"], x["v"], x["beta"], done, x["S0"])
        ref = dict(zip(("dq", "dk", "dv", "dbeta", "dS0"),
                       clib.delta_rule_bwd(x["q"], x["k"], x["v"], x["beta"], done, x["S0"], x["do"], x["dSl"])))
        ref.update(o=ro, S_last=rS)
        for n in ("o", "S_last", "dq", "dk", "dv", "dbeta", "dS0"):
            assert relerr(a[n], ref[n]) <= tol, (name, n, relerr(a[n], ref[n]))
            # against the units per episode: the same arithmetic up to the order of two sums in the backward's merged chunks
            bn = b[n].float().cpu().numpy()
            assert relerr(a[n], bn) <= (4e-3 if dtype == "bf16" else 2e-6), (name, n, relerr(a[n], bn))
        # the forward is the same arithmetic bit for bit, residuals included
        for n in ("o", "S_last", "S_chk", "Tm_chk"):
            assert torch.equal(a[n], b[n]), (name, n)


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_merged_with_the_prologue_and_without_optional_arguments(dtype):
    from memorax_amd import kernels as K
    B, T, H = 2, 130, 2
    rng = np.random.default_rng(3)
    done = rng.random((B, T)) < 0.05
    x = _case(B, T, H, 12, dtype, done)
    x["k"] = (rng.standard_normal((B, T, H, 64)) * 3).astype(np.float32)     # raw keys: normalised in the kernels
    x["beta"] = rng.standard_normal((B, T, H)).astype(np.float32)            # gate logits
    if dtype == "bf16":
        x["k"], x["beta"] = bf16_round(x["k"]), bf16_round(x["beta"])
    print(f"case merged prologue dtype={dtype}", flush=True)
    a = _run(K, x, dtype, "merged", prologue=True, S0=False, dSl=False)
    ref = G.deltanet_grads(x["q"], x["k"], x["v"], x["beta"], done, None, x["do"], None)
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    for n in ("o", "S_last", "dq", "dk", "dv", "dbeta"):
        assert relerr(a[n], ref[n]) <= tol, (n, relerr(a[n], ref[n]))


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_merged_falls_back_where_the_screen_fails(dtype):
    """NaN / Inf on one side of a reset inside a chunk, and magnitudes beyond the screen's bounds: the chunk
    takes the units per episode, whose zeros are put in by select; the other episodes are untouched."""
    from memorax_amd import kernels as K
    B, T, H = 1, 96, 1
    done = np.zeros((B, T), bool)
    done[0, [40, 50]] = True         # chunk 1 (rows 32..63) holds three episodes: 32..39, 40..49, 50..63
    x = _case(B, T, H, 13, dtype, done)
    x["v"][0, 44] = np.nan           # poison inside the middle episode: value, key, gate, gradient
    x["k"][0, 45] = np.inf
    x["beta"][0, 46] = np.nan
    x["do"][0, 47] = np.nan
    print(f"case merged poison dtype={dtype}", flush=True)
    a = _run(K, x, dtype, "merged", dSl=False)
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    cut = lambda z, lo, hi: z[:, lo:hi]  # noqa: E731
    # the episode before the poisoned one: steps 0..39 with the initial state
    r1 = G.delta_rule_grads(cut(x["q"], 0, 40), cut(x["k"], 0, 40), cut(x["v"], 0, 40), cut(x["beta"], 0, 40),
                            done[:, :40], x["S0"], cut(x["do"], 0, 40))
    # the episode after it: steps 50..95 from a zero state
    d3 = np.zeros((B, 46), bool)
    r3 = G.delta_rule_grads(cut(x["q"], 50, 96), cut(x["k"], 50, 96), cut(x["v"], 50, 96), cut(x["beta"], 50, 96),
                            d3, None, cut(x["do"], 50, 96))
    for n in ("o", "dq", "dk", "dv", "dbeta"):
        g = a[n].float().cpu().numpy()
        assert np.isfinite(g[:, :40]).all() and np.isfinite(g[:, 50:]).all(), n
        assert relerr(g[:, :40], r1[n]) <= tol and relerr(g[:, 50:], r3[n]) <= tol, n
    assert relerr(a["S_last"], r3["S_last"]) <= tol and relerr(a["dS0"], r1["dS0"]) <= tol
    # magnitudes beyond the bounds of the screen (values of 1e4): finite, so both paths agree with the oracle
    y = _case(B, T, H, 14, dtype, done)
    y["v"] *= 1e4
    if dtype == "bf16":
        y["v"] = bf16_round(y["v"])
    c = _run(K, y, dtype, "merged")
    ref = dict(zip(("dq", "dk", "dv", "dbeta", "dS0"),
                   clib.delta_rule_bwd(y["q"], y["k"], y["v"], y["beta"], done, y["S0"], y["do"], y["dSl"])))
    for n in ("dq", "dk", "dv", "dbeta", "dS0"):
        assert relerr(c[n], ref[n]) <= tol, n


def test_merged_at_the_torso_shape_through_the_functional_layer():
    """B = 64 of configuration 5's (B, 128, 4, 64) with its reset rate, bf16, prologue: functional.deltanet with
    resets="merged" against resets="passes" (outputs and every gradient), and the argument reaches the kernels
    (an unknown value is refused)."""
    import memorax_amd.functional as F
    B, T, H = 64, 128, 4
    g = torch.Generator().manual_seed(5)
    mk = lambda *s: torch.randn(*s, generator=g).cuda().to(torch.bfloat16)  # noqa: E731
    q, k, v, b = mk(B, T, H, 64), mk(B, T, H, 64), mk(B, T, H, 64), mk(B, T, H)
    done = (torch.rand(B, T, generator=g) < 0.01).cuda()
    S0 = (torch.randn(B, H, 64, 64, generator=g) * 0.1).cuda()
    gy = mk(B, T, H, 64)
    outs = []
    for mode in ("merged", "passes"):
        leaves = [t.clone().requires_grad_() for t in (q, k, v, b, S0)]
        o, Sl = F.deltanet(*leaves[:4], done, leaves[4], resets=mode)
        ((o.float() * gy.float()).sum() + Sl.sum()).backward()
        outs.append([o, Sl] + [t.grad for t in leaves])
    for a, b_ in zip(*outs):
        assert relerr(a, b_.detach().float().cpu().numpy()) <= 4e-3
    with pytest.raises(KeyError):
        F.deltanet(q, k, v, b, done, S0, resets="sometimes")
