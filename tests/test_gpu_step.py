"""GPU parity of the single-step (T = 1) kernels, through the C ABI, against the oracle recurrences.

A rollout calls the step T times, feeding the state back; the outputs and the final state must
equal what the oracle computes for the whole (B,T,...) sequence, resets included."""
import numpy as np
import pytest
import torch

from oracle import memoroid as M
from gpu_util import TOL_BF16, TOL_F32, attn_inputs, bf16_round, dev, relerr

pytestmark = pytest.mark.gpu


def _roll(step, T):
    outs = []
    for t in range(T):
        outs.append(step(t))
    return torch.stack(outs, dim=1)


@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 9, 2), (2, 17, 4)])
@pytest.mark.parametrize("p", [0.0, 0.2])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("fmap", ["none", "elu1"])
def test_linear_attention_step_rollout(shape, p, dtype, fmap):
    from memorax_amd import kernels as K
    B, T, H = shape
    x = attn_inputs(B, T, H, p=p, seed=11 * B + T + H, scale=1.0 / 8)
    print(f"case la_step shape={shape} p={p} dtype={dtype} fmap={fmap}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    if dtype == "bf16":
        for n in ("q", "k", "v"):
            x[n] = bf16_round(x[n])
    q, k, v, done = dev(x["q"], td), dev(x["k"], td), dev(x["v"], td), dev(x["done"])
    state = {"S": dev(x["S0"])}

    def step(t):
        o, state["S"], _ = K.linear_attn_step(q[:, t].contiguous(), k[:, t].contiguous(), v[:, t].contiguous(),
                                              done[:, t].contiguous(), state["S"], feature_map=fmap)
        return o

    o = _roll(step, T)
    ro, rS = M.linear_attention(x["q"], x["k"], x["v"], x["done"], x["S0"], fmap)
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    assert relerr(o, ro) <= tol, relerr(o, ro)
    assert relerr(state["S"], rS) <= (1e-5 if dtype == "f32" else tol), relerr(state["S"], rS)


@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 9, 2), (2, 17, 4)])
@pytest.mark.parametrize("p", [0.0, 0.2])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_delta_rule_step_rollout(shape, p, dtype):
    from memorax_amd import kernels as K
    B, T, H = shape
    x = attn_inputs(B, T, H, p=p, seed=13 * B + T + H, delta=True)
    print(f"case delta_step shape={shape} p={p} dtype={dtype}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    if dtype == "bf16":
        for n in ("q", "k", "v", "beta"):
            x[n] = bf16_round(x[n])
    q, k, v, beta = (dev(x[n], td) for n in ("q", "k", "v", "beta"))
    done = dev(x["done"])
    state = {"S": dev(x["S0"])}

    def step(t):
        o, state["S"] = K.delta_rule_step(q[:, t].contiguous(), k[:, t].contiguous(), v[:, t].contiguous(),
                                          beta[:, t].contiguous(), done[:, t].contiguous(), state["S"])
        return o

    o = _roll(step, T)
    ro, rS = M.delta_rule(x["q"], x["k"], x["v"], x["beta"], x["done"], x["S0"])
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    assert relerr(o, ro) <= tol, relerr(o, ro)
    assert relerr(state["S"], rS) <= (1e-5 if dtype == "f32" else tol), relerr(state["S"], rS)


@pytest.mark.parametrize("dims", [(64, 64), (32, 32), (16, 16), (8, 24)])
@pytest.mark.parametrize("p", [0.0, 0.2])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("fmap", ["none", "elu1"])
def test_gated_linear_attention_step_rollout(dims, p, dtype, fmap):
    """S' = (done ? 0 : exp(g) S) + v phi(k)^T, o = S' phi(q): a rollout of steps against the oracle's gated
    recurrence over the whole sequence, and the host mirror's T = 1 route against the chunked kernel."""
    from memorax_amd import functional as F
    from memorax_amd import kernels as K
    dk, dv = dims
    B, T, H = 3, 13, 2
    rng = np.random.default_rng(dk + dv + int(10 * p))
    x = {n: (rng.standard_normal((B, T, H, d)) / 4).astype(np.float32) for n, d in (("q", dk), ("k", dk), ("v", dv))}
    g = (-np.abs(rng.standard_normal((B, T, H))) * 0.5).astype(np.float32)
    done = rng.random((B, T)) < p
    S0 = (rng.standard_normal((B, H, dv, dk)) * 0.1).astype(np.float32)
    print(f"case gated_step dims={dims} p={p} dtype={dtype} fmap={fmap}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    if dtype == "bf16":
        for n in ("q", "k", "v"):
            x[n] = bf16_round(x[n])
    q, k, v, tg, dn = dev(x["q"], td), dev(x["k"], td), dev(x["v"], td), dev(g), dev(done)
    state = {"S": dev(S0)}

    def step(t):
        o, state["S"] = K.gated_linear_attn_step(q[:, t].contiguous(), k[:, t].contiguous(), v[:, t].contiguous(),
                                                 tg[:, t].contiguous(), dn[:, t].contiguous(), state["S"],
                                                 feature_map=fmap)
        return o

    o = _roll(step, T)
    ro, rS = M.gated_linear_attention(x["q"], x["k"], x["v"], g, done, S0, fmap)
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    assert o.shape == (B, T, H, dv) and relerr(o, ro) <= tol, relerr(o, ro)
    assert relerr(state["S"], rS) <= (1e-5 if dtype == "f32" else tol), relerr(state["S"], rS)
    # the host mirror takes the step kernel for T = 1 without gradients; same numbers as the chunked kernel
    S_mid = dev(S0)
    with torch.no_grad():
        o1, S1 = F.gated_linear_attention(q[:, :1], k[:, :1], v[:, :1], tg[:, :1], dn[:, :1], S_mid, fmap)
    o2, S2, _ = K.gated_linear_attn_fwd(q[:, :1].contiguous(), k[:, :1].contiguous(), v[:, :1].contiguous(),
                                        tg[:, :1].contiguous(), dn[:, :1].contiguous(), S_mid,
                                        {"none": 0, "elu1": 1}[fmap], save_chk=False)
    # (bf16: the chunked kernel rounds phi(k) to the I/O type before the products, the step kernel does not)
    assert relerr(o1, o2.float().cpu().numpy()) <= tol and relerr(S1, S2.cpu().numpy()) <= (1e-5 if dtype == "f32" else tol)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_linear_attention_step_normalised(dtype):
    """Fused denominator of LinearAttentionCell.read: o = S q / max(q . z, eps), z the running sum of phi(k)."""
    from memorax_amd import kernels as K
    B, T, H, d = 2, 12, 3, 64
    x = attn_inputs(B, T, H, p=0.15, seed=5, scale=1.0 / 8)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    if dtype == "bf16":
        for n in ("q", "k", "v"):
            x[n] = bf16_round(x[n])
    q, k, v, done = dev(x["q"], td), dev(x["k"], td), dev(x["v"], td), dev(x["done"])
    z0 = np.abs(np.random.default_rng(1).standard_normal((B, H, d))).astype(np.float32)
    S, z = dev(x["S0"]), dev(z0)
    outs = []
    for t in range(T):
        o, S, z = K.linear_attn_step(q[:, t].contiguous(), k[:, t].contiguous(), v[:, t].contiguous(),
                                     done[:, t].contiguous(), S, z, feature_map="elu1", normalise=True, eps=1e-6)
        outs.append(o)
    o = torch.stack(outs, dim=1)
    # oracle: numerator from the recurrence, normaliser = segmented running sum of phi(k) with carry z0
    num, _ = M.linear_attention(x["q"], x["k"], x["v"], x["done"], x["S0"], "elu1")
    fk, fq = M.elu1(x["k"].astype(np.float64)), M.elu1(x["q"].astype(np.float64))
    zz = z0.astype(np.float64).copy()
    ref = np.zeros_like(num)
    for t in range(T):
        zz = np.where(x["done"][:, t, None, None], 0.0, zz) + fk[:, t]
        den = np.maximum((fq[:, t] * zz).sum(-1, keepdims=True), 1e-6)
        ref[:, t] = num[:, t] / den
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    assert relerr(o, ref) <= tol, relerr(o, ref)
    assert relerr(z, zz) <= 1e-5, relerr(z, zz)


def test_step_inplace_zero_state_and_float_done():
    from memorax_amd import kernels as K
    B, H, d = 4, 2, 64
    x = attn_inputs(B, 1, H, p=0.0, seed=3, delta=True)
    q, k, v, beta = (dev(x[n][:, 0]) for n in ("q", "k", "v", "beta"))
    done_f = torch.tensor([0.0, 1.0, 0.0, 1.0], device="cuda")
    S = dev(x["S0"])
    S_keep = S.clone()
    o_ref, S_ref = K.delta_rule_step(q, k, v, beta, done_f, S)          # out of place, float32 done
    assert torch.equal(S, S_keep)
    o2, S2 = K.delta_rule_step(q, k, v, beta, done_f != 0, S, inplace=True)  # in place, bool done
    assert S2.data_ptr() == S.data_ptr()
    assert torch.equal(o2, o_ref) and torch.equal(S, S_ref)
    # rows whose done flag is set behave as if the state were absent
    o3, S3 = K.delta_rule_step(q, k, v, beta, torch.zeros(B, device="cuda"), None)
    assert torch.equal(o3[1], o_ref[1]) and torch.equal(S3[3], S_ref[3])
    # one step equals the chunked forward kernel at T = 1
    o4, S4, _ = K.delta_rule_fwd(q[:, None].contiguous(), k[:, None].contiguous(), v[:, None].contiguous(),
                                 beta[:, None].contiguous(), (done_f != 0)[:, None], S_keep, save_chk=False)
    assert relerr(o4[:, 0], o_ref.cpu().numpy()) <= 1e-5
    assert relerr(S4, S_ref.cpu().numpy()) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,H,d", [(1024, 4, 64), (5, 3, 32)])
def test_normalised_and_gated_steps_in_place_equal_the_steps_out_of_place(dtype, B, H, d):
    """Several steps in a row with the state (and the key sum) updated where they lie, against the same steps
    writing new arrays: outputs and states bit for bit.  The normaliser z is read by every row of a workgroup and
    written by one of them; many workgroups, so that rows that lag behind the writing one would show."""
    from memorax_amd import kernels as K
    g = torch.Generator(device="cuda").manual_seed(B + d)
    S, z = torch.randn(B, H, d, d, device="cuda", generator=g), torch.rand(B, H, d, device="cuda", generator=g) + 0.5
    S_in, z_in = S.clone(), z.clone()          # updated in place
    Sg, Sg_in = S.clone(), S.clone()
    print(f"case step in place dtype={dtype} B={B} H={H} d={d}", flush=True)
    for step in range(4):
        q, k, v = (torch.randn(B, H, d, device="cuda", generator=g).to(dtype) for _ in range(3))
        glog = -torch.rand(B, H, device="cuda", generator=g)
        done = torch.rand(B, device="cuda", generator=g) < 0.2
        o, S, z = K.linear_attn_step(q, k, v, done, S, z, "elu1", True, 1e-6)
        o2, S2, z2 = K.linear_attn_step(q, k, v, done, S_in, z_in, "elu1", True, 1e-6, inplace=True)
        assert S2.data_ptr() == S_in.data_ptr() and z2.data_ptr() == z_in.data_ptr()
        assert torch.equal(o2, o) and torch.equal(S_in, S) and torch.equal(z_in, z), step
        og, Sg = K.gated_linear_attn_step(q, k, v, glog, done, Sg, "none")
        og2, _ = K.gated_linear_attn_step(q, k, v, glog, done, Sg_in, "none", inplace=True)
        assert torch.equal(og2, og) and torch.equal(Sg_in, Sg), step


def test_step_rejects_bad_arguments():
    from memorax_amd import _lib
    lib = _lib.load()
    t = torch.zeros(64 * 64, device="cuda")
    p = t.data_ptr()
    args = lambda dk: (None, p, p, p, p, p, p, p, p, 1, 1, dk, 64, 0, 0)
    assert lib.mrx_delta_rule_step(*args(64)) == 0
    assert lib.mrx_delta_rule_step(*args(72)) == -2          # unsupported head dim
    assert lib.mrx_delta_rule_step(None, p, p, p, None, p, p, p, p, 1, 1, 64, 64, 0, 0) == -1  # beta missing
    assert lib.mrx_linear_attn_step(None, p, p, p, p, p, None, p, p, None, 1, 1, 64, 64, 0, 0, 7, 1e-6) == -1
    assert lib.mrx_gated_linear_attn_step(None, p, p, p, p, p, p, p, p, 1, 1, 64, 64, 0, 0, 0) == 0
    assert lib.mrx_gated_linear_attn_step(None, p, p, p, None, p, p, p, p, 1, 1, 64, 64, 0, 0, 0) == -1  # g missing
    assert lib.mrx_gated_linear_attn_step(None, p, p, p, p, p, p, p, p, 1, 1, 72, 72, 0, 0, 0) == -2
    torch.cuda.synchronize()
