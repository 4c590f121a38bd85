"""GPU parity of the DeltaNet entry points with the prologue fused (key L2-normalisation and
sigmoid gate inside the kernels) against the oracle composition and its torch-fp64 autograd."""
import numpy as np
import pytest
import torch

from oracle import grad as G
from oracle import memoroid as M
from gpu_util import TOL_BF16, TOL_F32, bf16_round, dev, relerr

pytestmark = pytest.mark.gpu

SHAPES = [(1, 64, 1), (2, 128, 2), (1, 1, 1), (2, 7, 1), (1, 65, 2), (2, 200, 3), (1, 33, 1)]


def _raw_inputs(B, T, H, p, seed, dtype, d=64):
    r = np.random.default_rng(seed)
    x = dict(q=r.standard_normal((B, T, H, d)), v=r.standard_normal((B, T, H, d)),
             k=r.standard_normal((B, T, H, d)) * np.exp(r.standard_normal((B, T, H, 1))),   # norms spread over a decade
             beta=r.standard_normal((B, T, H)) * 1.5, do=r.standard_normal((B, T, H, d)),
             S0=r.standard_normal((B, H, d, d)) * 0.1, dSl=r.standard_normal((B, H, d, d)) * 0.1)
    x = {n: a.astype(np.float32) for n, a in x.items()}
    x["done"] = r.random((B, T)) < p
    if dtype == "bf16":
        for n in ("q", "k", "v", "beta", "do"):
            x[n] = bf16_round(x[n])
    return x


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("p", [0.0, 0.05])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_deltanet_fwd_bwd(shape, p, dtype):
    from memorax_amd import kernels as K
    B, T, H = shape
    x = _raw_inputs(B, T, H, p, B * 100 + T + H + 91, dtype)
    print(f"case deltanet shape={shape} p={p} dtype={dtype}", flush=True)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    tq, tk, tv, tb, tdo = (dev(x[n], td) for n in ("q", "k", "v", "beta", "do"))
    dn = dev(x["done"])
    o, Sl, chk = K.delta_rule_fwd(tq, tk, tv, tb, dn, dev(x["S0"]), prologue=True)
    got = K.delta_rule_bwd(tq, tk, tv, tb, dn, chk, tdo, dev(x["dSl"]), prologue=True)
    ref = G.deltanet_grads(x["q"], x["k"], x["v"], x["beta"], x["done"], x["S0"], x["do"], x["dSl"])
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    errs = {"o": relerr(o, ref["o"]), "S_last": relerr(Sl, ref["S_last"])}
    errs.update({n: relerr(g, ref[n]) for n, g in zip(("dq", "dk", "dv", "dbeta", "dS0"), got)})
    assert all(e <= tol for e in errs.values()), errs
    # without a buffer for the triangular factors the sequential kernel inverts in place
    o3, Sl3, _ = K.delta_rule_fwd(tq, tk, tv, tb, dn, dev(x["S0"]), save_chk=False, prologue=True, tm_scratch=False)
    assert relerr(o3, ref["o"]) <= tol and relerr(Sl3, ref["S_last"]) <= tol
    # fp32: the prologue done by the caller and the plain entry points give the same numbers
    if dtype == "f32":
        kn = torch.nn.functional.normalize(tk, dim=-1)
        o2, Sl2, _ = K.delta_rule_fwd(tq, kn, tv, torch.sigmoid(tb), dn, dev(x["S0"]))
        assert relerr(o, o2.cpu().numpy()) <= 1e-5 and relerr(Sl, Sl2.cpu().numpy()) <= 1e-5


def test_deltanet_key_gradient_is_orthogonal_to_the_key_at_the_benchmark_shape():
    """Size-independent property at benchmark configuration 4's shape: the output is invariant to
    the scale of each key, so dk . k = 0 row by row (up to bf16 rounding of the two factors)."""
    from memorax_amd import kernels as K
    B, T, H = 64, 1024, 8
    g = torch.Generator(device="cuda").manual_seed(3)
    bf = torch.bfloat16
    q, k, v, do = (torch.randn((B, T, H, 64), device="cuda", generator=g).to(bf) for _ in range(4))
    k = (k.float() * torch.exp(torch.randn((B, T, H, 1), device="cuda", generator=g))).to(bf)
    braw = torch.randn((B, T, H), device="cuda", generator=g).to(bf)
    done = torch.rand((B, T), device="cuda", generator=g) < 0.002
    o, Sl, chk = K.delta_rule_fwd(q, k, v, braw, done, None, prologue=True)
    dq, dk, dv, db, _ = K.delta_rule_bwd(q, k, v, braw, done, chk, do, None, want_dS0=False, prologue=True)
    assert all(torch.isfinite(t.float()).all() for t in (o, Sl, dq, dk, dv, db))
    kf, dkf = k.float(), dk.float()
    cos = (kf * dkf).sum(-1).abs() / (kf.norm(dim=-1) * dkf.norm(dim=-1) + 1e-30)
    assert float(cos.max()) <= 2e-2, float(cos.max())
    # scaling the keys by powers of two changes nothing at all
    o2, Sl2, _ = K.delta_rule_fwd(q, (k.float() * 4).to(bf), v, braw, done, None, prologue=True)
    assert torch.equal(o, o2) and torch.equal(Sl, Sl2)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_deltanet_functional_autograd_rollout_and_other_head_dims(dtype):
    from memorax_amd import functional as F
    B, T, H, d = 2, 40, 2, 32
    x = _raw_inputs(B, T, H, 0.05, 7, dtype, d=d)
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    q, k, v, b = (dev(x[n], td).requires_grad_() for n in ("q", "k", "v", "beta"))
    S0 = dev(x["S0"]).requires_grad_()
    o, Sl = F.deltanet(q, k, v, b, dev(x["done"]), S0)
    ((o.float() * dev(x["do"])).sum() + (Sl * dev(x["dSl"])).sum()).backward()
    ref = G.deltanet_grads(x["q"], x["k"], x["v"], x["beta"], x["done"], x["S0"], x["do"], x["dSl"])
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    errs = {"o": relerr(o, ref["o"]), "S_last": relerr(Sl, ref["S_last"])}
    errs.update({n: relerr(t.grad, ref[n]) for n, t in (("dq", q), ("dk", k), ("dv", v), ("dbeta", b), ("dS0", S0))})
    assert all(e <= tol for e in errs.values()), errs
    # acting: T = 1 calls without gradients, state fed back
    with torch.no_grad():
        S, outs = S0.detach(), []
        for t in range(T):
            o1, S = F.deltanet(q[:, t:t + 1].detach(), k[:, t:t + 1].detach(), v[:, t:t + 1].detach(),
                               b[:, t:t + 1].detach(), dev(x["done"])[:, t:t + 1], S)
            outs.append(o1)
    assert relerr(torch.cat(outs, 1), ref["o"]) <= tol and relerr(S, ref["S_last"]) <= tol


def test_deltanet_poison_does_not_cross_episodes():
    from memorax_amd import kernels as K
    B, T, H = 1, 100, 1
    x = _raw_inputs(B, T, H, 0.0, 13, "f32")
    done = np.zeros((B, T), bool)
    done[0, 40] = True
    done[0, 70] = True
    clean = {n: dev(x[n]) for n in ("q", "k", "v", "beta", "do")}
    bad = {n: t.clone() for n, t in clean.items()}
    for n in bad:
        bad[n][0, 40:70] = float("nan")
    outs = []
    for inp in (clean, bad):
        o, Sl, chk = K.delta_rule_fwd(inp["q"], inp["k"], inp["v"], inp["beta"], dev(done), dev(x["S0"]), prologue=True)
        g = K.delta_rule_bwd(inp["q"], inp["k"], inp["v"], inp["beta"], dev(done), chk, inp["do"], dev(x["dSl"]),
                             prologue=True)
        outs.append((o, Sl) + tuple(g))
    keep = np.ones(T, bool)
    keep[40:70] = False
    for name, a, b_ in zip(("o", "S_last", "dq", "dk", "dv", "dbeta", "dS0"), outs[0], outs[1]):
        if a.dim() >= 3 and a.shape[1] == T:
            a, b_ = a[:, keep], b_[:, keep]
        bad_at = (a != b_).nonzero()
        assert bad_at.numel() == 0, (name, bad_at[:4].tolist(), a[a != b_][:4].tolist(), b_[a != b_][:4].tolist())


def test_chunk64_build_agrees_with_the_default_build():
    """libmemorax_amd_c64.so (the delta rule's bf16 kernels on 64-step chunks, loaded only by
    bench.py --all) computes the same function: forward and backward through its C ABI against the
    default library on the same inputs, ragged length, resets, non-zero initial state."""
    import ctypes
    import os
    from memorax_amd import _lib
    from memorax_amd import kernels as K
    path = os.path.join(os.path.dirname(_lib.LIB_PATH), "libmemorax_amd_c64.so")
    if not os.path.exists(path):
        pytest.skip("libmemorax_amd_c64.so not built")
    lib = ctypes.CDLL(path)
    for name in ("mrx_delta_rule_fwd", "mrx_delta_rule_bwd", "mrx_delta_chunk_size"):
        res, args = _lib.SIGNATURES[name]
        getattr(lib, name).restype, getattr(lib, name).argtypes = res, args
    assert lib.mrx_delta_chunk_size(_lib.MRX_BF16) == 64
    B, T, H = 3, 200, 2
    bf = torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(64)
    q, k, v, do = (torch.randn((B, T, H, 64), device="cuda", generator=g).to(bf) for _ in range(4))
    k = torch.nn.functional.normalize(k.float(), dim=-1).to(bf)
    beta = torch.rand((B, T, H), device="cuda", generator=g).to(bf)
    done = (torch.rand((B, T), device="cuda", generator=g) < 0.02).view(torch.uint8).contiguous()
    S0 = torch.randn((B, H, 64, 64), device="cuda", generator=g) * 0.1
    print("case chunk64 build", flush=True)
    o, Sl, chk = K.delta_rule_fwd(q, k, v, beta, done, S0)
    ref = (o, Sl) + tuple(K.delta_rule_bwd(q, k, v, beta, done, chk, do))
    NC = (T + 63) // 64
    p = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    st = torch.cuda.current_stream().cuda_stream
    o2, Sl2 = torch.empty_like(v), torch.empty_like(S0)
    S_chk = torch.empty((B, H, NC, 64, 64), dtype=bf, device="cuda")
    Tm_chk = torch.empty((B, H, NC, 64, 64), dtype=bf, device="cuda")
    rc = lib.mrx_delta_rule_fwd(st, p(q), p(k), p(v), p(beta), p(done), p(S0), p(o2), p(Sl2), p(S_chk), p(Tm_chk),
                                B, T, H, 64, 64, _lib.MRX_BF16, _lib.MRX_DONE_U8, _lib.MRX_FACTORS_AUTO, _lib.MRX_RESETS_AUTO)
    assert rc == 0, rc
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    db, dS0 = torch.empty_like(beta), torch.empty_like(S0)
    rc = lib.mrx_delta_rule_bwd(st, p(q), p(k), p(v), p(beta), p(done), p(S_chk), p(Tm_chk), p(do), None, p(dq), p(dk),
                                p(dv), p(db), p(dS0), B, T, H, 64, 64, _lib.MRX_BF16, _lib.MRX_DONE_U8, _lib.MRX_RESETS_AUTO)
    assert rc == 0, rc
    torch.cuda.synchronize()
    for name, a, b_ in zip(("o", "S_last", "dq", "dk", "dv", "dbeta", "dS0"), (o2, Sl2, dq, dk, dv, db, dS0), ref):
        assert relerr(a, b_.float().cpu().numpy()) <= TOL_BF16, name
    # the chunk-parallel factor kernel exists for 32-step chunks only
    rc = lib.mrx_delta_rule_fwd(st, p(q), p(k), p(v), p(beta), p(done), p(S0), p(o2), p(Sl2), p(S_chk), p(Tm_chk),
                                B, T, H, 64, 64, _lib.MRX_BF16, _lib.MRX_DONE_U8, _lib.MRX_FACTORS_PARALLEL, _lib.MRX_RESETS_AUTO)
    assert rc == -2, rc


def test_pattern_probe_of_the_measurement_build_moves_the_bytes_it_claims():
    """mrx_pattern_probe (libmemorax_amd_clk.so, loaded only by bench.py) is what the kernels' times are read
    against, so it has to touch what it says: every row of every output array is written (here: with the XOR of
    the inputs' rows, segments rotated by one, XOR the residual block of the chunk), the residual block written
    back, in both walking directions; bad arguments are refused before anything is launched."""
    import ctypes
    import os
    from memorax_amd import _lib
    path = os.path.join(os.path.dirname(_lib.LIB_PATH), "libmemorax_amd_clk.so")
    if not os.path.exists(path):
        pytest.skip("libmemorax_amd_clk.so not built")
    lib = ctypes.CDLL(path)
    vp, i64 = ctypes.c_void_p, ctypes.c_int64
    f = lib.mrx_pattern_probe
    f.argtypes = [vp, ctypes.POINTER(vp), ctypes.c_int, ctypes.POINTER(vp), ctypes.c_int, vp, ctypes.c_int, vp, ctypes.c_int,
                  i64, i64, i64, ctypes.c_int, ctypes.c_int]
    f.restype = ctypes.c_int
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator(device="cuda").manual_seed(7)
    for (n_in, n_out, C, res_in, res_out, reverse) in ((3, 1, 64, 0, 0, 0), (4, 3, 32, 4096, 0, 1), (3, 1, 32, 2048, 8192, 0)):
        B, T, H = 8, 4 * C, 2
        NC = T // C
        print(f"case pattern probe n_in={n_in} n_out={n_out} C={C}", flush=True)
        ins = [torch.randint(-2**31, 2**31 - 1, (B, T, H, 32), dtype=torch.int32, device="cuda", generator=g) for _ in range(n_in)]
        outs = [torch.zeros((B, T, H, 32), dtype=torch.int32, device="cuda") for _ in range(n_out)]
        rin = torch.randint(-2**31, 2**31 - 1, (B * H, NC, max(res_in, 16) // 4), dtype=torch.int32, device="cuda", generator=g)
        rout = torch.zeros((B * H, NC, max(res_out, 16) // 4), dtype=torch.int32, device="cuda")
        pi = (vp * n_in)(*[a.data_ptr() for a in ins])
        po = (vp * n_out)(*[a.data_ptr() for a in outs])
        rc = f(st, pi, n_in, po, n_out, rin.data_ptr(), res_in, rout.data_ptr(), res_out, B, T, H, C, reverse)
        assert rc == 0, rc
        torch.cuda.synchronize()
        x = ins[0]
        for a in ins[1:]:
            x = x ^ a
        # rows as 8 segments of 4 words: segment s of the output holds segment (s + 1) % 8 of the XOR of the inputs
        x = x.view(B, T, H, 8, 4).roll(-1, dims=3)
        # ... XOR, per thread, the words of the residual block that thread took (thread = 8 * row-in-pass + segment)
        if res_in:
            segs = res_in // 16
            r = rin.view(B, H, NC, segs, 4)
            acc = torch.zeros((B, H, NC, 256, 4), dtype=torch.int32, device="cuda")
            for s0 in range(0, segs, 256):
                blk = r[:, :, :, s0:s0 + 256]
                acc[:, :, :, :blk.shape[3]] ^= blk
            # thread tid handles rows tid // 8 + 32 p of the chunk, segment tid % 8
            acc = acc.view(B, H, NC, 32, 8, 4)                      # (row in pass, segment)
            per_row = acc.repeat(1, 1, 1, C // 32, 1, 1).view(B, H, NC * C, 8, 4).permute(0, 2, 1, 3, 4)
            x = x ^ per_row
        for o_ in outs:
            assert torch.equal(o_.view(B, T, H, 8, 4), x), (n_in, n_out, C)
        if res_out:
            want = torch.zeros_like(rout.view(B, H, NC, -1, 4))
            if res_in:
                segs_o = res_out // 16
                acc2 = torch.zeros((B, H, NC, 256, 4), dtype=torch.int32, device="cuda")
                r = rin.view(B, H, NC, res_in // 16, 4)
                for s0 in range(0, res_in // 16, 256):
                    blk = r[:, :, :, s0:s0 + 256]
                    acc2[:, :, :, :blk.shape[3]] ^= blk
                for s0 in range(0, segs_o, 256):
                    n = min(256, segs_o - s0)
                    want[:, :, :, s0:s0 + n] = acc2[:, :, :, :n]
            assert torch.equal(rout.view(B, H, NC, -1, 4), want)
    # refused: chunk length, ragged T, unsupported array counts, residual bytes without a pointer
    assert f(st, pi, 3, po, 1, None, 0, None, 0, 8, 100, 2, 32, 0) == -1
    assert f(st, pi, 3, po, 1, None, 0, None, 0, 8, 128, 2, 48, 0) == -1
    assert f(st, pi, 2, po, 1, None, 0, None, 0, 8, 128, 2, 32, 0) == -2
    assert f(st, pi, 3, po, 1, None, 64, None, 0, 8, 128, 2, 32, 0) == -1
