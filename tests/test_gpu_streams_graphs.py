"""The entry points only enqueue work on the stream they are given: results on a side stream
equal those on the default stream, and a captured HIP graph of a forward + backward pass replays
correctly on new input values (several replays, eager work and synchronisations in between)."""
import numpy as np
import pytest
import torch

from gpu_util import attn_inputs, bf16_round, dev

pytestmark = pytest.mark.gpu


def _delta_inputs(seed, B=2, T=160, H=2):
    x = attn_inputs(B, T, H, p=0.03, seed=seed, delta=True)
    bf = torch.bfloat16
    t = {n: dev(bf16_round(x[n]), bf) for n in ("q", "k", "v", "beta")}
    t["do"] = dev(bf16_round(np.random.default_rng(seed + 1).standard_normal((B, T, H, 64)).astype(np.float32)), bf)
    t["done"] = dev(x["done"])
    return t


def test_side_stream_equals_default_stream():
    from memorax_amd import kernels as K
    t = _delta_inputs(1)
    ref_f = K.delta_rule_fwd(t["q"], t["k"], t["v"], t["beta"], t["done"])
    ref_b = K.delta_rule_bwd(t["q"], t["k"], t["v"], t["beta"], t["done"], ref_f[2], t["do"], None)
    a = torch.rand(2, 50, 40, device="cuda")
    ref_s = K.linear_scan_fwd(a, a + 1, t["done"][:, :50].contiguous())
    torch.cuda.synchronize()
    side = torch.cuda.Stream()   # default priority
    with torch.cuda.stream(side):
        got_f = K.delta_rule_fwd(t["q"], t["k"], t["v"], t["beta"], t["done"])
        got_b = K.delta_rule_bwd(t["q"], t["k"], t["v"], t["beta"], t["done"], got_f[2], t["do"], None)
        got_s = K.linear_scan_fwd(a, a + 1, t["done"][:, :50].contiguous())
    side.synchronize()
    assert torch.equal(got_f[0], ref_f[0]) and torch.equal(got_f[1], ref_f[1])
    for g, r in zip(got_b, ref_b):
        assert torch.equal(g, r)
    assert torch.equal(got_s[0], ref_s[0])


def test_graph_replays_of_forward_and_backward():
    from memorax_amd import kernels as K
    K.init()   # per-device set-up (LDS limits of every kernel) before anything is captured; idempotent
    K.init(torch.cuda.current_device())
    static = _delta_inputs(2)
    # first calls outside the capture: they size the buffers
    o, Sl, chk = K.delta_rule_fwd(static["q"], static["k"], static["v"], static["beta"], static["done"])
    fwd_out = (o, Sl, chk[0], chk[1])
    bwd_out = K.delta_rule_bwd(static["q"], static["k"], static["v"], static["beta"], static["done"], chk,
                               static["do"], None, want_dS0=False)
    sa = torch.rand(4, 96, 128, device="cuda")
    sb = torch.randn(4, 96, 128, device="cuda")
    sdone = torch.rand(4, 96, device="cuda") < 0.05
    sh = torch.empty_like(sa)
    torch.cuda.synchronize()

    def work():
        K.delta_rule_fwd(static["q"], static["k"], static["v"], static["beta"], static["done"], out=fwd_out)
        K.delta_rule_bwd(static["q"], static["k"], static["v"], static["beta"], static["done"], chk, static["do"],
                         None, want_dS0=False, out=bwd_out)
        h, _, _ = K.linear_scan_fwd(sa, sb, sdone, want_P=False)
        sh.copy_(h)

    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work()   # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    with torch.cuda.graph(g):
        work()
    for rep in range(4):
        new = _delta_inputs(10 + rep)
        for n, tnew in new.items():
            static[n].copy_(tnew)
        sa.copy_(torch.rand_like(sa))
        sb.copy_(torch.randn_like(sb))
        g.replay()
        torch.cuda.synchronize()
        got = [x.clone() for x in (fwd_out[0], fwd_out[1]) + tuple(bwd_out[:4])] + [sh.clone()]
        # eager results on fresh buffers, with unrelated eager work before them
        _ = (torch.randn(256, 256, device="cuda") @ torch.randn(256, 256, device="cuda")).sum().item()
        ef = K.delta_rule_fwd(new["q"], new["k"], new["v"], new["beta"], new["done"])
        eb = K.delta_rule_bwd(new["q"], new["k"], new["v"], new["beta"], new["done"], ef[2], new["do"], None,
                              want_dS0=False)
        eh, _, _ = K.linear_scan_fwd(sa, sb, sdone, want_P=False)
        ref = [ef[0], ef[1]] + list(eb[:4]) + [eh]
        for i, (a, b) in enumerate(zip(got, ref)):
            assert torch.equal(a, b), (rep, i)


def test_graph_replays_of_the_chunk_parallel_pair_and_the_gated_backward():
    """The chunk-parallel pair enqueues three kernels per call, the gated backward carries its running
    sum for dg across chunks, and head dim 32 runs the library's second build: captured once, replayed
    on fresh inputs with eager work in between, every replay equal to the eager calls bit for bit."""
    from memorax_amd import kernels as K
    K.init()
    B, T, H, d = 2, 700, 2, 32
    gen = torch.Generator(device="cuda").manual_seed(3)

    def fresh():
        x = {n: (torch.randn((B, T, H, d), device="cuda", generator=gen) / 6).to(torch.bfloat16) for n in ("q", "k", "v", "do")}
        x["g"] = -torch.rand((B, T, H), device="cuda", generator=gen) * 0.3
        x["done"] = (torch.rand((B, T), device="cuda", generator=gen) < 0.01).to(torch.uint8)
        return x

    static = fresh()

    def work():
        o, Sl, chk = K.linear_attn_fwd(static["q"], static["k"], static["v"], static["done"], None, 1, chunk_parallel=True)
        gr = K.linear_attn_bwd(static["q"], static["k"], static["v"], static["done"], chk, static["do"], Sl, 1)
        o2, Sl2, chk2 = K.gated_linear_attn_fwd(static["q"], static["k"], static["v"], static["g"], static["done"], None, 0)
        gr2 = K.gated_linear_attn_bwd(static["q"], static["k"], static["v"], static["g"], static["done"], chk2,
                                      static["do"], Sl2, 0, S_last=Sl2)
        return [o, Sl, *gr, o2, Sl2, *gr2]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        outs = work()
    for rep in range(3):
        new = fresh()
        for n, t in new.items():
            static[n].copy_(t)
        g.replay()
        torch.cuda.synchronize()
        got = [x.clone() for x in outs]
        _ = (torch.randn(128, 128, device="cuda") @ torch.randn(128, 128, device="cuda")).sum().item()
        ref = work()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, ref)):
            assert torch.equal(a, b), (rep, i)
