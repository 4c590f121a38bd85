"""The acting step captured in a HIP graph (memorax_amd.rollout.GraphedStep): every replay against the eager step
on the same inputs, bit for bit, with eager work and synchronisations between the replays."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _torso(sm, Fe, d, H):
    torch.manual_seed(11)
    blocks = [sm.Residual(sm.PreNorm(sm.Memoroid(sm.DeltaNetCell(Fe, d, H)), Fe, norm=sm.RMSNorm)),
              sm.Residual(sm.PreNorm(sm.GatedLinearRecurrence(Fe), Fe, norm=sm.RMSNorm)),
              sm.Residual(sm.PreNorm(sm.LinearAttention(sm.LinearAttentionCell(Fe, d, H)), Fe)),
              sm.Residual(sm.PreNorm(sm.GLU(Fe, expansion_factor=2), Fe))]
    torso = sm.Stack(blocks).cuda()
    for p in torso.parameters():
        if p.dim() > 1:
            torch.nn.init.normal_(p, 0.0, 0.05)
    return torso


def _flat(tree, out):
    for v in tree:
        if isinstance(v, (tuple, list)):
            _flat(v, out)
        elif v is not None:
            out.append(v)
    return out


@pytest.mark.parametrize("autocast", [None, torch.bfloat16])
def test_graphed_step_equals_the_eager_step(autocast):
    from memorax_amd import sequence_models as sm
    from memorax_amd.rollout import GraphedStep
    B, Fe, d, H = 6, 128, 64, 2
    torso = _torso(sm, Fe, d, H)
    g = torch.Generator(device="cuda").manual_seed(5)
    xs = [torch.randn(B, 1, Fe, device="cuda", generator=g) for _ in range(6)]
    ds = [torch.rand(B, 1, device="cuda", generator=g) < 0.3 for _ in range(6)]

    def eager(x, done, carry):
        with torch.no_grad(), torch.autocast("cuda", dtype=autocast or torch.bfloat16, enabled=autocast is not None):
            return torso(x, done, carry)
    carry, want = torso.initialize_carry(None, (B, Fe)), []
    for x, done in zip(xs, ds):
        carry, y = eager(x, done, carry)
        want.append((y.clone(), [t.clone() for t in _flat(carry, [])]))
    act = GraphedStep(torso, B, Fe, autocast=autocast)
    assert len(act._pairs) < len(_flat(carry, []))     # the matrix states are updated where they lie, not copied back
    print(f"case graphed step autocast={autocast}", flush=True)
    for rep in range(2):                     # the second round after reset(): from the initial carry again
        for i, (x, done) in enumerate(zip(xs, ds)):
            y = act(x, done if i % 2 else done.float())      # flags of either type
            torch.cuda.synchronize()
            assert torch.equal(y, want[i][0]), (rep, i)
            for got, ref in zip(_flat(act.carry, []), want[i][1]):
                assert torch.equal(got, ref), (rep, i)
            _ = (torch.randn(256, 256, device="cuda") @ torch.randn(256, 256, device="cuda")).sum().item()   # eager work between replays
        act.reset()
    # a carry handed in: continue from step 3's carry with step 4's inputs
    mid, _ = eager(xs[0], ds[0], None)
    act.set_carry(mid)
    y = act(xs[1], ds[1])
    _, y_ref = eager(xs[1], ds[1], mid)
    assert torch.equal(y, y_ref)
    # weights written after the capture (an optimiser step) reach the graph's copies with the next call
    with torch.no_grad():
        for p in torso.parameters():
            p.add_(0.01 * torch.randn_like(p))
    act.set_carry(mid)
    y = act(xs[1], ds[1])
    _, y_ref = eager(xs[1], ds[1], mid)
    assert torch.equal(y, y_ref)
    # outside a GraphedStep a step leaves the carry it was given untouched
    before = [t.clone() for t in _flat(mid, [])]
    eager(xs[2], ds[2], mid)
    for a, b in zip(_flat(mid, []), before):
        assert torch.equal(a, b)

