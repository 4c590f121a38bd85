"""The stateless blocks and wrappers of the block library (blocks/{ffn,residual,stack}.py), which are
plain dense arithmetic around the sequence models: checked on the CPU against the formulas the
reference's modules spell out."""
import torch
import torch.nn.functional as F

from memorax_amd import sequence_models as sm


def _x(B=3, T=5, Fe=8, seed=0):
    return torch.randn((B, T, Fe), generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


def test_glu_splits_gate_then_value():
    m = sm.GLU(8, expansion_factor=2).double()
    x = _x()
    carry, y = m(x, done=None, initial_carry=None)
    u = x @ m.up_proj.weight.T
    g = u[..., :16]
    tanh_gelu = 0.5 * g * (1 + torch.tanh((2 / torch.pi) ** 0.5 * (g + 0.044715 * g ** 3)))   # jax.nn.gelu's default form
    want = (tanh_gelu * u[..., 16:]) @ m.down_proj.weight.T   # ffn.py:108-121
    assert carry is None and m.up_proj.bias is None and m.down_proj.bias is None
    assert torch.allclose(y, want, atol=1e-12)
    assert m.initialize_carry(None, (3, 8)) is None


def test_ffn_and_projection():
    m = sm.FFN(8, expansion_factor=4, activation=torch.tanh).double()
    x = _x(seed=1)
    carry, y = m(x)
    want = torch.tanh(x @ m.up.weight.T + m.up.bias) @ m.down.weight.T + m.down.bias   # ffn.py:31-45
    assert carry is None and torch.allclose(y, want, atol=1e-12)
    p = sm.Projection(8, 6, use_bias=False).double()
    carry, y = p(x)
    assert carry is None and p.proj.bias is None and torch.allclose(y, x @ p.proj.weight.T, atol=1e-12)


def test_gated_residual_gates_the_branch_not_the_input():
    inner = sm.FFN(8, 2).double()
    m = sm.GatedResidual(inner, 8).double()
    x = _x(seed=2)
    carry, y = m(x)
    gate = torch.sigmoid(x @ m.gate.weight.T + m.gate.bias)   # residual.py:54-60
    assert carry is None and torch.allclose(y, x + gate * inner(x)[1], atol=1e-12)


def test_stack_threads_one_carry_per_block_and_none_for_stateless_blocks():
    class Counter(torch.nn.Module):   # a block with a carry: running sum over time from the carry
        def forward(self, inputs, done=None, initial_carry=None, **kw):
            h = inputs.cumsum(dim=1) + (0 if initial_carry is None else initial_carry)
            return h[:, -1:], h

        def initialize_carry(self, key, input_shape):
            return torch.zeros((input_shape[0], 1, input_shape[1]), dtype=torch.float64)

    class Bare(torch.nn.Module):      # a block without initialize_carry (stack.py:53-58)
        def forward(self, inputs, done=None, initial_carry=None, **kw):
            return None, 2 * inputs

    blocks = [sm.Residual(sm.PreNorm(sm.GLU(8, 2), 8)), Counter(), Bare()]
    stack = sm.Stack(blocks).double()
    x = _x(seed=3)
    init = stack.initialize_carry(None, (3, 8))
    assert init[0] is None and init[2] is None and init[1].shape == (3, 1, 8)
    carries, y = stack(x, done=None, initial_carry=init)
    h = blocks[0](x)[1].cumsum(dim=1)
    assert carries[0] is None and carries[2] is None
    assert torch.allclose(carries[1], h[:, -1:]) and torch.allclose(y, 2 * h)
    # two halves with the carried tuple equal one call
    c1, y1 = stack(x[:, :2], initial_carry=init)
    c2, y2 = stack(x[:, 2:], initial_carry=c1)
    assert torch.allclose(torch.cat((y1, y2), dim=1), y) and torch.allclose(c2[1], carries[1])


def test_prenorm_defaults_to_layer_norm_and_takes_rms_norm():
    """normalization.py:22 defaults to flax's LayerNorm: mean subtracted, variance normalised with
    eps = 1e-6, learned scale and bias; the torso configuration passes RMSNorm explicitly."""
    inner = sm.Projection(8, 8).double()
    x = _x(seed=4) * 3 + 1.5
    m = sm.PreNorm(inner, 8).double()
    with torch.no_grad():
        m.norm.weight.copy_(torch.linspace(0.5, 1.5, 8))
        m.norm.bias.copy_(torch.linspace(-0.2, 0.2, 8))
    mu, var = x.mean(-1, keepdim=True), x.var(-1, unbiased=False, keepdim=True)
    xn = (x - mu) / torch.sqrt(var + 1e-6) * m.norm.weight + m.norm.bias
    carry, y = m(x)
    assert carry is None and torch.allclose(y, inner(xn)[1], atol=1e-12)
    r = sm.PreNorm(inner, 8, norm=sm.RMSNorm).double()
    xr = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6) * r.norm.scale
    assert torch.allclose(r(x)[1], inner(xr)[1], atol=1e-6)   # the RMS statistics are taken in fp32
    p = sm.PostNorm(inner, 8).double()                         # normalization.py:38-65
    yi = inner(x)[1]
    want = (yi - yi.mean(-1, keepdim=True)) / torch.sqrt(yi.var(-1, unbiased=False, keepdim=True) + 1e-6)
    assert torch.allclose(p(x)[1], want * p.norm.weight + p.norm.bias, atol=1e-12)


def test_mingru_cell_sows_the_mean_gate_when_it_is_read():
    """min_gru.py:63 records mean(z) of every call; here the mean is formed on first reading."""
    cell = sm.MinGRUCell(6, in_features=8)
    x = _x(seed=4).float()
    proj = cell(x)
    assert callable(dict.__getitem__(cell.intermediates, "gate"))     # nothing computed yet
    want = (x @ cell.z.weight.T).mean()
    assert torch.allclose(cell.intermediates["gate"], want, atol=1e-6)
    assert not callable(dict.__getitem__(cell.intermediates, "gate"))  # kept once read
    assert proj.z.shape == (3, 5, 6) and not cell.intermediates["gate"].requires_grad
