"""The entry point that allocates nothing: mrx_delta_rule_fwd_noalloc keeps the triangular factors in
the library's static device array.  Called through the C ABI (ctypes) with caller-owned inputs and
outputs and compared with mrx_delta_rule_fwd given the same factors buffer explicitly (same kernels:
bit-identical; the tolerance of the parity tests is asserted as well), on two calls in a row, the second
with a smaller input, so that stale factors of the first call sit in the array during the second."""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import TOL_BF16, TOL_F32, relerr

pytestmark = pytest.mark.gpu


def _inputs(B, T, H, dtype, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    q, k, v = (torch.randn((B, T, H, 64), device="cuda", generator=g) for _ in range(3))
    k = torch.nn.functional.normalize(k, dim=-1)
    beta = torch.rand((B, T, H), device="cuda", generator=g)
    done = (torch.rand((B, T), device="cuda", generator=g) < 0.02).view(torch.uint8).contiguous()
    S0 = torch.randn((B, H, 64, 64), device="cuda", generator=g) * 0.1
    return [t.to(dtype).contiguous() for t in (q, k, v, beta)] + [done, S0]


def _call_pair(lib, _lib, B, T, H, dtype, seed):
    q, k, v, beta, done, S0 = _inputs(B, T, H, dtype, seed)
    dt = _lib.MRX_BF16 if dtype == torch.bfloat16 else _lib.MRX_F32
    NC = (T + 31) // 32
    st = torch.cuda.current_stream().cuda_stream
    p = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    # reference: the existing entry point with a caller-owned factors buffer, no residual checkpoints
    o_ref, Sl_ref = torch.empty_like(v), torch.empty_like(S0)
    tm = torch.empty((B, H, NC, 32, 32), dtype=dtype, device="cuda")
    rc = lib.mrx_delta_rule_fwd(st, p(q), p(k), p(v), p(beta), p(done), p(S0), p(o_ref), p(Sl_ref), None, p(tm),
                                B, T, H, 64, 64, dt, _lib.MRX_DONE_U8, _lib.MRX_FACTORS_PARALLEL, _lib.MRX_RESETS_AUTO)
    assert rc == 0, rc
    # outputs pre-filled so that an entry point that wrote nothing cannot pass
    o, Sl = torch.full_like(v, float("nan")), torch.full_like(S0, float("nan"))
    rc = lib.mrx_delta_rule_fwd_noalloc(st, p(q), p(k), p(v), p(beta), p(done), p(S0), p(o), p(Sl),
                                        B, T, H, 64, 64, dt, _lib.MRX_DONE_U8)
    assert rc == 0, rc
    torch.cuda.synchronize()
    tol = TOL_BF16 if dtype == torch.bfloat16 else TOL_F32
    assert relerr(o, o_ref.float().cpu().numpy()) <= tol
    assert relerr(Sl, Sl_ref.cpu().numpy()) <= tol
    assert torch.equal(o, o_ref) and torch.equal(Sl, Sl_ref)
    return o, Sl


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_noalloc_matches_delta_rule_fwd_twice_in_a_row(dtype):
    from memorax_amd import _lib
    lib = _lib.load()
    assert lib.mrx_init(torch.cuda.current_device()) == 0
    print(f"case noalloc first call dtype={dtype}", flush=True)
    _call_pair(lib, _lib, 6, 200, 4, dtype, 11)   # 6*4*7 = 168 chunks, ragged last chunk
    print(f"case noalloc second, smaller call dtype={dtype}", flush=True)
    _call_pair(lib, _lib, 3, 70, 2, dtype, 12)    # 3*2*3 = 18 chunks over the stale factors of the first call


def test_noalloc_against_the_oracle():
    """The same call against the fp64 oracle recurrence (not only against the sibling entry point)."""
    from memorax_amd import kernels as K
    from oracle import memoroid as M
    x = M.make_inputs(4, (2, 100, 2, 64))
    bf = torch.bfloat16
    rb = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(bf).float().numpy()  # noqa: E731
    xb = {n: rb(x[n]) for n in ("q", "k", "v", "beta")}
    t = {n: torch.from_numpy(xb[n]).cuda().to(bf) for n in xb}
    print("case noalloc vs oracle", flush=True)
    o, Sl = K.delta_rule_fwd_noalloc(t["q"], t["k"], t["v"], t["beta"], torch.from_numpy(x["done"]).cuda())
    ro, rS = M.delta_rule(xb["q"], xb["k"], xb["v"], xb["beta"], x["done"])
    assert relerr(o, ro) <= TOL_BF16 and relerr(Sl, rS) <= TOL_BF16


def test_noalloc_rejects_problems_beyond_the_scratch_size():
    from memorax_amd import _lib
    lib = _lib.load()
    one = ctypes.c_void_p(256)
    # 16385 chunks of bf16: one more than MRX_NOALLOC_SCRATCH_BYTES holds -> refused before any launch
    rc = lib.mrx_delta_rule_fwd_noalloc(None, one, one, one, one, one, None, one, None, 16385, 32, 1, 64, 64,
                                        _lib.MRX_BF16, _lib.MRX_DONE_U8)
    assert rc == -4 and b"scratch" in lib.mrx_status_string(rc)
    rc = lib.mrx_delta_rule_fwd_noalloc(None, one, one, one, one, one, None, one, None, 8193, 32, 1, 64, 64,
                                        _lib.MRX_F32, _lib.MRX_DONE_U8)
    assert rc == -4
