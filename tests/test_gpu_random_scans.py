"""Seeded random sweep of the diagonal-scan kernels against the oracle: shapes on both sides of the planner's
thresholds (columns per row, sequences, time steps), float32 / complex64 / the MinGRU map, arrays in bfloat16
with float32 inside, time-invariant
coefficients, optional carries and final-state gradients, done as bool or float32, and operands that start
4 or 8 bytes off a 16-byte boundary (the planner then narrows its vectors)."""
import numpy as np
import pytest
import torch

from oracle import grad as G
from oracle import memoroid as M

pytestmark = pytest.mark.gpu
TOL = 1e-4
CASES_PER_SEED = 10
DS = [1, 3, 8, 31, 64, 65, 96, 128, 130, 192, 256, 258, 384, 512, 1000, 1024]
TS_ = [1, 2, 7, 8, 9, 63, 64, 65, 127, 128, 129, 200, 513, 1024, 1500]
BS = [1, 2, 3, 8, 17, 64, 130, 512]


def relerr(x, y):
    x = x.detach().cpu().numpy()
    return float(np.abs(x - y).max() / max(np.abs(y).max(), 1e-30))


def _dev(x, shift):
    """x on the device, its first element `shift` elements past a 16-byte boundary."""
    flat = torch.from_numpy(np.ascontiguousarray(x)).reshape(-1)
    buf = torch.empty(flat.numel() + shift, dtype=flat.dtype, device="cuda")
    out = buf[shift:]
    out.copy_(flat)
    return out.reshape(x.shape)


def _dev_bf16(x, shift):
    """x as bfloat16 on the device, its first element `shift` elements (2 bytes each) past a 16-byte boundary."""
    flat = torch.from_numpy(np.ascontiguousarray(x)).reshape(-1).bfloat16()
    buf = torch.empty(flat.numel() + shift, dtype=torch.bfloat16, device="cuda")
    out = buf[shift:]
    out.copy_(flat)
    return out.reshape(x.shape)


@pytest.mark.parametrize("seed", range(8))
def test_random_scans(seed):
    from memorax_amd import kernels as K
    rng = np.random.default_rng(2000 + seed)
    failures = []
    for it in range(CASES_PER_SEED):
        kind = str(rng.choice(["f32", "c64", "mingru", "f32", "mingru"]))
        half = kind != "c64" and bool(rng.integers(0, 3) == 0)  # the (B,T,D) arrays in bfloat16, float32 inside
        while True:
            B, T, D = int(rng.choice(BS)), int(rng.choice(TS_)), int(rng.choice(DS))
            if B * T * D <= 3_000_000:
                break
        ti = kind != "mingru" and bool(rng.integers(0, 4) == 0)  # time-invariant coefficients
        p = float(rng.choice([0.0, 0.02, 0.3]))
        shift = int(rng.choice([0, 0, 1, 2]))
        use_h0, use_P0, use_gl, done_f32 = (bool(rng.integers(0, 2)) for _ in range(4))
        desc = f"seed={seed} it={it} {kind}{'/bf16' if half else ''} B={B} T={T} D={D} ti={ti} p={p} shift={shift} h0={use_h0} P0={use_P0} gl={use_gl} done_f32={done_f32}"
        print("case", desc, flush=True)
        cplx = kind == "c64"
        rnd = (lambda *s: (rng.standard_normal(s) + 1j * rng.standard_normal(s)).astype(np.complex64)) if cplx \
            else (lambda *s: rng.standard_normal(s).astype(np.float32))
        done = rng.random((B, T)) < p
        tdone = torch.from_numpy(done.astype(np.float32) if done_f32 else done).cuda()
        rb = (lambda x: torch.from_numpy(x).bfloat16().float().numpy()) if half else (lambda x: x)  # round to bfloat16
        b, g = rb(rnd(B, T, D)), rb(rnd(B, T, D))
        h0 = rnd(B, D) if use_h0 else None
        gl = rnd(B, D) if use_gl else None
        d = lambda x: None if x is None else _dev(x, shift)                       # carries: float32 / complex64
        da_ = lambda x: d(x).bfloat16() if half and shift == 0 else (_dev_bf16(x, shift) if half else d(x))  # arrays
        tol = 2e-2 if half else TOL                                               # array outputs; carries stay at TOL
        errs = {}
        if kind == "mingru":
            z, x = rb(2 * b), rb(2 * rnd(B, T, D))
            h0 = None if h0 is None else np.exp(h0)
            P0 = rng.uniform(0.5, 1.0, (B, D)).astype(np.float32) if use_P0 else None
            h, hl, Pl = K.mingru_scan_fwd(da_(z), da_(x), tdone, d(h0), d(P0))
            a, bb = M.mingru_linear_coeffs(z, x)
            rh, rhl, rPl = M.diag_scan(a, bb, done, h0, P0)
            dz, dx, dh0 = K.mingru_scan_bwd(da_(z), da_(x), h, tdone, d(h0), da_(g), d(gl))
            da, lam, rdh0 = M.diag_scan_bwd(a, rh, done, g, h0, gl)
            s, x64 = M.sigmoid(z.astype(np.float64)), x.astype(np.float64)
            rdz = s * (1 - s) * (np.where(x64 >= 0, x64 + 0.5, M.sigmoid(x64)) * lam - da)
            rdx = lam * s * np.where(x64 >= 0, 1.0, M.sigmoid(x64) * (1 - M.sigmoid(x64)))
            errs = {"h": relerr(h.float(), rh), "dz": relerr(dz.float(), rdz), "dx": relerr(dx.float(), rdx)}
            carr = {"h_last": relerr(hl, rhl), "P_last": relerr(Pl, rPl)}
            if use_h0:
                errs["dh0"] = relerr(dh0, rdh0)
        else:
            ashape = (D,) if ti else (B, T, D)
            if cplx:
                a = (rng.uniform(0.8, 0.999, ashape) * np.exp(1j * rng.uniform(0, 3, ashape))).astype(np.complex64)
                P0 = (rng.uniform(0.5, 1.0, (B, D)) * np.exp(1j * rng.uniform(0, 3, (B, D)))).astype(np.complex64) if use_P0 else None
            else:
                a = rb(rng.uniform(0.8, 0.999, ashape).astype(np.float32))
                P0 = rng.uniform(0.5, 1.0, (B, D)).astype(np.float32) if use_P0 else None
            h, hl, Pl = K.linear_scan_fwd(da_(a), da_(b), tdone, d(h0), d(P0))
            rh, rhl, rPl = M.diag_scan(a, b, done, h0, P0)
            da, db, dh0 = K.linear_scan_bwd(da_(a), h, tdone, d(h0), da_(g), d(gl))
            ag = G.diag_scan_grads(np.broadcast_to(a, (B, T, D)).copy(), b, done, np.zeros_like(b[:, 0]) if h0 is None else h0, g, gl)
            cast = (lambda t: t.float()) if half else (lambda t: t)
            errs = {"h": relerr(cast(h), rh), "da": relerr(cast(da), ag["da"]), "db": relerr(cast(db), ag["db"])}
            carr = {"h_last": relerr(hl, rhl), "P_last": relerr(Pl, rPl)}
            if use_h0:
                errs["dh0"] = relerr(dh0, ag["dh0"])
        torch.cuda.synchronize()
        bad = {n: e for n, e in errs.items() if not e <= tol}
        bad.update({n: e for n, e in carr.items() if not e <= TOL})
        if bad:
            failures.append((desc, bad))
    assert not failures, failures
