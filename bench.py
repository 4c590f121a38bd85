#!/usr/bin/env python3
"""Benchmark of the memorax sequence-model hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--all]

One "step" = one forward + backward pass of the DeltaNet delta rule over the
synthetic batch of benchmark configuration 4 (B=64, H=8, T=1024, d=64, bf16 inputs,
fp32 state, reset mask Bernoulli(0.002)); inputs are resident in HBM before the
timed region.  Prints ONE JSON line.  Only one GPU is used: --gpus > 1 exits.

The other configurations (diagonal scan: configs[0]; linear attention: configs[1], configs[2];
the sequence kernels of the torso: configs[4]) are timed first and reported as secondary blocks of
the same line; the headline step is timed after them, on a device that is already at its clocks.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
MFMA_BF16_PEAK = 2.5e15    # MI355X dense bf16 matrix peak, flop/s, published
MFMA_F32_PEAK = 157.3e12   # MI355X fp32 matrix peak, flop/s, published
# Algorithmic HBM bytes per (b, t, h) token-head, d = 64, bf16:
#   forward : read q,k,v (3*128) + beta (2), write o (128)                    = 514
#   backward: read q,k,v,do (4*128) + beta (2), write dq,dk,dv (3*128) + dbeta (2) = 900
BYTES_FWD, BYTES_BWD = 514, 900
# HBM bytes one delta_bwd_kernel launch actually moves at this workload, from rocprofv3 --pmc
# FETCH_SIZE and WRITE_SIZE runs scaled by a plain elementwise kernel of known size
# (summary kept under profiles/).  The excess over the algorithmic bytes is the forward's
# per-chunk residuals (state checkpoints and triangular factors) being read back.
TRAFFIC_BWD_BYTES = 639.9e6
# Matrix-pipe busy fraction of delta_bwd_kernel from rocprofv3 --pmc (SQ_VALU_MFMA_BUSY_CYCLES over
# SQ_BUSY_CYCLES per SIMD), same workload; summary and command under profiles/.
MFMA_BUSY_BWD = 0.150
MFMA_BUSY_SOURCE = "profiles/delta_rule_kernels_counters_B64_T1024_H8_d64_bf16.md"
CLOCK_RAMP_S = 0.1         # untimed load before the warm-up steps, so that short runs see a device at its clocks


def delta_flops(C, d=64):
    """Matrix flops per (b, t, h) token-head of the delta rule in WY chunk form with C-step chunks
    (dense, no causal skip): forward 10 C d + 6 d^2 + 2/3 C^2, backward 2.5 x forward."""
    fwd = 10 * C * d + 6 * d * d + 2.0 * C * C / 3.0
    return fwd, 2.5 * fwd


def linear_attn_flops(C, d=64):
    """Chunk-form linear attention: forward 4 C d + 4 d^2, backward 10 C d + 10 d^2 per token-head."""
    return 4 * C * d + 4 * d * d, 10 * C * d + 10 * d * d


def synthetic(np, cfg, shape=None):
    """Seeded fp32 inputs of benchmark configuration cfg (1-based index into its list)."""
    rng = np.random.default_rng(1000 + cfg)
    if cfg == 2:
        B, T, H, d = shape or (64, 256, 4, 64)
        q, k, v = ((rng.standard_normal((B, T, H, d)) / 8.0).astype(np.float32) for _ in range(3))
        return dict(q=q, k=k, v=v, done=rng.random((B, T)) < 0.005)
    if cfg == 4:
        B, T, H, d = shape or (64, 1024, 8, 64)
        q = rng.standard_normal((B, T, H, d)).astype(np.float32)
        k = rng.standard_normal((B, T, H, d)).astype(np.float32)
        k /= np.linalg.norm(k, axis=-1, keepdims=True)
        v = rng.standard_normal((B, T, H, d)).astype(np.float32)
        beta = (1.0 / (1.0 + np.exp(-rng.standard_normal((B, T, H))))).astype(np.float32)
        return dict(q=q, k=k, v=v, beta=beta, done=rng.random((B, T)) < 0.002)
    raise ValueError(cfg)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--all", action="store_true",
                    help="also time the single-step kernels and the acting step, the RTRL scan, the mLSTM cell and the "
                         "block kernels")
    ap.add_argument("--headline-only", action="store_true", help="skip the secondary configurations")
    ap.add_argument("--ramp-ms", type=float, default=CLOCK_RAMP_S * 1e3,
                    help="untimed load before the warm-up steps (0 under a counter-collecting profiler)")
    ap.add_argument("--lib", default=None,
                    help="path of another build of the library to load (bench.py --all times the build with "
                         "64-step delta-rule chunks through this, in a child process)")
    ap.add_argument("--phase-clocks", action="store_true",
                    help="with --lib <the measurement build>: run the headline backward and print the share of "
                         "a wave's cycles spent inside matrix products (child process of the default run)")
    ap.add_argument("--no-children", action="store_true",
                    help="skip the two measurements that run in child processes (64-step-chunk build, product-phase "
                         "clocks): under a profiler the children would be traced into the same output")
    ap.add_argument("--torso-only", action="store_true",
                    help="time configuration 5's whole torso through the host mirror under bf16 autocast and nothing "
                         "else (seven updates: the run a kernel trace of the mirror's array-library side is taken from)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch a plain elementwise kernel of known size (256 MiB read, 256 MiB "
                         "written) so that a rocprofv3 --pmc FETCH_SIZE/WRITE_SIZE run can be scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU; this build has no multi-GPU path (--gpus must be 1)",
              file=sys.stderr)
        return 2

    import numpy as np
    import torch

    if args.lib:
        from memorax_amd import _lib
        _lib.LIB_PATH = os.path.abspath(args.lib)
    from memorax_amd import kernels as K

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    K.init()
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731

    if args.phase_clocks:
        print(json.dumps(phase_clocks_child(np, torch, K, dev)))
        return 0
    if args.torso_only:
        print(json.dumps(bench_torso_full(torch, K, variants=False)))
        return 0
    secondary = {}
    if not args.headline_only:
        secondary["hbm_copy"] = bench_copy(torch)
        secondary["scan"] = bench_scan(torch, K)
        secondary["linear_attention"] = bench_linear_attention(torch, K, np, dev)
        secondary["torso"] = bench_torso_kernels(torch, K)
        secondary["torso"].update(bench_torso_full(torch, K))
        if args.all:
            secondary["step"] = bench_step(torch, K)
            secondary["rtrl"] = bench_rtrl(torch, K)
            secondary["mlstm"] = bench_mlstm(torch)
            secondary["block"] = bench_block_kernels(torch, K)
        if not args.no_children:
            secondary["delta_rule_chunk64"] = bench_delta_chunk64()
        torch.cuda.empty_cache()
    if args.calibrate:
        cx = torch.zeros(64 * 1024 * 1024, device="cuda")  # 256 MiB fp32
        cy = torch.empty_like(cx)
        for _ in range(3):
            torch.add(cx, 1.0, out=cy)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del cx, cy

    bf = torch.bfloat16
    B, T, H, d = 64, 1024, 8, 64
    x = synthetic(np, 4, (B, T, H, d))
    do_np = np.random.default_rng(2004).standard_normal((B, T, H, d)).astype(np.float32)
    q, k, v, beta, do = (dev(a).to(bf) for a in (x["q"], x["k"], x["v"], x["beta"], do_np))
    done = dev(x["done"])
    torch.cuda.synchronize()

    # outputs and residuals are allocated once and reused, as a training loop's caching allocator does
    # The step runs the library's defaults (one unit of work per episode of a chunk that holds resets).  Episodes
    # end every five hundred steps in this configuration, where MRX_RESETS_MERGED (all episodes of a chunk in one
    # unit) is level with the default; it is timed beside it ("ms_per_step_merged_resets") and pays at the
    # torso's reset rate (the torso block).
    RESETS = None
    o, Sl, chk = K.delta_rule_fwd(q, k, v, beta, done, reset_path=RESETS)
    fwd_out = (o, Sl, chk[0], chk[1])
    bwd_out = K.delta_rule_bwd(q, k, v, beta, done, chk, do, None, want_dS0=False, reset_path=RESETS)

    def step(resets=RESETS):
        K.delta_rule_fwd(q, k, v, beta, done, out=fwd_out, reset_path=resets)
        return K.delta_rule_bwd(q, k, v, beta, done, chk, do, None, want_dS0=False, out=bwd_out, reset_path=resets)

    # The device needs some 30 ms of continuous load to reach its clocks (measured: 20-step batches
    # right after an idle stretch read 0.32, 0.29, 0.28, 0.27, 0.27 ms per step): an untimed ramp of the
    # same work comes first, outside the W warm-up steps and the K timed ones.
    t_ramp = time.perf_counter()
    while time.perf_counter() - t_ramp < args.ramp_ms * 1e-3:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    dt_merged = None
    if not args.lib:   # the other builds of the library (64-step chunks, clocks) have no use for it
        for _ in range(10):
            step("merged")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step("merged")
        torch.cuda.synchronize()
        dt_merged = (time.perf_counter() - t0) / args.steps

    # per-kernel durations with HIP events on the stream the kernels are launched on
    ev = lambda: torch.cuda.Event(enable_timing=True)  # noqa: E731
    tfs, tbs = [], []
    for _ in range(max(args.steps, 50)):
        e0, e1, e2 = ev(), ev(), ev()
        e0.record()
        K.delta_rule_fwd(q, k, v, beta, done, out=fwd_out, reset_path=RESETS)
        e1.record()
        K.delta_rule_bwd(q, k, v, beta, done, chk, do, None, want_dS0=False, out=bwd_out, reset_path=RESETS)
        e2.record()
        torch.cuda.synchronize()
        tfs.append(e0.elapsed_time(e1))
        tbs.append(e1.elapsed_time(e2))
    tf_ms, tb_ms = sum(tfs) / len(tfs), sum(tbs) / len(tbs)
    pct = lambda xs: {f"p{p}_ms": float(np.percentile(xs, p)) for p in (10, 50, 90)}  # noqa: E731
    nth = B * T * H
    bwd_gbs = BYTES_BWD * nth / (tb_ms * 1e-3) / 1e9
    fwd_gbs = BYTES_FWD * nth / (tf_ms * 1e-3) / 1e9
    C = K.chunk_size(bf, delta=True)
    fl_f, fl_b = delta_flops(C)
    mfma = lambda fl, ms: fl * nth / (ms * 1e-3) / MFMA_BF16_PEAK  # noqa: E731

    out = {
        "metric": "tokens/sec (B×T) fwd+bwd + % HBM/MFMA roofline, DeltaNet T=1024 on 1 GPU",
        "value": B * T / dt,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "clock_ramp_ms": args.ramp_ms,
        "config": {"workload": "configs[3]: DeltaNet delta rule fwd+bwd, B=64 H=8 T=1024 d=64, "
                               f"bf16 in / fp32 state, chunk {C}, resets p=0.002"
                               },
        "ms_per_step_merged_resets": None if dt_merged is None else dt_merged * 1e3,
        "roofline": {
            "bound": "hbm", "kernel": "delta_bwd_kernel", "achieved": bwd_gbs, "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": bwd_gbs / HBM_PEAK_GBS, "traffic": TRAFFIC_BWD_BYTES,
            "launch_ms": tb_ms, "algorithmic_bytes": BYTES_BWD * nth,
            # the matrix-pipe side of the same launch: chunk-form flops at the kernel's chunk length
            # over the launch time, against the dense bf16 peak; and the pipe's busy fraction by counter
            "mfma_frac": mfma(fl_b, tb_ms), "mfma_flops": fl_b * nth, "mfma_peak": MFMA_BF16_PEAK,
            "mfma_busy": MFMA_BUSY_BWD, "mfma_busy_source": MFMA_BUSY_SOURCE,
        },
        "kernels": {
            "delta_fwd": {"ms": tf_ms, "GB/s": fwd_gbs, "frac_hbm": fwd_gbs / HBM_PEAK_GBS,
                          "frac_mfma": mfma(fl_f, tf_ms), **pct(tfs)},
            "delta_bwd": {"ms": tb_ms, "GB/s": bwd_gbs, "frac_hbm": bwd_gbs / HBM_PEAK_GBS,
                          "frac_mfma": mfma(fl_b, tb_ms), **pct(tbs)},
            "fwd+bwd": {"ms": tf_ms + tb_ms,
                        "GB/s": (BYTES_FWD + BYTES_BWD) * nth / ((tf_ms + tb_ms) * 1e-3) / 1e9,
                        "frac_mfma": mfma(fl_f + fl_b, tf_ms + tb_ms)},
        },
    }
    if not args.headline_only:
        if not args.no_children:
            out["roofline"].update(bench_gemm_phase(MFMA_BUSY_BWD))
            ap_ = out["roofline"].get("access_pattern")
            if ap_:  # the kernels' times against what their access pattern alone costs (access_pattern_times)
                out["roofline"]["access_pattern_ms"] = ap_["delta_bwd_ms"]
                out["roofline"]["access_pattern_over_launch"] = ap_["delta_bwd_ms"] / tb_ms
                la3 = secondary.get("linear_attention", {}).get("cfg3_bf16_256x4096x8x64")
                if la3:
                    la3["access_pattern_ms"] = ap_["cfg3_fwd_ms"] + ap_["cfg3_bwd_ms"]
                    la3["access_pattern_over_ms"] = la3["access_pattern_ms"] / la3["ms"]
        if "hbm_copy" in secondary:
            out["roofline"]["hbm_copy_GB/s"] = secondary["hbm_copy"]["GB/s"]
            out["roofline"]["frac_of_copy_rate"] = bwd_gbs / secondary["hbm_copy"]["GB/s"]
    out.update(secondary)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(np, x, do_np)
    print(json.dumps(out))
    return 0


def bench_copy(torch):
    """What a plain streaming kernel reaches on this device: c = a + b over three float32 arrays of 512 MiB
    (two reads, one write, 1.6 GB per launch, far beyond the 256 MB last-level cache) -- the practical
    ceiling the HBM fractions of the bandwidth-bound kernels are to be read against."""
    n = 128 * 1024 * 1024
    a = torch.ones(n, device="cuda")
    b = torch.ones(n, device="cuda")
    c = torch.empty_like(a)
    ms = _time_ms(torch, lambda: torch.add(a, b, out=c), iters=20, warm=5)
    del a, b, c
    return {"ms": ms, "bytes": 12 * n, "GB/s": 12 * n / ms / 1e6, "frac_hbm_peak": 12 * n / ms / 1e6 / HBM_PEAK_GBS,
            "kernel": "torch.add(a, b, out=c), 3 x 512 MiB float32"}


MFMA_CYCLES_16x16x32_BF16 = 16   # 16 384 flop at the SIMD's peak of 1 024 flop per cycle (2.5 PFLOP/s / 1 024 SIMDs / 2.4 GHz)
MFMAS_PER_PASS_BWD = 48          # delta_bwd_kernel, bf16, 32-step chunks: MFMA instructions per wave and pass


def phase_clocks_child(np, torch, K, dev):
    """Runs in a child process on the measurement build (build.sh: MRX_PHASE_CLOCKS): the headline backward
    with every matrix product bracketed by shader-clock reads; returns the clock totals."""
    import ctypes
    from memorax_amd import _lib
    lib = _lib.load()
    lib.mrx_phase_clocks.argtypes = [ctypes.POINTER(ctypes.c_ulonglong), ctypes.c_int]
    lib.mrx_phase_clocks.restype = ctypes.c_int
    bf = torch.bfloat16
    B, T, H, d = 64, 1024, 8, 64
    x = synthetic(np, 4, (B, T, H, d))
    do_np = np.random.default_rng(2004).standard_normal((B, T, H, d)).astype(np.float32)
    q, k, v, beta, do = (dev(a).to(bf) for a in (x["q"], x["k"], x["v"], x["beta"], do_np))
    done = dev(x["done"])
    o, Sl, chk = K.delta_rule_fwd(q, k, v, beta, done)
    out = K.delta_rule_bwd(q, k, v, beta, done, chk, do, None, want_dS0=False)
    for _ in range(20):
        K.delta_rule_bwd(q, k, v, beta, done, chk, do, None, want_dS0=False, out=out)
    buf = (ctypes.c_ulonglong * 4)()
    assert lib.mrx_phase_clocks(buf, 1) == 0
    n = 20
    for _ in range(n):
        K.delta_rule_bwd(q, k, v, beta, done, chk, do, None, want_dS0=False, out=out)
    assert lib.mrx_phase_clocks(buf, 1) == 0
    C = K.chunk_size(bf, delta=True)
    dn = x["done"].reshape(B, T // C, C)
    passes = float((1 + dn.sum(-1)).sum()) / B   # units of work per sequence (every head of a batch row shares the resets)
    del q, k, v, beta, do, o, Sl, chk, out
    return {"product_clocks": int(buf[0]), "wave_clocks": int(buf[1]), "workgroups": int(buf[2]), "launches": n,
            "passes_per_sequence": passes, "access_pattern": access_pattern_times(torch, lib)}


def access_pattern_times(torch, lib):
    """What the chunked kernels' access pattern costs without their arithmetic (mrx_pattern_probe of the
    measurement build: one workgroup of four waves per (b, h), two per compute unit, 128-byte rows H rows apart,
    a chunk at a time with the next one requested ahead, results written row-wise; per-chunk residual blocks
    each way).  Milliseconds per launch for the delta rule at the headline shape (sequential forward kernel:
    q, k, v + 2 KB factor in, o + 8 KB checkpoint out per 32-row chunk; backward: q, k, v, dO + 10 KB in,
    dq, dk, dv out, last chunk first) and for plain linear attention at configuration 3's size (64-row chunks)."""
    import ctypes
    f = lib.mrx_pattern_probe
    vp, i64 = ctypes.c_void_p, ctypes.c_int64
    f.argtypes = [vp, ctypes.POINTER(vp), ctypes.c_int, ctypes.POINTER(vp), ctypes.c_int, vp, ctypes.c_int, vp, ctypes.c_int,
                  i64, i64, i64, ctypes.c_int, ctypes.c_int]
    f.restype = ctypes.c_int

    def time_case(B, T, H, C, n_in, n_out, res_in, res_out, reverse, iters):
        arrs = [torch.empty((B, T, H, 64), dtype=torch.bfloat16, device="cuda").fill_(1.0) for _ in range(n_in + n_out)]
        NC = T // C
        rin = torch.zeros((B * H * NC * max(res_in, 16),), dtype=torch.uint8, device="cuda")
        rout = torch.zeros((B * H * NC * max(res_out, 16),), dtype=torch.uint8, device="cuda")
        ins = (vp * n_in)(*[a.data_ptr() for a in arrs[:n_in]])
        outs = (vp * n_out)(*[a.data_ptr() for a in arrs[n_in:]])
        st = torch.cuda.current_stream().cuda_stream

        def go():
            rc = f(st, ins, n_in, outs, n_out, rin.data_ptr(), res_in, rout.data_ptr(), res_out, B, T, H, C, reverse)
            assert rc == 0, rc
        return _time_ms(torch, go, iters=iters)
    out = {"delta_fwd_sequential_ms": time_case(64, 1024, 8, 32, 3, 1, 2048, 8192, 0, 50),
           "delta_bwd_ms": time_case(64, 1024, 8, 32, 4, 3, 10240, 0, 1, 50),
           "cfg3_fwd_ms": time_case(256, 4096, 8, 64, 3, 1, 0, 0, 0, 5),
           "cfg3_bwd_ms": time_case(256, 4096, 8, 64, 4, 3, 0, 0, 1, 5)}
    return out


def bench_gemm_phase(mfma_busy):
    """MFMA utilisation inside the product phases of delta_bwd_kernel.  The measurement build brackets every
    matrix product of the kernel -- from before its first operand fragment is requested from LDS until its
    accumulators are in hand -- with reads of the shader clock; product_phase_share is the share of a wave's
    lifetime spent inside those brackets.  mfma_gemm_phase_frac is the rate at which a wave keeps its SIMD's
    matrix pipe busy while inside them: MFMAs per wave (48 per pass) x 16 cycles each / bracketed cycles per wave.
    Two waves share a SIMD at the headline shape, so the pipe's own utilisation while either is in a product
    lies between this figure and twice it; mfma_busy / product_phase_share (the whole-kernel busy counter spread
    over the product phases only) is reported beside it."""
    import subprocess
    lib = os.path.join(ROOT, "memorax_amd", "csrc", "libmemorax_amd_clk.so")
    if not os.path.exists(lib):
        return {"mfma_gemm_phase_frac": None, "mfma_gemm_phase_note": "libmemorax_amd_clk.so not built"}
    r = subprocess.run([sys.executable, os.path.abspath(__file__), "--lib", lib, "--phase-clocks"],
                       capture_output=True, text=True, timeout=300)
    if r.returncode != 0:
        return {"mfma_gemm_phase_frac": None, "mfma_gemm_phase_note": r.stderr[-300:]}
    d = json.loads(r.stdout.strip().splitlines()[-1])
    waves = 4 * d["workgroups"]
    prod_per_wave = d["product_clocks"] / waves
    share = d["product_clocks"] / d["wave_clocks"]
    mfma_cycles = MFMAS_PER_PASS_BWD * d["passes_per_sequence"] * MFMA_CYCLES_16x16x32_BF16
    return {"access_pattern": d.get("access_pattern"),
            "mfma_gemm_phase_frac": mfma_cycles / prod_per_wave, "product_phase_share": share,
            "mfma_busy_over_product_phase_share": mfma_busy / share,
            "mfma_gemm_phase_method": "shader-clock brackets around every product in the measurement build "
                                      "(libmemorax_amd_clk.so), 20 launches; per wave: 48 MFMAs/pass x 16 cycles / bracketed cycles"}


def bench_delta_chunk64():
    """The headline step on the build whose bf16 delta-rule kernels use 64-step chunks (the chunk length
    benchmark configuration 4 names; the library's default is 32), timed by this script in a child process
    that loads memorax_amd/csrc/libmemorax_amd_c64.so.  That build has no chunk-parallel factor kernel:
    the triangular inverse runs inside the sequential forward kernel."""
    import subprocess
    lib = os.path.join(ROOT, "memorax_amd", "csrc", "libmemorax_amd_c64.so")
    if not os.path.exists(lib):
        return {"skipped": "libmemorax_amd_c64.so not built"}
    r = subprocess.run([sys.executable, os.path.abspath(__file__), "--lib", lib, "--headline-only", "--no-cpu"],
                       capture_output=True, text=True, timeout=300)
    if r.returncode != 0:
        return {"failed": r.stderr[-300:]}
    d = json.loads(r.stdout.strip().splitlines()[-1])
    return {"workload": d["config"]["workload"], "ms_per_step": d["ms_per_step"], "tokens/s": d["value"],
            "fwd_ms": d["kernels"]["delta_fwd"]["ms"], "bwd_ms": d["kernels"]["delta_bwd"]["ms"]}


def _time_ms(torch, fn, iters=20, warm=3):
    for _ in range(warm):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def _graph_time_ms(torch, fn, n=50, reps=10):
    """Time per call of fn with n calls captured in a HIP graph and the graph replayed: what the
    kernels take back to back on the device, without the host's per-call cost (argument checks,
    output allocation, ctypes: some 15 us per call from Python, more than a small kernel runs)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(n):
            fn()
    for _ in range(2):
        g.replay()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    del g
    return e0.elapsed_time(e1) / (n * reps)


def bench_scan(torch, K):
    """Diagonal scan: configuration 1 (32,128,256), the torso's shape and a shape that saturates HBM.
    Configuration 1 moves 12.6 MB per call: its kernels are timed back to back inside a HIP graph
    (the per-call host cost from Python is larger than the kernel), the larger shapes call by call."""
    res = {}
    import numpy as np
    for name, shape in (("cfg1_32x128x256", (32, 128, 256)), ("torso_1024x128x256", (1024, 128, 256)),
                        ("sweep_512x1024x1024", (512, 1024, 1024))):
        Bn, Tn, Dn = shape
        if name.startswith("cfg1"):  # the configuration's own seeded inputs: a ~ U(0.9, 0.999), b ~ N(0, 1), resets p = 0.01
            rng = np.random.default_rng(1001)
            a = torch.from_numpy(rng.uniform(0.9, 0.999, shape).astype(np.float32)).cuda()
            b = torch.from_numpy(rng.standard_normal(shape).astype(np.float32)).cuda()
            dn = torch.from_numpy(rng.random((Bn, Tn)) < 0.01).cuda()
        else:                        # same distributions, drawn on the device (6.4 GB for the sweep shape)
            a = torch.rand(shape, device="cuda") * 0.099 + 0.9
            b = torch.randn(shape, device="cuda")
            dn = torch.rand((Bn, Tn), device="cuda") < 0.01
        small = 12 * Bn * Tn * Dn < 256e6
        timer = _graph_time_ms if small else (lambda t_, f_: _time_ms(t_, f_, iters=10))
        ms = timer(torch, lambda: K.linear_scan_fwd(a, b, dn, want_P=False))
        h, _, _ = K.linear_scan_fwd(a, b, dn, want_P=False)
        g = torch.randn(shape, device="cuda")
        msb = timer(torch, lambda: K.linear_scan_bwd(a, h, dn, None, g))
        by = 12 * Bn * Tn * Dn
        res[name] = {"fwd_ms": ms, "fwd_GB/s": by / ms / 1e6, "fwd_frac_hbm": by / ms / 1e6 / HBM_PEAK_GBS,
                     "fwd_tokens/s": Bn * Tn / ms * 1e3,
                     "bwd_ms": msb, "bwd_GB/s": 20 * Bn * Tn * Dn / msb / 1e6,
                     "bwd_frac_hbm": 20 * Bn * Tn * Dn / msb / 1e6 / HBM_PEAK_GBS,
                     "timed": "HIP graph of 50 calls" if small else "call by call"}
        if small:
            res[name]["fwd_ms_per_python_call"] = _time_ms(torch, lambda: K.linear_scan_fwd(a, b, dn, want_P=False), iters=20)
        if 12 * Bn * Tn * Dn < 256e6:
            # the working set fits the 256 MB Infinity Cache: also time it with the inputs rotated
            # through enough copies (> 512 MB) that every call reads them from HBM
            nset = int(512e6 // (8 * Bn * Tn * Dn)) + 1
            sets = [(a.clone(), b.clone()) for _ in range(nset)]
            it = [0]

            def rotated():
                aa, bb = sets[it[0] % nset]
                it[0] += 1
                K.linear_scan_fwd(aa, bb, dn, want_P=False)
            msr = _graph_time_ms(torch, rotated, n=2 * nset, reps=5)
            res[name]["fwd_ms_inputs_rotated"] = msr
            res[name]["fwd_GB/s_inputs_rotated"] = by / msr / 1e6
            del sets
        del a, b, g, h
    # MinGRU at the torso shape: gate arithmetic inside the scan kernels against the same recurrence
    # with the coefficients formed by elementwise torch kernels around the plain scan
    import memorax_amd.functional as Fn
    shape = (1024, 128, 256)
    z = torch.randn(shape, device="cuda").requires_grad_()
    x = torch.randn(shape, device="cuda").requires_grad_()
    dn = torch.rand(shape[:2], device="cuda") < 0.01
    g = torch.randn(shape, device="cuda")

    def fused():
        h, _, _ = Fn.mingru_scan(z, x, dn)
        h.backward(g)
        z.grad = x.grad = None

    def unfused():
        gx = torch.where(x >= 0, torch.relu(x) + 0.5, torch.sigmoid(x))
        h, _, _ = Fn.linear_scan(torch.sigmoid(-z), torch.sigmoid(z) * gx, dn)
        h.backward(g)
        z.grad = x.grad = None
    zd, xd = z.detach(), x.detach()
    h, _, _ = K.mingru_scan_fwd(zd, xd, dn, want_P=False)
    n = shape[0] * shape[1] * shape[2]
    mf = _time_ms(torch, lambda: K.mingru_scan_fwd(zd, xd, dn, want_P=False), iters=10)
    mb = _time_ms(torch, lambda: K.mingru_scan_bwd(zd, xd, h, dn, None, g), iters=10)
    # backward at this size: z, h~, g read, dz, dh~ written, and one row of h in eight (the others are formed again)
    res["mingru_1024x128x256"] = {"fwd_ms": mf, "fwd_GB/s": 12 * n / mf / 1e6, "bwd_ms": mb, "bwd_GB/s": 20.5 * n / mb / 1e6,
                                  "fwd+bwd_ms_fused_autograd": _time_ms(torch, fused, iters=10),
                                  "fwd+bwd_ms_elementwise_torch_around_the_plain_scan": _time_ms(torch, unfused, iters=10)}
    return res


def bench_linear_attention(torch, K, np, dev):
    """Configuration 2 (configs[1]: fp32, elu+1, resets) and configuration 3 (configs[2]: bf16, no resets),
    forward + backward, with the fractions of the roofline that binds each on paper: the fp32 matrix
    peak for configuration 2 (41 flop/B against a balance of 20), HBM for configuration 3."""
    res = {}
    x = synthetic(np, 2)
    q, k, v = (dev(x[n]) for n in ("q", "k", "v"))
    dn = dev(x["done"])
    do = torch.randn_like(v)

    def f2():
        o, Sl, chk = K.linear_attn_fwd(q, k, v, dn, None, 1)
        K.linear_attn_bwd(q, k, v, dn, chk, do, None, 1, want_dS0=False)
    ms = _time_ms(torch, f2)
    nth = 64 * 256 * 4
    ff, fb = linear_attn_flops(K.chunk_size(torch.float32))
    res["cfg2_f32_64x256x4x64"] = {"ms": ms, "tokens/s": 64 * 256 / ms * 1e3, "GB/s": 2816 * nth / ms / 1e6,
                                   "frac_hbm": 2816 * nth / ms / 1e6 / HBM_PEAK_GBS,
                                   "frac_mfma_f32": (ff + fb) * nth / (ms * 1e-3) / MFMA_F32_PEAK}
    del q, k, v, do
    # a grid that does not fill the device (32 sequences of 4096 steps, bf16): one workgroup per sequence
    # against the chunk-parallel pair the library's rule picks there
    Bn, Tn, Hn = 8, 4096, 4
    q, k, v, do = (torch.randn((Bn, Tn, Hn, 64), device="cuda").div_(8).to(torch.bfloat16) for _ in range(4))
    dn = torch.zeros((Bn, Tn), dtype=torch.bool, device="cuda")
    small = {}
    for name, par in (("ms_one_workgroup_per_sequence", False), ("ms_chunk_parallel", True)):
        def fs():
            o, Sl, chk = K.linear_attn_fwd(q, k, v, dn, None, 0, chunk_parallel=par)
            K.linear_attn_bwd(q, k, v, dn, chk, do, None, 0, want_dS0=False)
        small[name] = _time_ms(torch, fs)
    small["rule_picks_chunk_parallel"] = bool(K.linear_attn_chunk_parallel_pays(Bn, Tn, Hn, torch.bfloat16))
    small["tokens/s"] = Bn * Tn / min(small["ms_one_workgroup_per_sequence"], small["ms_chunk_parallel"]) * 1e3
    res["small_grid_bf16_8x4096x4x64"] = small
    del q, k, v, do
    # head dim 32 (the library's second build of the kernels) at 1024 environments x 128 steps x 4 heads,
    # beside the same token-heads at head dim 64 (what a 32-wide model paid when it was padded) and at
    # head dim 16 (the reference guides' size, which the 32-wide kernels take as it lies in memory)
    Bn, Tn, Hn = 1024, 128, 4
    dn = torch.rand((Bn, Tn), device="cuda") < 0.01
    hd = {}
    for d in (16, 32, 64):
        q, k, v, do = (torch.randn((Bn, Tn, Hn, d), device="cuda").div_(8).to(torch.bfloat16) for _ in range(4))

        def fh():
            o, Sl, chk = K.linear_attn_fwd(q, k, v, dn, None, 1)
            K.linear_attn_bwd(q, k, v, dn, chk, do, None, 1, want_dS0=False)
        hd[f"ms_d{d}"] = _time_ms(torch, fh)
        del q, k, v, do
    hd["tokens/s"] = Bn * Tn / hd["ms_d32"] * 1e3
    res["head_dim_32_bf16_1024x128x4"] = hd
    Bn, Tn, Hn = 256, 4096, 8   # configuration 3 at full size (11.8 GB of q, k, v, do, o, dq, dk, dv)
    q, k, v, do = (torch.randn((Bn, Tn, Hn, 64), device="cuda").div_(8).to(torch.bfloat16) for _ in range(4))
    dn = torch.zeros((Bn, Tn), dtype=torch.bool, device="cuda")

    def f3():
        o, Sl, chk = K.linear_attn_fwd(q, k, v, dn, None, 0)
        K.linear_attn_bwd(q, k, v, dn, chk, do, None, 0, want_dS0=False)
    ms = _time_ms(torch, f3, iters=5)
    nth = Bn * Tn * Hn
    ff, fb = linear_attn_flops(K.chunk_size(torch.bfloat16))
    res["cfg3_bf16_256x4096x8x64"] = {"ms": ms, "tokens/s": Bn * Tn / ms * 1e3, "GB/s": 1408 * nth / ms / 1e6,
                                      "frac_hbm": 1408 * nth / ms / 1e6 / HBM_PEAK_GBS,
                                      "frac_mfma": (ff + fb) * nth / (ms * 1e-3) / MFMA_BF16_PEAK}
    # the same shape with a per-step scalar decay (Mamba cell algebra); + g in, dg out: 8 B more per token-head
    g = -torch.rand((Bn, Tn, Hn), device="cuda") * 0.1

    def f3g():
        o, Sl, chk = K.gated_linear_attn_fwd(q, k, v, g, dn, None, 0)
        K.gated_linear_attn_bwd(q, k, v, g, dn, chk, do, None, 0, want_dS0=False)
    ms = _time_ms(torch, f3g, iters=5)
    res["gated_bf16_256x4096x8x64"] = {"ms": ms, "tokens/s": Bn * Tn / ms * 1e3,
                                       "GB/s": (1408 + 12) * Bn * Tn * Hn / ms / 1e6}
    # the same shape with the normalised read-out of LinearAttentionCell.read fused (elu+1 feature map);
    # + o read back in the backward call, den written and read: 136 B more per token-head
    def f3n():
        o, den, Sl, zl, chk = K.linear_attn_norm_fwd(q, k, v, dn, None, None, 1, 1e-6)
        K.linear_attn_norm_bwd(q, k, v, dn, chk, o, den, do, None, None, 1, 1e-6, want_d0=False)
    ms = _time_ms(torch, f3n, iters=5)
    res["normalised_bf16_256x4096x8x64"] = {"ms": ms, "tokens/s": Bn * Tn / ms * 1e3,
                                            "GB/s": (1408 + 136) * Bn * Tn * Hn / ms / 1e6}
    return res


def bench_mlstm(torch):
    """The mLSTM cell's scan through the host mirror (stabiliser kernels, gated chunked kernel, normaliser scan and
    the read-out's divisions; float32), forward and forward + backward, at a rollout-sized and a larger shape."""
    from memorax_amd import sequence_models as sm
    out = {}
    for (B, T, H, d) in ((64, 128, 4, 64), (256, 512, 4, 64)):
        cell = sm.mLSTMCell(64, hidden_dim=H * d, num_heads=H).cuda()
        g = torch.Generator(device="cuda").manual_seed(B)
        q, k, v = (torch.randn(B, T, H, d, device="cuda", generator=g).requires_grad_() for _ in range(3))
        li = torch.randn(B, T, H, device="cuda", generator=g).requires_grad_()
        lf = (-torch.rand(B, T, H, device="cuda", generator=g)).requires_grad_()
        done = torch.rand(B, T, device="cuda", generator=g) < 0.01
        carry = cell.initialize_carry(None, (B, 64))

        def fwd():
            with torch.no_grad():
                cell.scan((k, v, li, lf, q), carry, done)

        def step():
            h, c = cell.scan((k, v, li, lf, q), carry, done)
            (h.sum() + c[0].sum() + c[2].sum()).backward()
        out[f"scan_{B}x{T}x{H}x{d}"] = {"fwd_ms": _time_ms(torch, fwd, iters=10), "fwd+bwd_ms": _time_ms(torch, step, iters=10)}
    return out


def bench_rtrl(torch, K):
    """RTRL sensitivity update (memoroid.py:114-141): final state of a diagonal scan over
    H * param_size channels with the decay shared by param_size channels.  Bytes = one read of
    the Jacobians (+ decay, carry in and out).  Beside it: the reference's formulation on the
    general scan kernel (decay repeated param_size times, all states written)."""
    Bn, Tn, Hn, ps = 64, 128, 256, 64
    D = Hn * ps
    decay = torch.rand((Bn, Tn, Hn), device="cuda") * 0.1 + 0.9
    J = torch.randn((Bn, Tn, D), device="cuda")
    S = torch.randn((Bn, D), device="cuda")
    dn = torch.rand((Bn, Tn), device="cuda") < 0.01
    by = 4 * (Bn * Tn * D + Bn * Tn * Hn + 2 * Bn * D)
    ms = _time_ms(torch, lambda: K.linear_scan_last(decay, J, dn, S), iters=10)

    def general():
        a = decay.repeat_interleave(ps, dim=-1)
        K.linear_scan_fwd(a, J, dn, S, want_P=False)
    ms2 = _time_ms(torch, general, iters=5)
    return {"scan_last_64x128x(256x64)": {"ms": ms, "GB/s": by / ms / 1e6, "frac_hbm": by / ms / 1e6 / HBM_PEAK_GBS},
            "repeat_and_general_scan_ms": ms2}


def bench_step(torch, K):
    """Acting path: one time step for 1024 environments x 4 heads (the rollout of configuration 5),
    state updated in place.  Bytes = the fp32 state read once and written once (32 KiB per (b,h))
    plus q, k, v, o.  The chunked forward kernel at T = 1 is timed beside it."""
    Bn, Hn, d = 1024, 4, 64
    bf = torch.bfloat16
    q, k, v = (torch.randn((Bn, Hn, d), device="cuda").to(bf) for _ in range(3))
    k = torch.nn.functional.normalize(k.float(), dim=-1).to(bf)
    beta = torch.rand((Bn, Hn), device="cuda").to(bf)
    dn = torch.rand((Bn,), device="cuda") < 0.01
    S = torch.zeros((Bn, Hn, d, d), device="cuda")
    z = torch.zeros((Bn, Hn, d), device="cuda")
    by = Bn * Hn * (2 * d * d * 4 + 4 * d * 2)
    res = {}
    ms = _time_ms(torch, lambda: K.delta_rule_step(q, k, v, beta, dn, S, inplace=True), iters=50, warm=5)
    res["delta_rule_step_1024x4x64"] = {"ms": ms, "GB/s": by / ms / 1e6, "frac_hbm": by / ms / 1e6 / HBM_PEAK_GBS,
                                        "env_steps/s": Bn / ms * 1e3}
    ms = _time_ms(torch, lambda: K.linear_attn_step(q, k, v, dn, S, z, "elu1", True, 1e-6, True), iters=50, warm=5)
    res["linear_attn_step_normalised_1024x4x64"] = {"ms": ms, "GB/s": by / ms / 1e6,
                                                    "frac_hbm": by / ms / 1e6 / HBM_PEAK_GBS,
                                                    "env_steps/s": Bn / ms * 1e3}
    q1, k1, v1, b1, d1 = q[:, None].contiguous(), k[:, None].contiguous(), v[:, None].contiguous(), \
        beta[:, None].contiguous(), dn[:, None].contiguous()
    ms = _time_ms(torch, lambda: K.delta_rule_fwd(q1, k1, v1, b1, d1, S, save_chk=False), iters=50, warm=5)
    res["chunk_kernel_at_T1_for_comparison"] = {"ms": ms}
    res["torso_acting_step_1024_envs"] = bench_acting_step(torch)
    return res


def bench_acting_step(torch):
    """One acting step (T = 1, no gradients, bf16 autocast) of configuration 5's torso through the host mirror for
    1024 environments: issued kernel by kernel from the host, and replayed as one HIP graph
    (memorax_amd.rollout.GraphedStep)."""
    from memorax_amd import sequence_models as sm
    from memorax_amd.rollout import GraphedStep
    B, Fe, H, d = 1024, 256, 4, 64
    torch.manual_seed(5)
    blocks = []
    for _ in range(4):
        blocks += [sm.Residual(sm.PreNorm(sm.Memoroid(sm.DeltaNetCell(Fe, d, H)), Fe, norm=sm.RMSNorm)),
                   sm.Residual(sm.PreNorm(sm.GatedLinearRecurrence(Fe), Fe, norm=sm.RMSNorm))]
    torso = sm.Stack(blocks).cuda()
    x = torch.randn(B, 1, Fe, device="cuda")
    done = torch.rand(B, 1, device="cuda") < 0.01
    state = {"carry": torso.initialize_carry(None, (B, Fe))}

    def eager():
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
            state["carry"], _ = torso(x, done, state["carry"])
    ms_e = _time_ms(torch, eager, iters=30, warm=5)
    act = GraphedStep(torso, B, Fe, autocast=torch.bfloat16)
    ms_g = _time_ms(torch, lambda: act(x, done), iters=100, warm=5)
    return {"ms_issued_from_the_host": ms_e, "ms_as_a_graph": ms_g, "env_steps/s_as_a_graph": B / ms_g * 1e3}


def bench_block_kernels(torch, K):
    """The passes of a torso block around its recurrence, at configuration 5's size (131 072 rows of 256 features):
    the norms as a pre-norm block under bf16 autocast calls them (float32 residual stream in, bfloat16 out; the
    backward with the residual branch's gradient added), the read-out norm on bfloat16 rows, the gating product, and
    the array library's own operations for the same work beside them.  Bytes = every operand once."""
    rows, D = 1024 * 128, 256
    bf = torch.bfloat16
    x = torch.randn(rows, D, device="cuda")
    xb, gb, hb = (torch.randn(rows, D, device="cuda").to(bf) for _ in range(3))
    add = torch.randn(rows, D, device="cuda")
    sc, bi = torch.ones(D, device="cuda"), torch.zeros(D, device="cuda")
    n32, n16 = rows * D * 4, rows * D * 2
    out = {}

    def put(name, fn, nbytes):
        ms = _time_ms(torch, fn, iters=20, warm=3)
        out[name] = {"ms": ms, "GB/s": nbytes / ms / 1e6, "frac_hbm": nbytes / ms / 1e6 / HBM_PEAK_GBS}
    put("rms_norm_fwd_f32_to_bf16", lambda: K.rms_norm_fwd(x, sc, 1e-6, bf), n32 + n16)
    put("rms_norm_bwd_f32_with_residual_gradient", lambda: K.rms_norm_bwd(x, sc, gb, 1e-6, dx_add=add), 3 * n32 + n16)
    put("rms_norm_fwd_bf16", lambda: K.rms_norm_fwd(xb, sc), 2 * n16)
    put("rms_norm_bwd_bf16", lambda: K.rms_norm_bwd(xb, sc, gb), 3 * n16)
    put("layer_norm_fwd_f32_to_bf16", lambda: K.layer_norm_fwd(x, sc, bi, 1e-6, bf), n32 + n16)
    put("layer_norm_bwd_f32_with_residual_gradient", lambda: K.layer_norm_bwd(x, sc, gb, 1e-6, dx_add=add), 3 * n32 + n16)
    put("silu_gate_fwd_bf16", lambda: K.silu_gate_fwd(hb, gb), 3 * n16)
    put("silu_gate_bwd_bf16", lambda: K.silu_gate_bwd(hb, gb, xb), 5 * n16)
    # the array library on the same work: its fused norm kernels plus the cast and the addition around them
    F = torch.nn.functional
    xr = x.clone().requires_grad_()
    scr = sc.clone().requires_grad_()

    def lib_norm():
        xr.grad = scr.grad = None
        y = F.rms_norm(xr, (D,), scr, 1e-6).to(bf)
        y.backward(gb)
        return xr.grad + add
    ms = _time_ms(torch, lib_norm, iters=10, warm=2)
    mine = out["rms_norm_fwd_f32_to_bf16"]["ms"] + out["rms_norm_bwd_f32_with_residual_gradient"]["ms"]
    out["array_library_rms_norm_cast_backward_add"] = {"ms": ms, "over_the_kernels": ms / mine}
    hr, gr = hb.clone().requires_grad_(), gb.clone().requires_grad_()

    def lib_gate():
        hr.grad = gr.grad = None
        (hr * F.silu(gr)).backward(xb)
    ms = _time_ms(torch, lib_gate, iters=10, warm=2)
    mine = out["silu_gate_fwd_bf16"]["ms"] + out["silu_gate_bwd_bf16"]["ms"]
    out["array_library_gating_forward_backward"] = {"ms": ms, "over_the_kernels": ms / mine}
    return out


def bench_torso_kernels(torch, K):
    """Configuration 5 (configs[4]), the sequence kernels of one update: 4 blocks x (DeltaNet H=4, d=64
    forward + backward, diagonal recurrence forward + backward) over B=1024 envs x T=128, done p=0.01.
    The DeltaNet cell calls the kernels with its prologue inside (key normalisation and gate sigmoid on
    the raw projections, gradients taken back through them): that is the figure reported; the plain
    delta rule on ready-made unit keys and gates is timed beside it."""
    B, T, Fe, H, d = 1024, 128, 256, 4, 64
    bf = torch.bfloat16
    done = torch.rand(B, T, device="cuda") < 0.01
    q, k_raw, v = (torch.randn(B, T, H, d, device="cuda").to(bf) for _ in range(3))
    k_unit = torch.nn.functional.normalize(k_raw.float(), dim=-1).to(bf)
    b_raw = torch.randn(B, T, H, device="cuda").to(bf)
    beta = torch.sigmoid(b_raw.float()).to(bf)
    do = torch.randn_like(v)
    z, hx, g = (torch.randn(B, T, Fe, device="cuda") for _ in range(3))

    def kernels_only(prologue, resets=None):
        kk, bb = (k_raw, b_raw) if prologue else (k_unit, beta)
        for _ in range(4):
            o, Sl, chk = K.delta_rule_fwd(q, kk, v, bb, done, prologue=prologue, reset_path=resets)
            K.delta_rule_bwd(q, kk, v, bb, done, chk, do, None, want_dS0=False, prologue=prologue, reset_path=resets)
            h, _, _ = K.mingru_scan_fwd(z, hx, done, want_P=False)
            K.mingru_scan_bwd(z, hx, h, done, None, g)
    ms_k = _time_ms(torch, lambda: kernels_only(True), iters=10, warm=3)
    ms_p = _time_ms(torch, lambda: kernels_only(False), iters=10, warm=3)
    # episodes end every hundred steps here: the caller's choice of MRX_RESETS_MERGED (all episodes of a chunk in
    # one unit of work, behind a screen of the chunk's inputs) against the default of one unit per episode
    ms_m = _time_ms(torch, lambda: kernels_only(True, "merged"), iters=10, warm=3)
    # the same with the recurrence's arrays in bfloat16 (what a bf16 torso hands over; float32 arithmetic and
    # carries inside the kernels): half the bytes of the scans
    z, hx, g = (t.to(bf) for t in (z, hx, g))
    ms_h = _time_ms(torch, lambda: kernels_only(True), iters=10, warm=3)
    ms_hm = _time_ms(torch, lambda: kernels_only(True, "merged"), iters=10, warm=3)
    by = 4 * ((BYTES_FWD + BYTES_BWD) * B * T * H + 32.5 * B * T * Fe)   # + MinGRU scan: 12 B fwd, 20.5 B bwd per element
    return {"sequence_kernels_ms": ms_k, "sequence_kernels_tokens/s": B * T / ms_k * 1e3,
            "sequence_kernels_GB/s": by / ms_k / 1e6, "sequence_kernels_frac_hbm": by / ms_k / 1e6 / HBM_PEAK_GBS,
            "sequence_kernels_ms_merged_resets": ms_m, "sequence_kernels_tokens/s_merged_resets": B * T / ms_m * 1e3,
            "sequence_kernels_ms_plain_delta_rule": ms_p, "sequence_kernels_ms_bf16_recurrence_arrays": ms_h,
            "sequence_kernels_ms_bf16_recurrence_arrays_merged_resets": ms_hm,
            "sequence_kernels_tokens/s_bf16_recurrence_arrays": B * T / ms_h * 1e3,
            "sequence_kernels_frac_hbm_bf16_recurrence_arrays":
                4 * ((BYTES_FWD + BYTES_BWD) * B * T * H + 18 * B * T * Fe) / ms_h / 1e6 / HBM_PEAK_GBS}


def bench_torso_full(torch, K, variants=True):
    """Configuration 5 through the host mirror, dense projections in torch included: 4 blocks of
    [RMSNorm -> DeltaNet(H=4, d=64) -> +x ; RMSNorm -> gated linear recurrence -> +x], d_model 256,
    weights N(0, 0.02).  variants=False: the bf16-autocast update only, seven times (two of them warm-up)."""
    from memorax_amd import sequence_models as sm
    B, T, Fe, H, d = 1024, 128, 256, 4, 64
    torch.manual_seed(5)
    blocks = []
    for _ in range(4):
        blocks += [sm.Residual(sm.PreNorm(sm.Memoroid(sm.DeltaNetCell(Fe, d, H)), Fe, norm=sm.RMSNorm)),
                   sm.Residual(sm.PreNorm(sm.GatedLinearRecurrence(Fe), Fe, norm=sm.RMSNorm))]
    torso = sm.Stack(blocks).cuda()
    for p in torso.parameters():
        if p.dim() > 1:
            torch.nn.init.normal_(p, 0.0, 0.02)
    x = torch.randn(B, T, Fe, device="cuda")
    done = torch.rand(B, T, device="cuda") < 0.01
    gy = torch.randn(B, T, Fe, device="cuda")

    def full(autocast=True):
        for p in torso.parameters():
            p.grad = None
        # configuration 5 names bf16 weights: the dense projections run under bf16 autocast, the
        # recurrences in the precision their kernels take (bf16 in / fp32 state; fp32 for the scan)
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
            _, y = torso(x, done)
        y.backward(gy)   # the gradient a policy head would hand back
    ms_full = _time_ms(torch, full, iters=5, warm=2)
    if not variants:
        return {"full_torso_ms": ms_full, "full_torso_tokens/s": B * T / ms_full * 1e3}
    ms_full32 = _time_ms(torch, lambda: full(False), iters=3, warm=1)
    for blk in torso.blocks[0::2]:   # episodes end every hundred steps here: the caller's choice of merged episodes
        blk.module.module.cell.resets = "merged"
    ms_merged = _time_ms(torch, full, iters=5, warm=2)
    return {"full_torso_ms": ms_full, "full_torso_tokens/s": B * T / ms_full * 1e3,
            "full_torso_ms_merged_resets": ms_merged, "full_torso_ms_fp32_projections": ms_full32}


def cpu_baseline(np, x, do_np):
    """The C restatement (oracle/c, fp32 state, OpenMP) on a bounded sample of the same
    workload (configuration 4, forward + backward, one pass)."""
    from oracle import clib
    if not clib.available():
        return {"value": None, "unit": "tokens/s", "cores": 0, "kind": "port", "sample": "oracle not built"}
    Bs = 64  # the whole batch: about 20 core-seconds
    sl = {n: x[n][:Bs] for n in ("q", "k", "v", "beta", "done")}
    dos = do_np[:Bs]
    cores = clib.num_threads()
    clib.delta_rule_fwd(sl["q"][:1], sl["k"][:1], sl["v"][:1], sl["beta"][:1], sl["done"][:1], None, "f32")
    reps = 4   # about 1 s of wall time, 16 core-seconds of CPU work on the box's 16 host threads
    t0 = time.perf_counter()
    for _ in range(reps):
        clib.delta_rule_fwd(sl["q"], sl["k"], sl["v"], sl["beta"], sl["done"], None, "f32")
        clib.delta_rule_bwd(sl["q"], sl["k"], sl["v"], sl["beta"], sl["done"], None, dos, None, "f32")
    dt = (time.perf_counter() - t0) / reps
    T = sl["q"].shape[1]
    return {"value": Bs * T / dt, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"all {Bs} batch rows of configs[3] (H=8, T={T}, d=64), fwd+bwd, mean of {reps} runs after "
                      f"a warm-up, sequential recurrence in C (fp32 state), OpenMP over (b,h); {dt:.2f} s per run"}


if __name__ == "__main__":
    sys.exit(main())
