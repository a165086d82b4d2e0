#!/usr/bin/env python3
"""Headline benchmark: BF16 GEMM M=N=K=8192 on one MI355X through the C ABI of libneogemm.so.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--all]

Prints ONE JSON line.  A step is one GEMM (A [M,K] @ B [K,N], bf16 in, fp32 accumulate, bf16 out) on
inputs already resident in HBM.  `value` is 2*M*N*K / (wall time per step) in TFLOP/s; `roofline` prices
the kernel itself (HIP events on the launch stream) against the 2.5 PFLOP/s dense-BF16 peak;
`cpu_baseline` is the oracle's fp32 torch.matmul timed on the host cores of the same box (a reported
baseline, not a target); `vendor` is hipBLASLt/rocBLAS through torch.matmul on the same buffers.
With --all the other benchmark configurations are timed too and reported under `other_configs`.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = 2500.0   # MI355X dense BF16
PEAK_HBM_GBS = 8000.0  # MI355X HBM3E


def time_gpu(fn, steps, warmup, torch):
    """Wall time (host clock, sync on both sides) and HIP-event time per step."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    return wall * 1e3, e0.elapsed_time(e1) / steps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--all", action="store_true", help="also time the other benchmark configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy a few times, so that FETCH_SIZE / WRITE_SIZE "
                         "counters collected over this command can be scaled by what they read for a known size")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures ONE GPU (the GEMM path has no multi-GPU part); run with --gpus 1. "
                 "A multi-GPU job would shard M or N with no exchange, so N GPUs run N copies of this kernel.")

    import torch

    import gemm_amd as g
    from oracle import gemm_oracle as o   # cpu_baseline leg and the parity spot-check only

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    M = N = K = 8192
    A, B = o.make_inputs(M, N, K, seed=0)          # N(0,1)/sqrt(K) bf16, generated on the CPU
    Ad, Bd = A.to(dev), B.to(dev)
    C = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    variant, split_k = g.plan(M, N, K)

    def step():
        g.gemm_into(Ad, Bd, C, M, N, K, K, N, N, g.B_KN, g.C_ROW)

    wall_ms, ev_ms = time_gpu(step, args.steps, args.warmup, torch)
    flop = 2.0 * M * N * K
    value = flop / (wall_ms * 1e-3) / 1e12
    achieved = flop / (ev_ms * 1e-3) / 1e12

    # parity spot-check on a sample of rows (the full check lives in tests/test_gemm_gpu.py)
    idx = torch.randperm(M, generator=torch.Generator().manual_seed(1))[:128]
    rep = o.parity_report(C[idx.to(dev)], A[idx], B)
    parity_ok = (rep["finite"] and rep["rel_fro"] <= o.TOL_REL_FRO and rep["max_ulp_floored"] <= o.TOL_ULP
                 and rep["max_err_vs_bound"] <= 1.0)

    # vendor libraries on the same buffers (torch.matmul dispatches to hipBLASLt / rocBLAS)
    vend_ms = time_gpu(lambda: torch.matmul(Ad, Bd, out=C), max(10, args.steps // 2), 5, torch)[1]
    Bnk = Bd.t().contiguous()
    vend_nt_ms = time_gpu(lambda: torch.matmul(Ad, Bnk.t(), out=C), max(10, args.steps // 2), 5, torch)[1]
    ours_nt_ms = time_gpu(lambda: g.gemm_into(Ad, Bnk, C, M, N, K, K, K, N, g.B_NK, g.C_ROW), max(10, args.steps // 2), 5,
                          torch)[1]

    out = {
        "metric": "BF16 GEMM TFLOP/s at 8192^3 on 1 MI355X; % of dense-BF16 peak",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic: A [M,K], B [K,N] row-major, i.i.d. N(0,1)/sqrt(K) from seed 0 cast to bf16 on the CPU, "
                "copied to HBM before timing",
        "config": {"workload": "bf16 gemm M=N=K=8192, fp32 accumulate, bf16 C", "M": M, "N": N, "K": K,
                   "b_layout": "[K,N]", "kernel_variant": g.VARIANT_NAMES[variant], "split_k": split_k,
                   "entry": "neogemm_bf16 (C ABI) on torch's current stream"},
        "pct_of_peak": round(100.0 * value / PEAK_TFLOPS, 2),
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_TFLOPS, 4),
                     # HBM-side bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a plain copy
                     # (profiles/gemm_tile_256x256_w4_8192cubed.txt); the algorithmic figure is 402.7e6
                     "traffic": 1.762e9,
                     "kernel_ms": round(ev_ms, 5), "flop_per_launch": flop},
        "parity": {"ok": bool(parity_ok), "rows_checked": 128, **{k: rep[k] for k in ("max_ulp", "max_ulp_floored", "rel_fro")}},
        "vendor": {"lib": "torch.matmul (hipBLASLt/rocBLAS)", "tflops_b_kn": round(flop / vend_ms / 1e9, 2),
                   "tflops_b_nk": round(flop / vend_nt_ms / 1e9, 2), "neogemm_tflops_b_nk": round(flop / ours_nt_ms / 1e9, 2)},
    }

    if args.all:
        others = []
        for (m, n, k) in ((512, 512, 512), (4096, 4096, 4096), (16, 14336, 4096), (64, 14336, 4096),
                          (128, 14336, 4096), (3000, 5120, 3584), (1024, 1024, 32768)):
            a, b = o.make_inputs(m, n, k, seed=1)
            nbuf = 6 if m <= 128 else 1   # rotate weights larger than the 256 MB last-level cache
            ad, bds = a.to(dev), [b.to(dev).clone() for _ in range(nbuf)]
            c = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
            it = [0]

            def f():
                g.gemm_into(ad, bds[it[0] % nbuf], c, m, n, k, k, n, n, g.B_KN, g.C_ROW)
                it[0] += 1

            def fv():
                torch.matmul(ad, bds[it[0] % nbuf], out=c)
                it[0] += 1

            ms = time_gpu(f, 200 if m * n * k < 2e11 else 50, 20, torch)[1]
            vms = time_gpu(fv, 200 if m * n * k < 2e11 else 50, 20, torch)[1]
            fl, by = 2.0 * m * n * k, 2.0 * (m * k + k * n + m * n)
            v, s = g.plan(m, n, k)
            others.append({"M": m, "N": n, "K": k, "ms": round(ms, 5), "tflops": round(fl / ms / 1e9, 2),
                           "pct_of_2500": round(fl / ms / 1e9 / 25.0, 2), "gbps": round(by / ms / 1e6, 1),
                           "pct_of_8000": round(by / ms / 1e6 / 80.0, 2), "variant": g.VARIANT_NAMES[v], "split_k": s,
                           "vendor_ms": round(vms, 5)})
        out["other_configs"] = others

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["calibration_copy_bytes"] = 256 << 20

    if not args.no_cpu:
        # host baseline: the oracle's fp32 product, one full-size GEMM after a small warm-up
        nthreads = torch.get_num_threads()
        o.ref_gemm_f32(A[:256], B)
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            o.ref_gemm_f32(A, B)
            times.append(time.perf_counter() - t0)
        dt = sorted(times)[1]
        out["cpu_baseline"] = {"value": round(flop / dt / 1e12, 4), "unit": "TFLOP/s", "cores": nthreads, "kind": "port",
                               "sample": f"full M=N=K=8192 fp32 torch.matmul on the host, median of 3 ({dt:.1f} s each), "
                                         f"{os.cpu_count()} logical CPUs visible",
                               "seconds": round(dt, 2)}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
