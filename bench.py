#!/usr/bin/env python3
"""Headline benchmark: BF16 GEMM M=N=K=8192 on one MI355X through the C ABI of libneogemm.so.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--preheat-ms T] [--all]

Prints ONE JSON line.  A step is one GEMM (A [M,K] @ B [K,N], bf16 in, fp32 accumulate, bf16 out) on
inputs already resident in HBM.  Order of events:
  0. a host thread starts polling the board's telemetry (socket power, shader clocks: gemm_amd/telemetry.py, amdsmi;
     no GPU call, no process) and keeps doing so to the end: `roofline.power` holds what it read during each leg;
  1. (before this process touches the GPU) the stand-alone harness gemm_amd/vendor_bench/matmul_bench runs as a
     child: the matrix cores' power ceiling on N(0,1) operands (`roofline.power_ceiling`), and hipBLASLt (best of
     its heuristic candidates) / rocBLAS / libneogemm on the same buffers, both layouts of B (`vendor`); with --all
     also the other benchmark configurations, the same way (`other_configs`);
  2. an untimed, time-based preheat of the very GEMM that is measured (`preheat_ms`): the chip is power-limited
     on random data and the first launches after an idle period run slower until the clocks have settled;
  3. W warm-up steps, then exactly K timed steps between two synchronisations: `value` = 2*M*N*K / wall time per
     step.  The K steps are cut into batches, each bracketed by HIP events on the launch stream; the median batch
     is `roofline.kernel_ms`, the list is `roofline.batch_ms`;
  4. parity spot check against the CPU oracle, and the oracle's own fp32 product timed on the host cores
     (`cpu_baseline`: a reported baseline, not a target).
`roofline.frac_of_power_ceiling` divides by the ceiling of the MFMA order the timed kernel issues
(`roofline.power_ceiling_order`), measured in this run.
"""
import argparse
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = 2500.0   # MI355X dense BF16
PEAK_HBM_GBS = 8000.0  # MI355X HBM3E
MATMUL_BENCH = os.path.join(ROOT, "gemm_amd", "vendor_bench", "matmul_bench")
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "gemm_chain_256x256_8192cubed_traffic.json")


def run_harness(args, env_extra=None, timeout=300):
    """Run matmul_bench as a child and return its JSON lines (a list of dicts); [] if it is not built or fails."""
    if not os.path.exists(MATMUL_BENCH):
        return []
    env = dict(os.environ)
    env.update(env_extra or {})
    try:
        out = subprocess.run([MATMUL_BENCH] + [str(a) for a in args], env=env, capture_output=True, text=True,
                             timeout=timeout).stdout
    except (subprocess.TimeoutExpired, OSError):
        return []
    rows = []
    for line in out.splitlines():
        try:
            rows.append(json.loads(line))
        except ValueError:
            pass
    return rows


def vendor_leg(M, N, K, preheat_ms, sampler=None):
    """hipBLASLt best-of-heuristics, rocBLAS and libneogemm timed by one harness on the same buffers, B [K,N] and [N,K]."""
    out = {"harness": "gemm_amd/vendor_bench/matmul_bench (child process, HIP events, median of 5 batches of 40, "
                      f"{preheat_ms} ms preheat per library)"}
    for bl, name in ((0, "b_kn"), (1, "b_nk")):
        rows = run_harness([M, N, K, 40, bl], {"MATMUL_BENCH_PREHEAT_MS": str(preheat_ms)})
        for r in rows:
            if "lib" in r:
                out[f"{r['lib']}_tflops_{name}"] = r["tflops"]
                if r["lib"] == "hipblaslt":
                    out[f"hipblaslt_algos_tried_{name}"] = r.get("algos_tried")
                if sampler is not None and "t0" in r:
                    out.setdefault("power", {})[f"{r['lib']}_{name}"] = brief(sampler.summary(r["t0"], r["t1"]))
            elif r.get("check") == "neogemm_vs_vendor":
                out[f"rel_fro_vs_vendor_{name}"] = r["rel_fro"]
    return out


def brief(summary):
    """mean socket power and shader clock of a telemetry summary, for the per-leg tables"""
    if not summary.get("available") or summary.get("samples", 0) < 8:
        return None   # the board refreshes its readings every few tens of milliseconds: a leg shorter than that says nothing
    return {"socket_power_w": summary.get("socket_power_w", {}).get("mean"),
            "shader_clock_mhz": summary.get("shader_clock_mhz", {}).get("mean"), "samples": summary["samples"]}


# the other benchmark configurations: (M, N, K, weight buffers to rotate through, repetitions per batch)
OTHER_CONFIGS = ((512, 512, 512, 1, 200), (4096, 4096, 4096, 1, 40), (16, 14336, 4096, 8, 100), (64, 14336, 4096, 8, 100),
                 (128, 14336, 4096, 8, 100), (3000, 5120, 3584, 1, 40), (1024, 1024, 32768, 1, 40))


def other_configs_leg(preheat_ms, sampler=None):
    """Every other benchmark configuration the way the headline's vendor leg is measured: one child per shape and layout
    of B, libneogemm / hipBLASLt best of its heuristic candidates / rocBLAS on the same buffers, a time-based preheat of
    each library before it is timed, weights of the decode shapes rotating through 8 buffers (940 MB)."""
    rows_out = []
    for (m, n, k, nbuf, reps) in OTHER_CONFIGS:
        fl, by = 2.0 * m * n * k, 2.0 * (m * k + k * n + m * n)
        row = {"M": m, "N": n, "K": k, "weight_buffers": nbuf}
        for bl, name in ((0, "b_kn"), (1, "b_nk")):
            for r in run_harness([m, n, k, reps, bl, 0, 0, 0, nbuf], {"MATMUL_BENCH_PREHEAT_MS": str(preheat_ms)}):
                if "lib" not in r:
                    continue
                us = r["ms"] * 1e3
                if r["lib"] == "neogemm":
                    row[f"us_{name}"] = round(us, 2)
                    row[f"tflops_{name}"] = round(fl / us / 1e6, 2)
                    row[f"pct_of_2500_{name}"] = round(fl / us / 1e6 / 25.0, 2)
                    row[f"gbps_{name}"] = round(by / us / 1e3, 1)
                    row[f"pct_of_8000_{name}"] = round(by / us / 1e3 / 80.0, 2)
                    row[f"variant_{name}"], row[f"split_k_{name}"] = r.get("variant"), r.get("split_k")
                    if sampler is not None and "t0" in r:
                        row[f"power_{name}"] = brief(sampler.summary(r["t0"], r["t1"]))
                else:
                    row[f"{r['lib']}_us_{name}"] = round(us, 2)
        rows_out.append(row)
    return rows_out


def power_ceiling(preheat_ms, sampler=None):
    rows = [r for r in run_harness(["ceiling", preheat_ms]) if "ceiling" in r]
    if not rows:
        return None
    if sampler is not None:
        # what the board's telemetry read while each MFMA-only case was being timed
        tele = {}
        for r in rows:
            if "t0" not in r or r["ceiling"] == "gemm_like":
                continue
            key = (r.get("order") or ("16x16x32" if "16x16x32" in r["ceiling"] else "32x32x16")) + ", " + r["operands"]
            tele[key] = brief(sampler.summary(r["t0"], r["t1"]))
        power_ceiling.telemetry = tele
    out = {"what": "MFMA-only loop from registers, one wave per SIMD on 256 CUs, measured in this run before the GEMM "
                   "(matmul_bench ceiling): the rate the chip's power limit allows the matrix cores alone",
           "unit": "TFLOP/s"}
    for r in rows:
        if r["ceiling"] == "gemm_like":
            # the 16x16x32 sequence on N(0,1) operands next to the other parts of a GEMM main loop, at the tile kernel's rates
            out.setdefault("with_gemm_parts_" + r["operands"], {})[r["parts"]] = r["tflops"]
            continue
        if r["ceiling"] == "mfma_order":
            # the same 128 MFMAs of a wave tile in different orders (the tile kernel uses the 2x2-block walk)
            out.setdefault("by_mfma_order_" + r["operands"], {})[r["order"]] = r["tflops"]
            continue
        short = "16x16x32" if "16x16x32" in r["ceiling"] else "32x32x16"
        out[f"{short}_{r['operands']}"] = r["tflops"]
        out[f"{short}_{r['operands']}_mhz"] = r["implied_mhz"]
    return out


def measured_traffic():
    """HBM-side bytes per launch of the headline kernel from the tracked rocprofv3 --pmc summary (FETCH_SIZE and
    WRITE_SIZE, each scaled by what the same counter reads for a plain copy of known size)."""
    try:
        with open(TRAFFIC_FILE) as f:
            t = json.load(f)
        return float(t["fetch_kib"]) * 1024.0 * float(t["fetch_scale"]) + float(t["write_kib"]) * 1024.0 * float(t["write_scale"])
    except (OSError, ValueError, KeyError):
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--preheat-ms", type=float, default=1500.0,
                    help="untimed run of the measured GEMM before warm-up, until the clocks have settled")
    ap.add_argument("--all", action="store_true", help="also time the other benchmark configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline")
    ap.add_argument("--no-vendor", action="store_true", help="skip the vendor-library and power-ceiling child runs")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy a few times, so that FETCH_SIZE / WRITE_SIZE "
                         "counters collected over this command can be scaled by what they read for a known size")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures ONE GPU (the GEMM path has no multi-GPU part); run with --gpus 1. "
                 "A multi-GPU job would shard M or N with no exchange, so N GPUs run N copies of this kernel.")
    M = N = K = 8192

    # child runs first: this process has not initialised the GPU yet
    from gemm_amd.telemetry import Sampler   # imports neither torch nor HIP
    sampler = Sampler().start()
    ceiling = vendor = others = None
    power_ceiling.telemetry = {}
    if not args.no_vendor:
        ceiling = power_ceiling(700, sampler)
        vendor = vendor_leg(M, N, K, 1000, sampler)
        if args.all:
            others = other_configs_leg(300, sampler)

    import torch

    import gemm_amd as g
    from gemm_amd import _abi
    from oracle import gemm_oracle as o   # cpu_baseline leg and the parity spot-check only

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    A, B = o.make_inputs(M, N, K, seed=0)          # N(0,1)/sqrt(K) bf16, generated on the CPU
    Ad, Bd = A.to(dev), B.to(dev)
    C = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    variant, split_k = g.plan(M, N, K)
    need = g.workspace_bytes(M, N, K)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream()
    a_ptr, b_ptr, c_ptr, ws_ptr, st_ptr = Ad.data_ptr(), Bd.data_ptr(), C.data_ptr(), ws.data_ptr() if need else 0, stream.cuda_stream

    def step():
        st = _abi.gemm_raw(a_ptr, b_ptr, c_ptr, M, N, K, K, N, N, g.B_KN, g.C_ROW, ws_ptr, need, st_ptr)
        if st != _abi.OK:
            raise g.NeoGemmError(st)

    # 2. preheat (time-based, untimed)
    mono_pre = time.monotonic()
    t_pre = time.perf_counter()
    while (time.perf_counter() - t_pre) * 1e3 < args.preheat_ms:
        for _ in range(20):
            step()
        torch.cuda.synchronize()
    preheat_ms = (time.perf_counter() - t_pre) * 1e3
    # 3. warm-up, then exactly --steps timed steps in event-bracketed batches
    for _ in range(args.warmup):
        step()
    nb = min(10, args.steps) if args.steps >= 5 else args.steps
    sizes = [args.steps // nb + (1 if i < args.steps % nb else 0) for i in range(nb)]
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(nb + 1)]
    torch.cuda.synchronize()
    mono_t0 = time.monotonic()
    t0 = time.perf_counter()
    ev[0].record(stream)
    for i, n in enumerate(sizes):
        for _ in range(n):
            step()
        ev[i + 1].record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    mono_t1 = time.monotonic()
    batch_ms = [ev[i].elapsed_time(ev[i + 1]) / sizes[i] for i in range(nb)]
    kernel_ms = sorted(batch_ms)[nb // 2]
    flop = 2.0 * M * N * K
    value = flop / (wall_ms * 1e-3) / 1e12
    achieved = flop / (kernel_ms * 1e-3) / 1e12

    # parity spot-check on a sample of rows (the full check lives in tests/test_gemm_gpu.py)
    idx = torch.randperm(M, generator=torch.Generator().manual_seed(1))[:128]
    got = C[idx.to(dev)].cpu()
    ref = o.ref_gemm(A[idx], B)
    rep = o.parity_report(got, A[idx], B, ref=ref)
    parity_ok = (rep["finite"] and rep["rel_fro"] <= o.TOL_REL_FRO and rep["max_ulp_floored"] <= o.TOL_ULP
                 and rep["max_err_vs_bound"] <= 1.0 and rep["frac_gt1_ulp"] <= 2e-3)
    ulp = o.ulp_distance(o.bits_of(got), o.bits_of(ref))
    hist = {"0": int((ulp == 0).sum()), "1": int((ulp == 1).sum()), "2": int((ulp == 2).sum()),
            "3-4": int(((ulp >= 3) & (ulp <= 4)).sum()), "5-16": int(((ulp >= 5) & (ulp <= 16)).sum()),
            ">16": int((ulp > 16).sum())}

    roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / PEAK_TFLOPS, 4),
                # HBM-side bytes per launch from the tracked rocprofv3 --pmc summary; the algorithmic figure is 402.7e6
                "traffic": measured_traffic(),
                "kernel_ms": round(kernel_ms, 5), "batch_ms": [round(b, 5) for b in batch_ms],
                "flop_per_launch": flop, "algorithmic_bytes": 2.0 * (M * K + K * N + M * N)}
    # what the board itself reported while the timed kernel ran (and, for comparison, during the MFMA-only ceiling runs)
    roofline["power"] = {"timed_region": sampler.summary(mono_t0, mono_t1),
                         "preheat_and_timed": brief(sampler.summary(mono_pre, mono_t1)),
                         "mfma_only_ceiling_runs": power_ceiling.telemetry or None}
    if ceiling:
        roofline["power_ceiling"] = ceiling
        # the ceiling of the MFMA order the timed kernel issues: the chained kernel accumulates twice in a row into each
        # tile, the slab kernel walks 2x2 blocks of tiles
        order = ("2x2 blocks, both K steps of a tile back to back" if variant == g.VARIANT_C256x256_W4
                 else "2x2 blocks, serpentine")
        by_order = ceiling.get("by_mfma_order_randn", {})
        if by_order.get(order):
            roofline["power_ceiling_order"] = order
            roofline["frac_of_power_ceiling"] = round(achieved / by_order[order], 4)
        if ceiling.get("16x16x32_randn"):
            roofline["frac_of_plain_order_ceiling"] = round(achieved / ceiling["16x16x32_randn"], 4)

    out = {
        "metric": "BF16 GEMM TFLOP/s at 8192^3 on 1 MI355X; % of dense-BF16 peak",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "preheat_ms": round(preheat_ms, 1),
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
        "roofline": roofline,
        "parity": {"ok": bool(parity_ok), "rows_checked": 128,
                   **{k: rep[k] for k in ("max_ulp", "max_ulp_floored", "rel_fro", "frac_gt1_ulp", "max_err_vs_bound")},
                   "raw_ulp_histogram": hist},
    }
    if vendor:
        out["vendor"] = vendor

    def time_events(fn, steps, warmup):
        for _ in range(warmup):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(steps):
            fn()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps

    # torch.matmul (whatever torch dispatches to) on the same buffers, same process, clocks still warm
    n_t = max(10, args.steps // 2)
    Bnk = Bd.t().contiguous()
    out["torch_matmul"] = {
        "tflops_b_kn": round(flop / time_events(lambda: torch.matmul(Ad, Bd, out=C), n_t, 10) / 1e9, 2),
        "tflops_b_nk": round(flop / time_events(lambda: torch.matmul(Ad, Bnk.t(), out=C), n_t, 10) / 1e9, 2),
        "neogemm_tflops_b_nk": round(flop / time_events(
            lambda: g.gemm_into(Ad, Bnk, C, M, N, K, K, K, N, g.B_NK, g.C_ROW), n_t, 10) / 1e9, 2)}

    if others is not None:
        out["other_configs"] = {"method": "gemm_amd/vendor_bench/matmul_bench, one child per shape and layout of B, run before this "
                                          "process touched the GPU: 300 ms preheat per library, median of 5 event-timed batches; "
                                          "hipBLASLt = best of 8 heuristic candidates; columns *_b_kn: B [K,N], *_b_nk: B [N,K]",
                                "rows": others}

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["calibration_copy_bytes"] = 256 << 20

    if not args.no_cpu:
        # host baseline: the oracle's fp32 product, full-size GEMMs after a small warm-up
        nthreads = torch.get_num_threads()
        o.ref_gemm_f32(A[:256], B)
        times = []
        for _ in range(5):
            t0 = time.perf_counter()
            o.ref_gemm_f32(A, B)
            times.append(time.perf_counter() - t0)
        dt = sorted(times)[len(times) // 2]
        out["cpu_baseline"] = {"value": round(flop / dt / 1e12, 4), "unit": "TFLOP/s", "cores": nthreads, "kind": "port",
                               "sample": f"full M=N=K=8192 fp32 torch.matmul on the host, median of 5 ({dt:.1f} s each), "
                                         f"{os.cpu_count()} logical CPUs visible",
                               "seconds": round(dt, 2)}
    sampler.stop()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
