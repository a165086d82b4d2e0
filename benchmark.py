#!/usr/bin/env python3
"""Correctness printout and timing of the `neoGEMM` extension beside torch.matmul, one shape at a time.

The counterpart of the reference's driver (benchmark.py:1-100): same call pattern — bf16 A [M,K] and
B [N,K] on the GPU, `neoGEMM.neoGemmV1(A, B, C)` into a zeroed C whose storage then holds the product
column-major (benchmark.py:10-25) — followed by the same three blocks: error statistics against
`A @ B.t()` (benchmark.py:33-53), timing of torch (benchmark.py:57-77) and of the kernel
(benchmark.py:80-100), both as 2*M*N*K / t.  Unlike the reference it seeds its inputs, scales them by
1/sqrt(K), takes the shape from the command line (default: every benchmark configuration), times with
events on the stream instead of the host clock, and also times `neoGEMM.gemm(A, B)` with B [K,N].

    python benchmark.py                 # all configurations
    python benchmark.py 8192 8192 8192  # one shape
"""
import argparse
import math
import sys

import torch

CONFIGS = [(512, 512, 512), (4096, 4096, 4096), (8192, 8192, 8192), (16, 14336, 4096), (64, 14336, 4096),
           (128, 14336, 4096), (3000, 5120, 3584), (1024, 1024, 32768)]


def time_ms(fn, warmup, iters):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def run(M, N, K, warmup=10, iters=100, seed=0, out=sys.stdout):
    """One shape: returns a dict with the error statistics and the timings (also printed)."""
    import neoGEMM  # the built extension; needs `import torch` first (it links against torch's HIP runtime)

    def say(*a):
        print(*a, file=out)

    gen = torch.Generator().manual_seed(seed)
    A = (torch.randn(M, K, generator=gen) / math.sqrt(K)).to(torch.bfloat16).cuda()
    Bnk = (torch.randn(N, K, generator=gen) / math.sqrt(K)).to(torch.bfloat16).cuda()
    Bkn = Bnk.t().contiguous()
    C = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda")

    say(f"=== {M} x {N} x {K} ===")
    ref = A @ Bnk.t()
    neoGEMM.neoGemmV1(A, Bnk, C)
    got = C.view(N, M).t()  # the storage is the product column-major
    say("1. torch  A @ B.t():   shape", tuple(ref.shape), ref.dtype, "\n", ref[:3, :3])
    say("2. neoGEMM.neoGemmV1:  shape", tuple(got.shape), got.dtype, "\n", got[:3, :3])

    diff = (got.float() - ref.float()).abs()
    stats = {"max_err": diff.max().item(), "mean_err": diff.mean().item(),
             "rms_err": diff.pow(2).mean().sqrt().item(),
             "rel_fro": (diff.norm() / ref.float().norm().clamp_min(1e-30)).item()}
    say(f"max error {stats['max_err']:.8f}   mean {stats['mean_err']:.8f}   rms {stats['rms_err']:.8f}   "
        f"relative Frobenius {stats['rel_fro']:.3e}")
    say(f"value range: torch [{ref.min().item():.4f}, {ref.max().item():.4f}]   "
        f"neoGEMM [{got.min().item():.4f}, {got.max().item():.4f}]")
    for tol in (1e-2, 1e-3, 1e-4, 1e-5):
        ok = torch.allclose(got.float(), ref.float(), atol=tol, rtol=tol)
        say(f"  allclose at {tol:.0e}: {'pass' if ok else 'fail'}")
    stats["pct_within_1e-3"] = (diff < 1e-3).float().mean().item() * 100.0
    say(f"  elements within 1e-3: {stats['pct_within_1e-3']:.2f} %")

    flops = 2.0 * M * N * K
    Bt = Bnk.t()
    timings = {
        "torch  A @ B.t()  (B [N,K])": time_ms(lambda: torch.matmul(A, Bt), warmup, iters),
        "torch  A @ B      (B [K,N])": time_ms(lambda: torch.matmul(A, Bkn), warmup, iters),
        "neoGEMM.neoGemmV1 (B [N,K])": time_ms(lambda: neoGEMM.neoGemmV1(A, Bnk, C), warmup, iters),
        "neoGEMM.gemm      (B [K,N])": time_ms(lambda: neoGEMM.gemm(A, Bkn), warmup, iters),
    }
    for name, ms in timings.items():
        say(f"{name}: {ms:.4f} ms   {flops / ms / 1e9:.2f} TFLOP/s")
    stats["ms"] = timings
    return stats


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("shape", nargs="*", type=int, help="M N K (default: every benchmark configuration)")
    ap.add_argument("--iters", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    args = ap.parse_args()
    if args.shape and len(args.shape) != 3:
        ap.error("give M N K or nothing")
    if not torch.cuda.is_available():
        sys.exit("benchmark.py needs a GPU: the extension has no CPU path")
    for (m, n, k) in ([tuple(args.shape)] if args.shape else CONFIGS):
        run(m, n, k, args.warmup, args.iters)


if __name__ == "__main__":
    main()
