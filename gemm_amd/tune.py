"""Measure (variant, split-K) candidates for given shapes on the GPU and write the winners as a plan table.

    python -m gemm_amd.tune --out plan_table.json 512x512x512 256x256x8192 16x14336x4096
    NEOGEMM_PLAN_TABLE=plan_table.json python bench.py        # the library reads the table once, at first use
    python -m gemm_amd.tune --merge a.json b.json --inc gemm_amd/csrc/neogemm_default_plan.inc   # the table the library ships

The table is the JSON array libneogemm.so looks up before its cost model (neogemm_bf16_plan): objects
{"M","N","K","b_layout","c_layout","variant","split_k"}; an entry applies to exactly its shape and layouts
(--b-layout 1 tunes B [N,K], --c-layout 1 a column-major C: --b-layout 1 --c-layout 1 is the reference's call,
nemgemmV03.cu:343-391).  Only shapes whose best measured candidate beats the model's
choice by more than --margin are written.  The reference has nothing of the kind: its tile and stage
counts are template arguments (v01.cu:275-278, 304-311).
"""
import argparse
import json
import math
import sys

import torch

from . import _abi, gemm_into, plan
from ._abi import B_KN, B_NK, C_COL, C_ROW, ERR_UNSUPPORTED, NeoGemmError

CANDIDATE_VARIANTS = (_abi.VARIANT_T256x256_W4, _abi.VARIANT_C256x256_W4, _abi.VARIANT_T128x256_W4,
                      _abi.VARIANT_T256x128_W4, _abi.VARIANT_T128x128_W4, _abi.VARIANT_T64x128_W4,
                      _abi.VARIANT_T192x256_W4, _abi.VARIANT_T96x128_W4, _abi.VARIANT_T64x64_W4, _abi.VARIANT_SKINNY16, _abi.VARIANT_SKINNY32, _abi.VARIANT_SKINNY64,
                      _abi.VARIANT_SKINNY128, _abi.VARIANT_STRIP)
CANDIDATE_SPLITS = (1, 2, 3, 4, 6, 8, 12, 16, 24, 32)


def time_us(fn, warmup=5, iters=30, preheat_ms=0.0):
    """Microseconds per call: median of three event-bracketed batches, after `warmup` calls and, for launches long
    enough to be power-limited, `preheat_ms` of the same call (the first launches after an idle stretch run on clocks
    that have not settled: an 8192^3 GEMM takes 15 % longer there)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def batch(n):
        start.record()
        for _ in range(n):
            fn()
        stop.record()
        stop.synchronize()
        return start.elapsed_time(stop) * 1000.0 / n

    heated = 0.0
    while heated < preheat_ms * 1000.0:
        heated += batch(10) * 10
    per = max(1, iters // 3)
    return sorted(batch(per) for _ in range(3))[1]


def tune_shape(M, N, K, nbuf=1, log=sys.stderr, b_layout=B_KN, c_layout=C_ROW, dump=None):
    """Returns (model choice, its time, best choice, its time) for A [M,K], B in `b_layout`, C in `c_layout`."""
    gen = torch.Generator().manual_seed(0)
    A = (torch.randn(M, K, generator=gen) / math.sqrt(K)).to(torch.bfloat16).cuda()
    b_shape = (K, N) if b_layout == B_KN else (N, K)
    Bs = [(torch.randn(*b_shape, generator=gen) / math.sqrt(K)).to(torch.bfloat16).cuda() for _ in range(nbuf)]
    C = torch.empty((M, N) if c_layout == C_ROW else (N, M), dtype=torch.bfloat16, device="cuda")
    turn = [0]

    def call(variant, split):
        turn[0] += 1
        gemm_into(A, Bs[turn[0] % nbuf], C, M, N, K, K, b_shape[1], C.shape[1], b_layout, c_layout, variant, split, 0)

    model = plan(M, N, K, b_layout, c_layout)
    heat = 150.0 if 2.0 * M * N * K > 5e10 else 0.0   # GEMMs of tens of microseconds and more run into the power limit
    t_model = time_us(lambda: call(None, 0), preheat_ms=heat)
    best, t_best = model, t_model
    for v in CANDIDATE_VARIANTS:
        for s in CANDIDATE_SPLITS:
            if s > 1 and K // (64 * s) < 2:
                break
            try:
                # a short look first: a candidate a quarter behind the best so far is not worth a preheated measurement
                t_quick = time_us(lambda: call(v, s), warmup=2, iters=6)
                if t_quick > 1.25 * t_best:
                    if dump is not None:
                        dump.append({"M": M, "N": N, "K": K, "b_layout": b_layout, "c_layout": c_layout, "variant": v, "split_k": s,
                                     "us": round(t_quick, 2), "quick": True})
                    continue
                t = time_us(lambda: call(v, s), preheat_ms=heat)
                if dump is not None:
                    dump.append({"M": M, "N": N, "K": K, "b_layout": b_layout, "c_layout": c_layout, "variant": v, "split_k": s,
                                 "us": round(t, 2), "quick": False})
            except NeoGemmError as e:
                if e.status != ERR_UNSUPPORTED:
                    raise
                continue   # (a variant may refuse a shape unsplit and take it split: the strip kernel up to 64 rows)
            if t < t_best:
                best, t_best = (v, s), t
    t_model = min(t_model, time_us(lambda: call(None, 0), preheat_ms=heat))   # the first measurement ran on a cold clock
    if best == model or t_model <= t_best:
        best, t_best = model, t_model
    print(f"{M}x{N}x{K} b{b_layout} c{c_layout}: model {model} {t_model:.2f} us, best {best} {t_best:.2f} us", file=log)
    return model, t_model, best, t_best


def write_inc(tables, path):
    """Merge plan tables (lists of entries as this module writes them) into the initialiser list the library compiles in
    as its default table (gemm_amd/csrc/neogemm_default_plan.inc)."""
    seen, rows = set(), []
    for t in tables:
        for e in t:
            key = (e["M"], e["N"], e["K"], e.get("b_layout", 0), e.get("c_layout", 0))
            if key not in seen:
                seen.add(key)
                rows.append(key + (e["variant"], e["split_k"]))
    rows.sort(key=lambda r: (r[3], r[4], r[0], r[1], r[2]))
    with open(path, "w") as f:
        f.write("// {M, N, K, b_layout, c_layout, variant, split_k}: tuned exceptions to plan_model (see kDefaultPlan in neogemm.hip).\n"
                "// Written by `python -m gemm_amd.tune --merge ... --inc` from the tables a tuning sweep produced; the entry with all\n"
                "// fields zero keeps the array non-empty.\n{0, 0, 0, 0, 0, 0, 0},\n")
        for r in rows:
            f.write("{%d, %d, %d, %d, %d, %d, %d},\n" % r)
    return len(rows)


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("shapes", nargs="*", help="MxNxK")
    ap.add_argument("--out")
    ap.add_argument("--merge", nargs="+", metavar="TABLE.json", help="merge these tables instead of measuring (no GPU needed)")
    ap.add_argument("--inc", help="with --merge: write the merged table as the library's default-plan include file")
    ap.add_argument("--margin", type=float, default=0.03, help="minimum relative gain over the model's choice")
    ap.add_argument("--nbuf", type=int, default=1, help="rotate this many B buffers (streaming shapes)")
    ap.add_argument("--cold-weights-mb", type=float, default=0.0,
                    help="rotate as many B buffers as it takes to exceed this many MB (more than the last-level cache: every "
                         "launch then streams its B from HBM, as a layer's weights are in inference); overrides --nbuf")
    ap.add_argument("--dump", help="also write every candidate's time to this file, one JSON object per line (for fitting the "
                                   "cost model; a candidate that the short look dropped carries that look's time and quick: true)")
    ap.add_argument("--b-layout", type=int, default=B_KN, choices=(B_KN, B_NK), help="0: B [K,N], 1: B [N,K]")
    ap.add_argument("--c-layout", type=int, default=C_ROW, choices=(C_ROW, C_COL), help="0: row-major C, 1: column-major")
    args = ap.parse_args()
    if args.merge:
        if not args.inc:
            sys.exit("--merge needs --inc")
        tables = []
        for path in args.merge:
            with open(path) as f:
                tables.append(json.load(f))
        print(f"{write_inc(tables, args.inc)} entries written to {args.inc}", file=sys.stderr)
        return
    if not args.shapes or not args.out:
        sys.exit("give shapes and --out (or --merge ... --inc ...)")
    if not torch.cuda.is_available():
        sys.exit("tuning needs a GPU")
    table = []
    for sh in args.shapes:
        M, N, K = (int(x) for x in sh.lower().split("x"))
        nbuf = args.nbuf
        if args.cold_weights_mb > 0:
            nbuf = max(2, min(32, int(args.cold_weights_mb * 1e6 // (2.0 * N * K)) + 1))
        dump = [] if args.dump else None
        model, t_model, best, t_best = tune_shape(M, N, K, nbuf, b_layout=args.b_layout, c_layout=args.c_layout, dump=dump)
        if dump:
            with open(args.dump, "a") as f:
                for d in dump:
                    f.write(json.dumps(d) + "\n")
        if best != model and t_best < t_model * (1.0 - args.margin):
            table.append({"M": M, "N": N, "K": K, "b_layout": args.b_layout, "c_layout": args.c_layout,
                          "variant": best[0], "split_k": best[1]})
        # the table so far after every shape: a sweep that is cut short keeps what it has measured
        with open(args.out, "w") as f:
            json.dump(table, f, indent=1)
    print(f"{len(table)} entries written to {args.out}", file=sys.stderr)


if __name__ == "__main__":
    main()
