"""Writes the golden fixtures of tests/golden/*.npz with this repository's own CPU oracle.

The reference holds no golden vector, fixture or asserting test for the GEMM path (its benchmark.py
only prints, on unseeded inputs), and it cannot be built or imported here, so there is nothing of the
reference's to record.  These fixtures instead freeze the oracle itself — which tests/test_oracle.py
pins against hand-derived roundings, exact-integer products and an fp64 triple loop — so that a later
change to oracle/ (or to torch's CPU matmul) that alters a result is noticed, and so that the GPU box
checks against bytes that were produced here.

    python tests/golden/make_golden.py

Each file: A [M,K], B [K,N] (bf16 bit patterns as uint16), C = RNE_bf16(fp32-accumulated A @ B) from
the plain-C sequential-k oracle, C_torch from torch.matmul in fp32, shape and seed.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import gemm_oracle as o  # noqa: E402

CASES = [
    # name, M, N, K, seed
    ("tile64", 64, 64, 64, 101),          # one tile of the reference kernel (v01.cu:275-278)
    ("ragged", 96, 80, 72, 102),          # M, N, K not multiples of 64; K % 8 == 0
    ("odd", 33, 47, 19, 103),             # nothing aligned: generic path
    ("skinny16", 16, 64, 256, 104),      # decode-style: M = 16
    ("tallk", 16, 16, 1024, 105),         # long accumulation
]


def main():
    for name, M, N, K, seed in CASES:
        A, B = o.make_inputs(M, N, K, seed=seed)
        C = o.c_gemm(A, B)
        Ct = o.ref_gemm(A, B)
        path = os.path.join(HERE, f"{name}.npz")
        np.savez_compressed(path, A=o.bits_of(A), B=o.bits_of(B), C=o.bits_of(C), C_torch=o.bits_of(Ct),
                            shape=np.array([M, N, K]), seed=np.array([seed]))
        d = int((o.ulp_distance(o.bits_of(C), o.bits_of(Ct)) > 0).sum())
        print(f"{name}: {M}x{N}x{K} seed {seed} -> {os.path.getsize(path)} bytes; C vs C_torch differ in {d} elements")


if __name__ == "__main__":
    main()
