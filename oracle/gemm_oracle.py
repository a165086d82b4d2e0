"""TEST INFRASTRUCTURE — CPU oracle for the BF16 GEMM path.  Never imported by the product.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may use this module; gemm_amd/
and neoGEMM must not (and fail loudly without their HIP library instead).

The contract being restated (reference kernel v01.cu:189-270, launcher nemgemmV03.cu:343-391):
    C[i,j] = RNE_bf16( sum_k float(A[i,k]) * float(B[k,j]) ), accumulation in fp32, one rounding.
The reference cannot be built or imported here (CUDA + NVIDIA-only PTX; benchmark.py:2 needs the
built extension and allocates on `cuda` at import).  It also holds no golden vector, fixture or
asserting test for this path, so the oracle is pinned by what the mathematics fixes — see
tests/test_oracle.py: hand-derived rounding table, exact-integer products (order-independent, so
bit-exact), identity/one-hot selections, an fp64 triple loop on small odd shapes, agreement between
the three independent restatements below.

Restatements:
  ref_gemm            torch.matmul in fp32 on the CPU, rounded to bf16 — the oracle the task names.
  c_gemm / c_gemm_v1_tiles   plain C (oracle/gemm_oracle.c via ctypes): sequential-k fp32 sum, and the
                      reference's own walk (64x64x64 tiles, four k16 MMAs per slab, column-major C).
  ref_gemm_scaled     alpha * A*B + beta * C in fp32 with one rounding (neogemm_bf16_scaled).
  exact_gemm_f64      fp64 product of the bf16 inputs: the value both fp32 orders approximate.
  f32_to_bf16_bits    round-to-nearest-even written with integer arithmetic (numpy).
"""
import ctypes
import math
import os

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_CLIB_PATH = os.path.join(_HERE, "libgemm_oracle.so")
_clib = None


# ----------------------------------------------------------------------------- bf16 bit helpers
def f32_to_bf16_bits(x):
    """float32 ndarray -> uint16 bf16 bits, round-to-nearest-even (v01.cu:254, __float2bfloat16)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    r = np.where(nan, (u >> 16) | 0x0040, r)
    return r.astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def bits_of(t):
    """torch bf16 tensor (CPU) -> numpy uint16 bits."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(b):
    """numpy uint16 bits -> torch bf16 tensor (CPU)."""
    return torch.from_numpy(np.ascontiguousarray(b, dtype=np.uint16).view(np.int16)).view(torch.bfloat16)


def ordered(bits):
    """Map bf16 bit patterns to integers that are monotonic in the value (so differences count ulps)."""
    b = np.asarray(bits, dtype=np.uint16).astype(np.int32)
    return np.where(b & 0x8000, -(b & 0x7FFF), b)


def ulp_distance(a_bits, b_bits):
    """Element-wise distance in bf16 units in the last place between two bf16 bit arrays."""
    return np.abs(ordered(a_bits) - ordered(b_bits))


# ----------------------------------------------------------------------------- inputs
def make_inputs(M, N, K, seed=0, b_layout="kn"):
    """Seeded inputs of the benchmark configs: N(0,1)/sqrt(K) cast to bf16, generated on the CPU.

    A is [M,K]; B is [K,N] ("kn") or the same matrix stored [N,K] ("nk", the reference's layout).
    """
    g = torch.Generator().manual_seed(seed)
    s = 1.0 / math.sqrt(max(K, 1))
    A = (torch.randn(M, K, generator=g) * s).to(torch.bfloat16)
    B = (torch.randn(K, N, generator=g) * s).to(torch.bfloat16)
    if b_layout == "nk":
        B = B.t().contiguous()
    return A, B


# ----------------------------------------------------------------------------- oracles
def ref_gemm(A, B, b_layout="kn"):
    """fp32-accumulated CPU product rounded to bf16.  A [M,K]; B [K,N] or [N,K]."""
    Bf = B.float() if b_layout == "kn" else B.float().t()
    return torch.matmul(A.float(), Bf).to(torch.bfloat16)


def ref_gemm_f32(A, B, b_layout="kn"):
    Bf = B.float() if b_layout == "kn" else B.float().t()
    return torch.matmul(A.float(), Bf)


def ref_gemm_scaled(A, B, C0, alpha, beta, b_layout="kn"):
    """alpha * A*B + beta * C0 the way neogemm_bf16_scaled states it (the epilogue the reference's v4
    kernel declares, neogemmv4.cu:166,266): fp32 t = alpha * acc; if beta != 0: t = fma(beta, C0, t);
    one rounding to bf16.  With beta == 0, C0 is not looked at.  The fused multiply-add is taken in fp64
    (beta * C0 is exact there) and rounded to fp32."""
    acc = ref_gemm_f32(A, B, b_layout)
    t = acc * torch.tensor(alpha, dtype=torch.float32)
    if beta != 0.0:
        b32 = float(torch.tensor(beta, dtype=torch.float32))
        t = (b32 * C0.double() + t.double()).float()
    return t.to(torch.bfloat16)


def scaled_parity(C, A, B, C0, alpha, beta, b_layout="kn"):
    """(max error in bf16 ulps at max(|ref|, 2^-7 rms), relative Frobenius error) of C against ref_gemm_scaled."""
    ref = ref_gemm_scaled(A, B, C0, alpha, beta, b_layout).double()
    Cc = C.detach().cpu().double()
    rms = float(torch.sqrt(torch.mean(ref * ref))) if ref.numel() else 0.0
    mag = torch.clamp(ref.abs(), min=max(rms * 2.0 ** -7, 1e-38))
    ulp = torch.exp2(torch.floor(torch.log2(mag)) - 7)
    return float(((Cc - ref).abs() / ulp).max()), rel_frobenius(Cc, ref)


def exact_gemm_f64(A, B, b_layout="kn"):
    Bd = B.double() if b_layout == "kn" else B.double().t()
    return torch.matmul(A.double(), Bd)


def abs_gemm_f64(A, B, b_layout="kn"):
    """sum_k |a||b| — scale of the fp32 accumulation error of any summation order."""
    Bd = B.double().abs() if b_layout == "kn" else B.double().abs().t()
    return torch.matmul(A.double().abs(), Bd)


def _c():
    global _clib
    if _clib is None:
        if not os.path.exists(_CLIB_PATH):
            raise RuntimeError(f"{_CLIB_PATH} missing: run `make -C oracle` (or __graft_entry__.build())")
        lib = ctypes.CDLL(_CLIB_PATH)
        p16 = ctypes.c_void_p
        i64 = ctypes.c_int64
        lib.oracle_gemm_bf16.restype = None
        lib.oracle_gemm_bf16.argtypes = [p16, p16, p16, i64, i64, i64, i64, i64, i64, ctypes.c_int, ctypes.c_int]
        lib.oracle_gemm_v1_tiles.restype = ctypes.c_int
        lib.oracle_gemm_v1_tiles.argtypes = [p16, p16, p16, i64, i64, i64]
        lib.oracle_f32_to_bf16.restype = ctypes.c_uint16
        lib.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        _clib = lib
    return _clib


def c_f32_to_bf16(x):
    return int(_c().oracle_f32_to_bf16(float(x)))


def c_gemm(A, B, b_layout="kn", c_layout="row"):
    """Plain-C sequential-k oracle.  Returns bf16 tensor [M,N] (row) or the column-major buffer viewed [N,M]."""
    A = A.contiguous()
    B = B.contiguous()
    M, K = A.shape
    N = B.shape[1] if b_layout == "kn" else B.shape[0]
    a, b = bits_of(A), bits_of(B)
    out = np.zeros((M, N) if c_layout == "row" else (N, M), dtype=np.uint16)
    _c().oracle_gemm_bf16(a.ctypes.data, b.ctypes.data, out.ctypes.data, M, N, K, max(K, 1),
                          max(N if b_layout == "kn" else K, 1), max(N if c_layout == "row" else M, 1),
                          0 if b_layout == "kn" else 1, 0 if c_layout == "row" else 1)
    return from_bits(out)


def c_gemm_v1_tiles(A, B_nk):
    """The reference's walk (v01.cu): A [M,K], B [N,K] -> column-major C returned as a [N,M] tensor."""
    A = A.contiguous()
    B_nk = B_nk.contiguous()
    M, K = A.shape
    N = B_nk.shape[0]
    a, b = bits_of(A), bits_of(B_nk)
    out = np.zeros((N, M), dtype=np.uint16)
    st = _c().oracle_gemm_v1_tiles(a.ctypes.data, b.ctypes.data, out.ctypes.data, M, N, K)
    if st != 0:
        raise ValueError("M, N and K must be multiples of 64 (nemgemmV03.cu:375)")
    return from_bits(out)


# ----------------------------------------------------------------------------- parity metrics
def rel_frobenius(C, ref_f64):
    d = C.double().cpu() - ref_f64
    return float(torch.linalg.norm(d) / max(float(torch.linalg.norm(ref_f64)), 1e-300))


def parity_report(C, A, B, b_layout="kn", ref=None):
    """Compare a bf16 result C (any device) with the oracle for (A, B) on the CPU.

    Returns a dict:
      max_ulp          largest bf16-ulp distance to ref_gemm (raw)
      frac_gt1_ulp     fraction of elements more than 1 ulp from ref_gemm (raw)
      max_ulp_floored  largest distance in units of the bf16 ulp at max(|ref|, 2^-7 * rms(ref)):
                       fp32 sums taken in different orders differ by ~sqrt(K)*2^-24 of the partial
                       sums, which exceeds the ulp of elements that cancel to nearly zero, so raw
                       ulps of such elements say nothing about the kernel
      rel_fro          ||C - ref|| / ||ref|| with ref = ref_gemm (the bf16-rounded fp32 CPU product)
      rel_fro_exact    ||C - exact|| / ||exact|| with exact = the fp64 product; ~1.7e-3 for ANY correctly
                       rounded bf16 result (that is the rounding of the output itself), reported only
      max_err_vs_bound max over elements of |C - exact| / (half a bf16 ulp of |exact| plus
                       4*sqrt(K)*2^-24 * sum_k|a||b|): at most ~1 for any correct fp32-accumulating kernel
    """
    Cc = C.detach().cpu().contiguous()
    if ref is None:
        ref = ref_gemm(A, B, b_layout)
    exact = exact_gemm_f64(A, B, b_layout)
    cb, rb = bits_of(Cc), bits_of(ref)
    ulp = ulp_distance(cb, rb)
    K = A.shape[1]
    rf = ref.double()
    rms = float(torch.sqrt(torch.mean(rf * rf))) if rf.numel() else 0.0
    floor = max(rms * 2.0 ** -7, 1e-38)
    mag = torch.clamp(rf.abs(), min=floor)
    ulp_size = torch.exp2(torch.floor(torch.log2(mag)) - 7)
    floored = ((Cc.double() - rf).abs() / ulp_size)
    mag_e = torch.clamp(exact.abs(), min=1e-38)
    half_ulp = torch.exp2(torch.floor(torch.log2(mag_e)) - 8)
    bound = half_ulp * 1.0000001 + 4.0 * math.sqrt(max(K, 1)) * 2.0 ** -24 * abs_gemm_f64(A, B, b_layout)
    err = (Cc.double() - exact).abs()
    finite = bool(torch.isfinite(Cc.float()).all())
    return {
        "max_ulp": int(ulp.max()) if ulp.size else 0,
        "frac_gt1_ulp": float((ulp > 1).mean()) if ulp.size else 0.0,
        "max_ulp_floored": float(floored.max()) if floored.numel() else 0.0,
        "rel_fro": rel_frobenius(Cc, rf) if Cc.numel() else 0.0,
        "rel_fro_exact": rel_frobenius(Cc, exact) if Cc.numel() else 0.0,
        "max_err_vs_bound": float((err / bound).max()) if err.numel() else 0.0,
        "finite": finite,
    }


# Tolerance the task states: <= 1 bf16 ulp per element and <= 1e-3 relative Frobenius error against
# the fp32-accumulated CPU product rounded to bf16.
TOL_ULP = 1
TOL_REL_FRO = 1e-3


def assert_parity(C, A, B, b_layout="kn", ref=None, what=""):
    r = parity_report(C, A, B, b_layout, ref)
    assert r["finite"], f"{what}: non-finite output {r}"
    assert r["rel_fro"] <= TOL_REL_FRO, f"{what}: relative Frobenius error {r['rel_fro']:.3e} > {TOL_REL_FRO} {r}"
    assert r["max_ulp_floored"] <= TOL_ULP, f"{what}: {r['max_ulp_floored']} ulp (floored) > {TOL_ULP} {r}"
    assert r["max_err_vs_bound"] <= 1.0, f"{what}: error beyond half-ulp + fp32 accumulation bound {r}"
    # raw ulps may exceed 1 only on elements that cancel to nearly zero; that is rare
    assert r["frac_gt1_ulp"] <= 2e-3, f"{what}: {r['frac_gt1_ulp']:.2e} of elements more than 1 raw ulp off {r}"
    return r
