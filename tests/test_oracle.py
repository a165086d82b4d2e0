"""Pins the CPU oracle (oracle/) — the checker every GPU parity test relies on — without a GPU.

The reference has no golden vectors or asserting tests for the GEMM path and cannot be built here, so
the oracle is pinned by what the mathematics fixes:
  * a table of hand-derived bf16 roundings (ties to even, carries into the exponent, subnormals,
    infinities, NaN) for the epilogue convert (v01.cu:254-262, __float2bfloat16);
  * products whose fp32 sum is exact and therefore independent of summation order (small integers,
    powers of two, identity, one-hot selection) — expected values are computed with Python integers;
  * an fp64 triple loop on small odd shapes for indexing and layout flags (b_layout, c_layout);
  * agreement of the three independent restatements (torch fp32 matmul, plain-C sequential sum, the
    reference's 64x64x64 tile walk);
  * the committed fixtures of tests/golden.
A dropped k term, a transposed operand, a wrong leading dimension or a truncating convert fails at
least one of these.
"""
import glob
import os
import struct

import numpy as np
import pytest
import torch

from oracle import gemm_oracle as o

HERE = os.path.dirname(os.path.abspath(__file__))


def f32(bits):
    return struct.unpack("<f", struct.pack("<I", bits))[0]


# (fp32 bit pattern, expected bf16 bit pattern), derived by hand: keep the top 16 bits, round on bit 15
# with the lower 15 bits as sticky, ties go to the even (bit 16 == 0) neighbour.
ROUNDING_TABLE = [
    (0x3F800000, 0x3F80),  # 1.0 exact
    (0x3F808000, 0x3F80),  # 1 + 2^-8: tie, lsb 0 -> stays (even)
    (0x3F818000, 0x3F82),  # 1 + 3*2^-8: tie, lsb 1 -> up to even
    (0x3F808001, 0x3F81),  # just above the tie -> up
    (0x3F807FFF, 0x3F80),  # just below the tie -> down
    (0x43808000, 0x4380),  # 257.0 -> 256 (tie to even)
    (0x43818000, 0x4382),  # 259.0 -> 260 (tie to even)
    (0x43810000, 0x4381),  # 258.0 exact in bf16
    (0x3FFFFFFF, 0x4000),  # 1.99999988 -> 2.0: carry ripples into the exponent
    (0x7F7FFFFF, 0x7F80),  # FLT_MAX -> +inf (rounds up past the largest bf16)
    (0x7F7F7FFF, 0x7F7F),  # just below the last tie -> largest finite bf16
    (0x00000000, 0x0000),  # +0
    (0x80000000, 0x8000),  # -0 keeps its sign
    (0x00008000, 0x0000),  # fp32 subnormal at the tie with even neighbour 0 -> 0
    (0x00018000, 0x0002),  # subnormal tie, odd lsb -> up
    (0x00008001, 0x0001),  # subnormal just above the tie -> smallest bf16 subnormal
    (0xBF808000, 0xBF80),  # sign is untouched by rounding
    (0xBF818000, 0xBF82),
    (0x7F800000, 0x7F80),  # +inf
    (0xFF800000, 0xFF80),  # -inf
]


@pytest.mark.parametrize("fbits,expected", ROUNDING_TABLE)
def test_rounding_table(fbits, expected):
    x = np.array([fbits], dtype=np.uint32).view(np.float32)
    assert int(o.f32_to_bf16_bits(x)[0]) == expected          # numpy integer restatement
    assert o.c_f32_to_bf16(f32(fbits)) == expected            # plain C restatement
    t = torch.from_numpy(x.copy()).to(torch.bfloat16)          # torch's own convert
    assert int(o.bits_of(t)[0]) == expected


def test_rounding_nan_stays_nan():
    for fbits in (0x7FC00000, 0x7F800001, 0xFFC12345):
        x = np.array([fbits], dtype=np.uint32).view(np.float32)
        b = int(o.f32_to_bf16_bits(x)[0])
        assert (b & 0x7F80) == 0x7F80 and (b & 0x007F) != 0
        assert (b >> 15) == (fbits >> 31)
        c = o.c_f32_to_bf16(float("nan"))
        assert (c & 0x7F80) == 0x7F80 and (c & 0x007F) != 0


def test_rounding_exhaustive_against_torch():
    # every bf16 value, perturbed below / at / above the half-way point to the next one
    hi = np.arange(0, 0x7F80, dtype=np.uint32)  # positive finite bf16 patterns
    for low in (0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF):
        x = ((hi << 16) | low).astype(np.uint32).view(np.float32)
        mine = o.f32_to_bf16_bits(x)
        ref = o.bits_of(torch.from_numpy(x.copy()).to(torch.bfloat16))
        assert np.array_equal(mine, ref), f"low bits {low:#06x}"


def _int_matrix(rng, rows, cols, lo, hi):
    return torch.from_numpy(rng.integers(lo, hi + 1, size=(rows, cols)).astype(np.float32)).to(torch.bfloat16)


@pytest.mark.parametrize("M,N,K", [(5, 7, 9), (64, 64, 64), (17, 33, 130)])
def test_exact_integer_products(M, N, K):
    """|a|,|b| <= 8 and K <= 130: every partial sum is an integer below 2^24, so any fp32 summation order
    gives the same exact sum; the expected bf16 is the RNE rounding of that integer (done here with
    Python integers)."""
    rng = np.random.default_rng(7)
    A = _int_matrix(rng, M, K, -8, 8)
    B = _int_matrix(rng, K, N, -8, 8)
    exact = A.to(torch.int64) @ B.to(torch.int64)

    def rne_int_to_bf16_value(v):
        if v == 0:
            return 0.0
        s, a = (-1 if v < 0 else 1), abs(v)
        e = a.bit_length() - 1
        if e <= 7:
            return float(v)
        shift = e - 7
        q, r = a >> shift, a & ((1 << shift) - 1)
        half = 1 << (shift - 1)
        if r > half or (r == half and (q & 1)):
            q += 1
        return float(s * (q << shift))

    want = torch.tensor([[rne_int_to_bf16_value(int(v)) for v in row] for row in exact.tolist()])
    for name, got in (("torch", o.ref_gemm(A, B)), ("c", o.c_gemm(A, B)),
                      ("c nk/col", o.c_gemm(A, B.t().contiguous(), "nk", "col").t())):
        assert torch.equal(got.float(), want), name


def test_identity_and_selection():
    rng = np.random.default_rng(3)
    A, _ = o.make_inputs(40, 40, 40, seed=5)
    I = torch.eye(40, dtype=torch.bfloat16)
    for fn in (o.ref_gemm, o.c_gemm):
        assert torch.equal(fn(A, I), A)      # B = I  => C = A bit for bit
        assert torch.equal(fn(I, A), A)      # A = I  => C = B
    perm = torch.from_numpy(rng.permutation(40))
    P = torch.zeros(40, 40, dtype=torch.bfloat16)
    P[torch.arange(40), perm] = 1            # one-hot rows: (P @ A)[i] = A[perm[i]]
    assert torch.equal(o.c_gemm(P, A), A[perm])
    assert torch.equal(o.ref_gemm(P, A), A[perm])
    # powers of two scale exactly
    assert torch.equal(o.c_gemm((A.float() * 4).bfloat16(), I), (A.float() * 4).bfloat16())


def test_ones_sum_to_k():
    for K in (1, 8, 255, 256, 257, 259, 1000):
        A = torch.ones(3, K, dtype=torch.bfloat16)
        B = torch.ones(K, 2, dtype=torch.bfloat16)
        want = torch.tensor(float(K)).to(torch.bfloat16)   # 257 -> 256, 259 -> 260, 1000 -> 1000
        assert torch.all(o.c_gemm(A, B) == want) and torch.all(o.ref_gemm(A, B) == want)
    assert float(torch.tensor(257.0).to(torch.bfloat16)) == 256.0
    assert float(torch.tensor(259.0).to(torch.bfloat16)) == 260.0


@pytest.mark.parametrize("M,N,K", [(3, 5, 7), (9, 4, 33), (16, 18, 20)])
@pytest.mark.parametrize("b_layout", ["kn", "nk"])
@pytest.mark.parametrize("c_layout", ["row", "col"])
def test_triple_loop_fp64(M, N, K, b_layout, c_layout):
    """Independent fp64 triple loop with explicit indexing: pins b_layout / c_layout / leading dimensions."""
    A, Bkn = o.make_inputs(M, N, K, seed=M * 100 + N)
    B = Bkn if b_layout == "kn" else Bkn.t().contiguous()
    a, b = A.double().tolist(), B.double().tolist()
    want = [[0.0] * N for _ in range(M)]
    for i in range(M):
        for j in range(N):
            s = 0.0
            for k in range(K):
                s += a[i][k] * (b[k][j] if b_layout == "kn" else b[j][k])
            want[i][j] = s
    want = torch.tensor(want, dtype=torch.float64)
    got = o.c_gemm(A, B, b_layout, c_layout)
    if c_layout == "col":
        assert got.shape == (N, M)
        got = got.t()
    # fp64 sum vs fp32 sum: equal after rounding to bf16 except where the fp32 error crosses a rounding
    # boundary; at these sizes that is at most 1 ulp
    ulp = o.ulp_distance(o.bits_of(got.contiguous()), o.bits_of(want.to(torch.bfloat16)))
    assert ulp.max() <= 1
    assert torch.equal(o.ref_gemm(A, B, b_layout).float(), got.float()) or ulp.max() <= 1
    assert torch.allclose(o.exact_gemm_f64(A, B, b_layout), want, rtol=1e-12, atol=1e-12)


def test_three_restatements_agree():
    M, N, K = 128, 192, 256
    A, Bkn = o.make_inputs(M, N, K, seed=21)
    Bnk = Bkn.t().contiguous()
    r_torch = o.ref_gemm(A, Bkn)
    r_c = o.c_gemm(A, Bkn)
    r_tiles = o.c_gemm_v1_tiles(A, Bnk).t()      # column-major buffer viewed [N,M], transposed back
    for name, r in (("c", r_c), ("tiles", r_tiles)):
        rep = o.assert_parity(r, A, Bkn, ref=r_torch, what=name)
        assert rep["max_ulp"] <= 1
    # the tile walk and the sequential sum add in the same k order per element: identical bits
    assert torch.equal(r_tiles.contiguous(), r_c)
    with pytest.raises(ValueError):
        o.c_gemm_v1_tiles(A[:100], Bnk)           # the reference needs multiples of 64


def test_reference_call_contract():
    """benchmark.py:10-25: A [M,K], B [N,K], C buffer; after the call C.t() must equal A @ B.t()."""
    M = N = K = 64
    A, Bnk = o.make_inputs(M, N, K, seed=9, b_layout="nk")
    Cbuf = o.c_gemm(A, Bnk, "nk", "col")          # the column-major buffer, shaped [N, M]
    want = (A.float() @ Bnk.float().t()).to(torch.bfloat16)
    assert torch.equal(Cbuf.reshape(M, N).t().contiguous(), want) or \
        o.ulp_distance(o.bits_of(Cbuf.reshape(M, N).t().contiguous()), o.bits_of(want)).max() <= 1


def test_parity_report_catches_errors():
    A, B = o.make_inputs(64, 64, 512, seed=2)
    good = o.ref_gemm(A, B)
    o.assert_parity(good, A, B)
    # a dropped k term
    bad = (A[:, :-1].float() @ B[:-1].float()).to(torch.bfloat16)
    with pytest.raises(AssertionError):
        o.assert_parity(bad, A, B)
    # a transposed operand
    with pytest.raises(AssertionError):
        o.assert_parity(o.ref_gemm(A, B.t().contiguous().reshape(512, 64)), A, B)
    # truncation instead of round-to-nearest
    trunc = o.from_bits((o.ref_gemm_f32(A, B).numpy().view(np.uint32) >> 16).astype(np.uint16))
    with pytest.raises(AssertionError):
        o.assert_parity(trunc, A, B)
    # one element off by 2 ulp
    b = o.bits_of(good).copy()
    b[3, 4] += 2
    with pytest.raises(AssertionError):
        o.assert_parity(o.from_bits(b), A, B)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(HERE, "golden", "*.npz"))))
def test_golden_fixtures(path):
    z = np.load(path, allow_pickle=False)
    M, N, K = (int(v) for v in z["shape"])
    A, B = o.from_bits(z["A"]), o.from_bits(z["B"])
    assert A.shape == (M, K) and B.shape == (K, N)
    # the fixture's inputs are what the seeded generator makes today
    A2, B2 = o.make_inputs(M, N, K, seed=int(z["seed"][0]))
    assert np.array_equal(o.bits_of(A2), z["A"]) and np.array_equal(o.bits_of(B2), z["B"])
    assert np.array_equal(o.bits_of(o.c_gemm(A, B)), z["C"])
    assert np.array_equal(o.bits_of(o.ref_gemm(A, B)), z["C_torch"])
    assert o.ulp_distance(z["C"], z["C_torch"]).max() <= 1


def test_golden_fixtures_exist():
    assert len(glob.glob(os.path.join(HERE, "golden", "*.npz"))) >= 5


# ------------------------------------------------------------------------------------------------
# alpha/beta restatement (neogemm_bf16_scaled): pinned by exact integer cases and by its special cases
# ------------------------------------------------------------------------------------------------
def test_scaled_reduces_to_plain_gemm():
    A, B = o.make_inputs(37, 29, 53, seed=4)
    C0 = torch.full((37, 29), float("nan"), dtype=torch.bfloat16)   # beta == 0: never looked at
    assert np.array_equal(o.bits_of(o.ref_gemm_scaled(A, B, C0, 1.0, 0.0)), o.bits_of(o.ref_gemm(A, B)))


def test_scaled_exact_small_integers():
    g = torch.Generator().manual_seed(9)
    M, N, K = 12, 10, 7
    Ai = torch.randint(-3, 4, (M, K), generator=g)
    Bi = torch.randint(-3, 4, (K, N), generator=g)
    Ci = torch.randint(-8, 9, (M, N), generator=g)
    for alpha, beta in ((2.0, -3.0), (-1.0, 1.0), (0.0, 2.0), (4.0, 0.0), (0.5, 0.5)):
        want = [[alpha * sum(int(Ai[i, k]) * int(Bi[k, j]) for k in range(K)) + beta * int(Ci[i, j])
                 for j in range(N)] for i in range(M)]          # Python arithmetic: exact, |values| < 256
        got = o.ref_gemm_scaled(Ai.to(torch.bfloat16), Bi.to(torch.bfloat16), Ci.to(torch.bfloat16), alpha, beta)
        assert got.double().tolist() == want, (alpha, beta)


def test_scaled_power_of_two_alpha_is_exact_scaling():
    A, B = o.make_inputs(33, 40, 64, seed=6)
    C0 = torch.zeros(33, 40, dtype=torch.bfloat16)
    half = o.ref_gemm_scaled(A, B, C0, 0.5, 0.0)
    assert np.array_equal(o.bits_of(half), o.bits_of((o.ref_gemm_f32(A, B) * 0.5).to(torch.bfloat16)))
    assert torch.equal(half.float() * 2, o.ref_gemm(A, B).float())   # no subnormals here: exact


def test_scaled_against_fp64_formula():
    A, B = o.make_inputs(31, 27, 96, seed=8)
    C0 = (torch.randn(31, 27, generator=torch.Generator().manual_seed(1))).to(torch.bfloat16)
    alpha, beta = 1.75, -0.625
    want = alpha * o.exact_gemm_f64(A, B) + beta * C0.double()
    got = o.ref_gemm_scaled(A, B, C0, alpha, beta).double()
    half_ulp = torch.exp2(torch.floor(torch.log2(want.abs().clamp_min(1e-30))) - 8)
    slack = 8 * 2.0 ** -24 * (abs(alpha) * o.abs_gemm_f64(A, B) + abs(beta) * C0.double().abs())
    assert bool(((got - want).abs() <= half_ulp * 1.0000001 + slack).all())
    # a dropped beta term, a swapped sign or alpha applied to C as well must all fail this check
    for wrong in (alpha * o.exact_gemm_f64(A, B), alpha * o.exact_gemm_f64(A, B) - beta * C0.double(),
                  alpha * (o.exact_gemm_f64(A, B) + beta * C0.double())):
        assert not bool(((got - wrong).abs() <= half_ulp * 1.0000001 + slack).all())


def test_two_legal_fp32_orders_differ_by_more_than_one_raw_ulp():
    """Why the per-element criterion is measured at max(|ref|, 2^-7 rms) and not in raw ulps: two correct
    fp32-accumulating products of the same bf16 inputs, taken in different orders — torch's blocked CPU matmul
    (ref_gemm) and the plain-C sequential-k sum (c_gemm) — already disagree by more than 1 raw bf16 ulp on elements
    that cancel to nearly zero at K = 8192, while each passes assert_parity against the other as reference."""
    A, B = o.make_inputs(64, 64, 8192, seed=123)
    r_torch, r_c = o.ref_gemm(A, B), o.c_gemm(A, B)
    ulp = o.ulp_distance(o.bits_of(r_torch), o.bits_of(r_c))
    assert ulp.max() > 1, "expected the two summation orders to differ by more than one raw ulp somewhere"
    # the disagreement sits on elements far below the typical magnitude, nowhere else
    rms = float(r_torch.float().pow(2).mean().sqrt())
    big = np.abs(r_torch.float().numpy()) >= rms * 2.0 ** -5
    assert ulp[big].max() <= 1
    assert np.abs(r_torch.float().numpy())[ulp > 1].max() < rms * 2.0 ** -5
    o.assert_parity(r_c, A, B, ref=r_torch, what="sequential-k vs blocked")
    o.assert_parity(r_torch, A, B, ref=r_c, what="blocked vs sequential-k")
