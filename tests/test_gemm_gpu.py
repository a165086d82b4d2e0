"""GPU parity tests: the HIP path, called through the C ABI (gemm_amd -> ctypes -> libneogemm.so) and
through the built neoGEMM module, against the CPU oracle on the same seeded inputs.

Tolerance (stated by the task): <= 1 bf16 ulp per element and <= 1e-3 relative Frobenius error against
the fp32-accumulated CPU product rounded to bf16 — see oracle.gemm_oracle.assert_parity for how elements
that cancel to nearly zero are treated.  Known-answer cases (identity, one-hot, ones, small integers) do
not depend on summation order and are compared bit for bit.

The reference can only run M, N, K that are multiples of 64 (nemgemmV03.cu:375) and has no tests; ragged,
skinny and unaligned shapes are this build's own ground and are pinned by the oracle alone.
"""
import math

import numpy as np
import pytest
import torch

import gemm_amd as g
from gemm_amd import _abi
from oracle import gemm_oracle as o

pytestmark = pytest.mark.gpu

TILE_VARIANTS = [g.VARIANT_T256x256_W4, g.VARIANT_T128x128_W4, g.VARIANT_T256x128_W4,
                 g.VARIANT_T128x256_W4, g.VARIANT_T64x128_W4, g.VARIANT_T192x256_W4,
                 g.VARIANT_T96x128_W4, g.VARIANT_T64x64_W4]
ALL_VARIANTS = [g.VARIANT_GENERIC] + TILE_VARIANTS


TILE_SHAPE = {g.VARIANT_T256x256_W4: (256, 256), g.VARIANT_T128x128_W4: (128, 128),
              g.VARIANT_T256x128_W4: (256, 128), g.VARIANT_T128x256_W4: (128, 256), g.VARIANT_T64x128_W4: (64, 128),
              g.VARIANT_T192x256_W4: (192, 256), g.VARIANT_T96x128_W4: (96, 128),
              g.VARIANT_T64x64_W4: (64, 64)}


def supported(variant, b_layout, c_layout):
    """Whether a forced tile variant takes this pair of layouts.  The kernels write row-major output, so a
    column-major C exchanges the operands' roles; the side of the tile that an MN-major operand (B [K,N]) lands on
    must be a power of two of at least 128 rows.  Everything else is refused with ERR_UNSUPPORTED, never mis-run."""
    if variant is None or variant not in TILE_SHAPE:
        return True
    bm, bn = TILE_SHAPE[variant]
    ok = lambda rows: rows >= 128 and rows & (rows - 1) == 0
    if b_layout == g.B_NK:
        return True
    return ok(bn) if c_layout == g.C_ROW else ok(bm)


def cells(variants, b_layouts=(g.B_KN, g.B_NK), c_layouts=(g.C_ROW, g.C_COL)):
    return [(v, b, c) for v in variants for b in b_layouts for c in c_layouts if supported(v, b, c)]


def run_abi(A, B, dev, b_layout=g.B_KN, c_layout=g.C_ROW, variant=None, split_k=0, group_m=0, strict=True):
    """A [M,K] and B ([K,N] or [N,K]) are CPU bf16 tensors; returns the [M,N] result on the CPU."""
    M, K = A.shape
    N = B.shape[1] if b_layout == g.B_KN else B.shape[0]
    Ad, Bd = A.to(dev), B.to(dev)
    shape = (M, N) if c_layout == g.C_ROW else (N, M)
    C = torch.full(shape, float("nan"), dtype=torch.bfloat16, device=dev)   # poison: every element must be written
    try:
        g.gemm_into(Ad, Bd, C, M, N, K, max(K, 1), max(N if b_layout == g.B_KN else K, 1),
                    max(N if c_layout == g.C_ROW else M, 1), b_layout, c_layout, variant, split_k, group_m)
    except g.NeoGemmError:
        raise   # the parametrizations below only name (variant, layout) cells the library documents as supported
    torch.cuda.synchronize()
    C = C.cpu()
    return C if c_layout == g.C_ROW else C.t().contiguous()


def layouts(Bkn, b_layout):
    return Bkn if b_layout == g.B_KN else Bkn.t().contiguous()


# the 64x64 tile takes K-major operands only (B [N,K]); tests that force a variant on one layout use this one for it
NK_ONLY = (g.VARIANT_T64x64_W4,)


def home_layout(variant):
    return g.B_NK if variant in NK_ONLY else g.B_KN


# ------------------------------------------------------------------------------------------------
# known answers: bit-exact, every variant, every layout
# ------------------------------------------------------------------------------------------------
def test_unsupported_cells_are_refused(dev):
    A = torch.zeros(256, 256, dtype=torch.bfloat16, device=dev)
    refused = 0
    for v in TILE_VARIANTS:
        for b in (g.B_KN, g.B_NK):
            for c in (g.C_ROW, g.C_COL):
                if not supported(v, b, c):
                    st = _abi.gemm_raw(A.data_ptr(), A.data_ptr(), A.data_ptr(), 256, 256, 256, 256, 256, 256, b, c, 0, 0, 0, v, 1, 0)
                    assert st == _abi.ERR_UNSUPPORTED, (v, b, c, st)
                    refused += 1
    torch.cuda.synchronize()
    assert refused == 5   # 64x128, 192x256, 96x128 with B [K,N] and column-major C; 64x64 with B [K,N] either way


@pytest.mark.parametrize("variant,b_layout,c_layout", cells(ALL_VARIANTS))
def test_identity_and_permutation(dev, variant, b_layout, c_layout):
    n = 384
    A, _ = o.make_inputs(n, n, n, seed=1)
    I = torch.eye(n, dtype=torch.bfloat16)
    assert torch.equal(run_abi(A, layouts(I, b_layout), dev, b_layout, c_layout, variant), A)
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(2))
    P = torch.zeros(n, n, dtype=torch.bfloat16)
    P[torch.arange(n), perm] = 1
    assert torch.equal(run_abi(P, layouts(A, b_layout), dev, b_layout, c_layout, variant), A[perm])


@pytest.mark.parametrize("variant", ALL_VARIANTS)
def test_exact_small_integers(dev, variant):
    rng = np.random.default_rng(11)
    M, N, K = 264, 328, 200   # ragged in M and N, partial last K slab
    A = torch.from_numpy(rng.integers(-8, 9, size=(M, K)).astype(np.float32)).to(torch.bfloat16)
    B = torch.from_numpy(rng.integers(-8, 9, size=(K, N)).astype(np.float32)).to(torch.bfloat16)
    want = (A.to(torch.int64) @ B.to(torch.int64)).float().to(torch.bfloat16)   # |sum| < 2^24: fp32 exact
    for b_layout in (g.B_KN, g.B_NK):
        if b_layout == g.B_KN and variant in NK_ONLY:
            continue
        got = run_abi(A, layouts(B, b_layout), dev, b_layout, g.C_ROW, variant)
        assert torch.equal(got, want)
    if variant != g.VARIANT_GENERIC:
        bl = home_layout(variant)
        for split in (2, 3, 7):
            assert torch.equal(run_abi(A, layouts(B, bl), dev, bl, variant=variant, split_k=split), want)


@pytest.mark.parametrize("K", [8, 256, 264, 1000, 4096])
def test_ones(dev, K):
    A = torch.ones(40, K, dtype=torch.bfloat16)
    B = torch.ones(K, 264, dtype=torch.bfloat16)
    want = torch.tensor(float(K)).to(torch.bfloat16)   # 264 -> 264, 1000 -> 1000, exact sums then RNE
    for variant in (None, g.VARIANT_T128x128_W4, g.VARIANT_T256x256_W4):
        assert torch.all(run_abi(A, B, dev, variant=variant) == want)


def test_rounding_is_nearest_even(dev):
    # sums 257 and 259 sit exactly between two bf16 values: ties go to even (256, 260)
    A = torch.ones(16, 264, dtype=torch.bfloat16)
    for total, want in ((257, 256.0), (259, 260.0), (258, 258.0)):
        B = torch.zeros(264, 16, dtype=torch.bfloat16)
        B[:total] = 1
        C = run_abi(A, B, dev)
        assert torch.all(C.float() == want), (total, C[0, 0])


# ------------------------------------------------------------------------------------------------
# golden fixtures
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["tile64", "ragged", "odd", "skinny16", "tallk"])
def test_golden(dev, name):
    import os
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", f"{name}.npz"), allow_pickle=False)
    A, B = o.from_bits(z["A"]), o.from_bits(z["B"])
    want = o.from_bits(z["C_torch"])
    for b_layout in (g.B_KN, g.B_NK):
        for c_layout in (g.C_ROW, g.C_COL):
            got = run_abi(A, layouts(B, b_layout), dev, b_layout, c_layout)
            o.assert_parity(got, A, B, ref=want, what=f"{name} b{b_layout} c{c_layout}")


# ------------------------------------------------------------------------------------------------
# seeded random parity at the benchmark configurations
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("variant,b_layout,c_layout", cells([None] + ALL_VARIANTS))
def test_parity_512(dev, variant, b_layout, c_layout):
    A, Bkn = o.make_inputs(512, 512, 512, seed=0)
    got = run_abi(A, layouts(Bkn, b_layout), dev, b_layout, c_layout, variant)
    o.assert_parity(got, A, Bkn, what=f"512^3 v{variant} b{b_layout} c{c_layout}")


def check_big(dev, M, N, K, seed, b_layout=g.B_KN, variant=None, split_k=0, nrows=256, c_layout=g.C_ROW):
    """Full-size run.  Over the whole matrix, against the full fp32 CPU product: raw ulp, Frobenius error and the ulp
    measured at max(|ref|, 2^-7 rms) (see oracle.parity_report); the fp64-based bound, which needs a second full
    product in fp64, on a sample of rows (all rows when the problem is small)."""
    A, Bkn = o.make_inputs(M, N, K, seed=seed)
    got = run_abi(A, layouts(Bkn, b_layout), dev, b_layout, c_layout, variant, split_k)
    ref = o.ref_gemm(A, Bkn)
    ulp = o.ulp_distance(o.bits_of(got), o.bits_of(ref))
    assert bool(torch.isfinite(got.float()).all())
    assert (ulp > 1).mean() <= 2e-3, f"{(ulp > 1).mean():.2e} of elements more than 1 raw ulp off"
    rf = ref.float()
    rel = float(torch.linalg.norm(got.float() - rf) / torch.linalg.norm(rf))
    assert rel <= o.TOL_REL_FRO, rel
    floor = max(float(torch.sqrt(torch.mean(rf.double() ** 2))) * 2.0 ** -7, 1e-38)
    ulp_size = torch.exp2(torch.floor(torch.log2(torch.clamp(rf.abs(), min=floor))) - 7)
    floored = float(((got.float() - rf).abs() / ulp_size).max())
    assert floored <= o.TOL_ULP, f"{floored} ulp (floored) over the whole {M}x{N} matrix"
    idx = torch.arange(M) if M <= nrows else torch.cat([
        torch.tensor([0, M - 1]), torch.randperm(M, generator=torch.Generator().manual_seed(seed))[:nrows - 2]])
    return o.assert_parity(got[idx], A[idx], Bkn, ref=ref[idx], what=f"{M}x{N}x{K}")


@pytest.mark.parametrize("b_layout,c_layout", [(g.B_KN, g.C_ROW), (g.B_NK, g.C_ROW), (g.B_NK, g.C_COL)])
def test_parity_4096(dev, b_layout, c_layout):
    check_big(dev, 4096, 4096, 4096, seed=1, b_layout=b_layout, c_layout=c_layout)


def test_parity_8192_headline(dev):
    check_big(dev, 8192, 8192, 8192, seed=2)


def test_parity_8192_reference_call(dev):
    """The reference's own call at the headline size: B [N,K], column-major C (benchmark.py:10-25, nemgemmV03.cu:343-391):
    the chained kernel on exchanged operands, four rounds of workgroups; through the C ABI and through neoGEMM.neoGemmV1."""
    M = N = K = 8192
    assert g.plan(M, N, K, g.B_NK, g.C_COL) == (g.VARIANT_C256x256_W4, 1)
    check_big(dev, M, N, K, seed=3, b_layout=g.B_NK, c_layout=g.C_COL)
    import neoGEMM
    A, Bkn = o.make_inputs(M, N, K, seed=3)
    Ad, Bd = A.to(dev), Bkn.t().contiguous().to(dev)
    Cbuf = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    neoGEMM.neoGemmV1(Ad, Bd, Cbuf)                       # C storage receives the column-major product
    torch.cuda.synchronize()
    via_module = Cbuf.t().cpu()                            # benchmark.py:25
    via_abi = run_abi(A, Bkn.t().contiguous(), dev, g.B_NK, g.C_COL)
    assert torch.equal(via_module, via_abi)                # the same kernel on the same data, bit for bit


@pytest.mark.parametrize("M", [16, 64, 72, 100, 128])
@pytest.mark.parametrize("b_layout", [g.B_KN, g.B_NK])
def test_parity_skinny(dev, M, b_layout):
    check_big(dev, M, 14336, 4096, seed=3 + M, b_layout=b_layout)


@pytest.mark.parametrize("b_layout", [g.B_KN, g.B_NK])
def test_parity_irregular(dev, b_layout):
    check_big(dev, 3000, 5120, 3584, seed=5, b_layout=b_layout)


def test_parity_tall_k(dev):
    r = check_big(dev, 1024, 1024, 32768, seed=6)
    assert g.plan(1024, 1024, 32768)[1] > 1   # this shape runs split-K


@pytest.mark.parametrize("variant", TILE_VARIANTS)
@pytest.mark.parametrize("split", [2, 5, 16])
def test_split_k(dev, variant, split):
    M, N, K = 200, 392, 2056
    A, Bkn = o.make_inputs(M, N, K, seed=8)
    bl = home_layout(variant)
    got = run_abi(A, layouts(Bkn, bl), dev, bl, variant=variant, split_k=split)
    o.assert_parity(got, A, Bkn, what=f"split {split} v{variant}")


# ------------------------------------------------------------------------------------------------
# edges the reference never ran (it needs multiples of 64)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (1, 17, 5), (3, 1, 64), (7, 9, 8), (64, 64, 8), (65, 129, 72),
                                   (255, 257, 24), (300, 520, 200), (16, 8, 4096), (129, 40, 520), (40, 1000, 31)])
@pytest.mark.parametrize("b_layout", [g.B_KN, g.B_NK])
@pytest.mark.parametrize("c_layout", [g.C_ROW, g.C_COL])
def test_ragged_shapes(dev, M, N, K, b_layout, c_layout):
    A, Bkn = o.make_inputs(M, N, K, seed=M + 3 * N + 7 * K)
    got = run_abi(A, layouts(Bkn, b_layout), dev, b_layout, c_layout)
    o.assert_parity(got, A, Bkn, what=f"{M}x{N}x{K} b{b_layout} c{c_layout}")


@pytest.mark.parametrize("variant", TILE_VARIANTS)
@pytest.mark.parametrize("M,N,K", [(8, 8, 32), (264, 136, 40), (513, 520, 1032), (250, 1000, 72)])
def test_ragged_shapes_forced_tile_kernels(dev, variant, M, N, K):
    A, Bkn = o.make_inputs(M, N, K, seed=5 * M + N)
    for b_layout in (g.B_KN, g.B_NK):
        B = layouts(Bkn, b_layout)
        try:
            got = run_abi(A, B, dev, b_layout, g.C_ROW, variant, strict=True)
        except g.NeoGemmError as e:
            # an MN-major operand on a tile below 128 rows, or N % 8 != 0, is refused, never mis-run
            assert e.status == _abi.ERR_UNSUPPORTED and b_layout == g.B_KN
            continue
        o.assert_parity(got, A, Bkn, what=f"{M}x{N}x{K} v{variant} b{b_layout}")


# The tile kernels stage K in 64-deep tiles / 32-deep slabs with a prologue, a steady loop that is entered
# from seven K tiles on and unrolls two periods, and a tail: every K below walks a different way through
# them (tile counts 1..13, with and without a partial last tile), once per operand combination.
@pytest.mark.parametrize("variant", [g.VARIANT_T256x256_W4, g.VARIANT_T128x128_W4, g.VARIANT_T96x128_W4,
                                     g.VARIANT_T64x64_W4])
@pytest.mark.parametrize("b_layout,c_layout", [(g.B_KN, g.C_ROW), (g.B_NK, g.C_ROW), (g.B_KN, g.C_COL)])
def test_k_loop_transitions(dev, variant, b_layout, c_layout):
    if not supported(variant, b_layout, c_layout):
        b_layout = g.B_NK   # the same walk through the K loop on the layouts this tile takes
    M, N = 264, 392   # two tile rows/columns of the largest tile, ragged, both multiples of 8
    for K in (64, 72, 120, 128, 136, 192, 200, 256, 320, 384, 440, 448, 456, 512, 576, 640, 704, 768, 776, 832):
        A, Bkn = o.make_inputs(M, N, K, seed=K)
        got = run_abi(A, layouts(Bkn, b_layout), dev, b_layout, c_layout, variant)
        o.assert_parity(got, A, Bkn, what=f"{M}x{N}x{K} v{variant} b{b_layout} c{c_layout}")


def test_k_zero_writes_zeros(dev):
    A = torch.zeros(5, 0, dtype=torch.bfloat16, device=dev)
    B = torch.zeros(0, 9, dtype=torch.bfloat16, device=dev)
    C = g.gemm(A, B)
    assert C.shape == (5, 9) and torch.all(C == 0)


def test_empty_outputs(dev):
    A = torch.zeros(0, 8, dtype=torch.bfloat16, device=dev)
    B = torch.zeros(8, 4, dtype=torch.bfloat16, device=dev)
    assert g.gemm(A, B).shape == (0, 4)
    A2 = torch.zeros(4, 8, dtype=torch.bfloat16, device=dev)
    assert g.gemm(A2, B[:, :0]).shape == (4, 0)


def test_strided_and_unaligned_operands(dev):
    M, N, K = 96, 160, 256
    A, Bkn = o.make_inputs(M, N, K, seed=31)
    ref = o.ref_gemm(A, Bkn)
    # leading dimensions larger than the row length (views into wider buffers): MFMA path
    Aw = torch.zeros(M, K + 64, dtype=torch.bfloat16, device=dev)
    Aw[:, :K] = A.to(dev)
    Bw = torch.zeros(K, N + 32, dtype=torch.bfloat16, device=dev)
    Bw[:, :N] = Bkn.to(dev)
    o.assert_parity(g.gemm(Aw[:, :K], Bw[:, :N]), A, Bkn, ref=ref, what="wide ld")
    # base pointers off 16-byte alignment: generic path
    flatA = torch.zeros(M * K + 8, dtype=torch.bfloat16, device=dev)
    Au = flatA[3:3 + M * K].view(M, K)
    Au.copy_(A.to(dev))
    o.assert_parity(g.gemm(Au, Bkn.to(dev)), A, Bkn, ref=ref, what="unaligned A")
    # B given as the transposed view of an [N,K] tensor: taken as the reference's layout, no copy
    Bnk = Bkn.t().contiguous().to(dev)
    o.assert_parity(g.gemm(A.to(dev), Bnk.t()), A, Bkn, ref=ref, what="B = W.t()")
    # a column-sliced (non-contiguous rows) A is made contiguous by the wrapper
    o.assert_parity(g.gemm(Aw.t()[:K].t(), Bkn.to(dev)), A, Bkn, ref=ref, what="A view")


# ------------------------------------------------------------------------------------------------
# the reference's own call, as benchmark.py makes it
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("modname", ["gemm_amd", "neoGEMM"])
def test_reference_call_contract(dev, modname):
    """benchmark.py:10-25 with seeded inputs: C = zeros(M,N); neoGemmV1(A, B, C); C.t() == A @ B.t()."""
    mod = __import__(modname)
    M = N = K = 1024                                       # benchmark.py:6-8
    A, Bnk = o.make_inputs(M, N, K, seed=77, b_layout="nk")
    Ad, Bd = A.to(dev), Bnk.to(dev)
    C = torch.zeros(M, N, device=dev).to(torch.bfloat16)   # benchmark.py:12
    assert mod.neoGemmV1(A=Ad, B=Bd, C=C) is None          # keyword names of the binding, returns None
    torch.cuda.synchronize()
    o.assert_parity(C.t(), A, Bnk, b_layout="nk", what=f"{modname}.neoGemmV1")
    C2 = torch.zeros(M, N, device=dev).to(torch.bfloat16)
    mod.neogemm(Ad, Bd, C2)                                # the older module's name (v01.cu:314-317)
    torch.cuda.synchronize()
    assert torch.equal(C2, C)
    # non-square: the buffer is the column-major product, i.e. an [N,M] row-major matrix
    M2, N2 = 320, 192
    A2, B2 = o.make_inputs(M2, N2, K, seed=78, b_layout="nk")
    C3 = torch.zeros(M2 * N2, device=dev).to(torch.bfloat16).view(M2, N2)
    mod.neoGemmV1(A2.to(dev), B2.to(dev), C3)
    torch.cuda.synchronize()
    o.assert_parity(C3.view(N2, M2).t(), A2, B2, b_layout="nk", what=f"{modname}.neoGemmV1 non-square")


@pytest.mark.parametrize("M,N,K", [(1024, 6144, 8192), (4096, 1536, 8192), (1024, 1024, 32768), (3072, 1024, 16384)])
def test_reference_call_on_split_k_shapes(dev, M, N, K):
    """neoGemmV1's layout (B [N,K], column-major C: nemgemmV03.cu:343-391) on shapes whose plan for that layout
    splits K, or did at some stage of the cost model (the first two: the cells where the workspace query once fell
    short): both wrappers size the workspace with neogemm_bf16_workspace_bytes and the call must go through; the raw
    C-ABI call with a workspace of exactly the queried size likewise."""
    import neoGEMM
    if (M, N, K) in ((1024, 1024, 32768), (3072, 1024, 16384)):
        assert g.plan(M, N, K, g.B_NK, g.C_COL)[1] > 1
    A, Bnk = o.make_inputs(M, N, K, seed=M + N, b_layout="nk")
    Ad, Bd = A.to(dev), Bnk.to(dev)
    ref = o.ref_gemm(A, Bnk, b_layout="nk")
    rows = torch.randperm(M, generator=torch.Generator().manual_seed(5))[:192]
    results = []
    for mod in (g, neoGEMM):
        C = torch.full((M * N,), float("nan"), dtype=torch.bfloat16, device=dev).view(M, N)
        mod.neoGemmV1(Ad, Bd, C)
        torch.cuda.synchronize()
        got = C.view(N, M).t().cpu()
        o.assert_parity(got[rows], A[rows], Bnk, b_layout="nk", ref=ref[rows], what=f"{mod.__name__}.neoGemmV1 {M}x{N}x{K}")
        results.append(got)
    assert torch.equal(results[0], results[1])
    need = g.workspace_bytes(M, N, K)
    v, split = g.plan(M, N, K, g.B_NK, g.C_COL)
    assert need >= (split * M * N * 4 if split > 1 else 0)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
    C = torch.full((N, M), float("nan"), dtype=torch.bfloat16, device=dev)
    st = _abi.gemm_raw(Ad.data_ptr(), Bd.data_ptr(), C.data_ptr(), M, N, K, K, K, M, g.B_NK, g.C_COL, ws.data_ptr() if need else 0,
                       need, torch.cuda.current_stream().cuda_stream)
    assert st == _abi.OK, _abi.strerror(st)
    torch.cuda.synchronize()
    assert torch.equal(C.t().cpu(), results[0])


def test_split_k_on_two_streams(dev):
    """Two split-K GEMMs with different inputs queued on two streams with no host synchronisation in between, several
    times over: each stream has its own partials, so neither result is disturbed (the reference runs everything on
    the one default stream, nemgemmV03.cu:383)."""
    import neoGEMM
    M, N, K = 512, 512, 16384
    assert g.plan(M, N, K)[1] > 1 and g.workspace_bytes(M, N, K) > 0
    A1, B1 = o.make_inputs(M, N, K, seed=31)
    A2, B2 = o.make_inputs(M, N, K, seed=32)
    want1, want2 = o.ref_gemm(A1, B1), o.ref_gemm(A2, B2)
    d = [t.to(dev) for t in (A1, B1, A2, B2)]
    torch.cuda.synchronize()
    for mod in (g, neoGEMM):
        s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
        outs1, outs2 = [], []
        for it in range(6):
            with torch.cuda.stream(s1):
                outs1.append(mod.gemm(d[0], d[1]))
            with torch.cuda.stream(s2):
                outs2.append(mod.gemm(d[2], d[3]))
        s1.synchronize()
        s2.synchronize()
        for c in outs1:
            assert torch.equal(c, outs1[0])
        for c in outs2:
            assert torch.equal(c, outs2[0])
        o.assert_parity(outs1[0], A1, B1, ref=want1, what=f"{mod.__name__} stream 1")
        o.assert_parity(outs2[0], A2, B2, ref=want2, what=f"{mod.__name__} stream 2")
    # growing the buffer of a stream that still has work queued on it
    with torch.cuda.stream(s1):
        small = g.gemm(d[0], d[1])
        Abig, Bbig = o.make_inputs(1024, 1024, 32768, seed=33)
        big = g.gemm(Abig.to(dev, non_blocking=False), Bbig.to(dev))
    s1.synchronize()
    assert torch.equal(small, outs1[0])
    o.assert_parity(big[:128], Abig[:128], Bbig, what="grown workspace")


def test_module_gemm_matches_abi(dev):
    import neoGEMM
    for M, N, K in ((512, 512, 512), (200, 328, 136), (16, 14336, 4096)):
        A, B = o.make_inputs(M, N, K, seed=M)
        Ad, Bd = A.to(dev), B.to(dev)
        C1, C2 = neoGEMM.gemm(Ad, Bd), g.gemm(Ad, Bd)
        torch.cuda.synchronize()
        assert C1.dtype == torch.bfloat16 and C1.shape == (M, N) and C1.is_contiguous()
        assert torch.equal(C1, C2)
        o.assert_parity(C1, A, B, what=f"neoGEMM.gemm {M}x{N}x{K}")
    with pytest.raises(RuntimeError, match="inner dimensions"):
        neoGEMM.gemm(Ad, Ad)
    with pytest.raises(RuntimeError, match="bfloat16"):
        neoGEMM.gemm(Ad.float(), Bd.float())
    with pytest.raises(RuntimeError, match="M\\*N"):
        neoGEMM.neoGemmV1(Ad, Ad, torch.zeros(3, 3, dtype=torch.bfloat16, device=dev))


# ------------------------------------------------------------------------------------------------
# size-independent properties at full size
# ------------------------------------------------------------------------------------------------
def test_properties_full_size(dev):
    M = N = K = 4096
    A, B = o.make_inputs(M, N, K, seed=9)
    Ad, Bd = A.to(dev), B.to(dev)
    C = g.gemm(Ad, Bd)
    # deterministic: the same call gives the same bits
    assert torch.equal(C, g.gemm(Ad, Bd))
    # scaling by a power of two is exact in every partial sum
    assert torch.equal(g.gemm((Ad.float() * 4).bfloat16(), Bd), (C.float() * 4).bfloat16())
    assert torch.equal(g.gemm(Ad, (Bd.float() * 0.5).bfloat16()), (C.float() * 0.5).bfloat16())
    # (negating an operand is NOT asserted to negate the result bit for bit: the matrix cores' internal
    # adder is not sign-symmetric in its last bit, so -A gives results 1 ulp apart on a few elements)
    o.assert_parity(g.gemm(-Ad, Bd)[:64], -A[:64], B, what="negated A")
    # permuting rows of A permutes rows of C; permuting columns of B permutes columns of C (the
    # k-order of every dot product does not depend on where its output lies)
    perm = torch.randperm(M, generator=torch.Generator().manual_seed(1)).to(dev)
    assert torch.equal(g.gemm(Ad[perm], Bd), C[perm])
    assert torch.equal(g.gemm(Ad, Bd[:, perm].contiguous()), C[:, perm])
    # transposition identity: (A B)^T = B^T A^T, computed through the other layout flags
    Ct = torch.empty(N, M, dtype=torch.bfloat16, device=dev)
    g.gemm_into(Ad, Bd, Ct, M, N, K, K, N, M, g.B_KN, g.C_COL)
    assert torch.equal(Ct.t(), C)
    # checksum of checksums: sum over rows of C equals (1^T A) B up to the rounding of C itself
    ones_A = Ad.float().sum(0)                       # [K]
    lhs = C.float().sum(0).double()
    rhs = (ones_A.double() @ Bd.double())
    tol = 4.0 * math.sqrt(M) * 2.0 ** -9 * float(C.float().abs().mean()) * 4
    assert float((lhs - rhs).abs().max()) <= tol * math.sqrt(M)


# The chained 256x256 kernel (two MFMA steps per accumulator tile back to back, A's fragments resident, B's streamed)
# takes K in whole periods of 128, no split-K, and its rows from a K-major operand; on those problems it must give
# what the slab kernel gives, bit for bit (same sums in the same order).
CHAIN_CELLS = [(g.B_KN, g.C_ROW), (g.B_NK, g.C_ROW), (g.B_NK, g.C_COL)]


@pytest.mark.parametrize("b_layout,c_layout", CHAIN_CELLS)
def test_chain_kernel_known_answers(dev, b_layout, c_layout):
    v = g.VARIANT_C256x256_W4
    n = 384
    A, _ = o.make_inputs(n, n, n, seed=1)
    I = torch.eye(n, dtype=torch.bfloat16)
    assert torch.equal(run_abi(A, layouts(I, b_layout), dev, b_layout, c_layout, v), A)
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(2))
    P = torch.zeros(n, n, dtype=torch.bfloat16)
    P[torch.arange(n), perm] = 1
    assert torch.equal(run_abi(P, layouts(A, b_layout), dev, b_layout, c_layout, v), A[perm])
    rng = np.random.default_rng(11)
    M, N, K = 264, 328, 256   # ragged in M and N
    Ai = torch.from_numpy(rng.integers(-8, 9, size=(M, K)).astype(np.float32)).to(torch.bfloat16)
    Bi = torch.from_numpy(rng.integers(-8, 9, size=(K, N)).astype(np.float32)).to(torch.bfloat16)
    want = (Ai.to(torch.int64) @ Bi.to(torch.int64)).float().to(torch.bfloat16)
    for gm in (0, 1, 3):
        assert torch.equal(run_abi(Ai, layouts(Bi, b_layout), dev, b_layout, c_layout, v, group_m=gm), want)
    ones = torch.ones(40, 1024, dtype=torch.bfloat16)
    assert torch.all(run_abi(ones, layouts(torch.ones(1024, 264, dtype=torch.bfloat16), b_layout), dev, b_layout, c_layout, v) == 1024)


@pytest.mark.parametrize("b_layout,c_layout", CHAIN_CELLS)
def test_chain_kernel_k_loop_and_edges(dev, b_layout, c_layout):
    """Period counts 1..9 and 16 (the loop body holds two periods; the prologue holds two tiles), ragged M and N (row
    and column masks, two tile rows and columns), against the oracle and against the slab kernel bit for bit."""
    for M, N in ((264, 392), (8, 16), (520, 528)):
        for K in (128, 256, 384, 512, 640, 768, 896, 1024, 1152, 2048):
            A, Bkn = o.make_inputs(M, N, K, seed=M + K)
            B = layouts(Bkn, b_layout)
            got = run_abi(A, B, dev, b_layout, c_layout, g.VARIANT_C256x256_W4)
            o.assert_parity(got, A, Bkn, what=f"chain {M}x{N}x{K} b{b_layout} c{c_layout}")
            assert torch.equal(got, run_abi(A, B, dev, b_layout, c_layout, g.VARIANT_T256x256_W4)), (M, N, K)


def test_chain_kernel_matches_slab_kernel_on_random_shapes(dev):
    """Seeded random shapes (multiples of 8, up to 1100 x 1100, K up to 20 periods), every supported layout pair: the two
    256x256 kernels compute the same sums in the same order and must agree bit for bit, whatever the edges look like."""
    rng = np.random.default_rng(2024)
    for _ in range(36):
        M, N = (int(rng.integers(1, 138)) * 8 for _ in range(2))
        K = int(rng.integers(1, 21)) * 128
        b_layout, c_layout = CHAIN_CELLS[int(rng.integers(0, len(CHAIN_CELLS)))]
        A, Bkn = o.make_inputs(M, N, K, seed=M * 3 + N * 5 + K)
        B = layouts(Bkn, b_layout)
        got = run_abi(A, B, dev, b_layout, c_layout, g.VARIANT_C256x256_W4)
        assert torch.equal(got, run_abi(A, B, dev, b_layout, c_layout, g.VARIANT_T256x256_W4)), (M, N, K, b_layout, c_layout)
    # one case is checked against the oracle in full as well
    o.assert_parity(got, A, Bkn, what=f"chain {M}x{N}x{K}")


def test_chain_kernel_refuses_what_it_cannot_run(dev):
    A = torch.zeros(256, 512, dtype=torch.bfloat16, device=dev)
    v = g.VARIANT_C256x256_W4
    ws = torch.empty(4 * 256 * 256 * 4, dtype=torch.uint8, device=dev)
    call = lambda K, b, c, split: _abi.gemm_raw(A.data_ptr(), A.data_ptr(), A.data_ptr(), 256, 256, K, 512, 512, 256, b, c,
                                                ws.data_ptr(), ws.numel(), 0, v, split, 0)
    assert call(256, g.B_NK, g.C_ROW, 1) == _abi.OK
    assert call(192, g.B_NK, g.C_ROW, 1) == _abi.ERR_UNSUPPORTED     # K not in whole periods of 128
    assert call(256, g.B_NK, g.C_ROW, 2) == _abi.ERR_UNSUPPORTED     # no split-K
    assert call(256, g.B_KN, g.C_COL, 1) == _abi.ERR_UNSUPPORTED     # rows from an MN-major operand
    torch.cuda.synchronize()
    # the plan never sends such a problem there
    assert g.plan(4096, 4096, 4096 + 64)[0] != v and g.plan(4096, 4096, 4096, g.B_KN, g.C_COL)[0] != v
    assert g.plan(4096, 4096, 4096) == (v, 1) and g.plan(8192, 8192, 8192, g.B_NK, g.C_COL) == (v, 1)


def test_variants_agree_bitwise_on_exact_data(dev):
    rng = np.random.default_rng(5)
    M, N, K = 512, 768, 384
    A = torch.from_numpy(rng.integers(-4, 5, size=(M, K)).astype(np.float32)).to(torch.bfloat16)
    B = torch.from_numpy(rng.integers(-4, 5, size=(K, N)).astype(np.float32)).to(torch.bfloat16)
    base = run_abi(A, B, dev, variant=g.VARIANT_GENERIC)
    for v in TILE_VARIANTS:
        bl = home_layout(v)
        for gm in (1, 3, 8):
            assert torch.equal(run_abi(A, layouts(B, bl), dev, bl, variant=v, group_m=gm), base)


# ------------------------------------------------------------------------------------------------
# ABI behaviour on the device
# ------------------------------------------------------------------------------------------------
def test_error_codes_on_device(dev):
    M, N, K = 256, 256, 4096
    A = torch.zeros(M, K, dtype=torch.bfloat16, device=dev)
    B = torch.zeros(K, N, dtype=torch.bfloat16, device=dev)
    C = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    ws = torch.zeros(1024, dtype=torch.uint8, device=dev)
    # split-K without enough workspace
    st = _abi.gemm_raw(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, 0, ws.data_ptr(), 1024, 0,
                       g.VARIANT_T128x128_W4, 4, 0)
    assert st == _abi.ERR_WORKSPACE
    st = _abi.gemm_raw(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, 0, 0, 0, 0,
                       g.VARIANT_T128x128_W4, 4, 0)
    assert st == _abi.ERR_WORKSPACE
    # a tile kernel asked to run an unaligned problem
    st = _abi.gemm_raw(A.data_ptr() + 2, B.data_ptr(), C.data_ptr(), M, N, K - 8, K, N, N, 0, 0, 0, 0, 0,
                       g.VARIANT_T128x128_W4, 1, 0)
    assert st == _abi.ERR_UNSUPPORTED
    torch.cuda.synchronize()


def test_runs_on_the_callers_stream(dev):
    A, B = o.make_inputs(512, 512, 1024, seed=4)
    Ad, Bd = A.to(dev), B.to(dev)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        C = g.gemm(Ad, Bd)
        import neoGEMM
        C2 = neoGEMM.gemm(Ad, Bd)
    s.synchronize()
    o.assert_parity(C, A, B, what="side stream")
    assert torch.equal(C, C2)


def test_profile_entry_point(dev):
    lib = _abi.load()
    M = N = K = 1024
    A, B = o.make_inputs(M, N, K, seed=12)
    Ad, Bd = A.to(dev), B.to(dev)
    C = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    for variant, waves in ((g.VARIANT_T256x256_W4, 4),):
        nb = lib.neogemm_bf16_profile_bytes(M, N, variant)
        buf = torch.zeros(nb // 8, dtype=torch.int64, device=dev)
        st = lib.neogemm_bf16_profile(Ad.data_ptr(), Bd.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, None, variant, 0,
                                      buf.data_ptr(), nb)
        assert st == 0
        torch.cuda.synchronize()
        p = buf.cpu().view(-1, 4)
        assert p.shape[0] == 16 * waves
        assert torch.all(p[:, 0] > 0) and torch.all(p[:, 0] >= p[:, 1] + p[:, 2])
        o.assert_parity(C, A, B, what="profiled run")
        assert lib.neogemm_bf16_profile(Ad.data_ptr(), Bd.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, None, variant, 0,
                                        buf.data_ptr(), 8) == _abi.ERR_WORKSPACE
    # the instrumented build exists for that one kernel; retired variant numbers are refused everywhere
    for variant in (2, 8, g.VARIANT_T128x128_W4):
        assert lib.neogemm_bf16_profile(Ad.data_ptr(), Bd.data_ptr(), C.data_ptr(), M, N, K, K, N, N, 0, None, variant, 0,
                                        buf.data_ptr(), nb) == _abi.ERR_UNSUPPORTED
    for variant in (2, 8):
        with pytest.raises(g.NeoGemmError):
            g.gemm_into(Ad, Bd, C, M, N, K, K, N, N, g.B_KN, g.C_ROW, variant)


def test_benchmark_driver(dev):
    """benchmark.py (the reference driver's counterpart) on a small non-square shape: error block and timings."""
    import io

    import benchmark

    out = io.StringIO()
    st = benchmark.run(192, 320, 256, warmup=1, iters=2, seed=3, out=out)
    assert st["rel_fro"] < 1e-3 and st["pct_within_1e-3"] > 99.0
    text = out.getvalue()
    assert "neoGEMM.neoGemmV1" in text and text.count("TFLOP/s") == 4
    assert all(ms > 0 for ms in st["ms"].values())


# ------------------------------------------------------------------------------------------------
# C = alpha * A*B + beta * C (neogemm_bf16_scaled; the epilogue of neogemmv4.cu:166,266)
# ------------------------------------------------------------------------------------------------
def run_scaled(A, B, C0, dev, alpha, beta, b_layout=g.B_KN, c_layout=g.C_ROW):
    M, K = A.shape
    N = B.shape[1] if b_layout == g.B_KN else B.shape[0]
    Cd = (C0 if c_layout == g.C_ROW else C0.t().contiguous()).to(dev)
    g.gemm_into(A.to(dev), B.to(dev), Cd, M, N, K, max(K, 1), max(N if b_layout == g.B_KN else K, 1),
                max(N if c_layout == g.C_ROW else M, 1), b_layout, c_layout, alpha=alpha, beta=beta)
    torch.cuda.synchronize()
    C = Cd.cpu()
    return C if c_layout == g.C_ROW else C.t().contiguous()


def test_scaled_through_the_decode_kernels(dev):
    """alpha and beta through the skinny kernels the plan picks for decode shapes: 96 rows (SKINNY128), 120 rows (STRIP), 16-column strips
    (B [N,K], N = 4096) and staggered depths (K = 8192); exact on small integers, every layout of C."""
    gen = torch.Generator().manual_seed(23)
    for (M, N, K, b_layout, variant) in ((96, 14336, 2048, g.B_NK, g.VARIANT_SKINNY128), (96, 14336, 2048, g.B_KN, g.VARIANT_SKINNY128),
                                         (120, 14336, 2048, g.B_NK, g.VARIANT_STRIP),
                                         (16, 4096, 4096, g.B_NK, g.VARIANT_SKINNY16), (40, 8192, 8192, g.B_NK, g.VARIANT_SKINNY64)):
        A = torch.randint(-2, 3, (M, K), generator=gen).to(torch.bfloat16)
        B = torch.randint(-2, 3, (K, N), generator=gen).to(torch.bfloat16)
        C0 = torch.randint(-8, 9, (M, N), generator=gen).to(torch.bfloat16)
        for c_layout in (g.C_ROW, g.C_COL):
            assert g.plan(M, N, K, b_layout, c_layout)[0] == variant
            for alpha, beta in ((0.5, -3.0), (1.0, 1.0)):
                want = o.ref_gemm_scaled(A, B, C0, alpha, beta)
                got = run_scaled(A, layouts(B, b_layout), C0, dev, alpha, beta, b_layout, c_layout)
                assert np.array_equal(o.bits_of(got), o.bits_of(want)), (M, N, K, alpha, beta, b_layout, c_layout)


def test_scaled_exact_small_integers(dev):
    gen = torch.Generator().manual_seed(21)
    for (M, N, K) in ((24, 40, 16), (256, 512, 128), (130, 264, 72), (16, 2048, 1024)):   # generic, tile, ragged, split-K
        A = torch.randint(-3, 4, (M, K), generator=gen).to(torch.bfloat16)
        B = torch.randint(-3, 4, (K, N), generator=gen).to(torch.bfloat16)
        C0 = torch.randint(-8, 9, (M, N), generator=gen).to(torch.bfloat16)
        for alpha, beta in ((2.0, -3.0), (0.5, 0.0), (1.0, 1.0), (0.0, 2.0)):
            want = o.ref_gemm_scaled(A, B, C0, alpha, beta)          # exact integers / halves: order-independent
            for b_layout in (g.B_KN, g.B_NK):
                for c_layout in (g.C_ROW, g.C_COL):
                    got = run_scaled(A, layouts(B, b_layout), C0, dev, alpha, beta, b_layout, c_layout)
                    assert np.array_equal(o.bits_of(got), o.bits_of(want)), (M, N, K, alpha, beta, b_layout, c_layout)


@pytest.mark.parametrize("M,N,K", [(512, 512, 512), (2048, 2304, 1024), (300, 520, 200), (64, 14336, 4096),
                                   (1024, 1024, 8192), (7, 9, 8)])
def test_scaled_parity(dev, M, N, K):
    A, Bkn = o.make_inputs(M, N, K, seed=M + K)
    C0 = torch.randn(M, N, generator=torch.Generator().manual_seed(N)).to(torch.bfloat16)
    for alpha, beta in ((1.5, -0.75), (-2.0, 0.0), (1.0, 1.0)):
        for b_layout in (g.B_KN, g.B_NK):
            got = run_scaled(A, layouts(Bkn, b_layout), C0, dev, alpha, beta, b_layout)
            ulp, fro = o.scaled_parity(got, A, Bkn, C0, alpha, beta)
            # tolerance of the GEMM path itself: <= 1 bf16 ulp (floored at 2^-7 rms) and <= 1e-3 relative Frobenius
            assert ulp <= 1.0 and fro <= 1e-3, (M, N, K, alpha, beta, b_layout, ulp, fro)


def test_scaled_special_cases(dev):
    M, N, K = 384, 512, 256
    A, Bkn = o.make_inputs(M, N, K, seed=77)
    nan = torch.full((M, N), float("nan"), dtype=torch.bfloat16)
    plain = run_abi(A, Bkn, dev)
    # beta == 0 never reads C; alpha == 1 is the plain GEMM bit for bit; alpha == 0, beta == 1 leaves C as it is
    assert np.array_equal(o.bits_of(run_scaled(A, Bkn, nan, dev, 1.0, 0.0)), o.bits_of(plain))
    got = run_scaled(A, Bkn, nan, dev, 2.0, 0.0)
    assert torch.equal(got.float(), plain.float() * 2)               # power-of-two scaling is exact
    C0 = torch.randn(M, N, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    assert np.array_equal(o.bits_of(run_scaled(A, Bkn, C0, dev, 0.0, 1.0)), o.bits_of(C0 + 0.0))
    lib = _abi.load()
    Ad, Bd, Cd = A.to(dev), Bkn.to(dev), C0.to(dev)
    st = lib.neogemm_bf16_scaled(Ad.data_ptr(), Bd.data_ptr(), Cd.data_ptr(), M, N, K, K, N, N, 0, 0, float("nan"), 0.0,
                                 None, 0, None)
    assert st == _abi.ERR_BAD_ARG
    import neoGEMM
    C1 = C0.to(dev)
    neoGEMM.gemm_scaled(Ad, Bd, C1, alpha=1.5, beta=-0.75)
    C2 = g.gemm_scaled(Ad, Bd, C0.to(dev), 1.5, -0.75)
    torch.cuda.synchronize()
    assert np.array_equal(o.bits_of(C1.cpu()), o.bits_of(C2.cpu()))


def test_tuner_measures_candidates(dev):
    """gemm_amd/tune.py: every candidate it times is a valid (variant, split) and the best is no slower than the model's."""
    import io

    from gemm_amd import tune

    model, t_model, best, t_best = tune.tune_shape(256, 384, 2048, log=io.StringIO())
    assert model == g.plan(256, 384, 2048) and best[0] in tune.CANDIDATE_VARIANTS + (model[0],) and best[1] >= 1
    assert 0 < t_best <= t_model
    # the reference's layout (B [N,K], column-major C) is tuned on its own kernels
    model, t_model, best, t_best = tune.tune_shape(256, 384, 2048, log=io.StringIO(), b_layout=g.B_NK, c_layout=g.C_COL)
    assert model == g.plan(256, 384, 2048, g.B_NK, g.C_COL) and 0 < t_best <= t_model


# ------------------------------------------------------------------------------------------------
# batched (neogemm_bf16_batched): every problem of the batch against the oracle
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("batch,M,N,K", [(3, 256, 384, 512), (5, 130, 72, 200), (2, 1024, 1024, 1024), (4, 16, 2048, 4096),
                                         (7, 5, 9, 12), (1, 512, 512, 512)])
def test_batched_parity(dev, batch, M, N, K):
    As, Bs = zip(*(o.make_inputs(M, N, K, seed=100 * b + M) for b in range(batch)))
    A, B = torch.stack(As), torch.stack(Bs)
    C = g.gemm_batched(A.to(dev), B.to(dev))
    torch.cuda.synchronize()
    assert C.shape == (batch, M, N)
    for b in range(batch):
        o.assert_parity(C[b], As[b], Bs[b], what=f"batch {b} of {batch}x{M}x{N}x{K}")
    # a shared B (stride 0) and the extension's entry point
    C2 = g.gemm_batched(A.to(dev), Bs[0].to(dev))
    import neoGEMM
    C3 = neoGEMM.bmm(A.to(dev), B.to(dev))
    torch.cuda.synchronize()
    for b in range(batch):
        o.assert_parity(C2[b], As[b], Bs[0], what=f"shared B, batch {b}")
    assert np.array_equal(o.bits_of(C3.cpu().view(batch * M, N)), o.bits_of(C.cpu().view(batch * M, N)))
    # one problem of the batch is the plain call bit for bit when both take the same (variant, split)
    if g.plan(M, N, K) == tuple(_abi.plan(M, N, K)) and batch == 1:
        assert np.array_equal(o.bits_of(C[0].cpu()), o.bits_of(g.gemm(A[0].to(dev), B[0].to(dev)).cpu()))


@pytest.mark.parametrize("batch", [2, 7])
def test_batched_workspace_query_bounds_every_layout(dev, batch):
    """A workspace of exactly neogemm_bf16_batched_workspace_bytes(M,N,K,batch) must carry the batched call in every
    layout pair (the batched plan splits K differently from the single call's, and differently per layout): shapes
    with few output tiles and a deep K, where the plan splits."""
    lib = _abi.load()
    split_somewhere = False
    for (M, N, K) in ((128, 128, 8192), (256, 512, 16384), (64, 256, 4096), (1024, 1024, 8192)):
        need = int(lib.neogemm_bf16_batched_workspace_bytes(M, N, K, batch))
        split_somewhere |= need > 0
        assert need % (M * N * 4 * batch) == 0                      # a whole number of fp32 partials per problem
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
        A, Bkn = o.make_inputs(batch * M, N, K, seed=batch + M)    # a batch of different A, one shared B
        ref = o.ref_gemm(A, Bkn)
        for b_layout in (g.B_KN, g.B_NK):
            for c_layout in (g.C_ROW, g.C_COL):
                Ad, Bd = A.to(dev), layouts(Bkn, b_layout).to(dev)
                C = torch.full((batch, M, N) if c_layout == g.C_ROW else (batch, N, M), float("nan"), dtype=torch.bfloat16, device=dev)
                st = lib.neogemm_bf16_batched(Ad.data_ptr(), Bd.data_ptr(), C.data_ptr(), M, N, K, K, N if b_layout == g.B_KN else K,
                                              N if c_layout == g.C_ROW else M, M * K, 0, M * N, batch, b_layout, c_layout,
                                              ws.data_ptr() if need else None, need, None)
                assert st == _abi.OK, (M, N, K, batch, b_layout, c_layout, need, _abi.strerror(st))
                torch.cuda.synchronize()
                got = C.cpu() if c_layout == g.C_ROW else C.cpu().transpose(1, 2).contiguous()
                o.assert_parity(got.reshape(batch * M, N), A, Bkn, ref=ref, what=f"batched {batch}x{M}x{N}x{K} b{b_layout} c{c_layout}")
                if need:
                    # one byte less is refused, never overrun (where this layout pair's plan needs all of it, or less)
                    st = lib.neogemm_bf16_batched(Ad.data_ptr(), Bd.data_ptr(), C.data_ptr(), M, N, K, K, N if b_layout == g.B_KN else K,
                                                  N if c_layout == g.C_ROW else M, M * K, 0, M * N, batch, b_layout, c_layout,
                                                  ws.data_ptr(), M * N * 4 * batch - 1, None)
                    assert st in (_abi.OK, _abi.ERR_WORKSPACE)
                    torch.cuda.synchronize()
    assert split_somewhere


def test_batched_argument_checks(dev):
    lib = _abi.load()
    A = torch.zeros(2, 64, 64, dtype=torch.bfloat16, device=dev)
    C = torch.zeros(2, 64, 64, dtype=torch.bfloat16, device=dev)
    call = lambda sc, batch: lib.neogemm_bf16_batched(A.data_ptr(), A.data_ptr(), C.data_ptr(), 64, 64, 64, 64, 64, 64,
                                                      4096, 4096, sc, batch, 0, 0, None, 0, None)
    assert call(4096, 2) == _abi.OK
    assert call(100, 2) == _abi.ERR_BAD_ARG          # outputs would overlap
    assert call(4096, 70000) == _abi.ERR_BAD_ARG     # more than 65535 problems
    assert call(4096, 0) == _abi.OK                  # empty batch: nothing to do
    torch.cuda.synchronize()


# ------------------------------------------------------------------------------------------------
# skinny-M streaming kernels (M <= 16 / 32 / 64, and 128 as two row blocks): forced and through the plan
# ------------------------------------------------------------------------------------------------
SKINNY = [(g.VARIANT_SKINNY16, 16), (g.VARIANT_SKINNY32, 32), (g.VARIANT_SKINNY64, 64), (g.VARIANT_SKINNY128, 128)]


@pytest.mark.parametrize("variant,rows", SKINNY)
@pytest.mark.parametrize("b_layout", [g.B_KN, g.B_NK])
@pytest.mark.parametrize("c_layout", [g.C_ROW, g.C_COL])
def test_skinny_kernels(dev, variant, rows, b_layout, c_layout):
    # K: one step, a partial step, fewer steps than the four waves, more than the ring, a K tail;
    # N: one strip, a ragged strip (N % 64, N % 8 == 0), many strips; M: 1, ragged, full
    for (M, N, K) in ((1, 64, 64), (rows, 200, 72), (rows - 3, 1000, 520), (rows - 4, 1000, 520), (rows, 4096, 1032),
                      (5, 2048, 8200), (8, 2048, 8200), (rows, 64, 4096), (3, 72, 136), (rows, 14336, 512),
                      (rows // 2 + 1, 520, 1032), (rows // 2 + 4, 1096, 264), (rows - 16, 8, 256),
                      (rows, 12280, 136)):   # B [N,K]: 256 strips of 48 columns, the last one 40 wide
        A, Bkn = o.make_inputs(M, N, K, seed=M + N + K)
        try:
            got = run_abi(A, layouts(Bkn, b_layout), dev, b_layout, c_layout, variant, strict=True)
        except g.NeoGemmError as e:
            # a column-major C with ldc = M not a multiple of 4 is not on the aligned path: refused when forced
            assert e.status == _abi.ERR_UNSUPPORTED and c_layout == g.C_COL and M % 4 != 0
            continue
        o.assert_parity(got, A, Bkn, what=f"skinny v{variant} {M}x{N}x{K} b{b_layout} c{c_layout}")


@pytest.mark.parametrize("variant,rows", SKINNY)
def test_skinny_strip_widths_with_b_nk(dev, variant, rows):
    """B [N,K]: the strips are as wide as fills the CUs in whole rounds (16 to 64 columns, multiples of 8; instances with
    steps of 16, 32 and 64 columns); N need not be a multiple of 8 there, so the last strip can end anywhere."""
    for (M, N, K) in ((rows, 4096, 264), (rows - 1, 6152, 200), (rows, 5004, 136), (3, 1004, 520), (rows, 8192, 72),
                      (rows - 2, 14332, 136), (rows, 20480, 72), (rows, 24, 1032), (rows, 16388, 64),
                      # rows of B a multiple of 16 KiB apart: every strip starts at another depth of K
                      (rows, 520, 8192), (rows - 1, 4100, 16384)):
        A, Bkn = o.make_inputs(M, N, K, seed=M + N + K)
        for c_layout in (g.C_ROW, g.C_COL):
            if c_layout == g.C_COL and M % 4 != 0:
                continue   # ldc = M must be a multiple of 4 on the aligned path
            got = run_abi(A, layouts(Bkn, g.B_NK), dev, g.B_NK, c_layout, variant, strict=True)
            o.assert_parity(got, A, Bkn, what=f"skinny v{variant} {M}x{N}x{K} nk c{c_layout}")


def test_decode_shapes_through_the_plan_on_random_shapes(dev):
    """Seeded random decode shapes (1 to 136 rows on either side, 2000 to 28672 columns, K from 520 to 14336), all
    four layout pairs, through the auto plan: whatever kernel, strip width and ring the plan and the launcher pick, the
    result meets the oracle's bar; small-integer data in the same shapes must come out exact."""
    rng = np.random.default_rng(77)
    seen = set()
    for it in range(40):
        small = int(rng.integers(1, 137))
        wide = int(rng.choice([2048, 4096, 6144, 8192, 10240, 11008, 12288, 14336, 16384, 20480, 28672])) - 8 * int(rng.integers(0, 3))
        K = int(rng.choice([520, 1024, 2048, 4096, 4104, 8192, 14336]))
        if wide * K > 120e6:
            wide = int(120e6 // K) // 8 * 8
        tall = bool(rng.integers(0, 2))
        M, N = (wide, small) if tall else (small, wide)
        b_layout = g.B_NK if (tall or rng.integers(0, 2)) else g.B_KN
        if b_layout == g.B_KN:
            N = (N + 7) // 8 * 8          # whole 16-byte chunks of a row of B [K,N]
        c_layout = g.C_COL if rng.integers(0, 2) else g.C_ROW
        if (c_layout == g.C_COL and M % 4) or (c_layout == g.C_ROW and N % 4):
            c_layout = g.C_ROW if N % 4 == 0 else g.C_COL
        if (c_layout == g.C_COL and M % 4) or (c_layout == g.C_ROW and N % 4):
            continue                      # neither leading dimension of C would be aligned
        seen.add(g.plan(M, N, K, b_layout, c_layout)[0])
        A, Bkn = o.make_inputs(M, N, K, seed=1000 + it)
        got = run_abi(A, layouts(Bkn, b_layout), dev, b_layout, c_layout)
        o.assert_parity(got, A, Bkn, what=f"decode {M}x{N}x{K} b{b_layout} c{c_layout}")
        gen = torch.Generator().manual_seed(it)
        Ai = torch.randint(-2, 3, (M, K), generator=gen).to(torch.bfloat16)
        Bi = torch.randint(-2, 3, (K, N), generator=gen).to(torch.bfloat16)
        goti = run_abi(Ai, layouts(Bi, b_layout), dev, b_layout, c_layout)
        assert np.array_equal(o.bits_of(goti), o.bits_of(o.ref_gemm(Ai, Bi))), (M, N, K, b_layout, c_layout)
    assert {g.VARIANT_SKINNY16, g.VARIANT_SKINNY64, g.VARIANT_SKINNY128, g.VARIANT_STRIP} <= seen   # the draw reaches the decode kernels


def test_skinny_known_answers_and_refusals(dev):
    gen = torch.Generator().manual_seed(31)
    for variant, rows in SKINNY:
        M, N, K = rows, 320, 448
        A = torch.randint(-3, 4, (M, K), generator=gen).to(torch.bfloat16)
        B = torch.randint(-3, 4, (K, N), generator=gen).to(torch.bfloat16)
        want = o.ref_gemm(A, B)                                   # small integers: exact in any order
        for b_layout in (g.B_KN, g.B_NK):
            for c_layout in (g.C_ROW, g.C_COL):
                got = run_abi(A, layouts(B, b_layout), dev, b_layout, c_layout, variant, strict=True)
                assert np.array_equal(o.bits_of(got), o.bits_of(want))
        # too many rows, N % 8 != 0 with B [K,N]: refused, never mis-run
        lib = _abi.load()
        big = torch.zeros(rows + 1, 64, dtype=torch.bfloat16, device=dev)
        sq = torch.zeros(64, 64, dtype=torch.bfloat16, device=dev)
        call = lambda M_, N_, c_layout: lib.neogemm_bf16_variant(big.data_ptr(), sq.data_ptr(), big.data_ptr(), M_, N_, 64, 64,
                                                                   64, 64, 0, c_layout, None, 0, None, variant, 1, 0)
        assert call(rows + 1, 64, 0) == _abi.ERR_UNSUPPORTED
        assert call(rows, 60, 0) == _abi.ERR_UNSUPPORTED
    # the plan sends decode shapes there (both layouts of C: the reference's call writes column-major), and
    # alpha/beta pass through
    assert g.plan(16, 14336, 4096)[0] == g.VARIANT_SKINNY16 and g.plan(64, 14336, 4096)[0] == g.VARIANT_SKINNY64
    assert g.plan(16, 14336, 4096, c_layout=g.C_COL)[0] == g.VARIANT_SKINNY16
    assert g.plan(96, 14336, 4096)[0] == g.VARIANT_SKINNY128 and g.plan(96, 14336, 4096, b_layout=g.B_NK)[0] == g.VARIANT_SKINNY128
    assert g.plan(128, 14336, 4096, b_layout=g.B_NK)[0] == g.VARIANT_STRIP
    M, N, K = 16, 4096, 2048
    A, Bkn = o.make_inputs(M, N, K, seed=2)
    C0 = torch.randn(M, N, generator=gen).to(torch.bfloat16)
    assert g.plan(M, N, K)[0] == g.VARIANT_SKINNY16
    for c_layout in (g.C_ROW, g.C_COL):
        got = run_scaled(A, Bkn, C0, dev, 1.5, -0.5, g.B_KN, c_layout)
        ulp, fro = o.scaled_parity(got, A, Bkn, C0, 1.5, -0.5)
        assert ulp <= 1.0 and fro <= 1e-3


# ------------------------------------------------------------------------------------------------
# 65 to 128 rows: the eight-wave strip kernel (shared rings, rows split between the compute waves), forced
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("b_layout", [g.B_KN, g.B_NK])
@pytest.mark.parametrize("c_layout", [g.C_ROW, g.C_COL])
def test_strip_kernel(dev, b_layout, c_layout):
    # rows: every count of 16-row fragments from five to eight, whole and ragged (a wave then works on a copy of its last
    # fragment and drops it); K: less than a stage, a partial stage, fewer stages than the rings hold, many, a K tail in
    # the first and in the second half of a stage; N: one strip, ragged strips, two rounds of strips
    for (M, N, K) in ((65, 64, 64), (80, 200, 72), (81, 1000, 520), (96, 1000, 392), (100, 4096, 1032), (112, 2048, 8200),
                      (113, 64, 4096), (128, 72, 136), (128, 14336, 512), (127, 520, 1032), (124, 1096, 264), (68, 8, 256),
                      (128, 12280, 136), (96, 28672, 256), (128, 3000, 2048 + 40), (72, 4104, 2048 + 104)):
        if b_layout == g.B_KN and N % 8:
            continue   # whole 16-byte chunks of a row of B [K,N]
        A, Bkn = o.make_inputs(M, N, K, seed=M + N + K)
        try:
            got = run_abi(A, layouts(Bkn, b_layout), dev, b_layout, c_layout, g.VARIANT_STRIP, strict=True)
        except g.NeoGemmError as e:
            # a column-major C with ldc = M not a multiple of 4 is not on the aligned path: refused when forced
            assert e.status == _abi.ERR_UNSUPPORTED and c_layout == g.C_COL and M % 4 != 0
            continue
        o.assert_parity(got, A, Bkn, what=f"strip {M}x{N}x{K} b{b_layout} c{c_layout}")


def test_strip_kernel_known_answers_rings_and_refusals(dev):
    gen = torch.Generator().manual_seed(37)
    lib = _abi.load()
    for (M, N, K) in ((128, 328, 200), (72, 64, 264), (97, 136, 1032), (112, 2048, 4096)):
        A = torch.randint(-3, 4, (M, K), generator=gen).to(torch.bfloat16)
        B = torch.randint(-3, 4, (K, N), generator=gen).to(torch.bfloat16)
        want = o.ref_gemm(A, B)                                   # small integers: exact in any order
        for b_layout in (g.B_KN, g.B_NK):
            for c_layout in (g.C_ROW, g.C_COL):
                if c_layout == g.C_COL and M % 4:
                    continue
                # the default rings and forced ones (the group_m argument carries 16 * stages of A + stages of B); rings
                # that do not fit the 160 KiB of LDS, or with no stage in flight, are refused
                for rings in (0, 0x22, 0x33, 0x25, 0x43, 0x99):
                    Ad, Bd = A.to(dev), layouts(B, b_layout).to(dev)
                    C = torch.full((M, N) if c_layout == g.C_ROW else (N, M), float("nan"), dtype=torch.bfloat16, device=dev)
                    st = lib.neogemm_bf16_variant(Ad.data_ptr(), Bd.data_ptr(), C.data_ptr(), M, N, K, K, N if b_layout == g.B_KN else K,
                                                  N if c_layout == g.C_ROW else M, b_layout, c_layout, None, 0, None,
                                                  g.VARIANT_STRIP, 0, rings)
                    tmf = (M + 15) // 16
                    fits = rings == 0 or ((rings >> 4) * tmf * 4096 + (rings & 15) * 16384 <= 160 * 1024 and ((rings >> 4) - 2) * tmf <= 63)
                    assert st == (_abi.OK if fits else _abi.ERR_UNSUPPORTED), (M, N, K, rings, st)
                    if fits:
                        torch.cuda.synchronize()
                        got = C.cpu() if c_layout == g.C_ROW else C.cpu().t().contiguous()
                        assert np.array_equal(o.bits_of(got), o.bits_of(want)), (M, N, K, b_layout, c_layout, rings)
    # fewer than 65 or more than 128 rows on both sides, N % 8 != 0 with B [K,N]: refused, never mis-run
    big = torch.zeros(129, 136, dtype=torch.bfloat16, device=dev)
    call = lambda M_, N_, b_layout: lib.neogemm_bf16_variant(big.data_ptr(), big.data_ptr(), big.data_ptr(), M_, N_, 64, 64,
                                                               136 if b_layout == 0 else 64, 136, b_layout, 0, None, 0, None, g.VARIANT_STRIP, 1, 0)
    assert call(129, 136, 0) == _abi.ERR_UNSUPPORTED and call(64, 136, 0) == _abi.ERR_UNSUPPORTED
    assert call(128, 132, 0) == _abi.ERR_UNSUPPORTED
    assert call(129, 136, 1) == _abi.ERR_UNSUPPORTED   # B [N,K] with 136 rows: neither side has 65 to 128 rows
    torch.cuda.synchronize()


def test_strip_kernel_with_k_split(dev):
    """The strip kernel with K split over the workgroups of a strip: fp32 partial sums in the workspace, laid out as C is in
    memory, and the reduction kernel behind it.  Against the oracle on every layout pair, odd shapes and split counts (a split
    that would be empty is dropped), the transposed problem, twice in a row on one workspace (bit for bit the same); exact on
    small integers; a workspace that is too small is refused; and the plan sends few strips with deep K there."""
    lib = _abi.load()
    # (with K split the kernel also takes 64 rows and fewer, on four row fragments: unsplit those are refused)
    for (M, N, K) in ((128, 1024, 1024), (100, 2048, 4096), (120, 520, 2120), (65, 264, 392), (112, 4096, 14336), (64, 1024, 1024),
                      (40, 2048, 4096), (16, 520, 2120), (1, 264, 392)):
        for split_k in (2, 3, 8):
            for b_layout, c_layout in ((g.B_NK, g.C_ROW), (g.B_NK, g.C_COL), (g.B_KN, g.C_ROW), (g.B_KN, g.C_COL)):
                if c_layout == g.C_COL and M % 4:
                    continue
                A, Bkn = o.make_inputs(M, N, K, seed=M + N + K + split_k)
                got = [run_abi(A, layouts(Bkn, b_layout), dev, b_layout, c_layout, g.VARIANT_STRIP, split_k) for _ in range(2)]
                assert torch.equal(got[0], got[1])
                o.assert_parity(got[0], A, Bkn, what=f"strip {M}x{N}x{K} split {split_k} b{b_layout} c{c_layout}")
    for (M, N, K, split_k) in ((4096, 128, 4096, 2), (8192, 100, 2048, 4)):      # 65 .. 128 columns, B [N,K]: C^T = B * A^T
        for c_layout in (g.C_ROW, g.C_COL):
            A, Bkn = o.make_inputs(M, N, K, seed=M + N)
            got = run_abi(A, Bkn.t().contiguous(), dev, g.B_NK, c_layout, g.VARIANT_STRIP, split_k)
            o.assert_parity(got, A, Bkn, what=f"strip transposed {M}x{N}x{K} split {split_k} c{c_layout}")
    gen = torch.Generator().manual_seed(41)
    M, N, K = 128, 512, 1024
    A = torch.randint(-3, 4, (M, K), generator=gen).to(torch.bfloat16)
    B = torch.randint(-3, 4, (K, N), generator=gen).to(torch.bfloat16)
    for b_layout in (g.B_KN, g.B_NK):
        got = run_abi(A, layouts(B, b_layout), dev, b_layout, g.C_ROW, g.VARIANT_STRIP, 4)
        assert np.array_equal(o.bits_of(got), o.bits_of(o.ref_gemm(A, B)))
    Ad, Bd = A.to(dev), B.to(dev)
    C = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    ws = torch.zeros(4 * M * N, dtype=torch.float32, device=dev)
    call = lambda nbytes: lib.neogemm_bf16_variant(Ad.data_ptr(), Bd.data_ptr(), C.data_ptr(), M, N, K, K, N, N, g.B_KN, g.C_ROW,
                                                   ws.data_ptr(), nbytes, None, g.VARIANT_STRIP, 4, 0)
    assert call(4 * M * N * 4 - 16) == _abi.ERR_WORKSPACE and call(4 * M * N * 4) == _abi.OK
    torch.cuda.synchronize()
    with pytest.raises(g.NeoGemmError):
        run_abi(A[:64], B, dev, g.B_KN, g.C_ROW, g.VARIANT_STRIP, 1)
    assert g.plan(128, 8192, 8192, b_layout=g.B_NK) == (g.VARIANT_STRIP, 2)
    assert g.plan(64, 8192, 8192, b_layout=g.B_NK) == (g.VARIANT_STRIP, 2) and g.plan(16, 8192, 8192, b_layout=g.B_NK)[0] == g.VARIANT_SKINNY16
    check_big(dev, 64, 8192, 8192, seed=7, b_layout=g.B_NK)
    check_big(dev, 128, 8192, 8192, seed=5, b_layout=g.B_NK)
    check_big(dev, 8192, 128, 8192, seed=6, b_layout=g.B_NK, c_layout=g.C_COL)


def test_strip_kernel_on_the_transposed_problem_and_through_the_plan(dev):
    """N in 97 .. 128 < M with B [N,K] runs C^T = B * A^T on the strip kernel; the plan sends 97 to 128 rows with a K-major
    wide operand there when one round of strips about fills the CUs."""
    assert g.plan(128, 14336, 4096, b_layout=g.B_NK)[0] == g.VARIANT_STRIP
    assert g.plan(14336, 112, 4096, b_layout=g.B_NK, c_layout=g.C_COL)[0] == g.VARIANT_STRIP
    for (M, N, K) in ((14336, 128, 1024), (1000, 72, 520), (4100, 100, 2056), (14336, 112, 4096)):
        A, Bkn = o.make_inputs(M, N, K, seed=M + N)
        for c_layout in (g.C_ROW, g.C_COL):
            if (c_layout == g.C_COL and M % 4) or (c_layout == g.C_ROW and N % 4):
                continue
            for v in (g.VARIANT_STRIP, None):
                got = run_abi(A, layouts(Bkn, g.B_NK), dev, g.B_NK, c_layout, v, strict=True)
                o.assert_parity(got, A, Bkn, what=f"strip-n v{v} {M}x{N}x{K} c{c_layout}")
    # 128 x 14336 x 4096, the benchmark's decode shape, B [N,K], both layouts of C, bit-exact on small integers
    gen = torch.Generator().manual_seed(41)
    A = torch.randint(-2, 3, (128, 4096), generator=gen).to(torch.bfloat16)
    B = torch.randint(-2, 3, (4096, 14336), generator=gen).to(torch.bfloat16)
    want = o.ref_gemm(A, B)
    for c_layout in (g.C_ROW, g.C_COL):
        got = run_abi(A, layouts(B, g.B_NK), dev, g.B_NK, c_layout)
        assert np.array_equal(o.bits_of(got), o.bits_of(want))


def test_narrow_operands_run_the_tile_kernels(dev):
    """Leading dimensions below the tile width (N < 128 with B [K,N], K < 64) stay on the MFMA path."""
    for (M, N, K) in ((1024, 16, 512), (2048, 64, 4096), (300, 96, 200), (512, 512, 8), (512, 40, 24), (8, 8, 32),
                      (14336, 16, 4096)):
        assert g.plan(M, N, K)[0] != g.VARIANT_GENERIC
        A, Bkn = o.make_inputs(M, N, K, seed=N + K)
        for b_layout in (g.B_KN, g.B_NK):
            for c_layout in (g.C_ROW, g.C_COL):
                got = run_abi(A, layouts(Bkn, b_layout), dev, b_layout, c_layout)
                o.assert_parity(got, A, Bkn, what=f"{M}x{N}x{K} b{b_layout} c{c_layout}")
        for variant in (g.VARIANT_T128x128_W4, g.VARIANT_T256x256_W4):
            got = run_abi(A, Bkn, dev, g.B_KN, g.C_ROW, variant, strict=True)
            o.assert_parity(got, A, Bkn, what=f"{M}x{N}x{K} v{variant}")


def test_skinny_n_runs_the_transposed_problem(dev):
    """N <= 64 < M with B [N,K]: the skinny kernel computes C^T = B * A^T (small operand B, wide operand A)."""
    assert g.plan(14336, 16, 4096, b_layout=g.B_NK)[0] == g.VARIANT_SKINNY16
    assert g.plan(14336, 48, 4096, b_layout=g.B_NK, c_layout=g.C_COL)[0] == g.VARIANT_SKINNY64
    assert g.plan(14336, 16, 4096, b_layout=g.B_KN)[0] not in (g.VARIANT_SKINNY16, g.VARIANT_GENERIC)
    for variant, cols in SKINNY:
        for (M, N, K) in ((1000, cols, 520), (4096, cols - 4, 1032), (200, 8, 72), (14336, cols, 512)):
            A, Bkn = o.make_inputs(M, N, K, seed=M + N)
            for c_layout in (g.C_ROW, g.C_COL):
                for v in (variant, None):
                    got = run_abi(A, layouts(Bkn, g.B_NK), dev, g.B_NK, c_layout, v, strict=True)
                    o.assert_parity(got, A, Bkn, what=f"skinny-n v{v} {M}x{N}x{K} c{c_layout}")
        # with B [K,N] the small operand is not K-major: refused when forced
        A, Bkn = o.make_inputs(512, cols, 256, seed=1)
        with pytest.raises(g.NeoGemmError):
            run_abi(A, Bkn, dev, g.B_KN, g.C_ROW, variant, strict=True)


# ------------------------------------------------------------------------------------------------
# The tuned plan table compiled into the library, through the automatic plan (so the lookup is part of what is tested),
# against the oracle: every entry whose B has at most 60 M elements at its own shape, and of the larger ones the smallest
# per (layouts, variant, split-K) combination that the others do not cover
# ------------------------------------------------------------------------------------------------
def _shipped_plan_entries():
    import os
    import re
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "gemm_amd", "csrc", "neogemm_default_plan.inc")
    rows = sorted(tuple(int(x) for x in m.groups()) for m in
                  re.finditer(r"^\{(\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+)\},", open(inc).read(), re.M))
    rows = [r for r in rows if r[0] > 0]
    small = [r for r in rows if r[1] * r[2] <= 60e6]
    covered, extra = {r[3:] for r in small}, {}
    for r in rows:
        if r[1] * r[2] > 60e6 and r[3:] not in covered and (r[3:] not in extra or r[1] * r[2] < extra[r[3:]][1] * extra[r[3:]][2]):
            extra[r[3:]] = r
    return small + sorted(extra.values())


@pytest.mark.parametrize("entry", _shipped_plan_entries(), ids=lambda e: "{}x{}x{}-b{}c{}-v{}s{}".format(*e))
def test_shipped_plan_entries_parity(dev, entry):
    M, N, K, b_layout, c_layout, variant, split_k = entry
    assert g.plan(M, N, K, b_layout, c_layout) == (variant, split_k)
    check_big(dev, M, N, K, seed=M + N + K, b_layout=b_layout, c_layout=c_layout, nrows=64)
