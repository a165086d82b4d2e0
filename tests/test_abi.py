"""The C ABI of include/neogemm.h without a GPU: the library loads, exports every declared symbol, and
its host-only entry points (plan, workspace size, error text, argument validation that returns before any
HIP call) behave as documented.  No kernel is launched here."""
import ctypes
import os
import re

import pytest

from gemm_amd import _abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "neogemm.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(neogemm_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for must in ("neogemm_bf16", "neogemm_bf16_workspace_bytes", "neogemm_bf16_variant", "neogemm_bf16_plan",
                 "neogemm_bf16_profile", "neogemm_bf16_profile_bytes", "neogemm_strerror", "neogemm_version"):
        assert must in names


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_abi.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in include/neogemm.h but not exported"
    # and the ctypes prototypes cover exactly the header
    assert sorted(_abi.PROTOTYPES) == declared_functions()


def test_header_cites_the_reference_for_each_entry_point():
    text = open(HEADER).read()
    for cite in ("nemgemmV03.cu:343-391", "v01.cu:189-270", "v01.cu:254-262", "nemgemmV03.cu:387-390",
                 "v01.cu:304-311", "cublass/matmul.cu:99-106"):
        assert cite in text


def test_version_and_strerror():
    assert "gfx950" in _abi.version()
    assert _abi.strerror(0) == "success"
    for st in (_abi.ERR_BAD_ARG, _abi.ERR_WORKSPACE, _abi.ERR_UNSUPPORTED, _abi.ERR_LAUNCH, -99):
        s = _abi.strerror(st)
        assert isinstance(s, str) and s and s != "success"


def test_plan_for_the_benchmark_configs():
    # square compute-bound shapes run a 256x256 tile kernel without split-K
    for n in (4096, 8192):
        v, s = _abi.plan(n, n, n)
        assert v == _abi.VARIANT_C256x256_W4 and s == 1   # K in whole periods of 128, A K-major: the chained kernel
        assert _abi.plan(n, n, n, _abi.B_NK, _abi.C_COL) == (_abi.VARIANT_C256x256_W4, 1)   # the reference's call
        # B [K,N] with a column-major C puts the MN-major operand on the rows, K = 8256 is not whole periods: slab kernel
        assert _abi.plan(n, n, n, _abi.B_KN, _abi.C_COL)[0] == _abi.VARIANT_T256x256_W4
        assert _abi.plan(n, n, n + 64)[0] == _abi.VARIANT_T256x256_W4
    # shapes with few output tiles split K and need a workspace of split * M * N floats (skinny M with a row-major C
    # runs the streaming kernel instead, without split-K)
    for M, N, K in ((16, 14336, 4096), (64, 14336, 4096), (128, 14336, 4096), (1024, 1024, 32768), (512, 512, 512)):
        v, s = _abi.plan(M, N, K)
        assert v != _abi.VARIANT_GENERIC and s >= 1
        s = max(_abi.plan(M, N, K, b, c)[1] for b in (0, 1) for c in (0, 1))   # one query covers all four layouts
        assert _abi.workspace_bytes(M, N, K) == (s * M * N * 4 if s > 1 else 0)
    assert _abi.plan(1024, 1024, 32768)[1] > 1
    # 3072^3 and 6144^3: 144 / 576 tiles of 256x256 fill 256 CUs badly, 192 / 768 tiles of 192x256 do better; the
    # 192 rows must come from a K-major operand (A for a row-major C, B [N,K] for a column-major one)
    for n in (3072, 6144):
        assert _abi.plan(n, n, n) == (_abi.VARIANT_T192x256_W4, 1)
        assert _abi.plan(n, n, n, b_layout=_abi.B_NK, c_layout=_abi.C_COL) == (_abi.VARIANT_T192x256_W4, 1)
        assert _abi.plan(n, n, n, b_layout=_abi.B_KN, c_layout=_abi.C_COL)[0] != _abi.VARIANT_T192x256_W4
    # tall shapes with a skinny N stream through the skinny kernel when B is [N,K]
    assert _abi.plan(14336, 16, 4096, b_layout=_abi.B_NK) == (_abi.VARIANT_SKINNY16, 1)
    assert _abi.plan(14336, 16, 4096, b_layout=_abi.B_KN)[0] not in (_abi.VARIANT_SKINNY16, _abi.VARIANT_GENERIC)
    # 65 to 128 rows with one round of strips over the CUs and a K of a few thousand: the streaming kernel in one launch
    # (measured: it beats split-K tiles there except at 128 rows with B [K,N]); elsewhere the tiles
    # from 97 rows on with a K-major wide operand, the eight-wave strip kernel (shared rings, rows split between the waves)
    for M, want in ((65, _abi.VARIANT_SKINNY128), (96, _abi.VARIANT_SKINNY128), (97, _abi.VARIANT_STRIP), (128, _abi.VARIANT_STRIP)):
        assert _abi.plan(M, 14336, 4096, b_layout=_abi.B_NK) == (want, 1)
        assert _abi.plan(14336, M, 4096, b_layout=_abi.B_NK, c_layout=_abi.C_COL) == (want, 1)
    assert _abi.plan(96, 14336, 4096, b_layout=_abi.B_KN) == (_abi.VARIANT_SKINNY128, 1)
    assert _abi.plan(128, 14336, 4096, b_layout=_abi.B_KN)[0] not in (_abi.VARIANT_SKINNY128, _abi.VARIANT_STRIP)
    assert _abi.plan(128, 8192, 2048, b_layout=_abi.B_NK) == (_abi.VARIANT_STRIP, 1)   # 14.8 us against 19.1 for split-K tiles
    streaming = (_abi.VARIANT_SKINNY128, _abi.VARIANT_STRIP)
    for shape in ((128, 28672, 4096), (128, 14336, 1024), (96, 6144, 4096), (129, 14336, 4096), (128, 8192, 28672)):
        assert _abi.plan(*shape, b_layout=_abi.B_NK)[0] not in streaming
    # too few strips for one launch without a split, from 97 rows on: the strips split K (104 x 6144 x 4096: 20.8 us against
    # 23.6 for the tiles; with 96 rows they are level)
    assert _abi.plan(100, 6144, 4096, b_layout=_abi.B_NK) == (_abi.VARIANT_STRIP, 2)
    # few strips and deep K: the strip kernel with K split over the workgroups of a strip, one round of them in all
    # (128 x 8192 x 8192: 128 strips x 2, 38 us against 44 for split-K tiles), in the transposed problem as well
    assert _abi.plan(128, 8192, 8192, b_layout=_abi.B_NK) == (_abi.VARIANT_STRIP, 2)
    assert _abi.plan(112, 4096, 16384, b_layout=_abi.B_NK) == (_abi.VARIANT_STRIP, 4)
    assert _abi.plan(64, 8192, 8192, b_layout=_abi.B_NK) == (_abi.VARIANT_STRIP, 2)      # 31.7 us against 33.7 for the skinny kernel
    assert _abi.plan(16, 8192, 8192, b_layout=_abi.B_NK) == (_abi.VARIANT_SKINNY16, 1)   # 25.8 against 29.6
    assert _abi.plan(8192, 128, 8192, b_layout=_abi.B_NK, c_layout=_abi.C_COL) == (_abi.VARIANT_STRIP, 2)
    # below 33 rows where the skinny kernel is out (24 x 4096 x 11008: 24.1 us against 28.5 for the tiles), and with B [K,N]
    # from 33 rows on (64 x 4096 x 12288: 27.8 us against 29.4) but not below (16 x 4096 x 12288: 37 against 27)
    assert _abi.plan(24, 4096, 12288, b_layout=_abi.B_NK) == (_abi.VARIANT_STRIP, 4)
    assert _abi.plan(64, 4096, 12288, b_layout=_abi.B_KN) == (_abi.VARIANT_STRIP, 4)
    assert _abi.plan(16, 4096, 12288, b_layout=_abi.B_KN)[0] != _abi.VARIANT_STRIP
    # 65 to 96 rows as well (72 x 8192 x 8192: 36.6 us against 42.9 for the tiles; 80 x 4096 x 16384: 36.2 against 45.1)
    assert _abi.plan(72, 8192, 8192, b_layout=_abi.B_NK) == (_abi.VARIANT_STRIP, 2)
    assert _abi.plan(80, 4096, 16384, b_layout=_abi.B_NK) == (_abi.VARIANT_STRIP, 4)
    assert _abi.plan(8192, 80, 8192, b_layout=_abi.B_NK, c_layout=_abi.C_COL) == (_abi.VARIANT_STRIP, 2)
    # 128x128 tiles on weights from HBM: a few more workgroups than CUs means a second pass on some CUs at the pace of
    # the first (128 x 5120 x 27648 with B [N,K]: split 6, 240 workgroups, 69 us; split 8, 320 of them, 98)
    v, s = _abi.plan(104, 5120, 27648, b_layout=_abi.B_NK)
    assert not (v == _abi.VARIANT_T128x128_W4 and 256 < 40 * s <= 384)
    # in several rounds of strips gemm_skinny_kernel loses to the tiles (72 x 27648 x 5120: 69 us against 60)
    assert _abi.plan(88, 27648, 5120, b_layout=_abi.B_NK)[0] != _abi.VARIANT_SKINNY128
    assert _abi.workspace_bytes(128, 8192, 8192) >= 2 * 128 * 8192 * 4
    # unaligned problems go to the generic kernel
    # B [K,N] with fewer strips of 64 columns than CUs and weights too large for the caches: a strip streams no faster for the
    # chip being half empty, so split-K tiles take these (16 x 7168 x 7168: 29 us against 37 for the skinny kernel), while a
    # full round of strips stays on the skinny kernel
    skinny = (_abi.VARIANT_SKINNY16, _abi.VARIANT_SKINNY32, _abi.VARIANT_SKINNY64)
    for M in (16, 64):
        assert _abi.plan(M, 7168, 7168)[0] not in skinny and _abi.plan(M, 3072, 8192)[0] not in skinny
        assert _abi.plan(M, 12288, 4096)[0] in skinny and _abi.plan(M, 16384, 2048)[0] in skinny
    assert _abi.plan(100, 100, 100, aligned=False) == (_abi.VARIANT_GENERIC, 1)
    assert _abi.workspace_bytes(0, 5, 5) == 0 and _abi.workspace_bytes(5, 5, 0) == 0


def test_workspace_query_bounds_every_layout():
    """neogemm_bf16_workspace_bytes(M,N,K) must cover the split the call itself plans, for every (b_layout, c_layout)
    — the reference's own call is B [N,K] with a column-major C (nemgemmV03.cu:343-391) and must never be answered
    with 'workspace too small' after the caller sized the workspace by the query."""
    dims = [16, 64, 96, 128, 192, 256, 384, 512, 768, 1024, 1536, 2048, 3072, 4096, 6144, 8192, 14336]
    ks = [64, 256, 512, 1024, 2048, 4096, 8192, 16384, 32768]
    cells = 0
    for M in dims:
        for N in dims:
            for K in ks:
                have = _abi.workspace_bytes(M, N, K)
                for b in (_abi.B_KN, _abi.B_NK):
                    for c in (_abi.C_ROW, _abi.C_COL):
                        v, s = _abi.plan(M, N, K, b, c)
                        need = s * M * N * 4 if s > 1 else 0
                        assert need <= have, (M, N, K, b, c, v, s, have)
                        cells += 1
    assert cells >= 10000
    # the cells found failing before the query looked at every layout
    for M, N, K in ((1024, 6144, 8192), (2048, 3072, 8192), (512, 6144, 8192), (4096, 1536, 8192)):
        v, s = _abi.plan(M, N, K, _abi.B_NK, _abi.C_COL)
        assert _abi.workspace_bytes(M, N, K) >= (s * M * N * 4 if s > 1 else 0)
    # the batched query: a batch of one is the plain query; a larger batch asks for whole sets of fp32 partials (that the
    # queried size carries every layout pair's batched call is checked on the GPU, tests/test_gemm_gpu.py)
    lib = _abi.load()
    for M, N, K in ((128, 128, 8192), (256, 512, 16384), (1024, 6144, 8192)):
        assert lib.neogemm_bf16_batched_workspace_bytes(M, N, K, 1) == _abi.workspace_bytes(M, N, K)
        for batch in (2, 7):
            need = lib.neogemm_bf16_batched_workspace_bytes(M, N, K, batch)
            assert need % (M * N * 4 * batch) == 0 and need // (M * N * 4 * batch) in (0, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64)
    assert lib.neogemm_bf16_batched_workspace_bytes(128, 128, 8192, 2) > 0


def test_argument_validation_returns_before_touching_the_gpu():
    bad = _abi.ERR_BAD_ARG
    p = 0x1000  # never dereferenced: every call below is rejected, or is a no-op, on the host
    assert _abi.gemm_raw(p, p, p, -1, 4, 4, 4, 4, 4, 0, 0) == bad
    assert _abi.gemm_raw(p, p, p, 4, 4, 4, 4, 4, 4, 2, 0) == bad        # unknown b_layout
    assert _abi.gemm_raw(p, p, p, 4, 4, 4, 4, 4, 4, 0, 7) == bad        # unknown c_layout
    assert _abi.gemm_raw(p, p, p, 4, 4, 4, 3, 4, 4, 0, 0) == bad        # lda < K
    assert _abi.gemm_raw(p, p, p, 4, 4, 4, 4, 3, 4, 0, 0) == bad        # ldb < N for [K,N]
    assert _abi.gemm_raw(p, p, p, 4, 8, 4, 4, 3, 8, 1, 0) == bad        # ldb < K for [N,K]
    assert _abi.gemm_raw(p, p, p, 4, 4, 4, 4, 4, 3, 0, 0) == bad        # ldc < N row-major
    assert _abi.gemm_raw(p, p, p, 8, 4, 4, 4, 4, 4, 0, 1) == bad        # ldc < M column-major
    assert _abi.gemm_raw(0, p, p, 4, 4, 4, 4, 4, 4, 0, 0) == bad        # null A
    assert _abi.gemm_raw(p, p, 0, 4, 4, 4, 4, 4, 4, 0, 0) == bad        # null C
    assert _abi.gemm_raw(p, p, p, 4, 4, 4, 4, 4, 4, 0, 0, variant=99) == bad
    assert _abi.gemm_raw(p, p, p, 4, 4, 4, 4, 4, 4, 0, 0, variant=0, split_k=-1) == bad
    # empty problems are no-ops
    assert _abi.gemm_raw(0, 0, 0, 0, 4, 4, 4, 4, 4, 0, 0) == _abi.OK
    assert _abi.gemm_raw(0, 0, 0, 4, 0, 4, 4, 4, 4, 0, 0) == _abi.OK


def test_plan_rejects_null_outputs():
    lib = _abi.load()
    assert lib.neogemm_bf16_plan(4, 4, 4, 0, 0, 1, None, None) == _abi.ERR_BAD_ARG


def test_profile_bytes():
    lib = _abi.load()
    assert lib.neogemm_bf16_profile_bytes(8192, 8192, 2) == 0   # a retired variant number: nothing to profile
    assert lib.neogemm_bf16_profile_bytes(8192, 8192, _abi.VARIANT_T256x256_W4) == 1024 * 4 * 4 * 8
    assert lib.neogemm_bf16_profile_bytes(0, 8, _abi.VARIANT_T256x256_W4) == 0


def test_plan_table_overrides_the_model(tmp_path):
    """NEOGEMM_PLAN_TABLE: exact-shape entries win over the cost model; malformed entries are ignored."""
    import json
    import subprocess
    import sys

    table = tmp_path / "plan.json"
    table.write_text(json.dumps([
        {"M": 512, "N": 512, "K": 512, "c_layout": 0, "variant": _abi.VARIANT_T128x128_W4, "split_k": 2},
        {"M": 4096, "N": 4096, "K": 4096, "variant": _abi.VARIANT_T256x256_W4, "split_k": 1},   # c_layout defaults to 0
        {"M": 3072, "N": 3072, "K": 3072, "c_layout": 0, "variant": 2, "split_k": 1},            # a retired variant number
        {"M": 8192, "N": 8192, "K": 8192, "c_layout": 0, "variant": 99, "split_k": 1},           # unknown variant
        {"M": 1024, "N": 1024, "K": 1024, "c_layout": 0, "variant": _abi.VARIANT_T128x128_W4, "split_k": 0},  # bad split
        {"M": 2048, "N": 2048, "K": 2048, "b_layout": 1, "c_layout": 1, "variant": _abi.VARIANT_T128x256_W4, "split_k": 1},
    ]))
    code = ("from gemm_amd import _abi\n"
            "print(_abi.plan(512, 512, 512), _abi.plan(4096, 4096, 4096), _abi.plan(8192, 8192, 8192), "
            "_abi.plan(1024, 1024, 1024), _abi.plan(512, 512, 512, c_layout=1), _abi.workspace_bytes(512, 512, 512), "
            "_abi.plan(512, 512, 512, b_layout=1), _abi.plan(2048, 2048, 2048, 1, 1), _abi.plan(2048, 2048, 2048, 0, 1))")
    env = dict(os.environ, NEOGEMM_PLAN_TABLE=str(table))
    out = subprocess.run([sys.executable, "-c", code], env=env, cwd=ROOT, capture_output=True, text=True, check=True).stdout
    model = (_abi.plan(512, 512, 512), _abi.plan(8192, 8192, 8192), _abi.plan(1024, 1024, 1024))
    want = ((_abi.VARIANT_T128x128_W4, 2), (_abi.VARIANT_T256x256_W4, 1), model[1], model[2],
            _abi.plan(512, 512, 512, c_layout=1), 2 * 512 * 512 * 4,
            # an entry is keyed on both layouts: B [N,K] calls of a shape tuned with B [K,N] keep the model's choice
            _abi.plan(512, 512, 512, b_layout=1), (_abi.VARIANT_T128x256_W4, 1), _abi.plan(2048, 2048, 2048, 0, 1))
    assert out.strip() == " ".join(str(w) for w in want)
    # an unreadable file changes nothing
    env = dict(os.environ, NEOGEMM_PLAN_TABLE=str(tmp_path / "missing.json"))
    out = subprocess.run([sys.executable, "-c", "from gemm_amd import _abi\nprint(_abi.plan(512, 512, 512))"], env=env,
                         cwd=ROOT, capture_output=True, text=True, check=True).stdout
    assert out.strip() == str(model[0])


def test_shipped_plan_table():
    """The tuned exceptions compiled into the library (gemm_amd/csrc/neogemm_default_plan.inc): every entry names a kernel
    variant the planner may return and a sensible split, the planner returns it for exactly that shape and layout pair (and
    not for the others), and the workspace query covers its split."""
    import re
    inc = os.path.join(ROOT, "gemm_amd", "csrc", "neogemm_default_plan.inc")
    rows = [tuple(int(x) for x in m.groups()) for m in
            re.finditer(r"^\{(\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+)\},", open(inc).read(), re.M)]
    rows = [r for r in rows if r[0] > 0]
    assert len(rows) >= 10
    assert len({r[:5] for r in rows}) == len(rows)                       # one entry per shape and layout pair
    tile_variants = (_abi.VARIANT_T256x256_W4, _abi.VARIANT_T128x128_W4, _abi.VARIANT_T256x128_W4, _abi.VARIANT_T128x256_W4,
                     _abi.VARIANT_T64x128_W4, _abi.VARIANT_T192x256_W4, _abi.VARIANT_T96x128_W4, _abi.VARIANT_T64x64_W4,
                     _abi.VARIANT_C256x256_W4)
    for (M, N, K, b, c, v, s) in rows:
        assert b in (0, 1) and c in (0, 1) and 1 <= s <= 64 and s * 128 <= K
        assert v in tile_variants + (_abi.VARIANT_SKINNY16, _abi.VARIANT_SKINNY32, _abi.VARIANT_SKINNY64, _abi.VARIANT_SKINNY128,
                                     _abi.VARIANT_STRIP)
        if v in (_abi.VARIANT_C256x256_W4, _abi.VARIANT_SKINNY128) or v >= _abi.VARIANT_SKINNY16 and v <= _abi.VARIANT_SKINNY64:
            assert s == 1      # (the strip kernel is the one streaming kernel that splits K)
        assert _abi.plan(M, N, K, b, c) == (v, s), (M, N, K, b, c)
        assert _abi.workspace_bytes(M, N, K) >= (s * M * N * 4 if s > 1 else 0)
        assert _abi.plan(M, N, K, b, c, aligned=False) == (_abi.VARIANT_GENERIC, 1)   # the table is for the MFMA path only
