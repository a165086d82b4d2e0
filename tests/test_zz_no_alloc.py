"""neogemm_bf16_noalloc: the entry point for callers that cannot allocate device memory.  Its split-K partials go
to an array inside the library's code object instead of a caller's workspace; the kernels are the same, so the
result must equal neogemm_bf16's bit for bit.  Two calls in a row share the array, the second with a smaller
input; a shape whose partials do not fit the array is refused and nothing is written.

Collected last on purpose (the file name sorts after the other test files)."""
import pytest
import torch

import gemm_amd as g
from gemm_amd import _abi
from oracle import gemm_oracle as o

pytestmark = pytest.mark.gpu


def call_noalloc(Ad, Bd, C, M, N, K, b_layout, c_layout):
    lib = _abi.load()
    ldb = N if b_layout == g.B_KN else K
    ldc = N if c_layout == g.C_ROW else M
    return lib.neogemm_bf16_noalloc(Ad.data_ptr(), Bd.data_ptr(), C.data_ptr(), M, N, K, K, ldb, ldc, b_layout, c_layout,
                                    torch.cuda.current_stream().cuda_stream or None)


def call_with_workspace(Ad, Bd, C, M, N, K, b_layout, c_layout):
    need = g.workspace_bytes(M, N, K)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=Ad.device)
    ldb = N if b_layout == g.B_KN else K
    ldc = N if c_layout == g.C_ROW else M
    st = _abi.gemm_raw(Ad.data_ptr(), Bd.data_ptr(), C.data_ptr(), M, N, K, K, ldb, ldc, b_layout, c_layout,
                       ws.data_ptr() if need else 0, need, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()   # ws must outlive the kernels
    return st


@pytest.mark.parametrize("b_layout,c_layout", [(g.B_KN, g.C_ROW), (g.B_NK, g.C_COL)])
def test_noalloc_matches_the_workspace_entry_point(dev, b_layout, c_layout):
    # first a split-K shape that uses most of the array, then a smaller split-K shape, then one without split-K
    shapes = [(1024, 1024, 16384), (264, 392, 8200), (512, 640, 256)]
    assert g.plan(*shapes[0], b_layout, c_layout)[1] > 1 and g.plan(*shapes[1], b_layout, c_layout)[1] > 1
    assert 0 < g.workspace_bytes(*shapes[1]) < g.workspace_bytes(*shapes[0]) <= _abi.NOALLOC_SCRATCH_BYTES
    assert g.workspace_bytes(*shapes[2]) == 0
    for i, (M, N, K) in enumerate(shapes):
        A, Bkn = o.make_inputs(M, N, K, seed=40 + i)
        B = Bkn if b_layout == g.B_KN else Bkn.t().contiguous()
        Ad, Bd = A.to(dev), B.to(dev)
        cshape = (M, N) if c_layout == g.C_ROW else (N, M)
        want = torch.full(cshape, float("nan"), dtype=torch.bfloat16, device=dev)
        assert call_with_workspace(Ad, Bd, want, M, N, K, b_layout, c_layout) == _abi.OK
        got = torch.full(cshape, float("nan"), dtype=torch.bfloat16, device=dev)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        st = call_noalloc(Ad, Bd, got, M, N, K, b_layout, c_layout)
        torch.cuda.synchronize()
        free_after = torch.cuda.mem_get_info()[0]
        assert st == _abi.OK, _abi.strerror(st)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (M, N, K)
        res = got if c_layout == g.C_ROW else got.t()
        o.assert_parity(res[:128].cpu(), A[:128], Bkn, what=f"noalloc {M}x{N}x{K}")
        if i > 0:   # the library was loaded and its array placed by the first call at the latest
            assert free_before - free_after < max(g.workspace_bytes(M, N, K), 1 << 20), "device memory was allocated"


def test_noalloc_refuses_what_does_not_fit(dev):
    M, N, K = 1536, 1536, 32768   # split 6: 54 MiB of partials
    assert g.workspace_bytes(M, N, K) > _abi.NOALLOC_SCRATCH_BYTES
    A = torch.zeros(M, K, dtype=torch.bfloat16, device=dev)
    B = torch.zeros(N, K, dtype=torch.bfloat16, device=dev)
    C = torch.full((N, M), 7.0, dtype=torch.bfloat16, device=dev)
    st = call_noalloc(A, B, C, M, N, K, g.B_NK, g.C_COL)
    torch.cuda.synchronize()
    assert st == _abi.ERR_SCRATCH_LIMIT
    assert "NEOGEMM_NOALLOC_SCRATCH_BYTES" in _abi.strerror(st)
    assert bool((C == 7.0).all())   # nothing ran
    # the argument checks of neogemm_bf16 apply unchanged
    assert call_noalloc(A, B, C, 256, 256, 512, 5, g.C_COL) == _abi.ERR_BAD_ARG


def test_noalloc_under_graph_capture(dev):
    """The caller this entry point is for: a stream under HIP graph capture.  One warm-up call outside the capture (the
    first call on a device resolves the array's address, the first launch of a kernel instance raises its LDS limit:
    both are host-side set-up calls that a capturing stream does not allow), then the call is captured (kernel launches
    only: the split-K tile kernel and the reduce), and every replay, with eager work and synchronisations in between
    and fresh inputs each time, equals the eager result bit for bit."""
    M, N, K = 264, 392, 8200
    b_layout, c_layout = g.B_KN, g.C_ROW
    assert g.plan(M, N, K, b_layout, c_layout)[1] > 1
    gen = torch.Generator().manual_seed(5)
    A0, Bkn = o.make_inputs(M, N, K, seed=50)
    Ad, Bd = A0.to(dev), Bkn.to(dev)
    got = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    eager = torch.zeros(M, N, dtype=torch.bfloat16, device=dev)
    assert call_noalloc(Ad, Bd, eager, M, N, K, b_layout, c_layout) == _abi.OK      # warm-up, outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        st = call_noalloc(Ad, Bd, got, M, N, K, b_layout, c_layout)                 # on the capturing stream
    assert st == _abi.OK, _abi.strerror(st)
    for it in range(4):
        # fresh inputs in the same buffers (eager work between the replays), then replay and eager call
        Ad.copy_((torch.randn(M, K, generator=gen) / K ** 0.5).to(torch.bfloat16))
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert call_noalloc(Ad, Bd, eager, M, N, K, b_layout, c_layout) == _abi.OK
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), eager.view(torch.int16)), f"replay {it}"
    o.assert_parity(got[:64].cpu(), Ad[:64].cpu(), Bkn, what="noalloc under capture")
