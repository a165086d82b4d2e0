"""gemm_amd — host-side mirror of the reference's extension surface over libneogemm.so.

The drop-in module is `neoGEMM` (built by setup.py from csrc/neogemm_torch.cpp), with the reference's
`neoGemmV1(A, B, C)` (nemgemmV03.cu:396-399) plus `C = gemm(A, B)`.  This package offers the same
three functions through the C ABI with ctypes — which is what the parity tests and the bench use, so
that every measured call crosses the plain-pointer boundary of include/neogemm.h — and lets tests
force a kernel variant / split-K factor.

Nothing here computes: without libneogemm.so and a GPU every call raises.
"""
import torch

from . import _abi
from ._abi import (B_KN, B_NK, C_COL, C_ROW, NeoGemmError, VARIANT_AUTO, VARIANT_GENERIC, VARIANT_NAMES,  # noqa: F401
                   VARIANT_SKINNY16, VARIANT_SKINNY32, VARIANT_SKINNY64, VARIANT_SKINNY128, VARIANT_STRIP, VARIANT_T192x256_W4, VARIANT_T96x128_W4, VARIANT_T64x64_W4, VARIANT_C256x256_W4,
                   VARIANT_T128x128_W4, VARIANT_T128x256_W4, VARIANT_T256x128_W4, VARIANT_T256x256_W4,
                   VARIANT_T64x128_W4, plan, strerror, version, workspace_bytes)

__all__ = ["gemm", "neoGemmV1", "neogemm", "gemm_into", "plan", "workspace_bytes", "version", "NeoGemmError"]

_workspaces = {}        # (device index, stream) -> buffer, in order of last use
_MAX_WORKSPACES = 16    # streams come and go: the least recently used buffer is dropped beyond this many


def _check(t, name):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise ValueError(f"{name} must be a GPU tensor (there is no CPU path)")
    if t.dtype != torch.bfloat16:
        raise TypeError(f"{name} must be bfloat16, got {t.dtype}")
    if t.dim() != 2:
        raise ValueError(f"{name} must be 2-D, got {t.dim()}-D")


def _workspace(device, nbytes):
    """Split-K scratch for torch's current stream on `device`: one buffer per (device, stream), so that GEMMs on
    different streams never share partials.  A buffer is allocated while its stream is current and used on that
    stream only, so when a larger one replaces it, or it is dropped as the least recently used of too many, the
    caching allocator reuses the block in that stream's order."""
    with torch.cuda.device(device):
        key = (device.index if device.index is not None else torch.cuda.current_device(),
               torch.cuda.current_stream().cuda_stream)
        ws = _workspaces.pop(key, None)
        if ws is None or ws.numel() < nbytes:
            ws = None
            while len(_workspaces) >= _MAX_WORKSPACES:
                _workspaces.pop(next(iter(_workspaces)))
            ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
        _workspaces[key] = ws   # (re)inserted last: dicts keep insertion order
    return ws


def gemm_into(A, B, C, M, N, K, lda, ldb, ldc, b_layout, c_layout, variant=None, split_k=0, group_m=0, alpha=1.0,
              beta=0.0):
    """Call the C ABI on torch's current stream; A, B, C are torch tensors used as device buffers."""
    need = workspace_bytes(M, N, K)
    if variant is not None and split_k > 1:
        need = max(need, split_k * M * N * 4)
    ws_ptr = 0
    if need:
        ws_ptr = _workspace(C.device, need).data_ptr()
    with torch.cuda.device(C.device):
        stream = torch.cuda.current_stream().cuda_stream
        st = _abi.gemm_raw(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, lda, ldb, ldc, b_layout, c_layout,
                           ws_ptr, need, stream, variant, split_k, group_m, alpha, beta)
    if st != _abi.OK:
        raise NeoGemmError(st, f"M={M} N={N} K={K} b_layout={b_layout} c_layout={c_layout} variant={variant}")


def gemm(A, B, variant=None, split_k=0, group_m=0):
    """C[M,N] = A[M,K] @ B[K,N]; bf16 in, fp32 accumulate, bf16 out (new tensor)."""
    _check(A, "A")
    _check(B, "B")
    if A.shape[1] != B.shape[0]:
        raise ValueError(f"inner dimensions differ: A is {tuple(A.shape)}, B is {tuple(B.shape)}")
    if A.device != B.device:
        raise ValueError("A and B must be on the same device")
    if A.stride(1) != 1 and A.shape[1] > 1:
        A = A.contiguous()
    M, K = A.shape
    N = B.shape[1]
    lda = A.stride(0) if M > 1 else max(K, 1)
    if B.stride(1) == 1 or N <= 1:
        b_layout, ldb = B_KN, (B.stride(0) if K > 1 else max(N, 1))
    elif B.stride(0) == 1:
        b_layout, ldb = B_NK, (B.stride(1) if N > 1 else max(K, 1))
    else:
        B = B.contiguous()
        b_layout, ldb = B_KN, max(N, 1)
    C = torch.empty((M, N), dtype=torch.bfloat16, device=A.device)
    if M and N:
        gemm_into(A, B, C, M, N, K, lda, ldb, max(N, 1), b_layout, C_ROW, variant, split_k, group_m)
    return C


def neoGemmV1(A, B, C, variant=None, split_k=0, group_m=0):
    """Reference call (nemgemmV03.cu:343-391): A [M,K], B [N,K], C receives A @ B.T column-major."""
    _check(A, "A")
    _check(B, "B")
    _check(C, "C")
    if A.shape[1] != B.shape[1]:
        raise ValueError(f"A is [M,K] and B is [N,K]: K differs ({A.shape[1]} vs {B.shape[1]})")
    if not (A.is_contiguous() and B.is_contiguous() and C.is_contiguous()):
        raise ValueError("A, B and C must be contiguous")
    M, K = A.shape
    N = B.shape[0]
    if C.numel() != M * N:
        raise ValueError(f"C must hold M*N = {M * N} elements, has {C.numel()}")
    if M and N:
        gemm_into(A, B, C, M, N, K, max(K, 1), max(K, 1), M, B_NK, C_COL, variant, split_k, group_m)
    return None


neogemm = neoGemmV1


def gemm_scaled(A, B, C, alpha=1.0, beta=0.0):
    """C[M,N] = alpha * A[M,K] @ B[K,N] + beta * C, in place (C contiguous); neogemm_bf16_scaled."""
    _check(A, "A")
    _check(B, "B")
    _check(C, "C")
    if A.shape[1] != B.shape[0] or C.shape != (A.shape[0], B.shape[1]) or not C.is_contiguous():
        raise ValueError(f"shapes: A {tuple(A.shape)}, B {tuple(B.shape)}, C {tuple(C.shape)} (contiguous [M,N])")
    if A.stride(1) != 1 and A.shape[1] > 1:
        A = A.contiguous()
    M, K = A.shape
    N = B.shape[1]
    lda = A.stride(0) if M > 1 else max(K, 1)
    if B.stride(1) == 1 or N <= 1:
        b_layout, ldb = B_KN, (B.stride(0) if K > 1 else max(N, 1))
    elif B.stride(0) == 1:
        b_layout, ldb = B_NK, (B.stride(1) if N > 1 else max(K, 1))
    else:
        B = B.contiguous()
        b_layout, ldb = B_KN, max(N, 1)
    if M and N:
        gemm_into(A, B, C, M, N, K, lda, ldb, max(N, 1), b_layout, C_ROW, alpha=float(alpha), beta=float(beta))
    return C


def gemm_batched(A, B):
    """C[b,M,N] = A[b,M,K] @ B[b,K,N] (or B [K,N], shared by the batch) in one launch; neogemm_bf16_batched."""
    for t, name in ((A, "A"), (B, "B")):
        if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != torch.bfloat16:
            raise TypeError(f"{name} must be a bfloat16 GPU tensor")
    if A.dim() != 3 or B.dim() not in (2, 3) or A.shape[-1] != B.shape[-2] or (B.dim() == 3 and B.shape[0] != A.shape[0]):
        raise ValueError(f"shapes: A {tuple(A.shape)} must be [b,M,K], B {tuple(B.shape)} [b,K,N] or [K,N]")
    A, B = A.contiguous(), B.contiguous()
    batch, M, K = A.shape
    N = B.shape[-1]
    C = torch.empty((batch, M, N), dtype=torch.bfloat16, device=A.device)
    if batch == 0 or M == 0 or N == 0:
        return C
    lib = _abi.load()
    need = int(lib.neogemm_bf16_batched_workspace_bytes(M, N, K, batch))
    ws_ptr = _workspace(C.device, need).data_ptr() if need else 0
    with torch.cuda.device(C.device):
        stream = torch.cuda.current_stream().cuda_stream
        st = lib.neogemm_bf16_batched(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, max(K, 1), max(N, 1), max(N, 1),
                                      M * K, K * N if B.dim() == 3 else 0, M * N, batch, B_KN, C_ROW, ws_ptr or None,
                                      need, stream or None)
    if st != _abi.OK:
        raise NeoGemmError(st, f"batch={batch} M={M} N={N} K={K}")
    return C
