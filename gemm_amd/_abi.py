"""ctypes binding of the C ABI in include/neogemm.h (gemm_amd/libneogemm.so).

This is the binding the parity tests call through: plain pointers and sizes, no torch types cross it.
torch is used by callers only to own device memory and to name the stream.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libneogemm.so")

OK, ERR_BAD_ARG, ERR_WORKSPACE, ERR_UNSUPPORTED, ERR_LAUNCH, ERR_SCRATCH_LIMIT = 0, -1, -2, -3, -4, -5
NOALLOC_SCRATCH_BYTES = 32 * 1024 * 1024
B_KN, B_NK = 0, 1
C_ROW, C_COL = 0, 1
VARIANT_AUTO, VARIANT_GENERIC = 0, 1
VARIANT_T256x256_W4, VARIANT_T128x128_W4 = 3, 4   # 2 and 8 are retired numbers: the library refuses them
VARIANT_T256x128_W4, VARIANT_T128x256_W4 = 5, 6
VARIANT_T64x128_W4 = 7
VARIANT_SKINNY16, VARIANT_SKINNY32, VARIANT_SKINNY64 = 9, 10, 11
VARIANT_T192x256_W4 = 12
VARIANT_T96x128_W4, VARIANT_T64x64_W4 = 13, 14
VARIANT_C256x256_W4 = 15
VARIANT_SKINNY128 = 16
VARIANT_STRIP = 17
VARIANT_COUNT = 18
VARIANT_NAMES = {0: "auto", 1: "generic", 2: "retired", 3: "256x256_w4", 4: "128x128_w4", 5: "256x128_w4",
                 6: "128x256_w4", 7: "64x128_w4", 8: "retired", 9: "skinny16", 10: "skinny32", 11: "skinny64", 12: "192x256_w4", 13: "96x128_w4", 14: "64x64_w4",
                 15: "256x256_w4_chain", 16: "skinny128", 17: "strip"}

# every symbol include/neogemm.h declares, with its prototype
_i64, _int, _vp, _sz = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t
PROTOTYPES = {
    "neogemm_bf16": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _vp, _sz, _vp]),
    "neogemm_bf16_noalloc": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "neogemm_bf16_scaled": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, ctypes.c_float,
                                   ctypes.c_float, _vp, _sz, _vp]),
    "neogemm_bf16_batched": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int,
                                    _vp, _sz, _vp]),
    "neogemm_bf16_batched_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64]),
    "neogemm_bf16_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "neogemm_bf16_variant": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _vp, _sz, _vp,
                                    _int, _int, _int]),
    "neogemm_bf16_plan": (_int, [_i64, _i64, _i64, _int, _int, _int, ctypes.POINTER(_int), ctypes.POINTER(_int)]),
    "neogemm_bf16_profile": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _int, _vp, _int, _int, _vp, _sz]),
    "neogemm_bf16_profile_bytes": (_sz, [_i64, _i64, _int]),
    "neogemm_strerror": (ctypes.c_char_p, [_int]),
    "neogemm_version": (ctypes.c_char_p, []),
}

_lib = None


def load():
    """Load libneogemm.so (built by `python setup.py build_ext --inplace` or __graft_entry__.build()).

    There is no fallback: a missing library is an error, never a slower path.
    """
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python setup.py build_ext --inplace` "
                "(hipcc --offload-arch=gfx950); there is no CPU or PyTorch fallback for the GEMM path")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


class NeoGemmError(RuntimeError):
    def __init__(self, status, what=""):
        self.status = status
        msg = load().neogemm_strerror(status).decode()
        super().__init__(f"neogemm status {status}: {msg}{(' (' + what + ')') if what else ''}")


def strerror(status):
    return load().neogemm_strerror(status).decode()


def version():
    return load().neogemm_version().decode()


def workspace_bytes(M, N, K):
    return int(load().neogemm_bf16_workspace_bytes(M, N, K))


def plan(M, N, K, b_layout=B_KN, c_layout=C_ROW, aligned=True):
    v, s = _int(0), _int(0)
    st = load().neogemm_bf16_plan(M, N, K, b_layout, c_layout, int(aligned), ctypes.byref(v), ctypes.byref(s))
    if st != OK:
        raise NeoGemmError(st)
    return v.value, s.value


def gemm_raw(A_ptr, B_ptr, C_ptr, M, N, K, lda, ldb, ldc, b_layout, c_layout, ws_ptr=0, ws_bytes=0, stream=0,
             variant=None, split_k=0, group_m=0, alpha=1.0, beta=0.0):
    """Thin call-through; returns the status code (no exception)."""
    lib = load()
    if alpha != 1.0 or beta != 0.0:
        if variant is not None:
            raise ValueError("alpha/beta go through neogemm_bf16_scaled, which chooses the kernel itself")
        return lib.neogemm_bf16_scaled(A_ptr, B_ptr, C_ptr, M, N, K, lda, ldb, ldc, b_layout, c_layout, alpha, beta,
                                       ws_ptr or None, ws_bytes, stream or None)
    if variant is None:
        return lib.neogemm_bf16(A_ptr, B_ptr, C_ptr, M, N, K, lda, ldb, ldc, b_layout, c_layout, ws_ptr or None,
                                ws_bytes, stream or None)
    return lib.neogemm_bf16_variant(A_ptr, B_ptr, C_ptr, M, N, K, lda, ldb, ldc, b_layout, c_layout,
                                    ws_ptr or None, ws_bytes, stream or None, variant, split_k, group_m)
