"""Host-side logic without a GPU: the Python mirror of the reference's extension surface (gemm_amd) and
the built neoGEMM module reject what they must, and nothing falls back to a CPU computation."""
import pytest
import torch

import gemm_amd


def test_surface_names():
    # the reference's names (nemgemmV03.cu:396-399, v01.cu:314-317) plus C = gemm(A, B)
    for mod in (gemm_amd, __import__("neoGEMM")):
        assert callable(mod.gemm) and callable(mod.neoGemmV1) and callable(mod.neogemm)
    import neoGEMM
    assert neoGEMM.version() == gemm_amd.version()


def test_no_cpu_path():
    A = torch.zeros(8, 8, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="GPU"):
        gemm_amd.gemm(A, A)
    with pytest.raises(ValueError, match="GPU"):
        gemm_amd.neoGemmV1(A, A, A.clone())
    import neoGEMM
    with pytest.raises(RuntimeError, match="GPU"):
        neoGEMM.gemm(A, A)
    with pytest.raises(RuntimeError, match="GPU"):
        neoGEMM.neoGemmV1(A=A, B=A, C=A.clone())   # the reference's keyword names


def test_type_checks_come_first():
    with pytest.raises(TypeError):
        gemm_amd.gemm([1, 2], torch.zeros(2, 2))
    # dtype and rank are checked after the device in both wrappers; on CPU tensors the device error wins
    import neoGEMM
    with pytest.raises(RuntimeError):
        neoGEMM.gemm(torch.zeros(4, 4), torch.zeros(4, 4))


def test_missing_library_is_an_error(monkeypatch):
    from gemm_amd import _abi
    monkeypatch.setattr(_abi, "_lib", None)
    monkeypatch.setattr(_abi, "LIB_PATH", "/nonexistent/libneogemm.so")
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _abi.load()


def test_error_class_carries_status():
    e = gemm_amd.NeoGemmError(-3, "shape")
    assert e.status == -3 and "variant" in str(e)
