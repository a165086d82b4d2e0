"""Builds the `neoGEMM` PyTorch extension (counterpart of the reference's setup.py:4-24).

Two artefacts, both in-tree:
  gemm_amd/libneogemm.so   hand-written gfx950 HIP kernels behind a C ABI (hipcc, no torch)
  neoGEMM.*.so             pybind11/torch shim that unwraps tensors and calls that ABI

    python setup.py build_ext --inplace
"""
import os
import subprocess
import sys

from setuptools import setup
from torch.utils.cpp_extension import BuildExtension, CppExtension

ROOT = os.path.dirname(os.path.abspath(__file__))
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
LIB = os.path.join(ROOT, "gemm_amd", "libneogemm.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-DNDEBUG",
    # packed-fp32 VALU forms are kept off for every HIP file of this project
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def build_kernels():
    """hipcc -> gemm_amd/libneogemm.so (cross-compiles without a GPU)."""
    src = os.path.join(ROOT, "gemm_amd", "csrc", "neogemm.hip")
    cmd = [os.path.join(ROCM, "bin", "hipcc"), *HIPCC_FLAGS, "-I", os.path.join(ROOT, "include"), "-o", LIB, src]
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


class BuildWithKernels(BuildExtension):
    def run(self):
        build_kernels()
        super().run()


if __name__ == "__main__":
    setup(
        name="neoGEMM",
        version="0.1",
        ext_modules=[
            CppExtension(
                name="neoGEMM",
                sources=["gemm_amd/csrc/neogemm_torch.cpp"],
                include_dirs=[os.path.join(ROOT, "include"), os.path.join(ROCM, "include")],
                define_macros=[("__HIP_PLATFORM_AMD__", "1"), ("USE_ROCM", "1")],
                extra_compile_args=["-std=c++17", "-O2", "-Wno-unused-result"],
                library_dirs=[os.path.join(ROOT, "gemm_amd")],
                libraries=["neogemm", "c10_hip", "torch_hip"],
                extra_link_args=["-Wl,-rpath,$ORIGIN/gemm_amd"],
            )
        ],
        cmdclass={"build_ext": BuildWithKernels.with_options(use_ninja=False)},
    )
