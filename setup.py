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
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-DNDEBUG",
    # packed-fp32 VALU forms are kept off for every HIP file of this project
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
KERNEL_PARTS = 9  # NEOGEMM_PARTS in gemm_amd/csrc/neogemm.hip


def build_kernels():
    """hipcc -> gemm_amd/libneogemm.so (cross-compiles without a GPU).

    The one source file is compiled KERNEL_PARTS times in parallel, each time with a different share of the tile
    kernel's instances (-DNEOGEMM_PART=k), and the objects are linked into the library.
    """
    from concurrent.futures import ThreadPoolExecutor

    hipcc = os.path.join(ROCM, "bin", "hipcc")
    src = os.path.join(ROOT, "gemm_amd", "csrc", "neogemm.hip")
    objdir = os.path.join(ROOT, "build", "neogemm_parts")
    os.makedirs(objdir, exist_ok=True)

    def compile_part(k):
        obj = os.path.join(objdir, f"neogemm_part{k}.o")
        cmd = [hipcc, *HIPCC_FLAGS, f"-DNEOGEMM_PART={k}", "-I", os.path.join(ROOT, "include"), "-c", "-o", obj, src]
        print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
        return obj

    jobs = max(1, min(KERNEL_PARTS, int(os.environ.get("MAX_JOBS", os.cpu_count() or 1))))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_part, range(KERNEL_PARTS)))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
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
                depends=[os.path.join("include", "neogemm.h")],   # the shim is rebuilt when the C ABI changes
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
