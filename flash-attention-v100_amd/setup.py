"""Build script: hipcc for the gfx950 kernels, g++ for the thin PyTorch extension.

Takes the place of the reference's setup.py:116-149 (one CUDAExtension built by
nvcc for sm_70 with a CUTLASS include path).  Here there are two artefacts,
both placed in-tree next to this file:

  lib/libfused_mha.so        HIP kernels + the C ABI of include/fused_mha.h
                             (hipcc --offload-arch=gfx950; no third-party headers)
  flash_attn_v100_cuda.so    PyTorch extension (host C++ only) that validates,
                             allocates and calls the C ABI

Usage:  python setup.py build_ext --inplace      (or: python setup.py build_ext)
The functions build_kernels() / build_extension() can also be imported.
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
INCLUDE = os.path.join(ROOT, "include")
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
KERNEL_LIB = os.path.join(LIB_DIR, "libfused_mha.so")
EXT_LIB = os.path.join(HERE, "flash_attn_v100_cuda.so")
ROCM_HOME = os.environ.get("ROCM_HOME", "/opt/rocm")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed-fp32 VALU ops are kept off for every HIP translation unit
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _run(cmd):
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_kernels(extra_flags=()):
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = os.path.join(ROCM_HOME, "bin", "hipcc")
    _run([hipcc, *HIPCC_FLAGS, *extra_flags, "-I", INCLUDE, "-o", KERNEL_LIB,
          os.path.join(CSRC, "fused_mha_kernel.hip")])
    return KERNEL_LIB


def build_extension():
    import torch
    from torch.utils import cpp_extension

    if not os.path.exists(KERNEL_LIB):
        build_kernels()
    includes = cpp_extension.include_paths() + [INCLUDE, os.path.join(ROCM_HOME, "include"),
                                                sysconfig.get_paths()["include"]]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wno-deprecated-declarations",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=flash_attn_v100_cuda",
           "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    for inc in includes:
        cmd += ["-isystem", inc]
    cmd += [os.path.join(CSRC, "fused_mha_api.cpp"), "-o", EXT_LIB,
            "-L", torch_lib, "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_python",
            "-L", LIB_DIR, "-lfused_mha", "-Wl,-rpath,$ORIGIN/lib", "-Wl,--no-as-needed"]
    _run(cmd)
    return EXT_LIB


def build_all():
    build_kernels()
    build_extension()


if __name__ == "__main__":
    from setuptools import setup, Command

    class build_ext(Command):
        description = "build lib/libfused_mha.so (hipcc, gfx950) and flash_attn_v100_cuda.so in-tree"
        user_options = [("inplace", "i", "accepted for compatibility; the build is always in-tree")]

        def initialize_options(self):
            self.inplace = 1

        def finalize_options(self):
            pass

        def run(self):
            build_all()

    setup(
        name="flash_attn_v100",
        version="0.0.1",
        description="FlashAttention-2 forward/backward for MI355X (gfx950) behind the flash_attn_v100 API",
        packages=["flash_attn_v100"],
        cmdclass={"build_ext": build_ext},
        python_requires=">=3.8",
    )
