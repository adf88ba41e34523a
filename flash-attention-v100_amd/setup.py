"""Build script: hipcc for the gfx950 kernels, g++ for the thin PyTorch extension.

Takes the place of the reference's setup.py:116-172 (one CUDAExtension built by
nvcc for sm_70 with a CUTLASS include path, installed with `python setup.py
install`).  Here there are two artefacts:

  flash_attn_v100/lib/libfused_mha.so   HIP kernels + the C ABI of include/fused_mha.h
                                        (hipcc --offload-arch=gfx950; no third-party headers)
  flash_attn_v100_cuda.so               PyTorch extension (host C++ only) that validates,
                                        allocates and calls the C ABI; it finds the kernel
                                        library through the rpath $ORIGIN/flash_attn_v100/lib

Usage, as with the reference (README.md:21-23):
    python setup.py install                  (or: pip wheel . --no-build-isolation)
puts both files into the installed distribution, next to the flash_attn_v100
package;
    python setup.py build_ext --inplace
builds them in-tree, next to this file.  An install or wheel build reuses in-tree
artefacts that are newer than every source and compiles otherwise
(FLASH_ATTN_FORCE_BUILD=1 always compiles).
The functions build_kernels() / build_extension() can also be imported.
"""
import os
import shutil
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
INCLUDE = os.path.join(ROOT, "include")
CSRC = os.path.join(HERE, "csrc")
LIB_SUBDIR = os.path.join("flash_attn_v100", "lib")
LIB_DIR = os.path.join(HERE, LIB_SUBDIR)
KERNEL_LIB = os.path.join(LIB_DIR, "libfused_mha.so")
EXT_LIB = os.path.join(HERE, "flash_attn_v100_cuda.so")
ROCM_HOME = os.environ.get("ROCM_HOME", "/opt/rocm")
KERNEL_SOURCES = [os.path.join(CSRC, "fused_mha_kernel.hip"), os.path.join(CSRC, "block_map.h"),
                  os.path.join(INCLUDE, "fused_mha.h")]
EXT_SOURCES = [os.path.join(CSRC, "fused_mha_api.cpp"), os.path.join(INCLUDE, "fused_mha.h")]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed-fp32 VALU ops are kept off for every HIP translation unit
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _run(cmd):
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_kernels(extra_flags=(), out=KERNEL_LIB):
    os.makedirs(os.path.dirname(out), exist_ok=True)
    hipcc = os.path.join(ROCM_HOME, "bin", "hipcc")
    _run([hipcc, *HIPCC_FLAGS, *extra_flags, "-I", INCLUDE, "-I", CSRC, "-o", out,
          os.path.join(CSRC, "fused_mha_kernel.hip")])
    return out


def build_extension(out=EXT_LIB):
    """The extension links against libfused_mha.so in <dir of out>/flash_attn_v100/lib."""
    import torch
    from torch.utils import cpp_extension

    lib_dir = os.path.join(os.path.dirname(out), LIB_SUBDIR)
    if not os.path.exists(os.path.join(lib_dir, "libfused_mha.so")):
        build_kernels(out=os.path.join(lib_dir, "libfused_mha.so"))
    includes = cpp_extension.include_paths() + [INCLUDE, os.path.join(ROCM_HOME, "include"),
                                                sysconfig.get_paths()["include"]]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wno-deprecated-declarations",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=flash_attn_v100_cuda",
           "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    for inc in includes:
        cmd += ["-isystem", inc]
    cmd += [os.path.join(CSRC, "fused_mha_api.cpp"), "-o", out,
            "-L", torch_lib, "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_python",
            "-L", lib_dir, "-lfused_mha", "-Wl,-rpath,$ORIGIN/" + LIB_SUBDIR, "-Wl,--no-as-needed"]
    _run(cmd)
    return out


def build_all():
    build_kernels()
    build_extension()


def _fresh(artefact, sources):
    return (os.path.exists(artefact) and os.environ.get("FLASH_ATTN_FORCE_BUILD") != "1" and
            all(os.path.getmtime(artefact) >= os.path.getmtime(src) for src in sources))


if __name__ == "__main__":
    from setuptools import Extension, setup
    from setuptools.command.build_ext import build_ext as _build_ext

    class build_ext(_build_ext):
        """Builds both shared objects with the commands above instead of distutils' compiler,
        into the build directory (install, bdist_wheel) or in-tree (--inplace)."""

        def run(self):
            if self.inplace:
                build_all()
            else:
                super().run()

        def get_ext_filename(self, fullname):
            return fullname + ".so"  # the plain name the reference's module has (setup.py:118)

        def build_extension(self, ext):
            target = os.path.abspath(self.get_ext_fullpath(ext.name))
            kernel_target = os.path.join(os.path.dirname(target), LIB_SUBDIR, "libfused_mha.so")
            os.makedirs(os.path.dirname(kernel_target), exist_ok=True)
            for built, sources, dest, compile_it in (
                    (KERNEL_LIB, KERNEL_SOURCES, kernel_target, lambda: build_kernels(out=kernel_target)),
                    (EXT_LIB, EXT_SOURCES, target, lambda: build_extension(out=target))):
                if _fresh(built, sources):
                    print("copying", built, "->", dest, flush=True)
                    shutil.copy2(built, dest)
                else:
                    compile_it()

    setup(
        name="flash_attn_v100",
        version="0.0.1",
        description="FlashAttention-2 forward/backward for MI355X (gfx950) behind the flash_attn_v100 API",
        packages=["flash_attn_v100"],
        package_data={"flash_attn_v100": ["lib/*.so"]},
        ext_modules=[Extension("flash_attn_v100_cuda", sources=[])],
        cmdclass={"build_ext": build_ext},
        python_requires=">=3.8",
        zip_safe=False,
    )
