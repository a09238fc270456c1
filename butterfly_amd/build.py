"""Compile the native libraries in-tree for gfx950.

* ``libbutterfly_hip.so`` -- HIP kernels + C ABI (``include/butterfly_hip.h``), built with hipcc.
* ``_butterfly.so``       -- torch-library shim registering ``torch.ops.torch_butterfly.*``.
* ``_version.so``         -- ``torch_butterfly::cuda_version``.

The two shims carry no Python ABI suffix so a package initialiser can find them by bare
name next to itself (the reference does this in torch_butterfly/__init__.py:8-11).

    python -m butterfly_amd.build
"""
import os
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
ARCH = "gfx950"

LIB_HIP = os.path.join(PKG, "libbutterfly_hip.so")
LIB_OPS = os.path.join(PKG, "_butterfly.so")
LIB_VERSION = os.path.join(PKG, "_version.so")

# Packed-FP32 instructions are switched off for every device compile.
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_hip():
    _run(["hipcc", "-O3", f"--offload-arch={ARCH}", "-std=c++17", "-fPIC", "-shared"] + DEVICE_FLAGS +
         ["-o", LIB_HIP, os.path.join(CSRC, "butterfly_hip.hip")])
    return LIB_HIP


def _torch_flags():
    import torch
    from torch.utils import cpp_extension
    incs = cpp_extension.include_paths() + [sysconfig.get_paths()["include"]]
    libdir = cpp_extension.library_paths()[0]
    flags = ["-O2", "-std=c++17", "-fPIC", "-shared", "-w",
             f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
             "-DUSE_ROCM", "-D__HIP_PLATFORM_AMD__"]
    for i in incs:
        flags += ["-isystem", i]
    flags += ["-isystem", "/opt/rocm/include"]
    libs = [f"-L{libdir}", f"-Wl,-rpath,{libdir}", "-ltorch", "-ltorch_cpu", "-lc10"]
    return flags, libs


def build_ops():
    flags, libs = _torch_flags()
    _run(["g++"] + flags + [os.path.join(CSRC, "butterfly_ops.cpp"), "-o", LIB_OPS] + libs +
         ["-ltorch_hip", "-lc10_hip", f"-L{PKG}", "-lbutterfly_hip", "-Wl,-rpath,$ORIGIN"])
    return LIB_OPS


def build_version():
    flags, libs = _torch_flags()
    _run(["g++"] + flags + [os.path.join(CSRC, "version.cpp"), "-o", LIB_VERSION] + libs)
    return LIB_VERSION


def build_all():
    build_hip()
    build_ops()
    build_version()


if __name__ == "__main__":
    build_all()
    sys.exit(0)
