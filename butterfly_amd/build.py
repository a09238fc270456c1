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


# Kernels whose row pipelines wait for their LDS-direct row fetches with hand-counted
# `s_waitcnt vmcnt(N)`: N is right only while the compiler adds no memory operation of its own
# between request and wait, i.e. while nothing spills to scratch memory.  (Scalar registers that the
# compiler parks in the lanes of a vector register -- "SGPRs Spill" with a scratch size of 0 -- move
# no memory and are allowed: the forward variants compiled for eight wavefronts per SIMD have a few.)
GATED_KERNELS = ("fast_fw_kernel", "fast_bw_kernel", "wide_fw_kernel", "fast4_fw_kernel", "fast4_bw_kernel",
                 "fast4g_fw_kernel", "fast4g_bw_kernel")
RESOURCES = os.path.join(PKG, "kernel_resources.txt")


def parse_kernel_resources(text):
    """{mangled kernel name: {field: int}} from -Rpass-analysis=kernel-resource-usage remarks."""
    import re
    kernels, cur = {}, None
    for line in text.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            cur = kernels.setdefault(m.group(1), {})
            continue
        m = re.search(r"remark:\s+([A-Za-z ]+?)(?: \[[^\]]*\])?: (\d+)", line)
        if m and cur is not None:
            cur[m.group(1).strip()] = int(m.group(2))
    return kernels


def check_kernel_resources(path=RESOURCES):
    """Names of gated kernels that use scratch memory or spill registers (must be empty), and
    the number of gated kernels seen."""
    with open(path) as f:
        kernels = parse_kernel_resources(f.read())
    gated = {k: v for k, v in kernels.items() if any(g in k for g in GATED_KERNELS)}
    bad = [k for k, v in gated.items()
           if v.get("ScratchSize", 1) != 0 or v.get("VGPRs Spill", 1) != 0 or "SGPRs Spill" not in v]
    return bad, len(gated)


def build_hip():
    cmd = (["hipcc", "-O3", f"--offload-arch={ARCH}", "-std=c++17", "-fPIC", "-shared"] + DEVICE_FLAGS +
           ["-Rpass-analysis=kernel-resource-usage", "-o", LIB_HIP, os.path.join(CSRC, "butterfly_hip.hip")])
    print("+", " ".join(cmd), flush=True)
    r = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
    remarks = [l for l in r.stderr.splitlines() if "kernel-resource-usage" in l]
    other = [l for l in r.stderr.splitlines() if "kernel-resource-usage" not in l]
    if other:
        print("\n".join(other), file=sys.stderr, flush=True)
    if r.returncode != 0:
        raise subprocess.CalledProcessError(r.returncode, cmd)
    with open(RESOURCES, "w") as f:
        f.write("\n".join(remarks) + "\n")
    bad, seen = check_kernel_resources()
    if seen == 0:
        raise RuntimeError("no resource-usage remarks for the register-resident kernels: cannot check for spills")
    if bad:
        raise RuntimeError("kernels with hand-counted memory waits use scratch memory or spill: " + ", ".join(bad))
    print(f"{seen} register-resident kernels: no scratch memory, no vector-register spills", flush=True)
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
