"""Build recipe for the test oracle (TEST INFRASTRUCTURE ONLY).

* ``oracle/liboracle.so``        -- gcc build of ``butterfly_oracle.c`` (the repo's own
  CPU restatement).
* ``oracle/_ref/_butterfly_ref.so`` -- the reference's own ``csrc/butterfly.cpp`` +
  ``csrc/cpu/butterfly_cpu.cpp`` compiled where they lie with plain ``g++ -O2``
  (setuptools' default optimisation level) against the installed libtorch.  Built
  only when the reference tree is present; nothing is copied out of it.

Run ``python oracle/build.py`` (or call :func:`build_all`).
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE_ROOT = os.environ.get("BUTTERFLY_REFERENCE_ROOT", "/root/reference")
ORACLE_SO = os.path.join(HERE, "liboracle.so")
REF_DIR = os.path.join(HERE, "_ref")
REF_SO = os.path.join(REF_DIR, "_butterfly_ref.so")


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_oracle():
    _run(["gcc", "-O2", "-std=c99", "-ffp-contract=off", "-fPIC", "-shared",
          "-o", ORACLE_SO, os.path.join(HERE, "butterfly_oracle.c")])
    return ORACLE_SO


def reference_available():
    return os.path.isfile(os.path.join(REFERENCE_ROOT, "csrc", "cpu", "butterfly_cpu.cpp"))


def build_reference():
    """Compile the reference CPU op library from its own sources (no WITH_CUDA)."""
    if not reference_available():
        return None
    import torch
    from torch.utils import cpp_extension
    os.makedirs(REF_DIR, exist_ok=True)
    csrc = os.path.join(REFERENCE_ROOT, "csrc")
    incs = cpp_extension.include_paths() + [sysconfig.get_paths()["include"], csrc]
    libdir = cpp_extension.library_paths()[0]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-w",
           f"-D_GLIBCXX_USE_CXX11_ABI={abi}"]
    for i in incs:
        cmd += ["-isystem", i]
    cmd += [os.path.join(csrc, "butterfly.cpp"), os.path.join(csrc, "cpu", "butterfly_cpu.cpp"),
            "-o", REF_SO, f"-L{libdir}", f"-Wl,-rpath,{libdir}",
            "-ltorch", "-ltorch_cpu", "-lc10"]
    _run(cmd)
    return REF_SO


def build_all():
    build_oracle()
    build_reference()


if __name__ == "__main__":
    build_all()
    sys.exit(0)
