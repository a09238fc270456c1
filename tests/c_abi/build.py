"""Builds tests/c_abi/abi_check.out: the C ABI exercised from plain C++ (hipcc host compile,
linked against the in-tree libbutterfly_hip.so and, as the checker, oracle/liboracle.so)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(HERE, "abi_check.out")


def build():
    cmd = ["hipcc", "-O2", "-std=c++17", "--offload-arch=gfx950", os.path.join(HERE, "abi_check.cpp"),
           "-I", os.path.join(ROOT, "include"),
           "-L", os.path.join(ROOT, "butterfly_amd"), "-lbutterfly_hip",
           "-L", os.path.join(ROOT, "oracle"), "-loracle",
           "-Wl,-rpath,$ORIGIN/../../butterfly_amd", "-Wl,-rpath,$ORIGIN/../../oracle",
           "-o", OUT]
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    build()
    sys.exit(0)
