"""Build libngraph_hip.so (the gfx950 kernels + C ABI) in-tree with hipcc.

Usage: ``python build_ext.py`` or ``build_all()`` from Python.  hipcc
cross-compiles for gfx950 without a GPU present.  The library lands in
``ngraph_hip/lib/`` next to the ctypes loader that opens it.
"""
from __future__ import print_function
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB_DIR = os.path.join(HERE, "ngraph_hip", "lib")
LIB_PATH = os.path.join(LIB_DIR, "libngraph_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed-fp32 instruction forms are kept out of every kernel
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # a*b+c must round twice, as the NumPy statements of the CPU transformer do
    "-ffp-contract=off",
    "-fno-gpu-rdc", "-Wno-unused-command-line-argument",
]


def find_hipcc():
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        raise RuntimeError("hipcc not found; libngraph_hip.so cannot be built")
    return hipcc


def build_all(verbose=True):
    """Compile every HIP source into libngraph_hip.so; returns its path."""
    if not os.path.isdir(LIB_DIR):
        os.makedirs(LIB_DIR)
    cmd = [find_hipcc()] + HIPCC_FLAGS + os.environ.get("NGH_EXTRA_HIPCC_FLAGS", "").split() + [
        "-I", INCLUDE, "-I", CSRC,
        os.path.join(CSRC, "ngraph_hip.hip"),
        "-o", LIB_PATH + ".tmp",
    ]
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, universal_newlines=True)
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops" not in l and l.strip())
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + proc.stdout)
    if verbose and out:
        print(out)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_all(verbose="-q" not in sys.argv))
