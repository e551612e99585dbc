"""Builds csrc/libq4adamw.so for gfx950 with hipcc (cross-compiles without a GPU).

Counterpart of the reference's optim/setup.py:6-23 (a torch CUDAExtension built by
nvcc); here the product is a plain C-ABI shared library, so no torch headers and
no pybind11 are involved.

Usage:  python -m quantfour_adamw_cuda_amd.build
"""
import os
import shutil
import subprocess

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB = os.path.join(CSRC, "libq4adamw.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    # moment updates are individually rounded fp32 operations: never contract
    "-ffp-contract=off",
    # packed fp32 instructions are not to be generated on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-shared", "-fPIC",
]


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm)")


def build(verbose=False):
    """Compile unconditionally; returns the path of the library."""
    cmd = [hipcc_path()] + HIPCC_FLAGS + ["-o", LIB, os.path.join(CSRC, "q4adamw.hip")]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or proc.returncode != 0:
        print(proc.stdout)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + proc.stdout)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
