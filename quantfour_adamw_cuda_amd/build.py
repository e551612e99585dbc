"""Builds csrc/libq4adamw.so (the step) and csrc/libq4probe.so (the bench's memory-system
probes) for gfx950 with hipcc (cross-compiles without a GPU).

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
PROBE_LIB = os.path.join(CSRC, "libq4probe.so")
HOST_PASS_NOTE = "'-packed-fp32-ops' is not a recognized feature for this target (ignoring feature)"

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    # moment updates are individually rounded fp32 operations: never contract
    "-ffp-contract=off",
    # No packed fp32 instructions (v_pk_fma_f32 and its like) in the device code.  The feature
    # belongs to the gfx950 target: the device pass obeys it (tests/test_abi_and_tables.py
    # compiles a kernel both ways and counts them), and hipcc's host pass, which is handed the
    # same option, says that x86 does not know the feature and ignores it.  That message is
    # the only output of a clean build.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-shared", "-fPIC",
]


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm)")


def _compile(out, source, verbose):
    cmd = [hipcc_path()] + HIPCC_FLAGS + ["-o", out, os.path.join(CSRC, source)]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # anything besides the host pass's note about the device-only feature is a real diagnostic
    noise = [ln for ln in proc.stdout.splitlines() if ln.strip() and ln.strip() != HOST_PASS_NOTE]
    if verbose or proc.returncode != 0:
        print(proc.stdout)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + proc.stdout)
    if noise:
        raise RuntimeError(f"hipcc printed diagnostics for {source}; the build is kept warning-free:\n"
                           + "\n".join(noise))
    return out


def build(verbose=False):
    """Compile unconditionally; returns the path of the step library."""
    _compile(LIB, "q4adamw.hip", verbose)
    _compile(PROBE_LIB, "q4stream_probe.hip", verbose)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
