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
import tempfile

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
    "-fPIC",
]

# libq4adamw.so: the C ABI with its launchers and small kernels, and the step kernels'
# instantiations in translation units of their own, compiled side by side
STEP_SOURCES = ["q4adamw.hip", "q4adamw_pick_fused.hip", "q4adamw_pick_rank1_rows.hip",
                "q4adamw_pick_rank1_wide.hip", "q4adamw_pick_rank1_narrow.hip", "q4adamw_pick_rank1_any.hip"]
PROBE_SOURCES = ["q4stream_probe.hip"]


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm)")


def _checked(proc, what, verbose):
    # anything besides the host pass's note about the device-only feature is a real diagnostic
    noise = [ln for ln in proc.stdout.splitlines() if ln.strip() and ln.strip() != HOST_PASS_NOTE]
    if verbose or proc.returncode != 0:
        print(proc.stdout)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {what}:\n" + proc.stdout)
    if noise:
        raise RuntimeError(f"hipcc printed diagnostics for {what}; the build is kept warning-free:\n"
                           + "\n".join(noise))


def compile_library(out, sources, flags=None, verbose=False, check_output=True):
    """Compiles every source to an object file (all at once, one hipcc each) and links them
    into the shared library `out`.  flags: hipcc options in place of HIPCC_FLAGS."""
    flags = HIPCC_FLAGS if flags is None else flags
    hipcc = hipcc_path()
    with tempfile.TemporaryDirectory(prefix="q4adamw_build_") as tmp:
        jobs = []
        for src in sources:
            obj = os.path.join(tmp, os.path.splitext(src)[0] + ".o")
            cmd = [hipcc] + flags + ["-c", "-o", obj, os.path.join(CSRC, src)]
            jobs.append((src, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs = []
        for src, obj, job in jobs:
            job.stdout_text = job.communicate()[0]
        for src, obj, job in jobs:
            proc = subprocess.CompletedProcess(job.args, job.returncode, job.stdout_text)
            if check_output:
                _checked(proc, src, verbose)
            elif proc.returncode != 0:
                raise RuntimeError(f"hipcc failed for {src}:\n" + proc.stdout)
            objs.append(obj)
        link = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs,
                              stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if check_output:
            _checked(link, os.path.basename(out), verbose)
        elif link.returncode != 0:
            raise RuntimeError("link failed:\n" + link.stdout)
    return out


def build(verbose=False):
    """Compile unconditionally; returns the path of the step library."""
    compile_library(LIB, STEP_SOURCES, verbose=verbose)
    compile_library(PROBE_LIB, PROBE_SOURCES, verbose=verbose)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
