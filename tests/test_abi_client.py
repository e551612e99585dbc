"""The C ABI used from plain C: tests/native/abi_client.c includes include/q4adamw.h as C11,
links libq4adamw.so, the HIP runtime and the C oracle (as the checker), and runs steps on
memory from hipMalloc on the null stream -- what a non-Python host would do in place of the
reference's extension glue (optim/cuda_fused_interface.cc:19-64)."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def _compile(tmp_path):
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    from quantfour_adamw_cuda_amd import _lib
    from oracle import q4_oracle
    _lib.load()                       # raises if the library has not been built
    oracle_so = q4_oracle.build()
    exe = str(tmp_path / "abi_client")
    subprocess.check_call([
        gcc, "-std=c11", "-O1", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__",
        "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROCM, "include"),
        os.path.join(ROOT, "tests", "native", "abi_client.c"), _lib.LIB_PATH, oracle_so,
        "-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-lm",
        "-Wl,-rpath," + os.path.join(ROCM, "lib"), "-o", exe])
    return exe


def test_header_is_c11_and_client_links(tmp_path):
    """include/q4adamw.h compiles as C (no C++ in the ABI) and every symbol the client uses
    resolves against the built library"""
    assert os.path.exists(_compile(tmp_path))


@pytest.mark.gpu
def test_c_client_against_the_oracle(tmp_path):
    exe = _compile(tmp_path)
    out = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert out.returncode == 0, out.stdout
    assert out.stdout.strip().endswith("abi_client: all checks passed"), out.stdout
