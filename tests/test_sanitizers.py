"""Host code under AddressSanitizer and UndefinedBehaviorSanitizer (no GPU involved): a
build of libq4adamw.so's sources with sanitized host code and the C oracle, driven by tests/native/host_sanitize.c
through every refusal the C ABI makes before a launch and through the oracle on ragged sizes."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SAN = ["-fsanitize=address", "-fsanitize=undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer", "-g", "-O1"]


def test_host_code_under_sanitizers(tmp_path):
    from quantfour_adamw_cuda_amd import build as q4build
    try:
        hipcc = q4build.hipcc_path()
    except RuntimeError:
        pytest.skip("no hipcc")
    clang = shutil.which("amdclang") or os.path.join(os.path.dirname(os.path.realpath(hipcc)), "amdclang")
    if not os.path.exists(clang):
        pytest.skip("no amdclang")
    lib = str(tmp_path / "libq4adamw_hostsan.so")
    # sanitizers on the host side only (each option after -Xarch_host); the device code is
    # compiled as usual and not called by anything here
    host_san = [x for opt in SAN[:3] for x in ("-Xarch_host", opt)]
    q4build.compile_library(lib, q4build.STEP_SOURCES,
                            flags=["--offload-arch=gfx950", "-O1", "-std=c++17", "-ffp-contract=off",
                                   "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                                   *host_san, "-fPIC"], check_output=False)
    exe = str(tmp_path / "host_sanitize")
    subprocess.check_call([clang, "-std=c11", *SAN, "-I" + os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "native", "host_sanitize.c"),
                           os.path.join(ROOT, "oracle", "q4_oracle.c"), lib, "-lm",
                           "-Wl,-rpath," + str(tmp_path), "-o", exe])
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    out = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300, env=env)
    assert out.returncode == 0 and out.stdout.strip().endswith("host_sanitize: ok"), out.stdout[-4000:]
    assert "runtime error" not in out.stdout and "Sanitizer" not in out.stdout, out.stdout[-4000:]
