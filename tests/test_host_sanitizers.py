"""The library's host-side code (data layer, tile order, LDS swizzles) and the CPU checker under the address
and undefined-behaviour sanitizers: `make -C oracle asan` builds oracle/_asan/host_check, which exercises them
and exits 0 only if every check held and the sanitizers stayed silent.  CPU only."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLANG = "/opt/rocm/llvm/bin/clang++"


@pytest.mark.skipif(not os.path.exists(CLANG) or shutil.which("make") is None, reason="clang with sanitizer runtimes not installed")
def test_host_code_is_clean_under_address_and_ub_sanitizers():
    build = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "asan"], capture_output=True, text=True, timeout=600)
    assert build.returncode == 0, build.stdout[-2000:] + build.stderr[-2000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    run = subprocess.run([os.path.join(ROOT, "oracle", "_asan", "host_check"),
                          os.path.join(ROOT, "tests", "golden", "sample_points.csv")],
                         capture_output=True, text=True, timeout=600, env=env)
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-4000:]
    assert "all checks held" in run.stdout
    assert "runtime error" not in run.stderr and "AddressSanitizer" not in run.stderr
