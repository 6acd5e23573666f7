"""The C ABI's host code (argument validation, error text, workspace queries) under AddressSanitizer and UBSan.

`make -C trl_amd/csrc asan` builds `trl_amd/lib/libtrlk_asan.so`: the same device code objects, the host code
instrumented.  The checks of tests/test_abi.py and tests/test_host_logic.py run against it in a child process, with
the sanitizer runtime loaded first (an instrumented shared library inside an uninstrumented python needs that) and
every finding fatal.  No GPU is touched: each call in those files is rejected, or answered, on the host."""
import os
import subprocess
import sys

import pytest

from conftest import ROOT

ASAN_LIB = os.path.join(ROOT, "trl_amd", "lib", "libtrlk_asan.so")
CLANG = "/opt/rocm/lib/llvm/bin/clang++"


def _runtime():
    try:
        path = subprocess.run([CLANG, "-print-file-name=libclang_rt.asan-x86_64.so"], check=True, capture_output=True,
                              text=True).stdout.strip()
    except (OSError, subprocess.CalledProcessError):
        return None
    return path if os.path.isabs(path) and os.path.exists(path) else None


def test_host_code_is_clean_under_asan_and_ubsan():
    if not os.path.exists(ASAN_LIB):
        pytest.skip("trl_amd/lib/libtrlk_asan.so is not built (make -C trl_amd/csrc asan)")
    runtime = _runtime()
    if runtime is None:
        pytest.skip("the sanitizer runtime of the ROCm clang is not installed")
    env = dict(os.environ)
    env["LD_PRELOAD"] = " ".join(p for p in (runtime, env.get("LD_PRELOAD", "")) if p)
    env["TRLK_LIBRARY_PATH"] = ASAN_LIB
    # python itself and torch are not instrumented and never free what they hold at exit: leak reports are theirs
    env["ASAN_OPTIONS"] = "detect_leaks=0:abort_on_error=0:exitcode=99"
    env["UBSAN_OPTIONS"] = "halt_on_error=1:print_stacktrace=1:exitcode=98"
    run = subprocess.run([sys.executable, "-m", "pytest", "-q", "-x", "-p", "no:cacheprovider",
                          os.path.join(ROOT, "tests", "test_abi.py"), os.path.join(ROOT, "tests", "test_host_logic.py")],
                         env=env, cwd=ROOT, capture_output=True, text=True, timeout=600)
    report = run.stdout[-3000:] + run.stderr[-3000:]
    assert run.returncode == 0, report
    assert "AddressSanitizer" not in report and "runtime error:" not in report, report
    assert " passed" in run.stdout
