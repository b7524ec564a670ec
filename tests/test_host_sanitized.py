"""The host library (page bookkeeping, batch forming) under the address and undefined-behaviour sanitizers: the
cache manager's and the scheduler's tests, random request orders included, run in a child process against a
sanitized build (MLR_HOST_SANITIZE=1).  The reference runs its host tests the same way
(.github/workflows/ci.yml:60-71).  By hand:

    MLR_HOST_SANITIZE=1 LD_PRELOAD=$(gcc -print-file-name=libasan.so) ASAN_OPTIONS=detect_leaks=0 \\
        python -m pytest tests/test_cache_manager.py tests/test_scheduler.py -q -m "not gpu"
"""
import os
import shutil
import subprocess
import sys

import pytest

from conftest import ROOT


def test_cache_manager_and_scheduler_tests_pass_under_the_sanitizers():
    gcc = shutil.which("gcc") or shutil.which("g++")
    if gcc is None:
        pytest.skip("no gcc to ask for the sanitizer's runtime")
    runtime = subprocess.run([gcc, "-print-file-name=libasan.so"], capture_output=True, text=True).stdout.strip()
    if not os.path.isabs(runtime) or not os.path.exists(runtime):
        pytest.skip("the address sanitizer's runtime is not installed")
    env = dict(os.environ, MLR_HOST_SANITIZE="1", ASAN_OPTIONS="detect_leaks=0:abort_on_error=0:verify_asan_link_order=0",
               UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    env["LD_PRELOAD"] = ":".join(p for p in (runtime, os.environ.get("LD_PRELOAD", "")) if p)
    check = ("from mini_llm_runtime_amd.kernels import build; lib = build.load('host'); "
             "assert lib._mlr_path.endswith('libmlr_host_sanitized.so'), lib._mlr_path; print('sanitized library loaded')")
    done = subprocess.run([sys.executable, "-c", check], cwd=ROOT, env=env, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0 and "sanitized library loaded" in done.stdout, done.stdout + done.stderr
    done = subprocess.run([sys.executable, "-m", "pytest", "tests/test_cache_manager.py", "tests/test_scheduler.py", "-q",
                           "-m", "not gpu", "-p", "no:cacheprovider"], cwd=ROOT, env=env, capture_output=True, text=True,
                          timeout=900)
    tail = (done.stdout + done.stderr)[-3000:]
    assert done.returncode == 0, tail
    assert "passed" in done.stdout and "ERROR: AddressSanitizer" not in tail and "runtime error" not in tail, tail
