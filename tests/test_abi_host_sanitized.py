"""The boundary's host code under AddressSanitizer and UndefinedBehaviorSanitizer: builds the library's host side with
both (`python -m pypto_amd.build --sanitize`) and runs tests/test_abi_host.py against it in a child
process.  CPU only; sanitizers are for host code here, never for the GPU side."""
import os
import subprocess
import sys

import pytest

from pypto_amd import build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_abi_host_tests_pass_under_asan_and_ubsan():
    if os.environ.get("LD_PRELOAD") or os.path.exists("/etc/ld.so.preload"):
        pytest.skip("another library is preloaded here: the sanitizer runtime has to come first in the list")
    lib = build.build_sanitized()
    env = dict(os.environ, PYPTO_AMD_LIBRARY=lib, LD_PRELOAD=build.sanitizer_runtime(),
               ASAN_OPTIONS="detect_leaks=0:halt_on_error=1", UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    res = subprocess.run([sys.executable, "-m", "pytest", os.path.join(ROOT, "tests", "test_abi_host.py"), "-x", "-q",
                          "-p", "no:cacheprovider"], cwd=ROOT, env=env, capture_output=True, text=True, timeout=600)
    out = res.stdout + res.stderr
    assert "ERROR: AddressSanitizer" not in out and "runtime error:" not in out, out[-4000:]
    assert res.returncode == 0, out[-4000:]
    assert " passed" in out
