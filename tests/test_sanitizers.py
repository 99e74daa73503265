"""Host code under AddressSanitizer + UndefinedBehaviorSanitizer (CPU only, no GPU sanitizer).

The reference has no tooling of this kind and an unguarded race on its K/V staging buffers
(csrc/ring_attention.cu:611-619 with the barrier commented out at :457-459).  Here the host layer
of the library -- parameter validation, the schedule and table construction, plan lifetime, the
data generator -- is built with `hipcc --offload-host-only -fsanitize=address,undefined`, the
oracle with the same clang, and the CPU tests that exercise them run once more against those
builds in a child python with the sanitizer runtime preloaded."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpu_tests_pass_under_asan_and_ubsan(tmp_path):
    from oracle import build as oracle_build
    from ringattention_amd import _build
    try:
        clang, runtime = _build.sanitizer_runtime()
    except RuntimeError as e:
        pytest.skip(str(e))
    lib = _build.build_sanitized_library(str(tmp_path))
    ora = oracle_build.build_oracle_sanitized(clang, str(tmp_path))
    env = dict(os.environ)
    env["RINGATTN_LIB"] = lib
    env["ORACLE_LIB"] = ora
    # the sanitizer runtime must come first in the process; whatever is preloaded already stays
    env["LD_PRELOAD"] = runtime + (":" + env["LD_PRELOAD"] if env.get("LD_PRELOAD") else "")
    # python itself and its extension modules leak by design and are not instrumented
    env["ASAN_OPTIONS"] = "detect_leaks=0:detect_odr_violation=0:abort_on_error=1:handle_segv=0"
    env["UBSAN_OPTIONS"] = "halt_on_error=1:print_stacktrace=1"
    tests = [os.path.join(ROOT, "tests", t) for t in ("test_abi.py", "test_datagen.py", "test_oracle.py")]
    res = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-m", "not gpu", "-p", "no:cacheprovider"] + tests,
                         capture_output=True, text=True, env=env, cwd=ROOT, timeout=900)
    tail = (res.stdout + res.stderr)[-4000:]
    assert res.returncode == 0, tail
    assert "passed" in res.stdout and "ERROR: AddressSanitizer" not in tail and "runtime error:" not in tail, tail
