"""The argument validation of every entry point (tests/test_abi.py: fake pointers, bad shapes, nothing launched) run
once more against a build of the library whose host code carries AddressSanitizer and UndefinedBehaviorSanitizer.
Runs without a GPU; the device code is not instrumented."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_validation_layer_under_address_and_ub_sanitizers():
    from sla_amd import build
    try:
        lib = build.build_sanitized()
        runtime = build.asan_runtime()
    except (RuntimeError, OSError) as e:          # no hipcc / no sanitizer runtime on this machine
        pytest.skip(f"sanitized build unavailable: {e}")
    env = dict(os.environ)
    env["SLA_HIP_LIB"] = lib
    env["LD_PRELOAD"] = ":".join(x for x in (runtime, env.get("LD_PRELOAD", "")) if x)
    # the interpreter itself is not instrumented: no leak report at its exit, no complaint about the preload order
    env["ASAN_OPTIONS"] = "detect_leaks=0:verify_asan_link_order=0:abort_on_error=1"
    env["UBSAN_OPTIONS"] = "halt_on_error=1:print_stacktrace=1"
    res = subprocess.run([sys.executable, "-m", "pytest", os.path.join(ROOT, "tests", "test_abi.py"), "-x", "-q",
                          "-p", "no:cacheprovider"], cwd=ROOT, env=env, capture_output=True, text=True, timeout=900)
    tail = (res.stdout + res.stderr)[-3000:]
    assert res.returncode == 0, tail
    assert "AddressSanitizer" not in tail and "runtime error:" not in tail, tail
