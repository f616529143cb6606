"""Host code of the engine under ThreadSanitizer and Address/UB sanitizers: a host-only build (no device
code, host backend) driven by tests/cpp/engine_stress.cpp with three threads at work (caller, fetch thread,
predictor thread).  Any sanitizer report fails the run (non-zero exit / text on stderr)."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CPP = os.path.join(HERE, "cpp")
HIPCC = "/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc") else shutil.which("hipcc")


@pytest.mark.skipif(HIPCC is None, reason="needs hipcc for the host-only build")
@pytest.mark.parametrize("kind,policy", [("tsan", "nn"), ("tsan", "lru"), ("asan", "nn"), ("asan", "fifo")])
def test_engine_stress_under_sanitizer(kind, policy):
    r = subprocess.run(["make", "-C", CPP, kind, "HIPCC=" + HIPCC], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1", ASAN_OPTIONS="detect_leaks=1", UBSAN_OPTIONS="halt_on_error=1")
    r = subprocess.run([os.path.join(CPP, "engine_stress_" + kind), "600", policy], capture_output=True, text=True,
                       env=env, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-4000:]
    assert "WARNING: ThreadSanitizer" not in r.stderr and "ERROR: AddressSanitizer" not in r.stderr and \
        "runtime error" not in r.stderr, r.stderr[-4000:]
    assert "requests 3600" in r.stdout
