"""The host runtime (everything above the HIP FFI layer) under AddressSanitizer + UBSan and under
ThreadSanitizer: tests/hostshim/sanitize_driver.cpp drives the C ABI from four threads against
the host-memory stand-ins.  GPU code cannot run under a sanitizer on this hardware pool; host
code can, natively (no preloading into the Python process)."""
import os
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hostshim")


@pytest.mark.parametrize("kind,env", [("asan", {"ASAN_OPTIONS": "detect_leaks=1:abort_on_error=0",
                                                "UBSAN_OPTIONS": "halt_on_error=1:print_stacktrace=1"}),
                                      ("tsan", {"TSAN_OPTIONS": "halt_on_error=0"})])
def test_host_runtime_under_sanitizer(kind, env):
    exe = "sanitize_" + kind
    r = subprocess.run(["make", "-C", HERE, "-j8", exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    r = subprocess.run([os.path.join(HERE, exe)], capture_output=True, text=True, env=dict(os.environ, **env), timeout=600)
    out = r.stdout + r.stderr
    if "unexpected memory mapping" in out or "Shadow memory range interleaves" in out:
        pytest.skip("the sanitizer runtime cannot map its shadow memory in this environment")
    assert "threads ok" in out, out[-3000:]
    for bad in ("ERROR: AddressSanitizer", "ERROR: LeakSanitizer", "runtime error:", "WARNING: ThreadSanitizer"):
        assert bad not in out, out[-3000:]
    assert r.returncode == 0, out[-3000:]
