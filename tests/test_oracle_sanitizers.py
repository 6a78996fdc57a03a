"""The CPU oracle under AddressSanitizer + UndefinedBehaviorSanitizer: its golden-vector and invariant suites run
once more, in a child process, against a sanitizer build of oracle/rexsc_oracle.c.  The reference's own loops read
past their buffers in places (sc_matmul.cpp:428-438, 336-337); the checker that everything else is measured against
must not.  Host code only -- nothing here touches a GPU."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_oracle_suites_pass_under_asan_and_ubsan():
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import build as oracle_build
    try:
        so, runtime = oracle_build.build_oracle_sanitized()
    except Exception as e:  # a toolchain without the sanitizer runtimes
        pytest.skip("sanitizer build not available: %s" % e)
    if not os.path.isabs(runtime) or not os.path.exists(runtime):
        pytest.skip("libasan.so not found (%r)" % runtime)
    env = dict(os.environ)
    env["REXSC_ORACLE_SO"] = so
    # the ASan runtime has to be in the process before the library is: first in LD_PRELOAD, whatever else is there
    env["LD_PRELOAD"] = runtime + (":" + env["LD_PRELOAD"] if env.get("LD_PRELOAD") else "")
    env["ASAN_OPTIONS"] = "detect_leaks=0:verify_asan_link_order=0:abort_on_error=0:exitcode=66"
    env["UBSAN_OPTIONS"] = "print_stacktrace=1:halt_on_error=1"
    env["OMP_NUM_THREADS"] = "4"
    cmd = [sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider",
           os.path.join(ROOT, "tests", "test_oracle_golden.py"), os.path.join(ROOT, "tests", "test_oracle_invariants.py")]
    out = subprocess.run(cmd, env=env, cwd=ROOT, capture_output=True, text=True, timeout=900)
    text = out.stdout + out.stderr
    assert "AddressSanitizer" not in text and "runtime error:" not in text, text[-4000:]
    assert out.returncode == 0, text[-4000:]
    assert " passed" in out.stdout
