"""The host runtime (cache manager and scheduler) under the address and undefined-behaviour
sanitizers: its self-test program, built with LYAPUNOV_AMD_SANITIZE=1, drives both with random
requests, windows, pools small enough to preempt, aborts and end-of-sequence tokens, and checks the
manager's invariants after every step."""
import os
import subprocess
import sys

from conftest import ROOT


def test_random_requests_through_the_sanitized_runtime(tmp_path):
    env = dict(os.environ, LYAPUNOV_AMD_SANITIZE="1", LYAPUNOV_AMD_LIB_DIR=str(tmp_path))
    built = subprocess.run([sys.executable, "-c",
                            "import sys; sys.path.insert(0, %r); from lyapunov_engine_amd.kernels import build; "
                            "print(build.runtime_selftest())" % ROOT],
                           env=env, capture_output=True, text=True, timeout=600)
    assert built.returncode == 0, built.stderr[-2000:]
    program = built.stdout.strip().splitlines()[-1]
    assert "sanitized" in os.path.basename(program)
    run = subprocess.run([program, "60", "3"], capture_output=True, text=True, timeout=600,
                         env=dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1"))
    assert run.returncode == 0, (run.stdout + run.stderr)[-3000:]
    assert "every check held" in run.stdout
    assert "runtime error" not in run.stderr and "AddressSanitizer" not in run.stderr
    # the run is only worth something if requests were preempted and windows gave pages back
    counts = run.stdout[run.stdout.index("("):]
    numbers = [int(w) for w in counts.replace("(", " ").replace(",", " ").split() if w.isdigit()]
    steps, finished, preempted, refused, window_returns = numbers[:5]
    assert steps > 5000 and finished > 300 and preempted > 20 and refused > 5 and window_returns > 100, counts
