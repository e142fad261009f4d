"""The CPU oracle (oracle/*.c) under AddressSanitizer + UndefinedBehaviorSanitizer: oracle/san_check.c drives
every entry family over tile-edge shapes, zero / negative strides and ragged splits and compares each result
with a brute-force loop of its own. CPU only."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_oracle_is_clean_under_asan_and_ubsan():
    res = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "-B", "san_check"], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-3000:]
    env = dict(os.environ, OMP_NUM_THREADS="2", OMP_WAIT_POLICY="passive",
               ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    run = subprocess.run([os.path.join(ROOT, "oracle", "san_check")], capture_output=True, text=True, env=env, timeout=300)
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-4000:]
    assert " 0 mismatches" in run.stdout and "runtime error" not in run.stderr and "AddressSanitizer" not in run.stderr
