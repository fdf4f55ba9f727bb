"""The CPU checker under AddressSanitizer and UndefinedBehaviorSanitizer (host code only): `make -C oracle sanitize`
builds oracle/tab_oracle.c with a driver (oracle/sanitize_check.c) that runs every oracle function on exactly sized
heap buffers over the edge shapes of the parity tests; any out-of-bounds access or undefined operation aborts it."""
import os
import subprocess

ORACLE = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle")


def test_oracle_is_clean_under_asan_and_ubsan():
    build = subprocess.run(["make", "-C", ORACLE, "-B", "sanitize"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert build.returncode == 0, build.stdout
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1", OMP_NUM_THREADS="4")
    run = subprocess.run([os.path.join(ORACLE, "_ref", "sanitize_check")], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                         env=env, timeout=300)
    assert run.returncode == 0, run.stdout
    assert "0 failed" in run.stdout and "runtime error" not in run.stdout and "AddressSanitizer" not in run.stdout, run.stdout
