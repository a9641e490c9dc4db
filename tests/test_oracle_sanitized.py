"""The CPU oracle under AddressSanitizer + UndefinedBehaviorSanitizer: tests/c/oracle_sanitized.c includes oracle/oracle.c
as one translation unit and runs every block format (dequantization, matvec, the reference-algorithm matvec, GEMM) on
random bytes in buffers of exactly the documented sizes, the dense loops, attention and the decoder glue.  A read or a
write past a block, a row or an output, a misaligned access or a signed overflow in the checker ends the run."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_oracle_runs_clean_under_sanitizers(tmp_path):
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    exe = str(tmp_path / "oracle_sanitized")
    cmd = [gcc, "-std=gnu11", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
           "-fno-omit-frame-pointer", "-fopenmp", "-Wall", "-Wextra", "-o", exe,
           os.path.join(ROOT, "tests", "c", "oracle_sanitized.c"), "-lm"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0 and ("asan" in r.stderr or "ubsan" in r.stderr or "sanitize" in r.stderr):
        pytest.skip("this gcc has no sanitizer runtime: " + r.stderr.strip().splitlines()[-1])
    assert r.returncode == 0, r.stderr
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1", OMP_NUM_THREADS="4")
    r = subprocess.run([exe], capture_output=True, text=True, timeout=300, env=env)
    assert r.returncode == 0 and r.stdout.strip() == "ok", r.stdout + r.stderr
