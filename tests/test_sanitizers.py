"""AddressSanitizer + UndefinedBehaviorSanitizer build of the two host-only libraries — the APR builder
(csrc/aprcore.cpp) and the oracle (oracle/aprnet_oracle.cpp) — driven by tests/sanitize/san_driver.cpp, which builds an
APR of an odd-sized volume and runs every oracle operator on it.  The three sources are compiled into ONE instrumented
executable, so nothing has to be preloaded into the Python process.  (ThreadSanitizer is not run: libgomp is not
instrumented in this image, and its barriers then read as races.)"""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.timeout(600)
def test_aprcore_and_oracle_run_clean_under_asan_and_ubsan(tmp_path):
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("no g++")
    exe = str(tmp_path / "san_driver")
    cmd = [gxx, "-std=c++17", "-O1", "-g", "-fno-omit-frame-pointer", "-fopenmp",
           "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
           os.path.join(ROOT, "tests", "sanitize", "san_driver.cpp"),
           os.path.join(ROOT, "apr-cnn_amd", "csrc", "aprcore.cpp"),
           os.path.join(ROOT, "oracle", "aprnet_oracle.cpp"), "-o", exe]
    build = subprocess.run(cmd, capture_output=True, text=True)
    if build.returncode != 0 and ("asan" in build.stderr or "ubsan" in build.stderr):
        pytest.skip("sanitizer runtimes are not installed: " + build.stderr[-300:])
    assert build.returncode == 0, build.stderr[-3000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1",
               OMP_NUM_THREADS="4")
    run = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=500)
    assert run.returncode == 0, (run.stdout[-2000:] + "\n" + run.stderr[-6000:])
    assert run.stdout.strip().endswith("OK"), run.stdout[-2000:]
