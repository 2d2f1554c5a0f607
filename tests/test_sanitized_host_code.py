"""The host-side arithmetic once more under the undefined-behaviour sanitizer: the oracle's C restatement and the host
build of the product's integer helpers and stop rules (hyk_common.h, host/jacobi_stop.hpp through tests/host_math) are
compiled with -fsanitize=undefined (signed overflow, shifts, misaligned and out-of-bounds accesses the compiler can see,
float-to-int conversions), and the CPU tests that drive them run against those builds in a child process.  Any report
ends that process with an error."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SAN = ["-fsanitize=undefined,float-cast-overflow", "-fno-sanitize-recover=all", "-g", "-O1"]


def test_cpu_suites_under_ubsan(tmp_path):
    oracle = str(tmp_path / "libhyacin_oracle_ubsan.so")
    host_math = str(tmp_path / "libhost_math_ubsan.so")
    subprocess.check_call(["gcc"] + SAN + ["-mavx2", "-fopenmp", "-fPIC", "-ffp-contract=off", "-fno-fast-math", "-shared", "-o", oracle,
                           os.path.join(ROOT, "oracle", "hyacin_oracle.c"), "-lm"])
    subprocess.check_call(["g++"] + SAN + ["-std=c++17", "-shared", "-fPIC", "-I", os.path.join(ROOT, "hyacinth_amd", "csrc"),
                           os.path.join(ROOT, "tests", "host_math", "host_math.cpp"), "-o", host_math])
    env = dict(os.environ, HYACIN_ORACLE_LIBRARY=oracle, HYACIN_HOST_MATH_LIBRARY=host_math, UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1", OMP_NUM_THREADS="4")
    suites = ["test_host_math.py", "test_oracle_quantize.py", "test_oracle_gram.py", "test_oracle_tail.py", "test_oracle_planner.py", "test_golden.py"]
    r = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-m", "not gpu", "-p", "no:cacheprovider"] + [os.path.join(ROOT, "tests", t) for t in suites],
                       cwd=ROOT, env=env, capture_output=True, text=True, timeout=1500)
    assert r.returncode == 0 and "runtime error" not in r.stdout + r.stderr, (r.stdout + r.stderr)[-4000:]
