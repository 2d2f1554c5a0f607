"""Build libhyacin.so (HIP kernels + C++ drivers) for gfx950 with hipcc.

Usage: python -m hyacinth_amd.build [--jobs N]
The library lands next to this file (in-tree), which is where the loader looks.
"""
import argparse
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
ROOT = os.path.dirname(HERE)
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libhyacin.so")

KERNELS = ["exponent.hip", "quantize.hip", "gram_mfma.hip", "dequantize.hip", "potrfp.hip", "tail.hip", "tail_f32.hip", "matcopy.hip", "gemm.hip"]
HOST = ["host/handle.cpp", "host/herk.cpp", "host/tail.cpp", "host/lra.cpp"]

# -ffp-contract=off: the double-double code relies on error-free transforms.
# -packed-fp32-ops off: required on this hardware pool for all device code.
COMMON = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-Wall", "-Wextra", "-Wno-unused-parameter", "-Wno-unknown-attributes", "-Wno-pass-failed",
          "-I", os.path.join(ROOT, "include"), "-I", CSRC]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def compile_one(src, define=None):
    out = os.path.join(OBJ, ("timing_" if define else "") + src.replace("/", "_") + ".o")
    cmd = [hipcc(), "-x", "hip", "-c", os.path.join(CSRC, src), "-o", out] + COMMON + ([define] if define else [])
    r = subprocess.run(cmd, capture_output=True, text=True)
    log = "\n".join(l for l in (r.stdout + r.stderr).splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        return None, "hipcc failed for %s:\n%s" % (src, log)
    return out, log


def build(jobs=8, verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(compile_one, KERNELS + HOST))
    failed = [log for o, log in results if o is None]
    if failed:
        raise RuntimeError("\n".join(failed))
    objs = [o for o, _ in results]
    if verbose:
        for _, log in results:
            if log.strip():
                print(log)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=8)
    ap.add_argument("-v", "--verbose", action="store_true")
    a = ap.parse_args()
    print(build(a.jobs, a.verbose))
    sys.exit(0)
