"""The boundary as a caller of the reference sees it: include/hyacin.h is valid C and C++, and the reference's quick start
(README.md:109-167) compiles against it, links to libhyacin.so and, on a GPU, fits its 512 x 128 complex matrix."""
import os
import re
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")
LIBDIR = os.path.join(ROOT, "hyacinth_amd")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
FLAGS = ["-D__HIP_PLATFORM_AMD__", "-I", INC, "-I", os.path.join(ROCM, "include")]


def build_quickstart(tmp_path):
    exe = str(tmp_path / "quickstart")
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-Wextra"] + FLAGS + [os.path.join(ROOT, "tests", "quickstart", "quickstart.cpp"), "-o", exe,
           "-L", LIBDIR, "-lhyacin", "-L", os.path.join(ROCM, "lib"), "-lamdhip64", "-Wl,-rpath," + LIBDIR, "-Wl,-rpath," + os.path.join(ROCM, "lib")]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    return exe


@pytest.mark.parametrize("header", ["hyacin.h", "hyacin_kernels.h"])
def test_headers_are_valid_c(header, tmp_path):
    """Both headers declare a C ABI: they must go through a C compiler (C11, pedantic) as well as a C++ one."""
    src = tmp_path / "use.c"
    src.write_text('#include <%s>\nint use(void) { return (int)sizeof(hyacinHandle_t) + (int)HYACIN_QF_COMPLEX; }\n' % ("hyacin.h" if header == "hyacin.h" else "hyacin.h>\n#include <hyacin_kernels.h"))
    for cmd in (["gcc", "-x", "c", "-std=c11", "-pedantic", "-Wall", "-Werror=implicit-function-declaration"], ["g++", "-x", "c++", "-std=c++17", "-Wall"]):
        r = subprocess.run(cmd + FLAGS + ["-c", str(src), "-o", str(tmp_path / "use.o")], capture_output=True, text=True)
        assert r.returncode == 0, " ".join(cmd) + "\n" + r.stdout + r.stderr


def test_handle_layout_is_the_references(tmp_path):
    """112 bytes, the stream at offset 56, the reference's CUDA-typed names usable (include/hyacin.h:20-53 of the reference,
    built without NCCL)."""
    src = tmp_path / "layout.c"
    src.write_text('#include <stddef.h>\n#include <stdio.h>\n#include <hyacin.h>\nint main(void) { printf("%zu %zu %zu %zu %zu\\n", sizeof(hyacinHandle_t), offsetof(hyacinHandle_t, cudaStream), '
                   'offsetof(hyacinHandle_t, hipStream), offsetof(hyacinHandle_t, cublasHandle), offsetof(hyacinHandle_t, mempool)); return 0; }\n')
    exe = str(tmp_path / "layout")
    r = subprocess.run(["gcc", "-std=c11"] + FLAGS + [str(src), "-o", exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    out = subprocess.run([exe], capture_output=True, text=True).stdout.split()
    assert [int(v) for v in out] == [112, 56, 56, 64, 80]


def test_quickstart_compiles_and_links(tmp_path):
    build_quickstart(tmp_path)


@pytest.mark.gpu
def test_quickstart_runs(tmp_path):
    """rank 2 (the matrix is a sum of two rank-one terms), relative projection error at the level of eps, an orthonormal
    basis, and the two singular values numpy finds for the same matrix."""
    exe = build_quickstart(tmp_path)
    # this process first makes a cooperative launch of its own (a pivoted Cholesky): the quick start then runs as a second
    # process on the device, where the runtime refuses cooperative launches and the library has to start its kernel plainly
    import hyacinth_amd as ha
    from test_zz_no_alloc import spd, run
    assert run(ha.lib(), False, spd(np.random.default_rng(5), 200, 30, 0, False), 200, 200, 0, 1e-9)[0] > 0
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    print(r.stdout, r.stderr, flush=True)
    assert "failed" not in r.stderr
    m = re.search(r"rank = (\d+), relative projection error = (\S+), orthonormality defect = (\S+), S0 = (\S+), S1 = (\S+), S2 = (\S+)", r.stdout)
    assert m, r.stdout
    i, j = np.arange(512)[:, None], np.arange(128)[None, :]
    A = (1. + .01 * i) * (1. + .02 * j) + 1j * np.sin(.1 * i) * np.cos(.2 * j)
    want = np.linalg.svd(A, compute_uv=False)
    assert int(m.group(1)) == 2
    assert float(m.group(2)) <= 1e-9 and float(m.group(3)) <= 1e-12
    assert abs(float(m.group(4)) - want[0]) <= 1e-9 * want[0] and abs(float(m.group(5)) - want[1]) <= 1e-9 * want[0] and float(m.group(6)) == 0.0
