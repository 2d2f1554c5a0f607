"""Writes the known-answer fixtures of the Gram path, tests/golden/*.npz.

The reference ships no golden vectors, so these are made here: the CPU oracle runs the path on small seeded inputs, and
before anything is written every integer result is checked against exact arithmetic that does not follow the
reference's code (Python fractions for the quantization, Python integers for Q^H Q, the unique 63-bit-limb encoding), and
the dequantized Gram against the exact rational value.  A fixture is data only: the input matrix, the settings, and the
expected column exponents, integer Gram, Gram type and dequantized Gram.

    python tests/golden/make_fixtures.py        (from the repository root; rewrites every fixture)
"""
import json
import os
import sys
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

from oracle import closed_form as cf   # noqa: E402
from oracle import ho                  # noqa: E402
from util import rand_matrix           # noqa: E402

# name: (kind, M, N, eps, algorithm, bit correction, rows per slice, seed, what it covers)
CASES = {
    "real_f64_limbs": ("f64", 96, 12, 1e-10, "L", 7, 8192, 101, "limb path, 6 digits (the shape of benchmark configuration 1)"),
    "real_f64_crt": ("f64", 200, 10, 1e-12, "C", 7, 8192, 102, "real residues, 14 moduli (the shape of the benchmark target)"),
    "cplx_f64_crt": ("c128", 120, 8, 1e-12, "C", 7, 8192, 103, "complex residues with the square root of -1 (configuration 3)"),
    "cplx_f16_limbs": ("c32h", 150, 9, 1e-3, "L", 7, 8192, 104, "complex limb path, three digit groups (configuration 4)"),
    "real_f32_sliced": ("f32", 300, 7, 1e-5, "A", 7, 128, 105, "three row slices with different scales, a zero column, automatic choice"),
    "cplx_f64_extras": ("c128", 90, 5, 1e-15, "C", 20, 8192, 106, "more than 20 complex moduli: the three-product moduli"),
}


def make_input(kind, M, N, seed, name):
    rng = np.random.default_rng(seed)
    A = rand_matrix(rng, M, N, kind, 1.5)
    if name == "real_f32_sliced":
        A[128:256] *= np.float32(2.0 ** -9)
        A[:, 3] = 0
    return A


def exact_values(A, vexp, N):
    """Exact integer Gram of the exactly quantized matrix, packed triangle, as Python integers (real, imaginary)."""
    qre, qim = cf.quantize_matrix(A, vexp)
    re, im = cf.exact_gram(qre, qim)
    return cf.packed(re, N), (cf.packed(im, N) if qim is not None else None)


def check_against_mathematics(name, A, kind, eps, corr, g):
    M, N = A.shape[0], A.shape[1]
    pl, vexp, Cq = g["plan"], g["vexp"], g["C"]
    lP, T = pl["lP"], N * (N + 1) // 2
    # column scales: u - (floor(log2 max) + 1)
    if np.iscomplexobj(A):
        absmax = np.maximum(np.abs(A.real), np.abs(A.imag)).max(axis=0)
    elif A.ndim == 3:
        absmax = np.abs(A.astype(np.float64)).max(axis=(0, 2))
    else:
        absmax = np.abs(A.astype(np.float64)).max(axis=0)
    tiny = {"f64": 2.0 ** -1022, "c128": 2.0 ** -1022, "f32": 2.0 ** -126, "c64": 2.0 ** -126, "f16": 2.0 ** -126, "c32h": 2.0 ** -126}[kind]
    for j in range(N):
        assert vexp[j] == cf.column_exponent(absmax[j], pl["u"], tiny), (name, "exponent", j)
    # integer Gram: Python integers in the unique limb encoding
    re, im = exact_values(A, vexp, N)
    want = ho.int_to_limbs(re, lP)
    if im is not None:
        want = np.concatenate([want, ho.int_to_limbs(im, lP)])
    assert np.array_equal(Cq, want), (name, "integer Gram")
    # dequantized Gram: C 2^-(e_x + e_y), exact rational against the stored words
    gt = g["gtype"]
    dd = (gt & ~1) == ho.DD
    width = g["G"].shape[-1]
    parts = 2 if im is not None else 1
    per = width // parts
    for x in range(N):
        for y in range(x + 1):
            for part, vals in ((0, re), (1, im))[:parts]:
                v = vals[y + x * (x + 1) // 2]
                if vexp[x] == cf.INT_MAX or vexp[y] == cf.INT_MAX:
                    exact = Fraction(0)
                else:
                    exact = Fraction(v) / (Fraction(2) ** (int(vexp[x]) + int(vexp[y])))
                words = g["G"][x, y, part * per:(part + 1) * per]
                got = sum(Fraction(float(w)) for w in words)
                rel = Fraction(2) ** (-100 if dd else (-22 if (gt & ~1) == ho.F32 else -51))
                assert abs(got - exact) <= rel * abs(exact), (name, "dequantize", y, x, part)
    assert (gt & 1) == (1 if im is not None else 0)


def main():
    index = {}
    for name, (kind, M, N, eps, alg, corr, segK, seed, what) in CASES.items():
        A = make_input(kind, M, N, seed, name)
        g = ho.gram_pipeline(A, eps, alg=alg, corr=corr, segK=segK)
        check_against_mathematics(name, A, kind, eps, corr, g)
        pl = g["plan"]
        np.savez_compressed(os.path.join(HERE, name + ".npz"), A=A, vexp=g["vexp"], C=g["C"], G=g["G"])
        index[name] = dict(kind=kind, M=M, N=N, eps=eps, algorithm=alg, bit_correction=corr, rows_per_slice=segK, seed=seed, covers=what,
                           u=int(pl["u"]), cP=int(pl["cP"]), lP=int(pl["lP"]), batches=int(pl["batches"]), lastM=int(pl["lastM"]),
                           gtype=int(g["gtype"]), gbytes=int(g["gbytes"]), gram_bits=int(g["bits"]))
        print(name, index[name])
    with open(os.path.join(HERE, "index.json"), "w") as f:
        json.dump(index, f, indent=1, sort_keys=True)
        f.write("\n")


if __name__ == "__main__":
    main()
