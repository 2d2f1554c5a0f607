"""Oracle quantization stages against exact arithmetic (Fractions / Python ints)."""
import math

import numpy as np
import pytest

from oracle import closed_form as cf
from util import ALL_KINDS, INT_MAX, as_complex, rand_matrix

MIN_NORMAL = {"f64": 2.0**-1022, "c128": 2.0**-1022, "f32": 2.0**-126, "c64": 2.0**-126, "f16": 2.0**-126, "c32h": 2.0**-126}


def special_matrix(rng, kind, M=40, N=9):
    A = rand_matrix(rng, M, N, kind, 2.0)
    flat = A.reshape(M, N, -1) if A.ndim == 3 else A
    flat[:, 1] = 0                                   # all-zero column
    flat[3, 2] = 0
    if kind in ("f64", "c128"):
        flat[:, 3] = flat[:, 3] * 0 + 5e-324        # sub-normal column -> INT_MAX
        flat[0, 4] = 1.0; flat[1:, 4] = flat[1:, 4] * 0 + np.array([0.5 + 2.0**-30, 2.0**-40 * 1.5, -2.0**-40 * 2.5] * M)[:M - 1].reshape(flat[1:, 4].shape) if flat[1:, 4].ndim == 1 else flat[1:, 4]
    return A


@pytest.mark.parametrize("kind", ALL_KINDS)
def test_column_exponents(oracle, kind):
    rng = np.random.default_rng(1)
    M, N, segM = 70, 9, 16
    A = special_matrix(rng, kind, M, N)
    batches, lastM = (M + segM - 1) // segM, M - (M - 1) // segM * segM
    for u in (0, 23, 46):
        vexp = oracle.quantize_scale_batch(A, batches, segM, lastM, u)
        Ac = np.abs(as_complex(A).real) if not np.iscomplexobj(as_complex(A)) else np.maximum(np.abs(as_complex(A).real), np.abs(as_complex(A).imag))
        for b in range(batches):
            rows = Ac[b * segM:min(M, (b + 1) * segM)].astype(np.float64)
            for j in range(N):
                assert vexp[(1 + b) * N + j] == cf.column_exponent(rows[:, j].max(), u, MIN_NORMAL[kind])
        for j in range(N):
            assert vexp[j] == min(vexp[(1 + b) * N + j] for b in range(batches))
        segU = oracle.vector_range(batches, N, u, vexp)
        for b in range(batches):
            d = [int(vexp[j]) - int(vexp[(1 + b) * N + j]) for j in range(N) if vexp[(1 + b) * N + j] != INT_MAX]
            assert segU[b] == (u + max(d) if d else -2**31)
    assert (oracle.quantize_scale_batch(A, batches, segM, lastM, -1)[:N] == INT_MAX).all()


@pytest.mark.parametrize("kind", ALL_KINDS)
@pytest.mark.parametrize("u", [5, 23, 47, 62, 81])
def test_limb_digits_exact(oracle, kind, u):
    rng = np.random.default_rng(2)
    M, N = 33, 7
    A = special_matrix(rng, kind, M, N)
    vexp = oracle.quantize_scale_batch(A, 1, M, M, u)
    qre, qim = cf.quantize_matrix(A, vexp)
    # 12 digits are unreachable (the planner caps the bits at 81 < 87) and the reference's 12th digit only carries 7 bits
    for order in (1, 3, 6, 11):
        B = oracle.quantize("limbs", A, order, vexp, ldb=M + 5)
        groups = [[[a + b for a, b in zip(cr, ci)] for cr, ci in zip(qre, qim)], qre, qim] if qim is not None else [qre]
        for g, q in enumerate(groups):
            for j in range(N):
                for k in range(M):
                    digits = [int(B[g * order + l, j, k]) for l in range(order)]
                    assert digits == cf.balanced_digits(q[j][k], order)
                    assert (sum(d << (8 * l) for l, d in enumerate(digits)) - q[j][k]) % (256 ** order) == 0
        assert not B[:, :, M:].any()


@pytest.mark.parametrize("kind", ALL_KINDS)
@pytest.mark.parametrize("u", [5, 23, 47, 62, 81])
def test_crt_residues_exact(oracle, kind, u):
    rng = np.random.default_rng(3)
    M, N = 29, 6
    A = special_matrix(rng, kind, M, N)
    vexp = oracle.quantize_scale_batch(A, 1, M, M, u)
    qre, qim = cf.quantize_matrix(A, vexp)
    cplx = qim is not None
    moduli = cf.CPLX_MODULI if cplx else cf.REAL_MODULI
    for order in ((1, 7, 20, 21, 25) if cplx else (1, 8, 14, 24)):
        B = oracle.quantize("crt", A, order, vexp)
        for j in range(N):
            for k in range(M):
                for x in range(order):
                    m = moduli[x]
                    if not cplx:
                        assert int(B[x, j, k]) == cf.signed_residue(qre[j][k], m)
                    elif x < cf.CPLX_SPLIT:
                        roots = cf.sqrt_minus_one(m)
                        p, q = int(B[2 * x, j, k]), int(B[2 * x + 1, j, k])
                        ok = [i for i in roots if p == cf.signed_residue(qre[j][k] - i * qim[j][k], m) and q == cf.signed_residue(qre[j][k] + i * qim[j][k], m)]
                        assert ok, "p, q must be re -+ i*im for a square root i of -1"
                    else:
                        base = 40 + 3 * (x - 20)
                        assert int(B[base, j, k]) == cf.signed_residue(qre[j][k] + qim[j][k], m)
                        assert int(B[base + 1, j, k]) == cf.signed_residue(qre[j][k], m) and int(B[base + 2, j, k]) == cf.signed_residue(qim[j][k], m)


def test_rounding_ties_and_signs(oracle):
    # x * 2^e exactly half-way: ties go to even, symmetric in sign
    vals = np.array([[0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, 1.0 - 2.0**-53, 2.0**-1074, -(2.0**52 + 0.5), 0.0, 255.5, -128.5, 1e-300]], dtype=np.float64).T
    vexp = np.array([0], np.int32)
    B = oracle.quantize("limbs", vals, 8, vexp)
    got = [sum(int(B[l, 0, k]) << (8 * l) for l in range(8)) for k in range(vals.shape[0])]
    want = [cf.rne_scaled(float(v), 0) for v in vals[:, 0]]
    assert got == want == [0, 2, 2, 0, -2, -2, 4, 1, 0, -(2**52), 0, 256, -128, 0]
    # the same through a non-trivial exponent
    vexp = np.array([40], np.int32)
    x = np.array([[(2 * k + 1) * 2.0**-41 for k in range(-6, 6)]], dtype=np.float64).T
    B = oracle.quantize("limbs", x, 3, vexp)
    got = [sum(int(B[l, 0, k]) << (8 * l) for l in range(3)) for k in range(x.shape[0])]
    assert got == [cf.rne_scaled(float(v), 40) for v in x[:, 0]]
