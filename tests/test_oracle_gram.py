"""Oracle Gram pipeline: limb path == CRT path == exact big-integer Gram, in the unique 63-bit-limb encoding."""
import numpy as np
import pytest

from oracle import closed_form as cf
from util import ALL_KINDS, rand_matrix


def exact_C(oracle, A, vexp, lP):
    N = A.shape[1]
    qre, qim = cf.quantize_matrix(A, vexp)
    re, im = cf.exact_gram(qre, qim)
    want = oracle.int_to_limbs(cf.packed(re, N), lP)
    if qim is not None:
        want = np.concatenate([want, oracle.int_to_limbs(cf.packed(im, N), lP)])
    return want


@pytest.mark.parametrize("kind", ALL_KINDS)
@pytest.mark.parametrize("eps", [1e-3, 1e-10, 1e-15])
def test_paths_agree_with_exact(oracle, kind, eps):
    rng = np.random.default_rng(11)
    A = rand_matrix(rng, 150, 7, kind)
    at = oracle.atype_of(A)
    pl = oracle.fit_plan(150, 7, eps, at)
    vexp = oracle.quantize_scale_batch(A, pl["batches"], pl["batchIter"], pl["lastM"], pl["u"])
    want = exact_C(oracle, A, vexp, pl["lP"])
    for alg in "LCA":
        got = oracle.herk_batch(A, pl["batches"], pl["batchIter"], pl["lastM"], pl["u"], vexp, pl["lP"], alg=alg)
        assert np.array_equal(got, want), alg


@pytest.mark.parametrize("kind", ["f64", "c128", "f32"])
def test_sliced_buckets_and_zero_columns(oracle, kind):
    rng = np.random.default_rng(12)
    A = rand_matrix(rng, 700, 6, kind, 1.0)
    A[200:400] *= 1e-4            # slices that need fewer bits land in a limb bucket
    A[:, 3] = 0                   # INT_MAX column
    A[500:600] = 0                # all-zero slice is skipped
    at = oracle.atype_of(A)
    pl = oracle.fit_plan(700, 6, 1e-8, at, segK=100)
    assert pl["batches"] == 7
    vexp = oracle.quantize_scale_batch(A, pl["batches"], pl["batchIter"], pl["lastM"], pl["u"])
    want = exact_C(oracle, A, vexp, pl["lP"])
    for alg in "ALC":
        got = oracle.herk_batch(A, pl["batches"], pl["batchIter"], pl["lastM"], pl["u"], vexp, pl["lP"], alg=alg)
        assert np.array_equal(got, want), alg


def test_beta_accumulates_and_extra_moduli(oracle):
    rng = np.random.default_rng(13)
    A = rand_matrix(rng, 120, 5, "c128", 1.0)
    at = oracle.atype_of(A)
    pl = oracle.fit_plan(120, 5, 1e-15, at, corr=20)        # 72 bits -> 22 complex moduli: exercises the three-product extras
    assert oracle.gram_algorithm("C", 120, pl["u"] + 1, 1)[1] > cf.CPLX_SPLIT
    vexp = oracle.quantize_scale_batch(A, 1, 120, 120, pl["u"])
    want = exact_C(oracle, A, vexp, pl["lP"])
    got = oracle.herk_batch(A, 1, 120, 120, pl["u"], vexp, pl["lP"], alg="C")
    assert np.array_equal(got, want)
    # beta = 1 on top of C gives 2C
    twice = oracle.herk_batch(A, 1, 120, 120, pl["u"], vexp, pl["lP"], alg="C", beta=1, Cin=got)
    T = 15
    for plane in (0, 1):
        assert oracle.limbs_to_int(twice, pl["lP"], T, plane) == [2 * v for v in oracle.limbs_to_int(want, pl["lP"], T, plane)]


@pytest.mark.parametrize("cplx", [0, 1])
def test_reconstruct_is_centred_crt(oracle, cplx):
    rng = np.random.default_rng(14)
    moduli = cf.CPLX_MODULI if cplx else cf.REAL_MODULI
    for order in (1, 2, 5, 9, 14, len(moduli)):
        P = 1
        for m in moduli[:order]:
            P *= m
        lP = max(1, -(-(P.bit_length() + 1) // 63))
        vals = [0, 1, -1, P // 2 - 1, -(P // 2), 12345 % (P // 2)] + [int(rng.integers(-2**62, 2**62)) % P - P // 2 for _ in range(30)]
        res = np.array([[v % m for v in vals] for m in moduli[:order]], dtype=np.uint8)
        out = oracle.reconstruct(cplx, res, order, lP)
        got = oracle.limbs_to_int(out, lP, len(vals))
        assert got == [cf.crt_centered([v % m for m in moduli[:order]], moduli[:order]) for v in vals] == vals


def test_limb_encoding_roundtrip(oracle):
    rng = np.random.default_rng(15)
    for L in (1, 2, 3):
        bits = 63 * (L - 1) + 63
        vals = [0, 1, -1, 2**(bits - 1) - 1, -(2**(bits - 1))] + [int(rng.integers(-2**62, 2**62)) << int(rng.integers(0, bits - 62)) for _ in range(20)]
        enc = oracle.int_to_limbs(vals, L)
        assert oracle.limbs_to_int(enc, L, len(vals)) == vals
        T = len(vals)
        for l in range(L - 1):
            assert (enc[l * T:(l + 1) * T] < 2**63).all()
