"""Known-answer fixtures of the Gram path (tests/golden/*.npz, written by tests/golden/make_fixtures.py).

Without a GPU: the fixtures against exact arithmetic once more (so that a damaged file cannot pass for an answer) and the
oracle against the fixtures.  With a GPU: the hyacin.h stage functions against the fixtures, bit for bit for exponents and
the integer Gram, to the last bit of the high word for the dequantized Gram.
"""
import ctypes as C
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
with open(os.path.join(GOLDEN, "index.json")) as f:
    INDEX = json.load(f)
NAMES = sorted(INDEX)


def load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return INDEX[name], z["A"], z["vexp"], z["C"], z["G"]


@pytest.mark.parametrize("name", NAMES)
def test_fixture_is_the_exact_gram(oracle, name):
    from oracle import closed_form as cf
    meta, A, vexp, Cq, G = load(name)
    N, lP = meta["N"], meta["lP"]
    qre, qim = cf.quantize_matrix(A, vexp)
    re, im = cf.exact_gram(qre, qim)
    want = oracle.int_to_limbs(cf.packed(re, N), lP)
    if qim is not None:
        want = np.concatenate([want, oracle.int_to_limbs(cf.packed(im, N), lP)])
    assert np.array_equal(Cq, want)


@pytest.mark.parametrize("name", NAMES)
def test_oracle_reproduces_fixture(oracle, name):
    meta, A, vexp, Cq, G = load(name)
    assert oracle.atype_of(A) == {"f64": 0, "c128": 1, "f32": 2, "c64": 3, "f16": 4, "c32h": 5}[meta["kind"]]
    g = oracle.gram_pipeline(A, meta["eps"], alg=meta["algorithm"], corr=meta["bit_correction"], segK=meta["rows_per_slice"])
    pl = g["plan"]
    assert (pl["u"], pl["cP"], pl["lP"], pl["batches"], pl["lastM"]) == (meta["u"], meta["cP"], meta["lP"], meta["batches"], meta["lastM"])
    assert np.array_equal(g["vexp"], vexp)
    assert np.array_equal(g["C"], Cq)
    assert (g["gtype"], g["gbytes"], g["bits"]) == (meta["gtype"], meta["gbytes"], meta["gram_bits"])
    assert g["G"].dtype == G.dtype and np.array_equal(g["G"], G)


@pytest.mark.gpu
@pytest.mark.parametrize("name", NAMES)
def test_library_reproduces_fixture(oracle, name):
    import hyacinth_amd as ha
    from gpu_util import colmajor_bytes, zeros, ptr, sync, host, stream
    meta, A, vexp, Cq, G = load(name)
    N, M, at = meta["N"], meta["M"], oracle.atype_of(A)
    h = ha.create_handle(stream=stream().value, GramMatrixAlgorithm=meta["algorithm"].encode(), GramSegmentK=meta["rows_per_slice"],
                         QuantizeBitCorrection=meta["bit_correction"])
    try:
        L = ha.lib()
        u, cP, lP, stride = ha.herk_batch_init(h, meta["eps"], M, N, at)
        assert (u, cP, lP) == (meta["u"], meta["cP"], meta["lP"])
        seg = min(meta["rows_per_slice"], M)
        dA, lda, _ = colmajor_bytes(A)
        dv = zeros(4 * (meta["batches"] + 1) * N)
        dC = zeros(8 * cP * lP * stride)
        L.hyacinXquantizeScaleBatch(C.byref(h), meta["batches"], seg, meta["lastM"], N, at, ptr(dA), lda, u, ptr(dv))
        L.hyacinXherkBatch(C.byref(h), meta["batches"], seg, meta["lastM"], N, at, ptr(dA), lda, u, ptr(dv), 0, lP, ptr(dC))
        gt, gb = C.c_int(), C.c_int32()
        L.hyacinXdequantizeInit(C.byref(h), N, lP, ptr(dC), ptr(dv), at, C.byref(gt), C.byref(gb))
        assert (gt.value, gb.value) == (meta["gtype"], meta["gbytes"])
        dG = zeros(N * N * gb.value)
        L.hyacinXdequantize(C.byref(h), N, lP, ptr(dC), ptr(dv), gt.value, ptr(dG), N)
        sync()
        assert np.array_equal(host(dv, np.int32), vexp)
        assert np.array_equal(host(dC, np.uint64), Cq)
        got = host(dG, G.dtype, G.shape)
        if (meta["gtype"] & ~1) == 6:      # double-double: high words equal, low words to 2^-100 of the entry
            assert np.array_equal(got[..., 0::2], G[..., 0::2])
            assert np.all(np.abs(got[..., 1::2] - G[..., 1::2]) <= np.abs(G[..., 0::2]) * 2.0**-100)
        else:
            assert np.array_equal(got, G)
    finally:
        ha.destroy_handle(h)
