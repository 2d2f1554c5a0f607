"""Pins of the oracle's floating-point half: dequantization against exact rationals, the pivoted Cholesky against its
defining invariants and a plain numpy pivoted Cholesky, the SVD / interpolation tails and the residual check against
numpy's eigen-decomposition and QR."""
from fractions import Fraction

import numpy as np
import pytest

from oracle import closed_form as cf
from util import haar, rand_matrix

F64, F64C, F32, F32C, DD, DDC = 0, 1, 2, 3, 6, 7


def exact_entries(oracle, A, eps):
    """Exact rational Gram of the quantized matrix, G[y][x] = C[y, x] * 2^-(e_x + e_y) for y <= x, plus the plan."""
    g = oracle.gram_pipeline(A, eps)
    N = A.shape[1]
    qre, qim = cf.quantize_matrix(A, g["vexp"])
    re, im = cf.exact_gram(qre, qim)
    ex = [int(v) for v in g["vexp"][:N]]
    out = {}
    for x in range(N):
        for y in range(x + 1):
            s = Fraction(1, 2 ** (ex[x] + ex[y])) if ex[x] + ex[y] >= 0 else Fraction(2 ** -(ex[x] + ex[y]))
            out[(y, x)] = (re[(y, x)] * s, (im[(y, x)] * s) if qim is not None else Fraction(0))
    return g, out


def dd_value(hi, lo):
    return Fraction(float(hi)) + Fraction(float(lo))


@pytest.mark.parametrize("kind,eps", [("f64", 1e-4), ("f64", 1e-12), ("c128", 1e-12), ("f32", 1e-3), ("c64", 1e-6)])
def test_dequantize_against_exact_rationals(oracle, kind, eps):
    rng = np.random.default_rng(21)
    A = rand_matrix(rng, 90, 6, kind, 1.5)
    g, exact = exact_entries(oracle, A, eps)
    N, gt, G = 6, g["gtype"], g["G"]
    cplx = gt & 1
    base = gt & ~1
    assert base in (F32, F64, DD)
    # relative error bound of the conversion: 2 ulp of the target type; double-double keeps 104 bits
    tol = {F32: Fraction(1, 2 ** 22), F64: Fraction(1, 2 ** 51), DD: Fraction(1, 2 ** 103)}[base]
    for (y, x), (wre, wim) in exact.items():
        raw = G[x, y]            # raw layout [column][row][width]
        if base == DD:
            gre = dd_value(raw[0], raw[1])
            gim = dd_value(raw[2], raw[3]) if cplx else Fraction(0)
        else:
            gre = Fraction(float(raw[0]))
            gim = Fraction(float(raw[1])) if cplx else Fraction(0)
        scale = max(abs(wre), abs(wim), Fraction(1, 2 ** 1000))
        assert abs(gre - wre) <= tol * scale, (y, x)
        assert abs(gim - wim) <= tol * scale, (y, x)
        # Hermitian mirror
        mir = G[y, x]
        if base == DD:
            assert dd_value(mir[0], mir[1]) == gre and (not cplx or dd_value(mir[2], mir[3]) == -gim)
        else:
            assert Fraction(float(mir[0])) == gre and (not cplx or Fraction(float(mir[1])) == -gim)


def test_dequantize_type_follows_the_dominant_diagonal(oracle):
    """bits = bitlen(C_ii) - 2 vexp_i maximised over i, minus 2 corr: <= 23 FP32, <= 52 FP64, else double-double."""
    rng = np.random.default_rng(22)
    A = rand_matrix(rng, 64, 5, "f64", 1.0)
    seen = set()
    for eps in (1e-2, 1e-6, 1e-13):
        g = oracle.gram_pipeline(A, eps)
        N, lP = 5, g["plan"]["lP"]
        T = N * (N + 1) // 2
        ints = oracle.limbs_to_int(g["C"], lP, T)
        best = None
        for i in range(N):
            d = ints[i + i * (i + 1) // 2]
            key = (d.bit_length() - 2 * int(g["vexp"][i]), d.bit_length())
            best = key if best is None or key > best else best
        assert g["bits"] == best[1]          # the oracle reports the bit length itself
        bits = best[1] - 2 * 7
        want = F32 if bits <= 23 else F64 if bits <= 52 else DD
        assert g["gtype"] == want
        seen.add(want)
    assert seen == {F32, F64, DD}


def numpy_pivoted_cholesky(G, eps, K):
    """Textbook right-looking diagonal-pivoted Cholesky with the reference's stopping rule."""
    G = G.copy()
    N = G.shape[0]
    piv = np.arange(N)
    total = float(np.real(np.trace(G)))
    R = np.zeros_like(G)
    rank = 0
    for k in range(min(K, N)):
        d = np.real(np.diagonal(G))[k:]
        if float(d.sum()) <= eps * eps * total:
            break
        j = k + int(np.argmax(d))
        G[:, [k, j]] = G[:, [j, k]]
        G[[k, j], :] = G[[j, k], :]
        R[:, [k, j]] = R[:, [j, k]]
        piv[[k, j]] = piv[[j, k]]
        r = np.sqrt(np.real(G[k, k]))
        R[k, k] = r
        R[k, k + 1:] = G[k, k + 1:] / r
        G[k + 1:, k + 1:] -= np.outer(R[k, k + 1:].conj(), R[k, k + 1:])
        rank += 1
    return rank, piv, R


@pytest.mark.parametrize("cplx", [0, 1])
@pytest.mark.parametrize("gt", [F64, DD])
def test_potrfp_invariants_and_textbook(oracle, cplx, gt):
    rng = np.random.default_rng(23 + cplx)
    N, r = 24, 9
    U = haar(rng, N, N, bool(cplx))
    sig = np.concatenate([10.0 ** (-np.arange(r) / 3.0), 1e-9 * np.ones(N - r)])
    Gm = (U * sig ** 2) @ U.conj().T
    Gm = (Gm + Gm.conj().T) / 2
    gtype = gt + cplx
    width = {F64: 1, F64C: 2, DD: 2, DDC: 4}[gtype]
    raw = np.zeros((N, N, width))
    Gt = Gm.T                                   # raw layout is [column][row]
    if gt == F64:
        raw[..., 0] = Gt.real
        if cplx:
            raw[..., 1] = Gt.imag
    else:
        raw[..., 0] = Gt.real
        if cplx:
            raw[..., 2] = Gt.imag
    eps = 1e-6
    work = raw.copy()
    rank, jpiv = oracle.potrfp(work, gtype, eps, N)
    assert sorted(jpiv.tolist()) == list(range(1, N + 1))          # a permutation, 1-based
    assert 0 < rank <= N
    R = oracle.upper_factor(work, gtype, rank, jpiv).conj().T       # rank x N, columns back in original order
    resid = Gm - R.conj().T @ R
    p = jpiv - 1
    lead = resid[np.ix_(p[:rank], p[:rank])]
    assert np.abs(lead).max() <= 1e-13 * np.abs(Gm).max()           # leading block reproduced
    assert np.real(np.trace(resid)) <= eps * eps * np.real(np.trace(Gm)) * (1 + 1e-6)
    Rp = R[:, p]                                                    # pivoted order: upper triangular, diagonal non-increasing
    assert np.abs(np.tril(Rp[:, :rank], -1)).max() <= 1e-13 * np.abs(Rp).max()
    dg = np.abs(np.diagonal(Rp[:, :rank]))
    assert np.all(dg[:-1] >= dg[1:] * (1 - 1e-12))
    wrank, wpiv, wR = numpy_pivoted_cholesky(Gm, eps, N)
    assert rank == wrank
    assert np.array_equal(p[:rank], wpiv[:rank])                    # separated spectrum: no ties
    assert np.allclose(np.abs(np.diagonal(Rp[:, :rank])), np.abs(np.diagonal(wR)[:rank]), rtol=1e-9)


@pytest.mark.parametrize("kind", ["f64", "c128"])
def test_tsvd_tail_is_sqrt_eigvalsh(oracle, kind):
    rng = np.random.default_rng(25)
    M, N, r = 200, 12, 5
    cplx = kind == "c128"
    A = (haar(rng, M, r, cplx) * 10.0 ** (-np.arange(r))) @ haar(rng, N, r, cplx).conj().T
    A = A + 1e-13 * rand_matrix(rng, M, N, kind, 0.0)
    eps = 1e-8
    rank, S, V, g = oracle.tsvd_fit(A, eps, N)
    Gm = oracle.g_to_complex(g["G"], g["gtype"])
    ev = np.sqrt(np.maximum(np.linalg.eigvalsh(Gm)[::-1], 0))
    assert rank == r
    assert np.allclose(S[:rank], ev[:rank], rtol=10 * eps)
    assert np.all(S[rank:] == 0)
    # rank rule: keep i while the suffix energy exceeds eps^2 * total
    tot = float((ev ** 2).sum())
    want = sum(1 for i in range(N) if float((ev[i:] ** 2).sum()) > eps * eps * tot)
    assert rank == want
    assert np.allclose(V.conj().T @ V, np.eye(rank), atol=1e-10)
    assert oracle.check_norm(A, V) <= (2 * eps) ** 2 * np.linalg.norm(A) ** 2


def test_interp_tail_reproduces_columns(oracle):
    rng = np.random.default_rng(26)
    M, N, r = 150, 10, 4
    A = rng.standard_normal((M, r)) @ rng.standard_normal((r, N))
    rank, jpiv, X, g = oracle.interpolate_fit(A, 1e-9, N)
    assert rank == r
    p = jpiv - 1
    assert np.allclose(X[p[:rank], :], np.eye(rank), atol=0)          # identity rows at the pivots
    assert np.linalg.norm(A - A[:, p[:rank]] @ X.conj().T) <= 1e-7 * np.linalg.norm(A)


def test_check_norm_closed_form(oracle):
    rng = np.random.default_rng(27)
    A = rng.standard_normal((40, 8))
    U, s, Vt = np.linalg.svd(A, full_matrices=False)
    for k in (0, 3, 8):
        want = float((s[k:] ** 2).sum())
        got = oracle.check_norm(A, Vt[:k].T if k else None)
        assert abs(got - want) <= 1e-10 * float((s ** 2).sum())
