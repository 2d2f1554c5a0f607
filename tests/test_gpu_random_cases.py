"""Seeded random sweeps over the entry points: shapes, precisions, storage orders, algorithms, slice scales and accuracies
drawn at random, every case held to the oracle.  The integer Gram and the exponents bit for bit (reference:
src/fp_exponent.cu, src/hyacin_herk.cpp:283-384); the fits within the tolerances of test_gpu_api.py (singular values to
10 eps, projection residual within 2x of the oracle's, the vectors handed out orthonormal to sqrt(eps) or the storage
rounding; interpolation: identity rows on the pivots, residual within 2x)."""
import ctypes as C

import numpy as np
import pytest

from util import as_complex, rand_matrix
import test_gpu_api as api

pytestmark = pytest.mark.gpu

STORAGE_EPS = {0: 2.2e-16, 1: 2.2e-16, 2: 1.2e-7, 3: 1.2e-7, 4: 9.8e-4, 5: 9.8e-4}
KINDS = ["f64", "c128", "f32", "c64", "f16", "c32h"]


@pytest.fixture(scope="module")
def env():
    import hyacinth_amd as ha
    from gpu_util import stream
    h = ha.create_handle(stream=stream().value)
    yield ha, h
    ha.destroy_handle(h)


@pytest.mark.parametrize("seed", [101, 102, 103])
def test_random_gram_cases_bit_exact(env, oracle, seed):
    from gpu_util import zeros, ptr, sync, host, colmajor_bytes, stored_transpose
    ha, h = env
    L = ha.lib()
    rng = np.random.default_rng(seed)
    try:
        for case in range(60):
            kind = KINDS[rng.integers(6)]
            alg = [b"A", b"L", b"C"][rng.integers(3)]
            seg = int(rng.choice([128, 256, 384, 512, 1024]))
            M, N = int(rng.integers(1, 4000)), int(rng.integers(1, 600))
            eps = 10.0 ** -float(rng.uniform(1, 15.5))
            op = ["N", "T", "C"][rng.integers(3)]
            A = rand_matrix(rng, M, N, kind, float(rng.uniform(0.5, 3.0)))
            batches = (M + seg - 1) // seg
            for b in range(batches):                       # all-zero slices and slices far below the others (limb buckets)
                c = rng.integers(6)
                if c == 0:
                    A[b * seg:(b + 1) * seg] = 0
                elif c == 1:
                    A[b * seg:(b + 1) * seg] *= 2.0 ** -int(rng.integers(1, 40))
            if N > 2 and rng.integers(2):
                A[:, int(rng.integers(N))] = 0
            at = oracle.atype_of(A)
            h.GramMatrixAlgorithm = alg
            h.GramSegmentK = seg
            pl = oracle.fit_plan(M, N, eps, at, segK=seg)
            u, cP, lP, stride = ha.herk_batch_init(h, eps, M, N, at)
            assert (u, cP, lP, stride) == (pl["u"], pl["cP"], pl["lP"], pl["stride"])
            if op == "N":
                dA, lda, _ = colmajor_bytes(A)
            else:
                dA, lda, _ = stored_transpose(A, op, int(rng.integers(0, 5)) * (8 if at in (4, 5) else 1))
            vexp, Cd = zeros(4 * (pl["batches"] + 1) * N), zeros(8 * cP * max(lP, 1) * stride)
            print("random gram", seed, case, kind, alg, op, M, N, seg, "%.1e" % eps, flush=True)
            L.hykQuantizeScaleBatchOp(C.byref(h), op.encode(), pl["batches"], seg, pl["lastM"], N, at, ptr(dA), lda, u, ptr(vexp))
            L.hykHerkBatchOp(C.byref(h), op.encode(), pl["batches"], seg, pl["lastM"], N, at, ptr(dA), lda, u, ptr(vexp), 0, lP, ptr(Cd))
            sync()
            assert L.hykLastStatus() == 0
            v_o = oracle.quantize_scale_batch(A, pl["batches"], seg, pl["lastM"], u)
            assert np.array_equal(host(vexp, np.int32), v_o)
            if lP > 0:
                C_o = oracle.herk_batch(A, pl["batches"], seg, pl["lastM"], u, v_o, lP, alg=alg.decode())
                assert np.array_equal(host(Cd, np.uint64)[:len(C_o)], C_o)
    finally:
        h.GramMatrixAlgorithm = b"A"
        h.GramSegmentK = 8192


def _random_matrix(rng, at, max_n):
    M = int(rng.integers(60, 3000))
    N = int(rng.integers(4, min(M, max_n)))
    eps = 10.0 ** -float(rng.uniform(1, {0: 13.5, 1: 13.5, 2: 5.5, 3: 5.5, 4: 2.5, 5: 2.5}[at]))
    decay = float(rng.uniform(0.5, 0.97))
    opA = ["N", "T", "C"][rng.integers(3)]
    opA = "C" if (opA == "T" and at & 1) else ("T" if (opA == "C" and not at & 1) else opA)
    A0, _ = api.low_rank(rng, M, N, decay, cplx=bool(at & 1), noise=eps * 1e-2)
    return M, N, eps, decay, opA, A0


@pytest.mark.parametrize("seed", [201, 202])
def test_random_tsvd_fits(env, oracle, seed):
    ha, h = env
    rng = np.random.default_rng(seed)
    try:
        for case in range(25):
            at = int(rng.integers(6))
            M, N, eps, decay, opA, A0 = _random_matrix(rng, at, 400)
            K = int(rng.integers(1, N + 1))
            alg = [b"A", b"L", b"C"][rng.integers(3)]
            A = api.to_storage(A0, at)
            h.GramMatrixAlgorithm = alg
            print("random fit", seed, case, at, M, N, K, "%.1e" % eps, "%.2f" % decay, alg, opA, flush=True)
            rank, S, V, err, nrm = api.run_tsvd(env, A, eps, K, opA)
            assert ha.lib().hykLastStatus() == 0
            r_o, S_o, V_o, g = oracle.tsvd_fit(A, eps, K, alg=alg.decode())
            Ac = as_complex(A).astype(np.complex128 if at & 1 else np.float64)
            k = min(rank, r_o)
            # inside a noise floor below eps sigma_1 the energy cut is decided by values neither side resolves
            assert abs(rank - r_o) <= (1 if k == 0 or S_o[k - 1] > 4 * eps * S_o[0] else 4)
            tol = 10 * max(eps, STORAGE_EPS[at]) * S_o[0]
            if k:
                assert np.abs(S[:k] - S_o[:k]).max() <= tol
                defect = np.abs(V[:, :k].conj().T @ V[:, :k] - np.eye(k)).max()
                assert defect <= max({0: 1e-11, 1: 1e-11, 2: 5e-6, 3: 5e-6, 4: 2e-2, 5: 2e-2}[at], 2 * np.sqrt(eps))
            assert not S[rank:].any()
            mine = oracle.check_norm(Ac, V)
            ref = oracle.check_norm(Ac, V_o[:, :k]) if k else nrm
            assert mine <= max(2 * ref, (2 * eps) ** 2 * nrm) + (10 * tol) ** 2
    finally:
        h.GramMatrixAlgorithm = b"A"


@pytest.mark.parametrize("seed", [301])
def test_random_interpolations_and_segmented_fits(env, oracle, seed):
    from gpu_util import zeros, ptr, sync, host
    ha, h = env
    rng = np.random.default_rng(seed)
    for case in range(40):
        at = int(rng.integers(6))
        M, N, eps, decay, opA, A0 = _random_matrix(rng, at, 260)
        K = int(rng.integers(1, N + 1))
        if rng.integers(2):
            A0 = A0 * np.exp(rng.uniform(-4, 4, N) if at < 4 else rng.uniform(-1, 1, N))
        A = api.to_storage(A0, at)
        Ac = as_complex(A).astype(np.complex128 if at & 1 else np.float64)
        if rng.integers(2):
            print("random interpolation", seed, case, at, M, N, K, "%.1e" % eps, "%.2f" % decay, opA, flush=True)
            dA, lda = api.dev_matrix(A, opA)
            eb = {0: 8, 1: 16, 2: 4, 3: 8, 4: 2, 5: 4}[at]
            X, jp = zeros(eb * N * K), zeros(4 * N)
            rank = ha.lib().hyacinInterpolateFit(C.byref(h), eps, opA.encode(), M, N, K, ptr(dA), lda, ptr(jp), ptr(X), N, 0, at)
            sync()
            assert ha.lib().hykLastStatus() == 0
            jpiv = host(jp, np.int32)
            assert sorted(jpiv.tolist()) == list(range(1, N + 1))
            r_o, jp_o, X_o, g = oracle.interpolate_fit(A, eps, K)
            assert abs(rank - r_o) <= 1 and 0 <= rank <= K
            if rank == 0 or r_o > K:            # r_o > K: the reference counts a single remaining column in
                continue
            real = {8: np.float64, 4: np.float32, 2: np.float16}[eb // (1 + (at & 1))]
            Xh = host(X, real).astype(np.float64)
            Xh = (Xh.reshape(K, N, 2)[..., 0] + 1j * Xh.reshape(K, N, 2)[..., 1]).T if at & 1 else Xh.reshape(K, N).T
            Xh, sel = Xh[:, :rank], jpiv[:rank] - 1
            assert np.allclose(Xh[sel], np.eye(rank), atol=1e-3 if at >= 4 else (1e-6 if at >= 2 else 1e-12))
            resid = np.linalg.norm(Ac - Ac[:, sel] @ Xh.conj().T)
            sel_o = jp_o[:r_o] - 1
            resid_o = np.linalg.norm(Ac - Ac[:, sel_o] @ X_o.conj().T)
            assert resid <= 2 * resid_o + 50 * max(eps, STORAGE_EPS[at]) * np.linalg.norm(Ac) * max(1.0, np.abs(Xh).max())
        elif N >= 16:
            K = max(1, min(K, N // 4))
            print("random segmented fit", seed, case, at, M, N, K, "%.1e" % eps, "%.2f" % decay, opA, flush=True)
            rank, S, V, err, nrm = api.run_tsvd(env, A, eps, K, opA, segmented=True)
            assert ha.lib().hykLastStatus() == 0
            rank1, S1, V1, err1, _ = api.run_tsvd(env, A, eps, K, opA, segmented=False)
            assert 0 <= rank <= K and abs(rank - rank1) <= 2
            k = min(rank, rank1)
            if k:
                assert np.abs(S[:k] - S1[:k]).max() <= 20 * max(eps, STORAGE_EPS[at]) * S1[0]
            assert err <= 4 * err1 + (20 * max(eps, STORAGE_EPS[at])) ** 2 * nrm
