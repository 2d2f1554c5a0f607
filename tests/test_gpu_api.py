"""The hyacin.h entry points on the GPU against the oracle pipeline: bit-exact integer Gram, singular values and
Gram within 10*eps, fitted bases within 2x of the oracle's own projection residual."""
import ctypes as C

import numpy as np
import pytest

from util import as_complex, haar, rand_matrix

pytestmark = pytest.mark.gpu

NP_OF = {0: np.float64, 1: np.complex128, 2: np.float32, 3: np.complex64, 4: np.float16, 5: np.float16}


@pytest.fixture(scope="module")
def env():
    import torch
    import hyacinth_amd as ha
    from gpu_util import stream
    h = ha.create_handle(stream=stream().value)
    yield ha, h
    ha.destroy_handle(h)


def low_rank(rng, M, N, decay, cplx=False, noise=0.0):
    U, V = haar(rng, M, N, cplx), haar(rng, N, N, cplx)
    s = decay ** np.arange(N)
    A = (U * s) @ V.conj().T
    if noise:
        A = A + noise * (rng.standard_normal((M, N)) + (1j * rng.standard_normal((M, N)) if cplx else 0))
    return A, s


def to_storage(A, at):
    if at in (0, 1):
        return A.astype(NP_OF[at])
    if at in (2, 3):
        return A.astype(NP_OF[at])
    if at == 4:
        return A.real.astype(np.float16)
    return np.stack([A.real, A.imag], axis=-1).astype(np.float16)


def dev_matrix(A, opA):
    """Device copy of op^-1(A) so that op(stored) == A; returns (tensor, lda)."""
    from gpu_util import dev
    if A.ndim == 3:                       # complex half [M, N, 2]
        if opA == "N":
            return dev(np.ascontiguousarray(np.transpose(A, (1, 0, 2)))), A.shape[0]
        S = A.copy()
        if opA == "C":
            S[..., 1] = -S[..., 1]
        return dev(np.ascontiguousarray(S)), A.shape[1]      # stored N x M column-major == [m][n][2]
    if opA == "N":
        return dev(np.ascontiguousarray(A.T)), A.shape[0]
    S = A.conj() if opA == "C" else A
    return dev(np.ascontiguousarray(S)), A.shape[1]          # stored N x M column-major: element (n, m) at n + m*N


def run_tsvd(env, A, eps, K, opA="N", segmented=False):
    from gpu_util import zeros, ptr, sync, host
    from oracle import ho
    ha, h = env
    at = ho.atype_of(A)
    M, N = A.shape[0], A.shape[1]
    dA, lda = dev_matrix(A, opA)
    eb = {0: 8, 1: 16, 2: 4, 3: 8, 4: 2, 5: 4}[at]
    sb = eb // (1 + (at & 1))
    S, V = zeros(sb * K), zeros(eb * N * K)
    fn = ha.lib().hyacinTsvdFitSegmentN if segmented else ha.lib().hyacinTsvdFit
    rank = fn(C.byref(h), eps, opA.encode(), M, N, K, ptr(dA), lda, ptr(S), ptr(V), N, 0, at)
    sync()
    real = {8: np.float64, 4: np.float32, 2: np.float16}[sb]
    Sh = host(S, real).astype(np.float64)
    Vh = host(V, real).astype(np.float64)
    Vh = (Vh.reshape(K, N, 2)[..., 0] + 1j * Vh.reshape(K, N, 2)[..., 1]).T if at & 1 else Vh.reshape(K, N).T
    err = ha.lib().hyacinCheckNorm(C.byref(h), opA.encode(), M, N, ptr(dA), lda, rank, ptr(V), N, at)
    nrm = ha.lib().hyacinCheckNorm(C.byref(h), opA.encode(), M, N, ptr(dA), lda, 0, None, N, at)
    return rank, Sh, Vh[:, :rank], err, nrm


CASES = [
    # (type, M, N, K, eps, decay, alg, opA)
    (0, 2048, 96, 96, 1e-10, 10 ** (-1 / 6), b"L", "N"),
    (0, 2048, 96, 96, 1e-10, 10 ** (-1 / 6), b"A", "N"),
    (2, 4096, 128, 64, 1e-5, 2 ** (-1 / 4), b"A", "T"),
    (1, 3000, 80, 40, 1e-12, 10 ** (-1 / 5), b"A", "N"),
    (5, 4096, 96, 32, 1e-3, 0.8, b"L", "C"),
    (3, 1500, 70, 70, 1e-6, 0.7, b"A", "C"),
    (4, 1024, 64, 64, 1e-3, 0.85, b"A", "N"),
    (1, 1200, 60, 60, 1e-9, 0.6, b"L", "N"),
]


@pytest.mark.parametrize("at,M,N,K,eps,decay,alg,opA", CASES)
def test_tsvd_fit_parity(env, oracle, at, M, N, K, eps, decay, alg, opA):
    ha, h = env
    rng = np.random.default_rng(41)
    A0, s = low_rank(rng, M, N, decay, cplx=bool(at & 1), noise=eps * 1e-2)
    A = to_storage(A0, at)
    h.GramMatrixAlgorithm = alg
    print("tsvd", at, M, N, K, eps, alg, opA, flush=True)
    try:
        rank, S, V, err, nrm = run_tsvd(env, A, eps, K, opA)
    finally:
        h.GramMatrixAlgorithm = b"A"
    r_o, S_o, V_o, g = oracle.tsvd_fit(A, eps, K, alg=alg.decode())
    Ac = as_complex(A).astype(np.complex128 if at & 1 else np.float64)
    assert abs(nrm - np.linalg.norm(Ac) ** 2) <= 1e-10 * nrm
    # rank: the energy cut is decided on sigma values that agree to rounding; allow one at the threshold
    assert abs(rank - r_o) <= 1
    tol = 10 * max(eps, {0: 2.2e-16, 1: 2.2e-16, 2: 1.2e-7, 3: 1.2e-7, 4: 9.8e-4, 5: 9.8e-4}[at]) * S_o[0]
    k = min(rank, r_o)
    assert np.abs(S[:k] - S_o[:k]).max() <= tol
    assert not S[rank:].any()
    # projection residual: own CheckNorm agrees with the closed form, and is within 2x of the oracle basis' residual
    mine = oracle.check_norm(Ac, V)
    assert abs(err - mine) <= 1e-6 * nrm + 0.05 * mine
    ref = oracle.check_norm(Ac, V_o[:, :k]) if k else nrm
    floor = (10 * tol) ** 2
    assert oracle.check_norm(Ac, V[:, :k]) <= 2 * ref + floor
    assert mine <= max(2 * ref, (2 * eps) ** 2 * nrm) + floor


def test_gram_api_bit_exact_sliced(env, oracle):
    """hyacinXquantizeScaleBatch + hyacinXherkBatch against the oracle, sliced rows with uneven scales, beta chaining."""
    from gpu_util import dev, zeros, ptr, sync, host, colmajor_bytes
    ha, h = env
    rng = np.random.default_rng(42)
    for kind, alg in (("f64", b"A"), ("c128", b"A"), ("f32", b"L"), ("c64", b"C"), ("f16", b"A"), ("c32h", b"L")):
        M, N, seg = 3000, 150, 512
        A = rand_matrix(rng, M, N, kind, 1.5)
        A[512:1024] *= 2.0 ** -12
        A[2048:2560] = 0
        A[:, 7] = 0
        at = oracle.atype_of(A)
        h.GramMatrixAlgorithm = alg; h.GramSegmentK = seg
        try:
            pl = oracle.fit_plan(M, N, 1e-9, at, segK=seg)
            u, cP, lP, stride = ha.herk_batch_init(h, 1e-9, M, N, at)
            assert (u, cP, lP, stride) == (pl["u"], pl["cP"], pl["lP"], pl["stride"])
            dA, lda, _ = colmajor_bytes(A)
            vexp = zeros(4 * (pl["batches"] + 1) * N)
            ha.lib().hyacinXquantizeScaleBatch(C.byref(h), pl["batches"], seg, pl["lastM"], N, at, ptr(dA), lda, u, ptr(vexp))
            Cd = zeros(8 * cP * lP * stride)
            print("gram api", kind, alg, pl, flush=True)
            ha.lib().hyacinXherkBatch(C.byref(h), pl["batches"], seg, pl["lastM"], N, at, ptr(dA), lda, u, ptr(vexp), 0, lP, ptr(Cd))
            sync()
            v_o = oracle.quantize_scale_batch(A, pl["batches"], seg, pl["lastM"], u)
            assert np.array_equal(host(vexp, np.int32), v_o)
            C_o = oracle.herk_batch(A, pl["batches"], seg, pl["lastM"], u, v_o, lP, alg=alg.decode())
            assert np.array_equal(host(Cd, np.uint64), C_o)
            # dequantize: type choice and values
            gt, gb = C.c_int(), C.c_int32()
            ha.lib().hyacinXdequantizeInit(C.byref(h), N, lP, ptr(Cd), ptr(vexp), at, C.byref(gt), C.byref(gb))
            g_o, b_o, _ = oracle.dequantize_init(N, lP, C_o, v_o, at)
            assert (gt.value, gb.value) == (g_o, b_o)
        finally:
            h.GramMatrixAlgorithm = b"A"; h.GramSegmentK = 8192


@pytest.mark.parametrize("at,opA", [(0, "N"), (1, "N"), (2, "T"), (5, "C")])
def test_interpolate_fit(env, oracle, at, opA):
    from gpu_util import zeros, ptr, sync, host
    ha, h = env
    rng = np.random.default_rng(43)
    M, N, K, eps = 2000, 90, 30, {0: 1e-8, 1: 1e-8, 2: 1e-4, 5: 1e-2}[at]
    A0, _ = low_rank(rng, M, N, 0.6, cplx=bool(at & 1))
    A0 = A0 * np.exp(rng.uniform(-6, 6, N) if at < 4 else rng.uniform(-1, 1, N))     # badly scaled columns stress the exponent path
    A = to_storage(A0, at)
    dA, lda = dev_matrix(A, opA)
    eb = {0: 8, 1: 16, 2: 4, 5: 4}[at]
    X, jp = zeros(eb * N * K), zeros(4 * N)
    print("interp", at, opA, flush=True)
    rank = ha.lib().hyacinInterpolateFit(C.byref(h), eps, opA.encode(), M, N, K, ptr(dA), lda, ptr(jp), ptr(X), N, 0, at)
    sync()
    jpiv = host(jp, np.int32)
    assert sorted(jpiv.tolist()) == list(range(1, N + 1))
    r_o, jp_o, X_o, g = oracle.interpolate_fit(A, eps, K)
    assert abs(rank - r_o) <= 1 and 0 < rank <= K
    real = {8: np.float64, 16: np.float64, 4: np.float32 if at == 2 else np.float16}[eb]
    Xh = host(X, real).astype(np.float64)
    Xh = (Xh.reshape(K, N, 2)[..., 0] + 1j * Xh.reshape(K, N, 2)[..., 1]).T if at & 1 else Xh.reshape(K, N).T
    Xh = Xh[:, :rank]
    Ac = as_complex(A).astype(np.complex128 if at & 1 else np.float64)
    sel = jpiv[:rank] - 1
    assert np.allclose(Xh[sel], np.eye(rank), atol=1e-3 if at == 5 else 1e-12)
    resid = np.linalg.norm(Ac - Ac[:, sel] @ Xh.conj().T)
    sel_o = jp_o[:r_o] - 1
    resid_o = np.linalg.norm(Ac - Ac[:, sel_o] @ X_o.conj().T)
    storage_eps = {0: 2.2e-16, 1: 2.2e-16, 2: 1.2e-7, 5: 9.8e-4}[at]
    assert resid <= 2 * resid_o + 50 * max(eps, storage_eps) * np.linalg.norm(Ac)


def test_interpolate_fit_never_writes_past_k_columns(env):
    """K = N - 1 on a matrix of full rank: the reference's factorization counts the single remaining column in
    (src/hyacin_potrfp.cu:271) and its interpolation then writes N columns into an X sized for K (src/gram_id.cpp:41).
    Here the rank comes back as K and the memory behind the K columns of X stays as it was."""
    from gpu_util import dev, zeros, ptr, sync, host
    ha, h = env
    rng = np.random.default_rng(45)
    M, N, K = 700, 12, 11
    A = rng.standard_normal((M, N))
    dA, lda = dev_matrix(A, "N")
    X = dev(np.full(N * (K + 2), 7.5))                 # two guard columns behind the K the caller asked for
    jp = zeros(4 * N)
    rank = ha.lib().hyacinInterpolateFit(C.byref(h), 1e-10, b"N", M, N, K, ptr(dA), lda, ptr(jp), ptr(X), N, 0, 0)
    sync()
    assert rank == K and ha.lib().hykLastStatus() == 0
    Xh = host(X, np.float64).reshape(K + 2, N).T
    assert np.all(Xh[:, K:] == 7.5)
    sel = host(jp, np.int32)[:K] - 1
    assert np.allclose(Xh[sel, :K], np.eye(K), atol=1e-12)
    assert np.linalg.norm(A - A[:, sel] @ Xh[:, :K].T) <= 1e-9 * np.linalg.norm(A) + np.linalg.svd(A, compute_uv=False)[-1] * 50


def test_segmented_fit(env, oracle):
    ha, h = env
    rng = np.random.default_rng(44)
    for at, opA in ((0, "N"), (3, "C"), (5, "C")):
        M, N, K = 3000, 640, 40                       # floor(sqrt(640/40)) = 4 segments
        eps = {0: 1e-8, 3: 1e-4, 5: 1e-2}[at]
        A0, s = low_rank(rng, M, N, 0.75, cplx=bool(at & 1))
        A = to_storage(A0, at)
        print("segmented", at, opA, flush=True)
        rank, S, V, err, nrm = run_tsvd(env, A, eps, K, opA, segmented=True)
        rank1, S1, V1, err1, _ = run_tsvd(env, A, eps, K, opA, segmented=False)
        assert 0 < rank <= K and abs(rank - rank1) <= 2
        k = min(rank, rank1)
        storage_eps = {0: 2.2e-16, 3: 1.2e-7, 5: 9.8e-4}[at]
        assert np.abs(S[:k] - S1[:k]).max() <= 20 * max(eps, storage_eps) * S1[0]
        assert err <= 4 * err1 + (20 * max(eps, storage_eps)) ** 2 * nrm


def test_degenerate_inputs(env, oracle):
    from gpu_util import dev, zeros, ptr, sync, host
    ha, h = env
    A = np.zeros((300, 20))
    dA = dev(A.T.copy())
    S, V = zeros(8 * 20), zeros(8 * 20 * 20)
    L = ha.lib()
    assert L.hyacinTsvdFit(C.byref(h), 1e-8, b"N", 300, 20, 0, ptr(dA), 300, ptr(S), ptr(V), 20, 0, 0) == 0       # K <= 0
    assert L.hyacinTsvdFit(C.byref(h), 1e-8, b"N", 300, 20, 20, ptr(dA), 300, ptr(S), ptr(V), 20, 0, 99) == 0     # unknown precision
    assert L.hyacinTsvdFit(C.byref(h), 1e-8, b"N", 300, 20, 20, ptr(dA), 300, ptr(S), ptr(V), 20, 0, 0) == 0      # zero matrix
    sync()
    jp = zeros(4 * 20)
    assert L.hyacinInterpolateFit(C.byref(h), 1e-8, b"N", 300, 20, 5, ptr(dA), 300, ptr(jp), ptr(V), 20, 0, 0) == 0
    assert L.hyacinCheckNorm(C.byref(h), b"N", 300, 20, ptr(dA), 300, 0, None, 20, 0) == 0.0
    # timers: off by default -> sync only
    ms = (C.c_double * 3)(ord("D"), ord("R"), ord("C"))
    L.hyacinSync_TimerSegments(C.byref(h), ms, 3)
    # a single non-zero column: rank 1, exact direction
    A[:, 3] = np.arange(300) + 1.0
    dA = dev(A.T.copy())
    assert L.hyacinTsvdFit(C.byref(h), 1e-8, b"N", 300, 20, 20, ptr(dA), 300, ptr(S), ptr(V), 20, 0, 0) == 1
    sync()
    Sh, Vh = host(S, np.float64), host(V, np.float64).reshape(20, 20).T
    assert abs(Sh[0] - np.linalg.norm(A[:, 3])) <= 1e-9 * Sh[0] and abs(abs(Vh[3, 0]) - 1) < 1e-12


def test_timer_segments(oracle):
    import os
    import hyacinth_amd as ha
    from gpu_util import dev, zeros, ptr, sync, stream
    os.environ["HYACIN_CREATE_TIMER"] = "1"
    try:
        h = ha.create_handle(stream=stream().value)
    finally:
        del os.environ["HYACIN_CREATE_TIMER"]
    rng = np.random.default_rng(45)
    A = rng.standard_normal((4000, 64))
    dA = dev(A.T.copy())
    S, V = zeros(8 * 64), zeros(8 * 64 * 64)
    assert ha.lib().hyacinTsvdFit(C.byref(h), 1e-6, b"N", 4000, 64, 64, ptr(dA), 4000, ptr(S), ptr(V), 64, 0, 0) > 0
    ms = (C.c_double * 4)(ord("D"), ord("R"), ord("C"), ord("x"))
    ha.lib().hyacinSync_TimerSegments(C.byref(h), ms, 4)
    assert ms[0] > 0 and ms[1] > 0 and ms[2] == 0 and ms[3] == 0
    ha.destroy_handle(h)


def _kahan(n, c):
    s = np.sqrt(1.0 - c * c)
    return (s ** np.arange(n))[:, None] * (np.triu(-c * np.ones((n, n)), 1) + np.eye(n)) * (1.0 - 1e-3 * np.arange(n))[None, :]


@pytest.mark.parametrize("gtype", [0, 6])                     # Gram in FP64, in double-double
@pytest.mark.parametrize("case", ["floor left out", "floor taken back in", "floor never factored"])
def test_gevd_leaves_out_floor_columns(case, gtype, capfd, monkeypatch):
    """hyacinXGevd (src/gram_evd.cu:94-142) with fewer values wanted than the Cholesky factor has rows: the rows of a noise
    floor are left out of the Jacobi sweeps when they cannot move a value by more than 2 eps sigma_1 (first case: the log says
    so, and the values still agree with numpy's to 10 eps sigma_1).  The choice is made from the row norms; in the second case
    they mislead (a Kahan matrix: its last singular value is 3e-5 of its last row's norm), the test with the values found
    fails, and the sweeps must take rows back in: value K is then the floor's, not the Kahan block's.  Third case: a floor
    right under the K wanted values, light enough for the Cholesky itself to end after K + 1 columns (hykPotrfpWanted); the
    values found confirm it, and they are within (trace left) / (2 sigma_K) of numpy's."""
    import hyacinth_amd as ha
    from gpu_util import dev, zeros, ptr, stream, sync, host
    rng = np.random.default_rng(8)
    if case == "floor left out":
        N, K, eps = 300, 20, 1e-8
        V = haar(rng, N, N, False)
        R = (np.concatenate([10.0 ** -np.linspace(0, 6, 40), np.full(N - 40, 1e-8)])[:, None]) * V.T     # singular values: 40 graded ones over a floor
    elif case == "floor never factored":
        N, K, eps = 300, 20, 1e-4
        V = haar(rng, N, N, False)
        R = (np.concatenate([10.0 ** -np.linspace(0, 2, K), np.full(N - K, 1e-5)])[:, None]) * V.T       # 20 values down to 1e-2 over a floor of 1e-5
    else:
        N, K, eps = 64, 24, 1e-6
        R = np.zeros((N, N))
        R[:24, :24] = _kahan(24, 0.6)
        R[24:, 24:] = 1e-5 * np.eye(N - 24)
    G = R.T @ R
    want = np.linalg.svd(R, compute_uv=False)
    monkeypatch.setenv("HYACIN_VERBOSE", "1")
    h = ha.create_handle(stream=stream().value)
    try:
        raw = np.zeros((N, N, 2 if gtype == 6 else 1)); raw[..., 0] = G.T
        dG, dS, dX = dev(raw), zeros(8 * K), zeros(8 * N * K)
        capfd.readouterr()
        rank = ha.lib().hyacinXGevd(C.byref(h), eps, N, K, 0, ptr(dX), N, ptr(dS), gtype, ptr(dG), N)
        sync()
        C.CDLL(None).fflush(None)                       # the log goes through the C library's buffered stdout
        log = capfd.readouterr().out
    finally:
        ha.destroy_handle(h)
    S = host(dS, np.float64, (K,))
    X = host(dX, np.float64, (K, N))[:rank]
    assert "are left out of the sweeps" in log
    if case == "floor never factored":
        assert "POTRFP: ended after %d columns" % (K + 1) in log and "factoring again" not in log
        assert rank == K and np.abs(S - want[:K]).max() <= (N - K) * 1e-10 / (2 * want[K - 1]) + 1e-14
    assert ("weigh too much, the sweeps go on with" in log) == (case == "floor taken back in")
    # in the second case the Cholesky itself ends early at first (what is left after K steps is the floor, well within its
    # estimate of the budget), the values found refute the estimate, and the matrix is factored again in full
    assert ("POTRFP: ended after" in log and "factoring again, in full" in log) == (case == "floor taken back in")
    assert 0 < rank <= K and np.abs(S[:rank] - want[:rank]).max() <= 10 * eps * want[0]
    assert np.abs(X @ X.T - np.eye(rank)).max() <= max(1e-12, np.sqrt(eps))   # what is guaranteed with K below the factor's rank (the sweeps may end on the values)
    if case == "floor taken back in":
        assert rank >= 23 and abs(S[rank - 1] - want[rank - 1]) <= 1e-11 and (rank < 24 or abs(S[23] - 1e-5) <= 1e-11)
    # the basis captures the matrix up to the values that are not handed out
    resid2 = (R ** 2).sum() - ((R @ X.T) ** 2).sum()
    assert abs(resid2 - (want[rank:] ** 2).sum()) <= (10 * eps) ** 2 * (want ** 2).sum() + 1e-6 * (want[rank:] ** 2).sum()


@pytest.mark.parametrize("at", [0, 3])
def test_fit_hands_out_orthogonal_vectors(env, at):
    """Singular values 2 % apart: the values stop moving several sweeps before their vectors are orthogonal.  What
    hyacinTsvdFit hands out as singular vectors is orthonormal to sqrt(eps) all the same (the reference takes what three
    sweeps of gesvdj leave, src/gram_evd.cu:148-150), or to the rounding of the storage type where that is coarser."""
    rng = np.random.default_rng(90 + at)
    M, N, K, eps = 1500, 256, 128, 1e-5
    cplx = bool(at & 1)
    U, W = haar(rng, M, N, cplx), haar(rng, N, N, cplx)
    A = to_storage((U * 2.0 ** (-np.arange(N) / 32.0)) @ W.conj().T, at)
    rank, S, V, err, nrm = run_tsvd(env, A, eps, K, "N")
    assert rank == K
    defect = np.abs(V.conj().T @ V - np.eye(rank)).max()
    print("orthogonality", at, defect, flush=True)
    assert defect <= max(np.sqrt(eps), 1e-5 if at >= 2 else 0.0)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_orthonormalised_vectors_keep_their_span(env, seed, capfd, monkeypatch):
    """A fit whose values settle before its vectors are orthogonal and whose energy cut hands out fewer than K vectors (nearly
    all columns wanted, the last few below the cut).  The vectors are then made orthonormal directly (the log says so), and
    that has to happen to exactly the vectors that are handed out: orthonormalised together with vectors that are dropped
    afterwards they would carry a share of those directions and lose as much of their own, which shows as a projection
    residual far above the oracle's (complex FP64 at eps = 1e-13: 6e-22 against 2e-26 when it went wrong)."""
    from oracle import ho as oracle
    from util import as_complex
    ha, h = env
    rng = np.random.default_rng(600 + seed)
    M, N, K, eps = 2267, 373, 364, 8.9e-14
    A0, _ = low_rank(rng, M, N, 0.68, cplx=True, noise=eps * 1e-2)
    A = to_storage(A0, 1)
    monkeypatch.setenv("HYACIN_VERBOSE", "1")
    h2 = ha.create_handle(stream=h.hipStream)
    try:
        capfd.readouterr()
        rank, S, V, err, nrm = run_tsvd((ha, h2), A, eps, K, "C")
        C.CDLL(None).fflush(None)
        log = capfd.readouterr().out
    finally:
        ha.destroy_handle(h2)
    r_o, S_o, V_o, g = oracle.tsvd_fit(A, eps, K)
    k = min(rank, r_o)
    print("rank", rank, "oracle", r_o, "orthonormalised" if "after an orthonormalisation step" in log else "by sweeps alone", flush=True)
    assert 0 < rank < K and abs(rank - r_o) <= 4
    assert "after an orthonormalisation step" in log
    Ac = as_complex(A).astype(np.complex128)
    mine, ref = oracle.check_norm(Ac, V), oracle.check_norm(Ac, V_o[:, :k])
    assert mine <= 2 * ref + (100 * eps * S_o[0]) ** 2, (mine, ref)
    assert np.abs(V[:, :rank].conj().T @ V[:, :rank] - np.eye(rank)).max() <= 2 * np.sqrt(eps)


@pytest.mark.parametrize("at,eps", [(0, 1e-12), (1, 1e-9), (2, 1e-5)])
def test_fit_with_global_rows(env, at, eps):
    """globalM above M (the rows of other devices, include/hyacin.h:67-113): the integer Gram gets the head-room of
    nextpow2(globalM) (src/hyacin_herk.cpp:52,57: one 63-bit limb more in the first case) and carries the same value, so the fit
    returns what it returns for globalM = M."""
    from gpu_util import zeros, ptr, sync, host
    ha, h = env
    rng = np.random.default_rng(95 + at)
    M, N, K = 1800, 120, 60
    A0, _ = low_rank(rng, M, N, 0.8, cplx=bool(at & 1), noise=eps * 1e-2)
    A = to_storage(A0, at)
    dA, lda = dev_matrix(A, "N")
    eb = {0: 8, 1: 16, 2: 4}[at]
    sb = eb // (1 + (at & 1))
    out = []
    for globalM in (0, 1 << 40):
        u, cP, lP, stride = ha.herk_batch_init(h, eps, globalM or M, N, at)
        S, V = zeros(sb * K), zeros(eb * N * K)
        rank = ha.lib().hyacinTsvdFit(C.byref(h), eps, b"N", M, N, K, ptr(dA), lda, ptr(S), ptr(V), N, globalM, at)
        sync()
        assert ha.lib().hykLastStatus() == 0
        real = {8: np.float64, 4: np.float32}[sb]
        out.append((rank, lP, host(S, real).astype(np.float64).copy(), host(V, real).astype(np.float64).copy()))
    (r0, l0, S0, V0), (r1, l1, S1, V1) = out
    assert l1 >= l0 + (at == 0) and r1 == r0 and r0 > 0           # the FP64 case crosses into a third limb
    tol = 4 * {0: 2.2e-16, 1: 2.2e-16, 2: 1.2e-7}[at]
    assert np.abs(S1 - S0).max() <= tol * S0[0]
    assert np.abs(V1 - V0).max() <= max(1e-9, 100 * tol)


def test_tail_options_of_the_handle(env):
    """QRCPTruncateRank and JacobiSVDSweeps (include/hyacin.h:44, src/gram_evd.cu:148-150): without the rank cut in the
    Cholesky (QRCPTruncateRank = 0, where the sweep count is |min(0, JacobiSVDSweeps)|, 0 standing for the backend without a
    budget) and with other sweep budgets the fit returns the values of the default settings; a budget of one (five plain
    sweeps here) still returns a basis whose projection residual is within a factor of the converged one."""
    ha, h = env
    rng = np.random.default_rng(97)
    M, N, K, eps = 1500, 96, 40, 1e-9
    A0, _ = low_rank(rng, M, N, 0.7, noise=1e-12)
    A = to_storage(A0, 0)
    base = run_tsvd(env, A, eps, K, "N")
    try:
        for trunc, sweeps, converged in ((0, 3, True), (0, -4, True), (1, -6, True), (1, 6, True), (1, 1, False)):
            h.QRCPTruncateRank, h.JacobiSVDSweeps = trunc, sweeps
            rank, S, V, err, nrm = run_tsvd(env, A, eps, K, "N")
            assert ha.lib().hykLastStatus() == 0
            print("tail options", trunc, sweeps, rank, err / nrm, flush=True)
            assert abs(rank - base[0]) <= (1 if converged else 3)
            k = min(rank, base[0])
            assert np.abs(S[:k] - base[1][:k]).max() <= (10 * eps if converged else 1e-3) * base[1][0]
            assert err <= (4 if converged else 100) * base[3] + (20 * eps) ** 2 * nrm
    finally:
        h.QRCPTruncateRank, h.JacobiSVDSweeps = 1, 3


def test_handle_settings_from_the_environment(monkeypatch):
    """hyacinCreate reads its settings from the environment variables the reference reads (src/utils.cpp:64-72), with the
    reference's defaults when they are not set."""
    import hyacinth_amd as ha
    from gpu_util import stream
    fields = ("GramMatrixAlgorithm", "StrideBatchPerfPenalty", "GramSegmentK", "TCGemmTargetK", "QuantizeBitCorrection", "QRCPTruncateRank", "JacobiSVDSweeps")
    names = ("HYACIN_GRAM_ALGORITHM", "HYACIN_STRIDE_BATCH_PERF_PENALTY", "HYACIN_GRAM_SEGMENT_K", "HYACIN_TCGEMM_TARGET_K", "HYACIN_QUANTIZE_BITS_CORR",
             "HYACIN_QRCP_TRUNCATE_RANK", "HYACIN_JACOBI_SVD_SWEEPS")
    for n in names:
        monkeypatch.delenv(n, raising=False)
    h = ha.create_handle(stream=stream().value)
    try:
        assert tuple(getattr(h, f) for f in fields) == (b"A", 1.3, 8192, 8192, 7, 1, 3)
    finally:
        ha.destroy_handle(h)
    for n, v in zip(names, ("L", "2.5", "4096", "1024", "12", "0", "-5")):
        monkeypatch.setenv(n, v)
    h = ha.create_handle(stream=stream().value)
    try:
        assert tuple(getattr(h, f) for f in fields) == (b"L", 2.5, 4096, 1024, 12, 0, -5)
    finally:
        ha.destroy_handle(h)


def test_two_handles_on_two_threads():
    """Two handles, each on a stream and a host thread of its own, fit different matrices at the same time: every result
    equals, bit for bit, what the same handle gives when it runs alone.  (The reference keeps all state on the handle,
    include/hyacin.h:20-53; a handle itself is used by one thread at a time.)"""
    import threading
    import torch
    import hyacinth_amd as ha
    from gpu_util import zeros, ptr
    from oracle import ho
    L = ha.lib()
    rng = np.random.default_rng(77)
    jobs = []
    for (M, N, K, cplx, eps) in ((2048, 192, 96, False, 1e-10), (1536, 128, 128, True, 1e-8)):
        A, _ = low_rank(rng, M, N, 0.9, cplx, noise=1e-13)
        A = to_storage(A, 1 if cplx else 0)
        at = ho.atype_of(A)
        dA, lda = dev_matrix(A, "N")
        eb = 16 if cplx else 8
        st = torch.cuda.Stream()
        jobs.append(dict(M=M, N=N, K=K, eps=eps, at=at, dA=dA, lda=lda, S=zeros(8 * K), V=zeros(eb * N * K), stream=st,
                         h=ha.create_handle(stream=st.cuda_stream)))
    torch.cuda.synchronize()

    def fit(j):
        j["S"].zero_(); j["V"].zero_(); torch.cuda.synchronize()
        rank = L.hyacinTsvdFit(C.byref(j["h"]), j["eps"], b"N", j["M"], j["N"], j["K"], ptr(j["dA"]), j["lda"], ptr(j["S"]), ptr(j["V"]), j["N"], 0, j["at"])
        j["stream"].synchronize()
        return rank, L.hykLastStatus(), j["S"].cpu().numpy().copy(), j["V"].cpu().numpy().copy()

    try:
        alone = [fit(j) for j in jobs]
        assert all(r[0] > 0 and r[1] == 0 for r in alone)
        together = [[], []]
        start = threading.Barrier(2)

        def worker(i):
            start.wait()
            for _ in range(4):
                together[i].append(fit(jobs[i]))

        threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        for i in range(2):
            assert len(together[i]) == 4
            for rank, status, S, V in together[i]:
                assert status == 0 and rank == alone[i][0]
                assert np.array_equal(S, alone[i][2]) and np.array_equal(V, alone[i][3])
    finally:
        torch.cuda.synchronize()
        for j in jobs:
            ha.destroy_handle(j["h"])


def test_two_gevd_tails_at_the_same_time():
    """hyacinXGevd (src/gram_evd.cu:94-142) on two handles, streams and host threads at once, at sizes whose Jacobi rounds put
    two workgroups on every block pair and fill the device (N = r = 2048 and N = r = 1024, real): while the other handle's
    kernels hold compute units, the two partners of a pair start at different times.  The rounds read one copy of the factor
    and write another, so the values and vectors are, bit for bit, those of each handle running alone."""
    import threading
    import torch
    import hyacinth_amd as ha
    from gpu_util import dev, zeros, ptr
    L = ha.lib()
    rng = np.random.default_rng(78)
    jobs = []
    for N in (2048, 1024):
        W = haar(rng, N, N, False)
        R = (2.0 ** (-np.arange(N) / (N / 24.0)))[:, None] * W.T                 # a dense factor, singular values over seven digits
        G = R.T @ R
        st = torch.cuda.Stream()
        jobs.append(dict(N=N, G0=dev(np.ascontiguousarray(G.T)), G=zeros(8 * N * N), S=zeros(8 * N), X=zeros(8 * N * N), stream=st, h=ha.create_handle(stream=st.cuda_stream)))
    torch.cuda.synchronize()

    def tail(j):
        with torch.cuda.stream(j["stream"]):                                        # the call overwrites G; no device-wide wait, the other handle keeps running
            j["G"].copy_(j["G0"]); j["S"].zero_(); j["X"].zero_()
        rank = L.hyacinXGevd(C.byref(j["h"]), 1e-9, j["N"], j["N"], 0, ptr(j["X"]), j["N"], ptr(j["S"]), 0, ptr(j["G"]), j["N"])
        j["stream"].synchronize()
        return rank, L.hykLastStatus(), j["S"].cpu().numpy().copy(), j["X"].cpu().numpy().copy()

    try:
        alone = [tail(j) for j in jobs]
        assert all(r[0] > j["N"] // 2 and r[1] == 0 for r, j in zip(alone, jobs))
        for (rank, _, S, X), j in zip(alone, jobs):                                  # and the vectors are an orthonormal set
            V = X.view(np.float64).reshape(j["N"], j["N"])[:rank]
            assert np.abs(V @ V.T - np.eye(rank)).max() <= 1e-9
        together = [[], []]
        start = threading.Barrier(2)

        def worker(i):
            start.wait()
            for _ in range(3 if i == 0 else 8):
                together[i].append(tail(jobs[i]))

        threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        for i in range(2):
            for rank, status, S, X in together[i]:
                assert status == 0 and rank == alone[i][0]
                assert np.array_equal(S, alone[i][2]) and np.array_equal(X, alone[i][3])
    finally:
        torch.cuda.synchronize()
        for j in jobs:
            ha.destroy_handle(j["h"])
