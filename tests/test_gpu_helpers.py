"""The small kernels around the factorizations, each called directly through the C ABI and held to numpy:
converting copies and transposes (src/matcopy.cu:23-96), sums of squares (the nrm2 calls of src/lra.cpp:170,204),
the panel padding (the memset of src/hyacin_herk.cpp:154,261,275), the copies around the SVD and the interpolation
(src/gram_evd.cu:110-137, src/gram_id.cpp:40-46, scatter modes 'U' / 'I' of src/matcopy.cu:48-52) and the
re-orthonormalisation (geqrf + orgqr of src/lra.cpp:176-191)."""
import numpy as np
import pytest

import hyacinth_amd as ha

pytestmark = pytest.mark.gpu

NP_REAL = {ha.F64: np.float64, ha.F32: np.float32, ha.F16: np.float16}


@pytest.fixture(scope="module")
def L():
    return ha.lib()


def to_storage(Z, t):
    """Complex or real numpy matrix -> bytes of a column-major array of precision t with leading dimension ld (padding NaN)."""
    real = NP_REAL[t & ~1]
    if t & 1:
        return np.stack([Z.real, Z.imag], axis=-1).astype(real)
    return Z.astype(real)


def colmajor(Zs, ld, fill=np.nan):
    """[rows, cols(, 2)] storage array -> [cols, ld(, 2)] buffer (column-major with padding rows)."""
    rows, cols = Zs.shape[0], Zs.shape[1]
    buf = np.full((cols, ld) + Zs.shape[2:], fill, dtype=Zs.dtype)
    buf[:, :rows] = np.swapaxes(Zs, 0, 1)
    return buf


def from_buffer(buf, rows):
    out = np.swapaxes(buf[:, :rows], 0, 1)
    return out[..., 0].astype(np.float64) + 1j * out[..., 1].astype(np.float64) if out.ndim == 3 else out.astype(np.float64)


@pytest.mark.parametrize("mode", ["A", "T", "C"])
@pytest.mark.parametrize("src,dst", [(ha.F64, ha.F64), (ha.F32, ha.F64), (ha.F16, ha.F64), (ha.F64, ha.F32), (ha.F64, ha.F16), (ha.F32, ha.F32), (ha.F16, ha.F16),
                                     (ha.F64C, ha.F64C), (ha.F32C, ha.F64C), (ha.F16C, ha.F64C), (ha.F64C, ha.F32C), (ha.F16C, ha.F16C), (ha.F32C, ha.F32C)])
@pytest.mark.parametrize("M,N,pa,pb", [(45, 19, 0, 0), (77, 130, 5, 3), (256, 64, 1, 0)])
def test_matcopy(L, mode, src, dst, M, N, pa, pb):
    """B (M x N, ldb) = op(A) with conversion; A is M x N for 'A' and N x M for 'T' / 'C'.  Sizes off the 32 x 32 tiles,
    padded leading dimensions on both sides; the padding of B is left alone."""
    from gpu_util import dev, ptr, stream, sync, host
    rng = np.random.default_rng(50 + src * 12 + dst)
    cplx = src & 1
    Z = rng.standard_normal((M, N)) + (1j * rng.standard_normal((M, N)) if cplx else 0)
    Zs = to_storage(Z, src)                                        # what the source really holds after its rounding
    Zv = from_buffer(colmajor(Zs, M), M)
    srcM = Zs if mode == "A" else np.swapaxes(Zs, 0, 1)            # stored matrix: M x N, or N x M for the transposed modes
    if mode == "C" and cplx:
        srcM = srcM.copy(); srcM[..., 1] = -srcM[..., 1]           # stored = conj(transpose) so that op(stored) = Z
    lda, ldb = srcM.shape[0] + pa, M + pb
    dA = dev(colmajor(srcM, lda))
    out0 = np.full((N, ldb) + ((2,) if cplx else ()), 7.0, dtype=NP_REAL[dst & ~1])
    dB = dev(out0)
    assert L.hykMatcopy(stream(), mode.encode(), M, N, src, ptr(dA), lda, dst, ptr(dB), ldb) == 0
    sync()
    got = host(dB, NP_REAL[dst & ~1], out0.shape)
    want = to_storage(Zv, dst)
    assert np.array_equal(np.swapaxes(got[:, :M], 0, 1), want)
    assert (got[:, M:] == 7.0).all()


def test_matcopy_limits(L):
    from gpu_util import zeros, ptr, stream
    t = zeros(64)
    assert L.hykMatcopy(stream(), b"A", 0, 5, ha.F64, ptr(t), 1, ha.F64, ptr(t), 1) == 0          # empty: nothing to do
    assert L.hykMatcopy(stream(), b"A", 1, 1, ha.F64, ptr(t), 1, ha.F64C, ptr(t), 1) == -1        # real -> complex is not a copy
    assert L.hykMatcopy(stream(), b"A", 1, 1, ha.DD, ptr(t), 1, ha.F64, ptr(t), 1) == -1


@pytest.mark.parametrize("M,N,pad", [(1, 1, 0), (300, 7, 5), (5000, 300, 0), (70000, 3, 11)])
def test_sum_squares(L, M, N, pad):
    from gpu_util import dev, ptr, stream, sync, host
    rng = np.random.default_rng(60)
    A = rng.standard_normal((N, M + pad))
    dA, out = dev(A), dev(np.array([2.5]))
    assert L.hykSumSquares(stream(), M, N, ptr(dA), M + pad, ptr(out)) == 0
    sync()
    want = 2.5 + (A[:, :M] ** 2).sum()
    assert abs(host(out, np.float64)[0] - want) <= 1e-13 * want


def test_zero_rows(L):
    from gpu_util import dev, ptr, stream, sync, host
    ldb, cols = 640, 37
    B = np.full((cols, ldb), 9, np.int8)
    for row0, row1 in ((0, 0), (5, 6), (131, 256), (500, 640), (3, 637)):
        dB = dev(B)
        assert L.hykZeroRows(stream(), ptr(dB), ldb, cols, row0, row1) == 0
        sync()
        want = B.copy(); want[:, row0:row1] = 0
        assert np.array_equal(host(dB, np.int8, B.shape), want)


@pytest.mark.parametrize("wide", [1, 0])
@pytest.mark.parametrize("cplx", [0, 1])
@pytest.mark.parametrize("dd", [0, 1])
def test_factor_to_b(L, cplx, dd, wide):
    """B[c, k] = conj(R[k, c]) (high words of a double-double factor), src/gram_evd.cu:110-117, in doubles or rounded to floats
    (the precision the SVD of that storage type runs in, src/gram_evd.cu:96-98)."""
    from gpu_util import dev, zeros, ptr, stream, sync, host
    rng = np.random.default_rng(61)
    N, rank, ldr = 70, 33, 40
    WR = 2 if dd else 1
    WE = WR * (2 if cplx else 1)
    Rt = rng.standard_normal((N, ldr, WE))
    real = np.float64 if wide else np.float32
    dR, B = dev(Rt), zeros(N * rank * (8 if wide else 4) * (1 + cplx))
    assert L.hykFactorToB(stream(), N, rank, (6 if dd else 0) + cplx, ptr(dR), ldr, (0 if wide else 2) + cplx, ptr(B)) == 0
    sync()
    got = host(B, real, (rank, N, 1 + cplx))
    assert np.array_equal(got[..., 0], Rt[:, :rank, 0].T.astype(real))
    if cplx:
        assert np.array_equal(got[..., 1], (-Rt[:, :rank, WR].T).astype(real))
    assert L.hykFactorToB(stream(), N, rank, (6 if dd else 0) + cplx, ptr(dR), ldr, 1 - cplx, ptr(B)) == -1     # real factor, complex B


@pytest.mark.parametrize("wide", [1, 0])
@pytest.mark.parametrize("atype", [ha.F64, ha.F32, ha.F16, ha.F64C, ha.F32C, ha.F16C])
def test_basis_and_values_out(L, atype, wide):
    """X[:, j] = B[:, order[j]] / sigma[order[j]] in the storage type (a zero column stays zero); S in the real storage type."""
    from gpu_util import dev, ptr, stream, sync, host
    rng = np.random.default_rng(62)
    cplx, real = atype & 1, NP_REAL[atype & ~1]
    N, r, ldx = 50, 9, 57
    B = rng.standard_normal((r, N, 1 + cplx)).astype(np.float64 if wide else np.float32)
    sigma = rng.uniform(0.5, 2.0, r); sigma[4] = 0.0
    order = rng.permutation(r).astype(np.int32)[:7]
    X0 = np.full((7, ldx, 1 + cplx), 3.0, real)
    dB, dS, dO, dX = dev(B), dev(sigma), dev(order), dev(X0)
    assert L.hykBasisOut(stream(), N, 7, atype, (0 if wide else 2) + cplx, ptr(dB), ptr(dS), ptr(dO), ptr(dX), ldx) == 0
    sync()
    got = host(dX, real, X0.shape)
    inv = np.where(sigma > 0, 1.0 / np.where(sigma > 0, sigma, 1.0), 0.0)
    want = (B[order].astype(np.float64) * inv[order][:, None, None]).astype(real)
    assert np.array_equal(got[:, :N], want) and (got[:, N:] == 3.0).all()
    S = rng.uniform(0, 3, 11)
    dSi, dSo = dev(S), dev(np.zeros(11, real))
    assert L.hykValuesOut(stream(), 11, atype, ptr(dSi), ptr(dSo)) == 0
    sync()
    assert np.array_equal(host(dSo, real), S.astype(real))


@pytest.mark.parametrize("atype", [ha.F64, ha.F32C, ha.F16])
def test_interp_out(L, atype):
    """Row jpiv[x]-1 of X is the unit row x (x < K) or conj(T[:, x-K]) (scatter mode 'I', src/matcopy.cu:48-52)."""
    from gpu_util import dev, ptr, stream, sync, host
    rng = np.random.default_rng(63)
    cplx, real = atype & 1, NP_REAL[atype & ~1]
    N, K, ldx = 41, 13, 44
    jpiv = (rng.permutation(N) + 1).astype(np.int32)
    T = rng.standard_normal((N - K, K, 1 + cplx))                  # [column x-K][row y]
    X0 = np.full((K, ldx, 1 + cplx), 5.0, real)
    dJ, dT, dX = dev(jpiv), dev(T), dev(X0)
    assert L.hykInterpOut(stream(), N, K, atype, ptr(dJ), ptr(dT), ptr(dX), ldx) == 0
    sync()
    got = host(dX, real, X0.shape)
    want = X0.copy()
    for x in range(N):
        row = jpiv[x] - 1
        if x < K:
            want[:, row, :] = 0
            want[x, row, 0] = 1
        else:
            want[:, row, 0] = T[x - K, :, 0].astype(real)
            if cplx:
                want[:, row, 1] = (-T[x - K, :, 1]).astype(real)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("cplx", [0, 1])
@pytest.mark.parametrize("N,r", [(64, 1), (300, 40), (1100, 130)])
def test_orthonormalize(L, cplx, N, r):
    """Columns become orthonormal and keep their span (the Q of a QR factorization spans the same space)."""
    from gpu_util import dev, zeros, ptr, stream, sync, host
    rng = np.random.default_rng(64 + N)
    V = rng.standard_normal((N, r)) + (1j * rng.standard_normal((N, r)) if cplx else 0)
    V = V @ (np.eye(r) + 0.3 * rng.standard_normal((r, r)))       # correlated columns
    buf = np.stack([V.real, V.imag], axis=-1) if cplx else V
    dV = dev(np.ascontiguousarray(np.swapaxes(buf, 0, 1)))
    work = zeros(r * 16 + 64)
    assert L.hykOrthonormalize(stream(), cplx, N, r, ptr(dV), N, ptr(work)) == 0
    sync()
    g = host(dV, np.float64, (r, N, 2) if cplx else (r, N))
    Q = (g[..., 0] + 1j * g[..., 1]).T if cplx else g.T
    assert np.abs(Q.conj().T @ Q - np.eye(r)).max() <= 1e-12
    Qr, _ = np.linalg.qr(V)
    assert np.abs(Q - Qr @ (Qr.conj().T @ Q)).max() <= 1e-12       # nothing of Q lies outside span(V)
    assert L.hykOrthonormalize(stream(), cplx, N, r, ptr(dV), N + 1, ptr(work)) == -1


@pytest.mark.parametrize("cplx", [0, 1])
@pytest.mark.parametrize("wide", [1, 0])
@pytest.mark.parametrize("n,pad", [(2, 0), (37, 3), (300, 0)])
def test_max_cosine(L, cplx, n, pad, wide):
    """hykMaxCosine: the largest |G[p, q]|^2 / (G[p, p] G[q, q]) over the marked pairs of a Gram matrix, against numpy;
    unmarked columns do not count, a zero diagonal entry under a non-zero product counts as 1."""
    from gpu_util import dev, zeros, ptr, stream, sync, host
    rng = np.random.default_rng(70 + n)
    X = rng.standard_normal((2 * n, n)) + (1j * rng.standard_normal((2 * n, n)) if cplx else 0)
    X[:, 0] *= 1e-9
    G = X.conj().T @ X
    ld = n + pad
    buf = np.full((n, ld, 2) if cplx else (n, ld), np.nan, np.float64 if wide else np.float32)   # [column][row]: column-major with padding rows
    if cplx:
        buf[:, :n, 0] = G.real.T
        buf[:, :n, 1] = G.imag.T
    else:
        buf[:, :n] = G.T
    mark = (rng.random(n) < 0.7).astype(np.int32)
    mark[:2] = 1
    dG, dM, out = dev(buf), dev(mark), zeros(8)
    assert L.hykMaxCosine(stream(), (0 if wide else 2) + cplx, n, ptr(dG), ld, ptr(dM), ptr(out)) == 0
    sync()
    if not wide:                                                    # what the kernel saw
        G = (buf[:, :n, 0] + 1j * buf[:, :n, 1]).T.astype(np.complex128) if cplx else buf[:, :n].T.astype(np.float64)
    d = np.real(np.diag(G))
    c2 = np.abs(G) ** 2 / np.outer(d, d)
    keep = np.outer(mark, mark).astype(bool) & ~np.eye(n, dtype=bool)
    want = c2[keep].max()
    got = host(out, np.float64)[0]
    assert abs(got - want) <= 1e-12 * want
    assert L.hykMaxCosine(stream(), (0 if wide else 2) + cplx, n, ptr(dG), n - 1, ptr(dM), ptr(out)) == -1


@pytest.mark.parametrize("cplx", [0, 1])
@pytest.mark.parametrize("wide", [1, 0])
@pytest.mark.parametrize("n,pad", [(1, 0), (37, 3), (300, 0)])
def test_max_defect(L, cplx, n, pad, wide):
    """hykMaxDefect: the largest |G[p, q] - delta_pq|^2 over p <= q of the Gram matrix of nearly orthonormal columns, against
    numpy; once with the largest entry on the diagonal (a column whose norm is off), once off it."""
    from gpu_util import dev, zeros, ptr, stream, sync, host
    rng = np.random.default_rng(75 + n)
    for where in ("diagonal", "off"):
        Q, _ = np.linalg.qr(rng.standard_normal((2 * n + 3, n)) + (1j * rng.standard_normal((2 * n + 3, n)) if cplx else 0))
        X = Q + 1e-3 * (rng.standard_normal(Q.shape) + (1j * rng.standard_normal(Q.shape) if cplx else 0)) / np.sqrt(Q.shape[0])
        if where == "diagonal":
            X[:, n // 2] *= 1.01
        elif n > 1:
            X[:, 0] += 0.02 * X[:, n - 1]
        G = X.conj().T @ X
        ld = n + pad
        buf = np.full((n, ld, 2) if cplx else (n, ld), np.nan, np.float64 if wide else np.float32)   # [column][row]
        if cplx:
            buf[:, :n, 0] = G.real.T
            buf[:, :n, 1] = G.imag.T
        else:
            buf[:, :n] = G.T
        dG, out = dev(buf), zeros(8)
        assert L.hykMaxDefect(stream(), (0 if wide else 2) + cplx, n, ptr(dG), ld, ptr(out)) == 0
        sync()
        if not wide:                                                # what the kernel saw
            G = (buf[:, :n, 0] + 1j * buf[:, :n, 1]).T.astype(np.complex128) if cplx else buf[:, :n].T.astype(np.float64)
        want = (np.abs(np.triu(G - np.eye(n)).T) ** 2).max()        # entries p <= q (column q, row p)
        got = host(out, np.float64)[0]
        assert abs(got - want) <= 1e-12 * want
        assert (np.argmax(np.abs(G - np.eye(n))) % (n + 1) == 0) == (where == "diagonal" or n == 1)
    assert L.hykMaxDefect(stream(), (0 if wide else 2) + cplx, 5, ptr(dG), 4, ptr(out)) == -1
    # hykNewtonSchulzFactor: G <- (3 I - G) / 2 in place, padding rows untouched
    assert L.hykNewtonSchulzFactor(stream(), (0 if wide else 2) + cplx, n, ptr(dG), ld) == 0
    sync()
    got = host(dG, buf.dtype, buf.shape)
    T = (got[:, :n, 0] + 1j * got[:, :n, 1]).T if cplx else got[:, :n].T
    assert np.allclose(T, (3 * np.eye(n) - G) / 2, rtol=0, atol=1e-6 if not wide else 1e-15)
    assert np.isnan(got[:, n:]).all()
    assert L.hykNewtonSchulzFactor(stream(), (0 if wide else 2) + cplx, 5, ptr(dG), 4) == -1
