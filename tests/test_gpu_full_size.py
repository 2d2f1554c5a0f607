"""Size-independent checks at the full sizes of the benchmark configurations.

The oracle cannot finish M = 131072 ... 1048576 rows in seconds, but the path has an exact closed form for a matrix made
of a small integer block repeated down the rows: with integer entries every column scale is a power of two that keeps the
entries integral, so quantization is exact, the integer Gram is (M / m0) * A0^H A0 scaled by 2^(e_x + e_y), and the
dequantized Gram must equal (M / m0) * A0^H A0 to the last bit (in FP64 when it fits 52 bits, else in double-double).
One run therefore checks exponents, quantization, the int8 contraction over the full K with all its K splits and chunks,
reconstruction and dequantization at the real shape, through the hyacin.h stage API.
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

F64, F64C, F32, F32C, F16, F16C, DD, DDC = range(8)

# (name, type, M, N, eps, algorithm, |entries| bound, rows of the repeated block)
CASES = [
    ("target: real FP64 131072 x 2048, eps 1e-12, CRT", F64, 131072, 2048, 1e-12, b"A", 1 << 20, 64),
    ("config 2: real FP32 65536 x 1024, eps 1e-5, CRT", F32, 65536, 1024, 1e-5, b"A", 1 << 10, 64),
    ("config 3: complex FP64 131072 x 2048, eps 1e-12, CRT complex", F64C, 131072, 2048, 1e-12, b"A", 1 << 20, 64),
    ("config 4: complex FP16 262144 x 4096, eps 1e-3, limbs", F16C, 262144, 4096, 1e-3, b"L", 30, 32),
    ("config 5: real FP64 1048576 x 4096, eps 1e-8, CRT", F64, 1048576, 4096, 1e-8, b"A", 1 << 16, 32),
    ("config 1 at full size: real FP64 4096 x 256, eps 1e-10, limbs", F64, 4096, 256, 1e-10, b"L", 1 << 20, 64),
]


@pytest.fixture(scope="module")
def env():
    import torch
    import hyacinth_amd as ha
    from gpu_util import stream
    h = ha.create_handle(stream=stream().value)
    yield ha, h, torch
    ha.destroy_handle(h)


def block_and_gram(rng, at, N, bound, m0):
    """Integer block A0 (m0 x N, real or complex parts in [-bound, bound], last column scaled down to vary the exponents)
    and its exact Gram A0^H A0 as int64 (real, imaginary)."""
    re = rng.integers(-bound, bound + 1, (m0, N)).astype(np.int64)
    im = rng.integers(-bound, bound + 1, (m0, N)).astype(np.int64) if at & 1 else None
    re[:, N // 3] = 0                     # one all-zero column: INT_MAX exponent
    re[:, N // 2] //= max(1, bound // 3)  # one column with small entries: a different scale
    if im is not None:
        im[:, N // 3] = 0
        im[:, N // 2] //= max(1, bound // 3)
    if im is None:
        return re, None, re.T @ re, None
    gre = re.T @ re + im.T @ im
    gim = re.T @ im - im.T @ re           # Im (A^H A)[y, x] = sum re_y im_x - im_y re_x
    return re, im, gre, gim


@pytest.mark.parametrize("name,at,M,N,eps,alg,bound,m0", CASES, ids=[c[0].split(":")[0] for c in CASES])
def test_repeated_integer_block(env, name, at, M, N, eps, alg, bound, m0):
    ha, h, torch = env
    L = ha.lib()
    rng = np.random.default_rng(51)
    re, im, gre, gim = block_and_gram(rng, at, N, bound, m0)
    reps = M // m0
    real_t = {F64: torch.float64, F64C: torch.float64, F32: torch.float32, F32C: torch.float32, F16: torch.float16, F16C: torch.float16}[at]
    comps = 2 if at & 1 else 1
    blk = np.stack([re, im], axis=-1) if im is not None else re[..., None]            # [m0][N][comps]
    blk_d = torch.from_numpy(np.ascontiguousarray(np.transpose(blk, (1, 0, 2)))).to("cuda").to(real_t)   # [N][m0][comps]
    A = blk_d.unsqueeze(1).expand(N, reps, m0, comps).reshape(N, M, comps).contiguous()   # column-major M x N
    assert A.element_size() * A.numel() == M * N * comps * {torch.float64: 8, torch.float32: 4, torch.float16: 2}[real_t]
    print(name, "device bytes", A.element_size() * A.numel(), flush=True)

    h.GramMatrixAlgorithm = alg
    try:
        u, cP, lP, stride = ha.herk_batch_init(h, eps, M, N, at)
        seg = min(h.GramSegmentK, M)
        batches, lastM = (M + seg - 1) // seg, M - (M - 1) // seg * seg
        vexp = torch.zeros((batches + 1) * N, dtype=torch.int32, device="cuda")
        Cq = torch.zeros(cP * lP * stride, dtype=torch.int64, device="cuda")
        pA, pV, pC = C.c_void_p(A.data_ptr()), C.c_void_p(vexp.data_ptr()), C.c_void_p(Cq.data_ptr())
        L.hyacinXquantizeScaleBatch(C.byref(h), batches, seg, lastM, N, at, pA, M, u, pV)
        L.hyacinXherkBatch(C.byref(h), batches, seg, lastM, N, at, pA, M, u, pV, 0, lP, pC)
        gt, gb = C.c_int(), C.c_int32()
        L.hyacinXdequantizeInit(C.byref(h), N, lP, pC, pV, at, C.byref(gt), C.byref(gb))
        G = torch.zeros(N * N * gb.value, dtype=torch.uint8, device="cuda")
        L.hyacinXdequantize(C.byref(h), N, lP, pC, pV, gt.value, C.c_void_p(G.data_ptr()), N)
        torch.cuda.synchronize()
    finally:
        h.GramMatrixAlgorithm = b"A"
    del A

    # every column scale keeps the integer entries integral
    ve = vexp[:N].cpu().numpy()
    col_max = np.abs(re).max(axis=0) if im is None else np.maximum(np.abs(re).max(axis=0), np.abs(im).max(axis=0))
    assert np.all((ve == 2**31 - 1) == (col_max == 0))
    assert np.all(ve[col_max > 0] >= 0)

    gtype = gt.value
    assert (gtype & 1) == (at & 1) and (gtype & ~1) in (F32, F64, DD)
    width = {F32: 1, F64: 1, DD: 2}[gtype & ~1] * comps
    Gh = G.cpu().numpy().view(np.float32 if (gtype & ~1) == F32 else np.float64).reshape(N, N, width)   # [column x][row y][width]
    want_re = (gre * reps).T                                    # exact int64, indexed [x][y]
    want_im = (gim * reps).T if gim is not None else None
    assert np.abs(gre).max() * reps < 2**62
    if (gtype & ~1) == DD:
        got_re = Gh[..., 0].astype(np.int64) + Gh[..., 1].astype(np.int64)
        got_im = (Gh[..., 2].astype(np.int64) + Gh[..., 3].astype(np.int64)) if comps == 2 else None
        assert np.all(Gh == np.rint(Gh))
    else:
        assert np.abs(want_re).max() < 2**53 and ((gtype & ~1) == F64 or np.abs(want_re).max() < 2**24)
        got_re = Gh[..., 0].astype(np.float64).astype(np.int64)
        got_im = Gh[..., 1].astype(np.float64).astype(np.int64) if comps == 2 else None
        assert np.all(Gh == np.rint(Gh))
    assert np.array_equal(got_re, want_re), name
    if comps == 2:
        assert np.array_equal(got_im, want_im), name


@pytest.mark.parametrize("at,M,N,K,eps", [(F64, 16384, 2048, 1024, 1e-12), (F64C, 8192, 1024, 512, 1e-12), (F64, 8192, 4096, 256, 1e-7), (F64C, 6144, 3000, 128, 1e-6)],
                         ids=["real", "complex", "real-4096", "complex-3000"])
def test_fit_at_full_width(env, at, M, N, K, eps):
    """hyacinTsvdFit with the column counts of the benchmark configurations (the Cholesky and Jacobi kernels then run on
    every compute unit, with many workgroups exchanging data; above 2048 columns they take other variants): singular values against sqrt(eigvalsh(A^H A)) computed by
    torch in FP64, an orthonormal basis, and the same bits on a second run (every reduction order is fixed)."""
    ha, h, torch = env
    L = ha.lib()
    g = torch.Generator(device="cuda")
    g.manual_seed(97)
    cplx = at & 1
    scale = torch.pow(10.0, -torch.arange(N, device="cuda", dtype=torch.float64) / (N / 8.0))
    A = (torch.randn((N, M, 2 if cplx else 1), generator=g, device="cuda", dtype=torch.float64) * scale[:, None, None]).contiguous()
    outs = []
    for rep in range(2):
        S = torch.zeros(K, dtype=torch.float64, device="cuda")
        V = torch.zeros(N * K * (2 if cplx else 1), dtype=torch.float64, device="cuda")
        rank = L.hyacinTsvdFit(C.byref(h), eps, b"N", M, N, K, C.c_void_p(A.data_ptr()), M, C.c_void_p(S.data_ptr()), C.c_void_p(V.data_ptr()), N, 0, at)
        torch.cuda.synchronize()
        outs.append((rank, S, V))
    rank, S, V = outs[0]
    assert rank == K
    Am = torch.view_as_complex(A).reshape(N, M) if cplx else A.reshape(N, M)       # row j = column j of A
    G = Am.conj() @ Am.T                                                            # G[y, x] = sum_k conj(a_ky) a_kx
    ev = torch.linalg.eigvalsh(G).flip(0).clamp_min(0).sqrt()
    if eps <= 1e-10:
        rel = ((S - ev[:K]).abs() / ev[:K]).max().item()
        assert rel <= 1e-9, rel
    else:                                                        # the bar of the path: 10 eps of the largest value
        assert ((S - ev[:K]).abs().max() / ev[0]).item() <= 10 * eps
    Vm = (torch.view_as_complex(V.reshape(K, N, 2)) if cplx else V.reshape(K, N))   # row i = basis vector i
    eye = torch.eye(K, device="cuda", dtype=Vm.dtype)
    assert (Vm.conj() @ Vm.T - eye).abs().max().item() <= max(1e-12, eps)    # rotations stop at cosines of eps / 16
    # the basis spans the dominant right singular subspace: the residual of A outside it is the tail of the spectrum
    resid2 = (Am.abs() ** 2).sum().item() - ((Vm @ Am).abs() ** 2).sum().item()   # row i of Vm @ Am = (A v_i)^T
    tail2 = (ev[K:] ** 2).sum().item()
    assert abs(resid2 - tail2) <= 1e-6 * tail2 + max(1e-12, (10 * eps) ** 2) * (ev ** 2).sum().item()
    assert outs[1][0] == rank and torch.equal(outs[1][1], S) and torch.equal(outs[1][2], V)


# (name, entry point, type, opA, M, N, K, eps, algorithm, |entries| bound, rows of the repeated block)
API_CASES = [
    ("config 2: hyacinTsvdFit opA=T real FP32 65536 x 1024", "hyacinTsvdFit", F32, "T", 65536, 1024, 512, 1e-5, b"A", 1 << 10, 64),
    ("config 4: hyacinTsvdFit opA=C complex FP16 262144 x 4096, limbs", "hyacinTsvdFit", F16C, "C", 262144, 4096, 256, 1e-3, b"L", 30, 32),
    ("config 4 segmented: hyacinTsvdFitSegmentN on the same matrix (four column segments, complex FP16 stage products)", "hyacinTsvdFitSegmentN", F16C, "C", 262144, 4096, 256, 1e-3, b"L", 30, 32),
    ("config 5: hyacinInterpolateFit real FP64 1048576 x 4096", "hyacinInterpolateFit", F64, "N", 1048576, 4096, 2048, 1e-8, b"A", 1 << 16, 32),
    ("config 3: hyacinTsvdFitSegmentN complex FP64 131072 x 2048", "hyacinTsvdFitSegmentN", F64C, "N", 131072, 2048, 1024, 1e-12, b"A", 1 << 20, 64),
]


@pytest.mark.parametrize("name,fit,at,opA,M,N,K,eps,alg,bound,m0", API_CASES, ids=[c[0].split(":")[0] + " fit" for c in API_CASES])
def test_fit_entry_points_at_configuration_size(env, name, fit, at, opA, M, N, K, eps, alg, bound, m0):
    """The fit each configuration names (include/hyacin.h:67-113), at its size, storage order and type, on the repeated
    integer block: the matrix has exactly the rank of the block (its rows), so the fit must stop there; its singular values
    are sqrt(M / m0) times the block's; the basis must capture the matrix (hyacinCheckNorm <= (10 eps)^2 |A|^2), the
    interpolation must reproduce the block from the chosen columns."""
    ha, h, torch = env
    L = ha.lib()
    rng = np.random.default_rng(77)
    re, im, _, _ = block_and_gram(rng, at, N, bound, m0)
    re[:, N // 3] = rng.integers(1, bound + 1, m0)        # no all-zero column here: every column can be a pivot
    if im is not None:
        im[:, N // 3] = rng.integers(1, bound + 1, m0)
    reps = M // m0
    cplx = at & 1
    real_t = {F64: torch.float64, F64C: torch.float64, F32: torch.float32, F16C: torch.float16}[at]
    A0 = (re + 1j * im) if cplx else re.astype(np.float64)                              # the block, m0 x N
    if at in (F16, F16C):
        A0 = A0 * 2.0 ** -6                      # singular values of the order of 2000: the half-precision S can hold them
    stored = np.conj(A0) if opA == "C" else A0                                          # op(stored) = A
    blk = np.stack([stored.real, stored.imag], axis=-1) if cplx else stored[..., None]  # [m0][N][comps]
    comps = 2 if cplx else 1
    if opA == "N":                                                                      # column-major M x N: [N][M][comps]
        blk_d = torch.from_numpy(np.ascontiguousarray(np.transpose(blk, (1, 0, 2)))).to("cuda").to(real_t)
        A = blk_d.unsqueeze(1).expand(N, reps, m0, comps).reshape(N, M, comps).contiguous(); lda = M
    else:                                                                               # the stored N x M matrix: [M][N][comps]
        blk_d = torch.from_numpy(np.ascontiguousarray(blk)).to("cuda").to(real_t)
        A = blk_d.unsqueeze(0).expand(reps, m0, N, comps).reshape(M, N, comps).contiguous(); lda = N
    print(name, "device bytes", A.element_size() * A.numel(), flush=True)
    pA = C.c_void_p(A.data_ptr())
    S = torch.zeros(max(K, N), dtype=torch.float64, device="cuda")
    V = torch.zeros(N * K * comps, dtype=real_t, device="cuda")
    h.GramMatrixAlgorithm = alg
    try:
        rank = getattr(L, fit)(C.byref(h), eps, opA.encode(), M, N, K, pA, lda, C.c_void_p(S.data_ptr()), C.c_void_p(V.data_ptr()), N, 0, at)
        torch.cuda.synchronize()
        assert L.hykLastStatus() == 0
        assert rank == m0, (rank, m0)
        want = np.linalg.svd(A0, compute_uv=False) * np.sqrt(reps)
        storage_eps = {torch.float64: 2.2e-16, torch.float32: 6e-8, torch.float16: 4.9e-4}[real_t]
        if fit == "hyacinInterpolateFit":
            jp = S.view(torch.int32)[:N].cpu().numpy()
            assert sorted(jp.tolist()) == list(range(1, N + 1))
            X = V.cpu().numpy().reshape(K, N).T[:, :rank]                               # N x rank
            sel = jp[:rank] - 1
            assert np.allclose(X[sel], np.eye(rank), atol=1e-12)
            assert np.linalg.norm(A0 - A0[:, sel] @ X.T) <= 50 * max(eps, storage_eps) * np.linalg.norm(A0)
        else:
            Sh = S.view(real_t)[:K].double().cpu().numpy()
            assert np.all(Sh[rank:] == 0)
            assert np.abs(Sh[:rank] - want[:rank]).max() <= 10 * max(eps, storage_eps) * want[0]
            err = L.hyacinCheckNorm(C.byref(h), opA.encode(), M, N, pA, lda, rank, C.c_void_p(V.data_ptr()), N, at)
            nrm = L.hyacinCheckNorm(C.byref(h), opA.encode(), M, N, pA, lda, 0, None, N, at)
            assert abs(nrm - (np.abs(A0) ** 2).sum() * reps) <= 1e-9 * nrm
            assert err <= (10 * max(eps, storage_eps)) ** 2 * nrm, (err, nrm)
    finally:
        h.GramMatrixAlgorithm = b"A"
