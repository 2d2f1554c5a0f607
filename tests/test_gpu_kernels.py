"""HIP kernel layer against the CPU oracle, through the C ABI. Integer results must be bit-exact."""
import ctypes as C

import numpy as np
import pytest

from util import ALL_KINDS, INT_MAX, haar, rand_matrix

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gl():
    from gpu_util import Lib
    return Lib()


def special(rng, M, N, kind):
    A = rand_matrix(rng, M, N, kind, 2.0)
    flat = A
    flat[:, 1] = 0
    flat[min(3, M - 1), 2] = 0
    return A


@pytest.mark.parametrize("kind", ALL_KINDS)
def test_column_exponents(gl, oracle, kind):
    rng = np.random.default_rng(31)
    for (M, N, segM) in [(70, 9, 16), (1000, 33, 256), (513, 5, 513)]:
        A = special(rng, M, N, kind)
        batches, lastM = (M + segM - 1) // segM, M - (M - 1) // segM * segM
        for u in (23, 46, -1):
            got = gl.column_exponents(A, batches, segM, lastM, u)
            want = oracle.quantize_scale_batch(A, batches, segM, lastM, u)
            n = len(want) if u >= 0 else N
            print("exponents", kind, M, N, segM, u, flush=True)
            assert np.array_equal(got[:n], want[:n])


def test_slice_range_and_gram_range(gl, oracle):
    import torch
    from gpu_util import dev, zeros, ptr, stream, sync, host
    rng = np.random.default_rng(32)
    A = rand_matrix(rng, 640, 40, "f64", 1.0)
    A[128:256] *= 1e-5
    A[384:512] = 0
    vexp = oracle.quantize_scale_batch(A, 5, 128, 128, 33)
    dv, segU = dev(vexp), zeros(4 * 5)
    assert gl.L.hykSliceRange(stream(), 5, 40, 33, ptr(dv), ptr(segU)) == 0
    sync()
    assert np.array_equal(host(segU, np.int32), oracle.vector_range(5, 40, 33, vexp))
    for lP, eps in ((1, 1e-3), (2, 1e-10), (3, 1e-15)):
        pl = oracle.fit_plan(640, 40, eps, 0, corr=7 if lP < 3 else 20, segK=128)
        v = oracle.quantize_scale_batch(A, 5, 128, 128, pl["u"])
        Cq = oracle.herk_batch(A, 5, 128, 128, pl["u"], v, pl["lP"])
        out = zeros(4)
        dC, dv = dev(Cq), dev(v)                  # named: a temporary would hand its memory back before the kernel has run
        assert gl.L.hykGramRange(stream(), 40, pl["lP"], ptr(dC), ptr(dv), ptr(out)) == 0
        sync()
        assert host(out, np.int32)[0] == oracle.dequantize_init(40, pl["lP"], Cq, v, 0)[2]


@pytest.mark.parametrize("kind", ALL_KINDS)
def test_quantize_panels_bit_exact(gl, oracle, kind):
    rng = np.random.default_rng(33)
    cplx = kind.startswith("c")
    for (M, N) in [(37, 5), (1029, 12)]:
        A = special(rng, M, N, kind)
        for u in (5, 23, 46, 62, 81):
            vexp = oracle.quantize_scale_batch(A, 1, M, M, u)
            for order in (1, 3, 6, 11):
                print("limbs", kind, M, N, u, order, flush=True)
                want = oracle.quantize("limbs", A, order, vexp, ldb=M + 11)
                got = gl.quantize("limbs", A, order, vexp, ldb=M + 11)
                assert np.array_equal(got, want)
            for order in ((1, 7, 15, 20, 21, 25) if cplx else (1, 8, 14, 24)):
                print("crt", kind, M, N, u, order, flush=True)
                want = oracle.quantize("crt", A, order, vexp, ldb=M + 3)
                for mb in (0, u + 1):
                    got = gl.quantize("crt", A, order, vexp, ldb=M + 3, max_bits=mb)
                    assert np.array_equal(got, want)
    # rows appended at an odd offset of an existing panel set (byte-store path)
    A = special(rng, 50, 4, kind)
    vexp = oracle.quantize_scale_batch(A, 1, 50, 50, 30)
    want = oracle.quantize("limbs", A, 4, vexp)
    got = gl.quantize("limbs", A, 4, vexp, ldb=64, row_offset=7)
    assert np.array_equal(got[:, :, 7:57], want) and not got[:, :, :7].any() and not got[:, :, 57:].any()


@pytest.mark.parametrize("cplx", [False, True])
def test_limb_digits_at_the_integer_width_limits(gl, oracle, cplx):
    """The limb encoder takes the digits of small values from 32- and 64-bit integers (below 2^29 and 2^50) and of the rest
    from the 96-bit path: integers on both sides of the two limits, of both signs, alone in their group of four rows and
    mixed with small ones, must give the oracle's digits (reference: src/quantize_limbs.cu:14-58)."""
    edge = [2 ** 29 - 1, 2 ** 29, 2 ** 29 + 1, 2 ** 50 - 1, 2 ** 50, 2 ** 50 + 1, 2 ** 52 + 1, 3, 0, 1]
    vals = []
    for e in edge:
        vals += [e, 0, 0, 0, -e, 1, -1, 2, 5, e, -7, 100, -e, -e, e, e]          # groups of four rows
    vals += [2 ** 28, 2 ** 28, 2 ** 28, 2 ** 28, -(2 ** 49), 2 ** 49, 2 ** 49, -(2 ** 49)]
    col = np.array(vals, dtype=np.float64)
    M = len(col)
    A = np.zeros((M, 3), dtype=np.complex128 if cplx else np.float64)
    A[:, 0] = col
    A[:, 1] = col[::-1]
    A[:, 2] = np.roll(col, 5)
    if cplx:
        A[:, 0] += 1j * np.roll(col, 3)          # re + im reaches 2^53: the sum's own carry into the next width
        A[:, 1] -= 1j * col
    A[0, :] = 2.0 ** 60                          # the column maximum: with u = 61 the exponent is 0 and q = x
    vexp = oracle.quantize_scale_batch(A, 1, M, M, 61)
    assert not vexp[:3].any()
    for order in (4, 8, 11):
        want = oracle.quantize("limbs", A, order, vexp, ldb=M + 4)
        got = gl.quantize("limbs", A, order, vexp, ldb=M + 4)
        assert np.array_equal(got, want), order
        got_t = gl.quantize_op("limbs", A, "C" if cplx else "T", order, vexp, ldb=M + 4)
        assert np.array_equal(got_t, want), order


@pytest.mark.parametrize("op", ["T", "C"])
@pytest.mark.parametrize("kind", ALL_KINDS)
def test_transposed_storage_bit_exact(gl, oracle, kind, op):
    """opA = 'T' / 'C' without a transposed copy (the reference copies first, src/lra.cpp:63-69): exponents and panels read
    from the stored N x M matrix equal the oracle's on op(A), bit for bit.  Leading dimension above N, sizes off the
    128 x 32 / 64 tiles, several row slices, a zero column, both residue paths, limbs."""
    rng = np.random.default_rng(133)
    cplx = kind.startswith("c")
    for (M, N, segM, pad) in [(70, 9, 16, 0), (300, 45, 128, 3), (1029, 70, 1029, 8), (257, 130, 100, 1)]:
        A = special(rng, M, N, kind)
        batches, lastM = (M + segM - 1) // segM, M - (M - 1) // segM * segM
        for u in (23, 46):
            print("transposed exponents", kind, op, M, N, segM, u, flush=True)
            want = oracle.quantize_scale_batch(A, batches, segM, lastM, u)
            got = gl.column_exponents_op(A, op, batches, segM, lastM, u, pad)
            assert np.array_equal(got[:len(want)], want)
        for u in (23, 62):
            vexp = oracle.quantize_scale_batch(A, 1, M, M, u)
            print("transposed limbs", kind, op, M, N, u, flush=True)
            assert np.array_equal(gl.quantize_op("limbs", A, op, 4, vexp, ldb=M + 5, pad=pad), oracle.quantize("limbs", A, 4, vexp, ldb=M + 5))
            order = 21 if cplx else 14
            want = oracle.quantize("crt", A, order, vexp, ldb=M + 3)
            for mb in (0, u + 1):
                print("transposed crt", kind, op, M, N, u, order, mb, flush=True)
                assert np.array_equal(gl.quantize_op("crt", A, op, order, vexp, ldb=M + 3, max_bits=mb, pad=pad), want)


def random_panels(rng, p, N, K, rows, lo=-128, hi=128):
    P = rng.integers(lo, hi, size=(p, N, K), dtype=np.int64).astype(np.int8)
    P[:, :, rows:] = 0
    return P


GRAM_SHAPES = [(7, 128, 128), (130, 384, 300), (300, 1152, 1100), (513, 256, 256)]


@pytest.mark.parametrize("N,K,rows", GRAM_SHAPES)
@pytest.mark.parametrize("cplx,order", [(0, 1), (0, 14), (1, 2), (1, 15), (1, 22)])
def test_gram_crt_bit_exact(gl, oracle, N, K, rows, cplx, order):
    rng = np.random.default_rng(34)
    panels = random_panels(rng, oracle.n_panels("crt", order, cplx), N, K, rows, -125, 126)
    orderC = 3
    print("gram crt", N, K, rows, cplx, order, flush=True)
    want = oracle.i8herk("crt", cplx, N, order, panels, 0, orderC)
    got = gl.gram("crt", cplx, N, order, panels, orderC)
    assert np.array_equal(got, want)
    want2 = oracle.i8herk("crt", cplx, N, order, panels, 1, orderC, Cin=want)
    got2 = gl.gram("crt", cplx, N, order, panels, orderC, beta=1, Cin=got)
    assert np.array_equal(got2, want2)


@pytest.mark.parametrize("N,K,rows", GRAM_SHAPES)
@pytest.mark.parametrize("cplx,order", [(0, 1), (0, 6), (1, 3), (0, 11), (1, 6), (1, 9), (1, 11)])
def test_gram_limbs_bit_exact(gl, oracle, N, K, rows, cplx, order):
    """Complex orders 9 and 11 make 3 o^2 > 192 panel pairs in 3 (2 o - 1) > 48 groups: the plan no longer fits one launch's
    tables and is cut between groups, also between the three groups of one level."""
    rng = np.random.default_rng(35)
    panels = random_panels(rng, oracle.n_panels("limbs", order, cplx), N, K, rows)
    orderC = 3 if order > 6 else 2
    print("gram limbs", N, K, rows, cplx, order, flush=True)
    want = oracle.i8herk("limbs", cplx, N, order, panels, 0, orderC)
    got = gl.gram("limbs", cplx, N, order, panels, orderC)
    assert np.array_equal(got, want)
    want2 = oracle.i8herk("limbs", cplx, N, order, panels, 1, orderC, Cin=want)
    got2 = gl.gram("limbs", cplx, N, order, panels, orderC, beta=1, Cin=got)
    assert np.array_equal(got2, want2)


@pytest.mark.parametrize("kind,cplx,order", [("crt", 0, 3), ("crt", 1, 4), ("crt", 1, 22), ("limbs", 0, 2), ("limbs", 1, 3), ("limbs", 1, 9)])
def test_gram_split_along_k(gl, oracle, kind, cplx, order):
    """A K long enough for the few tiles of a small N to be cut along K: the parts of a tile add into the same sums.  Complex
    CRT order 22 has moduli whose three products share planes, complex limb order 9 does not fit one launch's tables."""
    rng = np.random.default_rng(37)
    N, K, rows, orderC = 70, 16384, 16300, 3
    panels = random_panels(rng, oracle.n_panels(kind, order, cplx), N, K, rows, -125, 126)
    want = oracle.i8herk(kind, cplx, N, order, panels, 0, orderC)
    print("gram split along K", kind, cplx, order, flush=True)
    got = gl.gram(kind, cplx, N, order, panels, orderC)
    assert np.array_equal(got, want)
    want2 = oracle.i8herk(kind, cplx, N, order, panels[:, :, :4096], 1, orderC, Cin=want)
    assert np.array_equal(gl.gram(kind, cplx, N, order, panels[:, :, :4096], orderC, beta=1, Cin=got), want2)


def test_gram_extreme_values_and_long_k(gl, oracle):
    """All -128 digits over a K that needs several int32-safe splits; all-(-125) residues over K = 131072 rows are covered by the bound."""
    N, K = 20, 16384 * 3
    panels = np.full((2, N, K), -128, np.int8)
    want = oracle.i8herk("limbs", 0, N, 2, panels, 0, 2)
    assert np.array_equal(gl.gram("limbs", 0, N, 2, panels, 2), want)
    panels = np.full((2, N, K), -125, np.int8)
    panels[0] = -128
    want = oracle.i8herk("crt", 0, N, 2, panels, 0, 2)
    assert np.array_equal(gl.gram("crt", 0, N, 2, panels, 2), want)


def test_gram_rows_too_long_for_tile_offsets(gl, oracle):
    """Panel rows so long that the 256 rows of a tile do not fit 32-bit byte offsets: the launch takes the register-staged
    kernel and gives the same bits as the compact layout."""
    import torch
    import hyacinth_amd as ha
    from gpu_util import ptr, stream, sync, host, zeros, check, DEV
    rng = np.random.default_rng(41)
    N, K, order, orderC = 5, 640, 2, 2
    ldb = 16_900_096                               # 255 * ldb > 2^32, a multiple of 16
    panels = random_panels(rng, order, N, K, 600, -125, 126)
    want = oracle.i8herk("crt", 0, N, order, panels, 0, orderC)
    wide = torch.zeros((order, N, ldb), dtype=torch.int8, device=DEV)
    wide[:, :, :K] = torch.from_numpy(panels).to(DEV)
    T = N * (N + 1) // 2
    Cd = zeros(8 * orderC * T)
    wsb = gl.L.hykGramWorkspaceBytes(ha.GRAM_CRT, 0, N, order)
    ws = torch.zeros(int(wsb), dtype=torch.uint8, device=DEV)
    print("gram crt, ldb", ldb, flush=True)
    check(gl.L.hykGramCrt(stream(), 0, N, order, ptr(wide), ldb, K, 0, orderC, ptr(Cd), ptr(ws)))
    sync()
    assert np.array_equal(host(Cd, np.uint64), want)


@pytest.mark.parametrize("slab", [0, 2, 64, 128])
@pytest.mark.parametrize("cplx,order,K,rows", [(0, 3, 640, 600), (1, 2, 1536, 1500), (0, 2, 4224, 4200)])
def test_gram_kernel_variants(gl, oracle, slab, cplx, order, K, rows):
    """Every contraction kernel variant (direct-to-LDS rings with 64- and 128-byte rows, register-staged K slabs) gives the same bits."""
    rng = np.random.default_rng(36)
    panels = random_panels(rng, oracle.n_panels("crt", order, cplx), 270, K, rows, -125, 126)
    want = oracle.i8herk("crt", cplx, 270, order, panels, 0, 2)
    try:
        assert gl.L.hykGramSetSlab(slab) == 0
        got = gl.gram("crt", cplx, 270, order, panels, 2)
    finally:
        gl.L.hykGramSetSlab(0)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("cplx", [0, 1])
def test_dequantize(gl, oracle, cplx):
    from gpu_util import dev, zeros, ptr, stream, sync, host
    rng = np.random.default_rng(37)
    N = 45
    A = rand_matrix(rng, 300, N, "c128" if cplx else "f64", 2.0)
    A[:, 4] = 0
    at = oracle.atype_of(A)
    for eps, corr in ((1e-3, 7), (1e-10, 7), (1e-15, 20)):
        pl = oracle.fit_plan(300, N, eps, at, corr=corr)
        vexp = oracle.quantize_scale_batch(A, 1, 300, 300, pl["u"])
        Cq = oracle.herk_batch(A, 1, 300, 300, pl["u"], vexp, pl["lP"])
        for gtype in (oracle.F32 + cplx, oracle.F64 + cplx, oracle.DD + cplx):
            want = oracle.dequantize(N, pl["lP"], Cq, vexp, gtype)
            G = zeros(want.nbytes)
            dC, dv = dev(Cq), dev(vexp)
            assert gl.L.hykDequantize(stream(), N, pl["lP"], ptr(dC), ptr(dv), gtype, ptr(G), N) == 0
            sync()
            got = host(G, want.dtype, want.shape)
            if gtype in (oracle.DD, oracle.DDC):
                # double-double: compare the represented values (hi + lo) to 2^-100 relative, exactly where the lo word is zero
                assert np.array_equal(got[..., 0::2], want[..., 0::2])
                scale = np.abs(want[..., 0::2]).max()
                assert (np.abs(got[..., 1::2] - want[..., 1::2]) <= scale * 2.0**-100).all()
            else:
                assert np.array_equal(got, want)


def spd_raw(rng, N, r, cplx, gbase, floor=1e-9):
    """Hermitian positive matrix with a separated spectrum (r leading values 10^(-i/3), the rest `floor`) in the raw
    Gram layout [column][row][width]; a double-double matrix carries a non-zero low word."""
    U = haar(rng, N, N, bool(cplx))
    sig = np.concatenate([10.0 ** (-np.arange(r) / 3.0), floor * np.ones(N - r)])
    Gm = (U * sig ** 2) @ U.conj().T
    Gm = (Gm + Gm.conj().T) / 2
    Gt = Gm.T
    dd = gbase == 6
    raw = np.zeros((N, N, (2 if dd else 1) * (2 if cplx else 1)))
    step = 2 if dd else 1
    raw[..., 0] = Gt.real
    if cplx:
        raw[..., step] = Gt.imag
    if dd:
        low = np.abs(Gt.real) * 2.0**-55 * rng.uniform(-1, 1, (N, N))
        low = (low + low.T) / 2                 # keeps the matrix Hermitian
        raw[..., 1] = low
    return raw


def spd_exact_dd(rng, N, r, cplx):
    """B^H B of an r x N integer matrix whose row i is scaled by 2^-i, computed in Python integers and split exactly into
    double-double words: a positive semi-definite matrix of rank r that is exact to the last bit of the low word, with
    a spectrum spanning 2^(-2 r): what only double-double arithmetic can factor down to the last row."""
    br = rng.integers(-2**15, 2**15, (r, N)).astype(object)
    bi = rng.integers(-2**15, 2**15, (r, N)).astype(object) if cplx else None
    gre = np.zeros((N, N), object)
    gim = np.zeros((N, N), object)
    for i in range(r):
        w = 1 << (2 * (r - 1 - i))
        gre += w * np.outer(br[i], br[i])
        if cplx:
            gre += w * np.outer(bi[i], bi[i])
            gim += w * (np.outer(br[i], bi[i]) - np.outer(bi[i], br[i]))      # Im G[y, x] = sum re_y im_x - im_y re_x
    raw = np.zeros((N, N, 4 if cplx else 2))
    sh = -2 * (r - 1)
    for y in range(N):
        for x in range(N):
            for part, g in ((0, gre), (2, gim)) if cplx else ((0, gre),):
                v = int(g[y, x])
                hi = float(v)
                lo = float(v - int(hi))
                raw[x, y, part] = np.ldexp(hi, sh)
                raw[x, y, part + 1] = np.ldexp(lo, sh)
    return raw


# (N, leading values, K, eps for FP64, eps for double-double, floor, compute units offered)
POTRFP_CASES = [(24, 9, 24, 1e-6, 1e-6, 1e-9, 256), (150, 40, 150, 1e-6, 1e-10, 1e-13, 256), (150, 15, 150, 0.0, 0.0, 1e-5, 3),
                (150, 60, 17, 1e-12, 1e-12, 1e-15, 256), (700, 64, 700, 1e-6, 1e-9, 1e-12, 256), (700, 64, 16, 1e-12, 1e-12, 1e-12, 11),
                (130, 50, 18, 1e-12, 1e-12, 1e-12, 2)]


@pytest.mark.parametrize("entry", ["hykPotrfp", "hykPotrfpLeftLooking"])
@pytest.mark.parametrize("gbase", [0, 6])        # FP64, double-double
@pytest.mark.parametrize("cplx", [0, 1])
@pytest.mark.parametrize("N,r,K,eps64,epsdd,floor,units", POTRFP_CASES)
def test_potrfp_kernel(gl, oracle, entry, gbase, cplx, N, r, K, eps64, epsdd, floor, units):
    """Both kernels (blocked right-looking, left-looking) against the oracle's pivoted Cholesky (src/hyacin_potrfp.cu:119-318): same rank, same pivots, factor rows equal
    to rounding (the two sum in different orders, and row t carries the rounding of the Schur complement it came from, so
    the bound grows with d_0 / d_t).  The cut-off sits well above the rounding level of the arithmetic and well above the
    floor of the spectrum, so the rank is not decided by rounding.  `units` limits the workgroups, so that wavefronts
    own several columns."""
    from gpu_util import dev, zeros, ptr, stream, sync, host
    rng = np.random.default_rng(41 + cplx + gbase)
    gtype = gbase + cplx
    eps = epsdd if gbase == 6 else eps64
    exact = gbase == 6 and N <= 150 and eps > 0.
    raw = spd_exact_dd(rng, N, min(r, 30), cplx) if exact else spd_raw(rng, N, r, cplx, gbase, floor)
    work = raw.copy()
    want_rank, want_piv = oracle.potrfp(work, gtype, eps, K)
    if exact:
        assert want_rank == min(min(r, 30), K)
    width = raw.shape[2]
    ldr = min(N, K + 1)
    Rt = zeros(N * ldr * width * 8)
    jp = zeros(N * 4)
    rk = zeros(4)
    ws = zeros(gl.L.hykPotrfpWorkspaceBytes(N, gtype))
    dG = dev(raw)
    print(entry, "N", N, "K", K, "gtype", gtype, "units", units, flush=True)
    assert getattr(gl.L, entry)(stream(), units, eps, K, N, gtype, ptr(dG), N, ptr(Rt), ldr, ptr(jp), ptr(ws), ptr(rk)) == 0
    sync()
    rank = int(host(rk, np.int32)[0])
    piv = host(jp, np.int32)
    assert rank == want_rank
    assert sorted(piv.tolist()) == list(range(1, N + 1))
    assert np.array_equal(piv[:rank], want_piv[:rank])
    got = host(Rt, np.float64, (N, ldr, width))                    # [column l][row t]
    ref = np.transpose(work, (1, 0, 2))                           # oracle: row t of R in row t of the column-permuted matrix
    p = want_piv - 1
    unit = 2.0**-100 if gbase == 6 else 2.0**-53
    d0 = ref[0, 0, 0] ** 2
    for t in range(rank):
        a = got[p[t:], t, :]                                      # R[t, columns in pivot order from the diagonal on]
        b = ref[t, t:, :]
        if gbase == 6:
            a = a[..., 0::2] + a[..., 1::2]
            b = b[..., 0::2] + b[..., 1::2]
        scale = np.abs(b).max()
        bound = 1e3 * unit * d0 / ref[t, t, 0] ** 2
        assert np.abs(a - b).max() <= bound * scale, (t, np.abs(a - b).max(), scale, bound)
    # entries below the diagonal (in pivot order) stay zero
    for t in range(1, rank):
        assert not got[p[:t], t, :].any()


@pytest.mark.parametrize("entry", ["hykPotrfp", "hykPotrfpLeftLooking"])
@pytest.mark.parametrize("gbase,cplx,N", [(0, 0, 600), (6, 1, 300), (6, 0, 2048)])
def test_potrfp_plain_launch(gl, entry, gbase, cplx, N):
    """hykPotrfpSetPlainLaunch: the same kernels started with a plain launch (for runs under a kernel-tracing profiler) give
    the rank, pivots and factor bits of the cooperative launch."""
    from gpu_util import dev, zeros, ptr, stream, sync, host
    rng = np.random.default_rng(43 + cplx + gbase)
    gtype = gbase + cplx
    raw = spd_raw(rng, N, min(N, 120), cplx, gbase, 1e-9)
    width = raw.shape[2]
    outs = []
    try:
        for plain in (0, 1):
            assert gl.L.hykPotrfpSetPlainLaunch(plain) == 0
            Rt, jp, rk, ws, dG = zeros(N * N * width * 8), zeros(N * 4), zeros(4), zeros(gl.L.hykPotrfpWorkspaceBytes(N, gtype)), dev(raw)
            print(entry, "plain launch", plain, "N", N, "gtype", gtype, flush=True)
            assert getattr(gl.L, entry)(stream(), 256, 1e-7, N, N, gtype, ptr(dG), N, ptr(Rt), N, ptr(jp), ptr(ws), ptr(rk)) == 0
            sync()
            outs.append((int(host(rk, np.int32)[0]), host(jp, np.int32).copy(), host(Rt, np.float64).copy()))
    finally:
        gl.L.hykPotrfpSetPlainLaunch(0)
    assert outs[0][0] > 0 and outs[0][0] == outs[1][0] and np.array_equal(outs[0][1], outs[1][1]) and np.array_equal(outs[0][2], outs[1][2])


@pytest.mark.parametrize("gbase,cplx", [(0, 0), (0, 1), (6, 0), (6, 1)])
def test_potrfp_wanted(gl, gbase, cplx):
    """hykPotrfpWanted: the factorization for a caller that uses `wanted` values only.  Twelve graded values over a floor of
    288 columns of 1e-6: what is left of G after twelve steps (2.9e-10) is within 32 b for cut = 1e-6 (b = 1e-6 nu_1 nu_w, the norms
    of rows 1 and w of the factor: about 2e-10), so the factorization ends at the first step that leaves at most b, with the
    pivots of the full run up to there and the trace of what is left in traceOut.  With cut = 1e-8 the floor is far above 32 b
    and with cut = 0 there is no rule: both give the full run's rank and pivots and report 0."""
    from gpu_util import dev, zeros, ptr, stream, sync, host
    rng = np.random.default_rng(47 + cplx + gbase)
    gtype, N, wanted = gbase + cplx, 300, 12
    raw = spd_raw(rng, N, wanted, cplx, gbase, 1e-6)
    width = raw.shape[2]
    def run(cut):
        Rt, jp, rk, tr, ws, dG = zeros(N * N * width * 8), zeros(N * 4), zeros(4), zeros(8), zeros(gl.L.hykPotrfpWorkspaceBytes(N, gtype)), dev(raw)
        print("hykPotrfpWanted gtype", gtype, "cut", cut, flush=True)
        assert gl.L.hykPotrfpWanted(stream(), 256, 1e-9, N, wanted, cut, N, gtype, ptr(dG), N, ptr(Rt), N, ptr(jp), ptr(ws), ptr(rk), ptr(tr)) == 0
        sync()
        R = host(Rt, np.float64, (N, N, width))[..., 0] + (1j * host(Rt, np.float64, (N, N, width))[..., 2 if gbase == 6 else 1] if cplx else 0)   # [column][row]
        return int(host(rk, np.int32)[0]), host(jp, np.int32).copy(), float(host(tr, np.float64)[0]), R
    full = run(0.0)
    assert full[0] == N and full[2] == 0.0
    far = run(1e-8)
    assert far[0] == full[0] and np.array_equal(far[1], full[1]) and far[2] == 0.0
    rank, piv, left, R = run(1e-6)
    rows2 = (np.abs(full[3]) ** 2).sum(axis=0)                                   # squared norms of the rows of the full factor, in pivot order
    b = 1e-6 * np.sqrt(rows2[0] * rows2[wanted - 1])
    assert wanted < rank < N and np.array_equal(piv[:rank], full[1][:rank])
    tail = lambda t: rows2[t:].sum()                                             # the trace of what is left after t steps
    ideal = next(t for t in range(wanted + 1, N) if tail(t) <= b)                # the first step that leaves at most b
    assert abs(rank - ideal) <= 1                                                # (the kernel's running trace carries the rounding of its updates: a step of the floor is 0.5 % of b)
    assert abs(left - tail(rank)) <= 1e-2 * tail(rank)
    assert np.allclose(R[:, :rank], full[3][:, :rank], rtol=0, atol=1e-13)


@pytest.mark.parametrize("gtype", [0, 1, 6, 7])
def test_mirror_lower(gl, gtype):
    """hykMirrorLower: the strict upper triangle written again as the conjugate of the lower one; diagonal and lower triangle
    untouched, also with a padded leading dimension."""
    from gpu_util import dev, ptr, stream, sync, host
    rng = np.random.default_rng(48 + gtype)
    N, ld, cplx, w = 77, 80, gtype & 1, 2 if gtype >= 6 else 1
    raw = rng.standard_normal((N, ld, w * (1 + cplx)))                          # [column][row][words]
    d = dev(raw)
    print("hykMirrorLower gtype", gtype, flush=True)
    assert gl.L.hykMirrorLower(stream(), N, gtype, ptr(d), ld) == 0
    sync()
    got, want = host(d, np.float64, raw.shape), raw.copy()
    for x in range(N):
        for y in range(x):
            want[x, y] = raw[y, x]
            if cplx:
                want[x, y, w:] = -raw[y, x, w:]
    assert np.array_equal(got, want)


@pytest.mark.parametrize("cplx", [0, 1])
@pytest.mark.parametrize("opA", ["N", "T", "C"])
@pytest.mark.parametrize("M,N,K,pad", [(300, 70, 45, 0), (128, 128, 64, 0), (1000, 260, 333, 8), (257, 129, 1, 0), (96, 40, 200, 3)])
def test_f16_products(gl, cplx, opA, M, N, K, pad):
    """hykMatmulCf16 / hykGemm on FP16 operands (src/matmul_fp16_complex.cu:21-89, the GemmEx calls of src/lra.cpp:86-105):
    C = op(A) B against numpy in FP32 on the same half-rounded inputs.  Ragged tiles, K tails inside a 16-byte piece, padded
    leading dimensions; pad = 3 makes the leading dimensions unaligned, which takes the vector-ALU kernel."""
    from gpu_util import dev, zeros, ptr, stream, sync, host
    rng = np.random.default_rng(77 + cplx)
    comps = 2 if cplx else 1
    rowsA, colsA = (M, K) if opA == "N" else (K, M)
    lda, ldb, ldc = rowsA + (8 - rowsA % 8) % 8 + pad, K + (8 - K % 8) % 8 + pad, M + pad
    def rand(rows, cols, ld):
        buf = np.zeros((cols, ld, comps), np.float16)
        buf[:, :rows, :] = rng.standard_normal((cols, rows, comps)).astype(np.float16)
        v = buf[:, :rows, :].astype(np.float32)
        m = (v[..., 0] + 1j * v[..., 1]).T if cplx else v[..., 0].T        # rows x cols
        return buf, m
    bufA, mA = rand(rowsA, colsA, lda)
    bufB, mB = rand(K, N, ldb)
    opm = mA if opA == "N" else (mA.T if opA == "T" else mA.conj().T)
    want = opm.astype(np.complex64 if cplx else np.float32) @ mB
    Cd = zeros(N * ldc * comps * 2)
    dA, dB = dev(bufA), dev(bufB)
    if cplx:
        rc = gl.L.hykMatmulCf16(stream(), opA.encode(), M, N, K, ptr(dA), lda, ptr(dB), ldb, ptr(Cd), ldc)
    else:
        rc = gl.L.hykGemm(stream(), opA.encode(), b"N", M, N, K, C.c_double(1.0), 4, ptr(dA), C.c_int64(lda), ptr(dB), C.c_int64(ldb), C.c_double(0.0), ptr(Cd), C.c_int64(ldc))
    assert rc == 0
    sync()
    got = host(Cd, np.float16, (N, ldc, comps))[:, :M, :].astype(np.float32)
    got = (got[..., 0] + 1j * got[..., 1]).T if cplx else got[..., 0].T
    scale = np.sqrt(np.mean(np.abs(want) ** 2))
    assert np.all(np.abs(got - want) <= 2.0**-10 * np.abs(want) + 2.0**-12 * scale + 1e-6)
    assert not host(Cd, np.float16, (N, ldc, comps))[:, M:, :].any()       # nothing written into the padding


@pytest.mark.parametrize("cplx", [0, 1])
@pytest.mark.parametrize("opA", ["N", "T", "C"])
@pytest.mark.parametrize("M,N,K,pad", [(300, 70, 45, 0), (128, 128, 64, 0), (1000, 260, 333, 4), (257, 129, 1, 0), (96, 40, 200, 3), (2048, 512, 2048, 0)])
def test_f32_products(gl, cplx, opA, M, N, K, pad):
    """hykGemm on FP32 / complex FP32 operands in the form C = op(A) B (the stage products of the column-segmented fit, the
    GemmEx calls of src/lra.cpp:90-93,102-105) against numpy in FP64 on the same inputs, at the bound of test_gemm_fp64 with
    the FP32 unit roundoff: 2^-24 / 2^-53 times its 1e-13.  Ragged tiles, K tails inside a 16-byte piece, padded leading
    dimensions; pad = 3 makes the leading dimensions unaligned, which takes the vector-ALU kernel."""
    from gpu_util import dev, zeros, ptr, stream, sync, host
    rng = np.random.default_rng(177 + cplx)
    comps = 2 if cplx else 1
    rowsA, colsA = (M, K) if opA == "N" else (K, M)
    lda, ldb, ldc = rowsA + (4 - rowsA % 4) % 4 + pad, K + (4 - K % 4) % 4 + pad, M + pad
    def rand(rows, cols, ld):
        buf = np.zeros((cols, ld, comps), np.float32)
        buf[:, :rows, :] = rng.standard_normal((cols, rows, comps)).astype(np.float32)
        v = buf[:, :rows, :].astype(np.float64)
        m = (v[..., 0] + 1j * v[..., 1]).T if cplx else v[..., 0].T        # rows x cols
        return buf, m
    bufA, mA = rand(rowsA, colsA, lda)
    bufB, mB = rand(K, N, ldb)
    want = (mA if opA == "N" else (mA.T if opA == "T" else mA.conj().T)) @ mB
    Cd = zeros(N * ldc * comps * 4)
    dA, dB = dev(bufA), dev(bufB)
    rc = gl.L.hykGemm(stream(), opA.encode(), b"N", M, N, K, C.c_double(1.0), 3 if cplx else 2, ptr(dA), C.c_int64(lda), ptr(dB), C.c_int64(ldb), C.c_double(0.0), ptr(Cd), C.c_int64(ldc))
    assert rc == 0
    sync()
    full = host(Cd, np.float32, (N, ldc, comps))
    got = full[:, :M, :].astype(np.float64)
    got = (got[..., 0] + 1j * got[..., 1]).T if cplx else got[..., 0].T
    assert np.abs(got - want).max() <= 1e-13 * 2.0**29 * np.abs(want).max() * max(1, K) ** 0.5
    assert not full[:, M:, :].any()                                        # nothing written into the padding


@pytest.mark.parametrize("cplx", [0, 1])
@pytest.mark.parametrize("N,K", [(40, 7), (150, 32), (300, 75), (700, 257)])
def test_interp_solve(gl, cplx, N, K):
    """hykInterpSolve (cuBLAS trsm of src/gram_id.cpp:40-46): T = R11^-1 R12 for a factor given column-wise in pivot order,
    against numpy's triangular solve; K below, at and across the block size of the blocked back substitution."""
    from gpu_util import dev, zeros, ptr, stream, sync, host
    rng = np.random.default_rng(91 + cplx)
    W = 2 if cplx else 1
    R = rng.standard_normal((K, N)) + (1j * rng.standard_normal((K, N)) if cplx else 0)
    R[:, :K] = np.triu(R[:, :K])
    R[np.arange(K), np.arange(K)] = 2.0 + np.abs(R[np.arange(K), np.arange(K)])      # real positive diagonal, well conditioned
    piv = rng.permutation(N).astype(np.int32) + 1                                     # column at pivot position x is piv[x] - 1
    ldr = K + 3
    Rt = np.zeros((N, ldr, W))                                                        # Rt[column][row]
    for x in range(N):
        col = piv[x] - 1
        Rt[col, :K, 0] = R[:, x].real
        if cplx:
            Rt[col, :K, 1] = R[:, x].imag
    dRt, dp = dev(Rt), dev(piv)
    R11 = zeros(K * K * W * 8)
    T = zeros(K * (N - K) * W * 8)
    assert gl.L.hykInterpSolve(stream(), N, K, 1 if cplx else 0, ptr(dRt), ldr, ptr(dp), ptr(R11), ptr(T)) == 0
    sync()
    got = host(T, np.float64, (N - K, K, W))
    got = (got[..., 0] + 1j * got[..., 1]).T if cplx else got[..., 0].T
    want = np.linalg.solve(R[:, :K], R[:, K:])
    assert np.abs(got - want).max() <= 1e-11 * np.abs(want).max()
    g11 = host(R11, np.float64, (K, K, W))
    g11 = (g11[..., 0] + 1j * g11[..., 1]).T if cplx else g11[..., 0].T
    assert np.array_equal(g11, R[:, :K])


@pytest.mark.parametrize("cplx", [0, 1])
@pytest.mark.parametrize("opA,opB", [("N", "N"), ("T", "N"), ("C", "N"), ("N", "C"), ("N", "T"), ("C", "T")])
@pytest.mark.parametrize("M,N,K", [(70, 33, 19), (600, 130, 75), (1025, 257, 64)])
def test_gemm_fp64(gl, cplx, opA, opB, M, N, K):
    """hykGemm in FP64 / complex FP64 (the cuBLAS gemm calls of src/lra.cpp:86-105,202-203): C = alpha op(A) op(B) + beta C
    against numpy, all operand forms, sizes on both the 64 x 64 and the 128 x 128 tile paths, ragged edges."""
    from gpu_util import dev, ptr, stream, sync, host
    rng = np.random.default_rng(5 + cplx)
    W = 2 if cplx else 1
    def rand(r, c):
        return rng.standard_normal((r, c)) + (1j * rng.standard_normal((r, c)) if cplx else 0)
    def op(X, o):
        return X if o == "N" else (X.T if o == "T" else X.conj().T)
    def store(X, ld):                                   # column-major with leading dimension ld, interleaved complex
        buf = np.zeros((X.shape[1], ld, W))
        buf[:, :X.shape[0], 0] = X.real.T
        if cplx:
            buf[:, :X.shape[0], 1] = X.imag.T
        return buf
    A = rand(*((M, K) if opA == "N" else (K, M)))
    B = rand(*((K, N) if opB == "N" else (N, K)))
    C0 = rand(M, N)
    alpha, beta = -1.5, 0.75
    want = alpha * op(A, opA) @ op(B, opB) + beta * C0
    lda, ldb, ldc = A.shape[0] + 3, B.shape[0] + 1, M + 2
    dA, dB, dC = dev(store(A, lda)), dev(store(B, ldb)), dev(store(C0, ldc))
    rc = gl.L.hykGemm(stream(), opA.encode(), opB.encode(), M, N, K, C.c_double(alpha), 1 if cplx else 0, ptr(dA), C.c_int64(lda), ptr(dB), C.c_int64(ldb), C.c_double(beta), ptr(dC), C.c_int64(ldc))
    assert rc == 0
    sync()
    got = host(dC, np.float64, (N, ldc, W))[:, :M, :]
    got = (got[..., 0] + 1j * got[..., 1]).T if cplx else got[..., 0].T
    assert np.abs(got - want).max() <= 1e-13 * np.abs(want).max() * max(1, K) ** 0.5


@pytest.mark.parametrize("wide", [1, 0])
@pytest.mark.parametrize("variant,carry", [(0, 0), (0, 1), (1, 0), (2, 0), (2, 1)])
@pytest.mark.parametrize("cplx,N,r", [(0, 300, 40), (0, 1000, 130), (0, 2048, 96), (0, 2500, 70), (0, 4096, 40), (1, 600, 50), (1, 2048, 40), (1, 3000, 24), (1, 4096, 36), (0, 64, 64), (0, 700, 20), (0, 701, 40), (0, 1023, 64), (0, 2047, 33), (0, 2048, 256)])
def test_jacobi_sweep_kernels(gl, variant, carry, cplx, N, r, wide):
    """One-sided Jacobi sweeps on a graded N x r factor: every kernel behind hykJacobiSweep / hykJacobiSweepCarry (Gram-space
    rounds with blocks of 8 and of 4 columns, with and without the products inside a block carried from round to round in
    memory that starts as NaN, the step kernel, the pair kernel for few columns) must leave orthogonal columns whose norms are
    the singular values numpy finds, to 32 sqrt(r) eps of the largest (a column takes part in a few hundred rotations), and
    whose span is unchanged.  Odd N takes the kernels' element-wise loads (columns not aligned to a pair of rows); r = 256
    gives the 16 block pairs of a round that are numbered by XCD.  wide = 0: the factor in floats (the SVD of FP32 / FP16
    storage, src/gram_evd.cu:96-98), eps that of single precision; above 2048 rows a workgroup then takes all rows at once."""
    from gpu_util import dev, host, ptr, stream, sync, zeros
    rng = np.random.default_rng(1000 * N + r + cplx)
    real, eps = (np.float64, 2.220446049250313e-16) if wide else (np.float32, 1.1920929e-07)
    cpx = np.complex128 if wide else np.complex64
    btype = (0 if wide else 2) + cplx
    B = rng.standard_normal((N, r)) + (1j * rng.standard_normal((N, r)) if cplx else 0)
    mix = np.triu(rng.standard_normal((r, r))) * 0.1 + np.eye(r)          # columns correlated
    B = ((B @ mix) * 10.0 ** ((-6.0 if wide else -3.0) * np.arange(r) / r)).astype(cpx if cplx else real)   # graded like a pivoted Cholesky factor
    want = np.linalg.svd(B.astype(np.complex128 if cplx else np.float64), compute_uv=False)
    dB = dev(np.ascontiguousarray(B.T)); counter = zeros(64)
    carried = zeros(gl.L.hykJacobiCarryBytes(r)); carried.fill_(255)       # all-ones bytes: NaN, must never be read before written
    tol = float(eps * np.sqrt(N))
    assert gl.L.hykJacobiSetVariant(variant) == 0
    try:
        sweeps = 0
        while True:
            counter.zero_()
            print("jacobi", variant, cplx, N, r, "wide", wide, "sweep", sweeps, flush=True)
            if carry:
                assert gl.L.hykJacobiSweepCarry(stream(), btype, N, r, ptr(dB), tol, ptr(counter), ptr(carried)) == 0
            else:
                assert gl.L.hykJacobiSweep(stream(), btype, N, r, ptr(dB), tol, ptr(counter)) == 0
            sync(); sweeps += 1
            rotations = int(host(counter, np.int32)[0]); cos2 = float(host(counter, np.float64)[1])
            assert int(host(counter, np.int32)[1]) == 0
            if rotations == 0:
                break
            assert sweeps < 30, "no convergence"
        assert cos2 <= (8 * tol) ** 2
    finally:
        gl.L.hykJacobiSetVariant(0)
    U = host(dB, cpx if cplx else real, (r, N)).T.astype(np.complex128 if cplx else np.float64)
    got = np.sort(np.linalg.norm(U, axis=0))[::-1]
    assert np.max(np.abs(got - want)) <= 32 * eps * want[0] * np.sqrt(r)
    sig = zeros(8 * r)                                                     # hykColumnNorms on the same memory
    assert gl.L.hykColumnNorms(stream(), btype, N, r, ptr(dB), ptr(sig)) == 0
    sync()
    assert np.max(np.abs(host(sig, np.float64) - np.linalg.norm(U, axis=0))) <= 1e-12 * want[0]
    Un = U / np.linalg.norm(U, axis=0)
    assert np.max(np.abs(Un.conj().T @ Un - np.eye(r))) <= 16 * tol
    Qb, _ = np.linalg.qr(B.astype(np.complex128 if cplx else np.float64))                                               # same column space
    assert np.linalg.norm(Un - Qb @ (Qb.conj().T @ Un)) <= (1e-9 if wide else 1e-3) * np.sqrt(r)


@pytest.mark.parametrize("N,r", [(2048, 96), (1000, 130), (2047, 33), (2048, 256)])
def test_jacobi_split_rounds_with_a_late_partner(gl, N, r):
    """The rounds that put two workgroups on a block pair, with the dispatch order forced from the host: the workgroup of
    one half arrives only when its partner has taken the whole pair, finds that in the pair's word and leaves; the partner has
    rotated and stored both halves.  Either way round the sweep leaves exactly the bits of the sweep in which the partners
    start together (same sums, same rotations, same arithmetic on every row).  With a partner that arrives and then never
    reports its loads, the waiting workgroup gives up: rotations[1] is set."""
    from gpu_util import dev, host, ptr, stream, sync, zeros
    rng = np.random.default_rng(7 * N + r)
    B = rng.standard_normal((N, r)) @ (np.triu(rng.standard_normal((r, r))) * 0.1 + np.eye(r)) * 10.0 ** (-6.0 * np.arange(r) / r)
    tol = float(2.220446049250313e-16 * np.sqrt(N))
    out = {}
    try:
        for mode in (0, 1, 2, 3):
            assert gl.L.hykJacobiSetSplitTest(mode) == 0
            dB = dev(np.ascontiguousarray(B.T)); counter = zeros(64); carried = zeros(gl.L.hykJacobiCarryBytes(r)); carried.fill_(255)
            flags = []
            for sweep in range(1 if mode == 3 else 3):
                counter.zero_()
                print("split rounds", N, r, "mode", mode, "sweep", sweep, flush=True)
                assert gl.L.hykJacobiSweepCarry(stream(), 0, N, r, ptr(dB), tol, ptr(counter), ptr(carried)) == 0
                sync()
                flags.append(int(host(counter, np.int32)[1]))
            out[mode] = (host(dB, np.float64, (r, N)).copy(), int(host(counter, np.int32)[0]), flags)
    finally:
        gl.L.hykJacobiSetSplitTest(0)
    assert out[0][2] == [0, 0, 0] and out[1][2] == [0, 0, 0] and out[2][2] == [0, 0, 0]
    assert out[0][1] > 0
    for mode in (1, 2):
        assert out[mode][1] == out[0][1] and np.array_equal(out[mode][0], out[0][0])
    assert out[3][2] == [1]


@pytest.mark.parametrize("variant,carry", [(0, 1), (0, 0), (1, 0), (2, 1)])
@pytest.mark.parametrize("cplx,N,r,head,top", [(0, 1000, 130, 37, 37), (0, 2048, 96, 40, 64), (1, 600, 50, 9, 9), (1, 2048, 40, 12, 20), (0, 700, 20, 5, 20), (0, 300, 40, 0, 0)])
def test_jacobi_sweeps_with_limits(gl, variant, carry, cplx, N, r, head, top):
    """hykJacobiSweepTop: pairs of two columns from `top` on are never rotated, and only the pairs with a column before
    `head` are reported.  The columns behind `head` are 1e-5 of the others (the separation under which the host uses the
    limits).  Sweeps run until the reported cosine is at the threshold's level; then the columns before `head` are
    orthogonal to every other column, so the singular values are their norms together with those of the block behind
    them, and the span is unchanged.  With head = top = r the sweep is the plain one, bit for bit."""
    from gpu_util import dev, host, ptr, stream, sync, zeros
    rng = np.random.default_rng(7000 + N + r + cplx)
    B = rng.standard_normal((N, r)) + (1j * rng.standard_normal((N, r)) if cplx else 0)
    B = (B @ (np.triu(rng.standard_normal((r, r))) * 0.1 + np.eye(r))) * 10.0 ** (-2.0 * np.arange(r) / r)
    B[:, head:] *= 1e-5
    want = np.linalg.svd(B, compute_uv=False)
    tol = float(2.220446049250313e-16 * np.sqrt(N))
    assert gl.L.hykJacobiSetVariant(variant) == 0
    try:
        dB = dev(np.ascontiguousarray(B.T)); counter = zeros(64)
        carried = zeros(gl.L.hykJacobiCarryBytes(r)); carried.fill_(255)
        for sweeps in range(30):
            counter.zero_()
            print("jacobi limits", variant, carry, cplx, N, r, head, top, "sweep", sweeps, flush=True)
            assert gl.L.hykJacobiSweepTop(stream(), cplx, N, r, head, top, ptr(dB), tol, ptr(counter), ptr(carried) if carry else None) == 0
            sync()
            if float(host(counter, np.float64)[1]) <= (8 * tol) ** 2:
                break
        else:
            raise AssertionError("no convergence")
        # one plain sweep through both entry points: identical bits
        d1, d2 = dev(np.ascontiguousarray(B.T)), dev(np.ascontiguousarray(B.T)); c1, c2 = zeros(64), zeros(64)
        assert gl.L.hykJacobiSweep(stream(), cplx, N, r, ptr(d1), tol, ptr(c1)) == 0
        assert gl.L.hykJacobiSweepTop(stream(), cplx, N, r, r, r, ptr(d2), tol, ptr(c2), None) == 0
        sync()
        assert np.array_equal(host(d1, np.uint8), host(d2, np.uint8)) and np.array_equal(host(c1, np.uint8), host(c2, np.uint8))
    finally:
        gl.L.hykJacobiSetVariant(0)
    U = host(dB, np.complex128 if cplx else np.float64, (r, N)).T
    G = U.conj().T @ U
    nrm = np.sqrt(np.abs(np.diagonal(G)))
    Gn = G / np.outer(nrm, nrm)
    off = Gn - np.diag(np.diagonal(Gn))
    assert np.abs(off[:head, :]).max(initial=0.0) <= 64 * tol             # leading columns: orthogonal to everything
    sv = np.sort(np.concatenate([nrm[:head], np.linalg.svd(U[:, head:], compute_uv=False)]))[::-1]
    assert np.max(np.abs(sv - want)) <= 32 * 2.220446049250313e-16 * want[0] * np.sqrt(r)
    Qb, _ = np.linalg.qr(B)                                               # same column space
    Un = U / nrm
    assert np.linalg.norm(Un - Qb @ (Qb.conj().T @ Un)) <= 1e-9 * np.sqrt(r)
