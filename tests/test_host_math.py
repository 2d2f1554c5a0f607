"""The integer helpers the HIP kernels are built from (hyk_common.h), compiled for the host and checked against exact arithmetic."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

from oracle import closed_form as cf

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "host_math", "host_math.cpp")
LIB = os.environ.get("HYACIN_HOST_MATH_LIBRARY") or os.path.join(ROOT, "tests", "host_math", "libhost_math.so")   # (the variable: a build made elsewhere, e.g. with a sanitizer)


@pytest.fixture(scope="module")
def hm():
    hdr = os.path.join(ROOT, "hyacinth_amd", "csrc", "hyk_common.h")
    stop = os.path.join(ROOT, "hyacinth_amd", "csrc", "host", "jacobi_stop.hpp")
    if not os.environ.get("HYACIN_HOST_MATH_LIBRARY") and (not os.path.exists(LIB) or os.path.getmtime(LIB) < max(os.path.getmtime(SRC), os.path.getmtime(hdr), os.path.getmtime(stop))):
        subprocess.check_call(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-I", os.path.join(ROOT, "hyacinth_amd", "csrc"), SRC, "-o", LIB])
    L = C.CDLL(LIB)
    L.hm_frexp.restype = C.c_int32
    L.hm_reduce_i32.restype = C.c_int32
    L.hm_jacobi_done.argtypes = [C.c_int, C.c_double, C.c_double, C.c_double]
    L.hm_jacobi_done.restype = C.c_int
    L.hm_jacobi_tail_start.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_double]
    L.hm_jacobi_tail_start.restype = C.c_int
    L.hm_jacobi_settled.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_double]
    L.hm_jacobi_head.argtypes = [C.c_void_p, C.c_int, C.c_int]
    L.hm_jacobi_head.restype = C.c_int
    L.hm_jacobi_columns_needed.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_double]
    L.hm_jacobi_columns_needed.restype = C.c_int
    L.hm_jacobi_truncation_holds.argtypes = [C.c_double, C.c_double, C.c_double, C.c_double]
    L.hm_jacobi_truncation_holds.restype = C.c_int
    L.hm_jacobi_settled.restype = C.c_int
    return L


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def samples(rng, dtype, n=400):
    x = rng.standard_normal(n) * np.exp(rng.standard_normal(n) * 8)
    x = np.clip(x, -float(np.finfo(dtype).max), float(np.finfo(dtype).max)).astype(dtype)
    tiny = np.finfo(dtype).tiny
    special = np.array([0.0, -0.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, tiny, tiny / 2, -tiny / 4, 1.0, -1.0, 255.5, -128.5, 0.99999], dtype=dtype)
    return np.concatenate([special, x])


TYPES = [(0, np.float64), (2, np.float32), (4, np.float16)]


@pytest.mark.parametrize("tcode,dtype", TYPES)
def test_round_scaled(hm, tcode, dtype):
    rng = np.random.default_rng(21)
    x = samples(rng, dtype)
    for expon in (-30, -3, 0, 1, 17, 40, 62, 81):
        xs = x[np.abs(x.astype(np.float64)) * 2.0**expon < 2.0**90]
        out = np.zeros(2 * len(xs), np.int64)
        hm.hm_round(tcode, _p(xs), C.c_int64(len(xs)), C.c_int32(expon), _p(out))
        for i, v in enumerate(xs):
            got = (int(out[2 * i]) & (2**64 - 1)) + (int(out[2 * i + 1]) << 64)
            assert got == cf.rne_scaled(float(v), expon), (float(v), expon)


@pytest.mark.parametrize("tcode,dtype", TYPES)
def test_digits_and_residues(hm, tcode, dtype):
    rng = np.random.default_rng(22)
    x = samples(rng, dtype, 200)
    for expon in (0, 20, 44):
        xs = x[np.abs(x.astype(np.float64)) * 2.0**expon < 2.0**47]
        q = [cf.rne_scaled(float(v), expon) for v in xs]
        for order in (1, 4, 8, 12):
            out = np.zeros(len(xs) * order, np.int8)
            hm.hm_digits(tcode, _p(xs), C.c_int64(len(xs)), C.c_int32(expon), order, _p(out))
            assert out.reshape(len(xs), order).tolist() == [cf.balanced_digits(v, order) for v in q]
        for table, moduli in ((0, cf.REAL_MODULI), (1, cf.CPLX_MODULI)):
            for dots in (2, 3):
                out = np.zeros(len(xs) * len(moduli), np.int8)
                hm.hm_residues(table, dots, tcode, _p(xs), C.c_int64(len(xs)), C.c_int32(expon), len(moduli), _p(out))
                assert out.reshape(len(xs), len(moduli)).tolist() == [[cf.signed_residue(v, m) for m in moduli] for v in q]
    # wide values need all three dwords
    big = np.array([1.0, -1.0, 0.75, -0.3, 1 - 2.0**-52], dtype=np.float64).astype(dtype)
    for expon in (60, 75, 81):
        q = [cf.rne_scaled(float(v), expon) for v in big]
        out = np.zeros(len(big) * 24, np.int8)
        hm.hm_residues(0, 3, tcode, _p(big), C.c_int64(len(big)), C.c_int32(expon), 24, _p(out))
        assert out.reshape(len(big), 24).tolist() == [[cf.signed_residue(v, m) for m in cf.REAL_MODULI] for v in q]


def test_dot_residues_at_the_range_limits(hm):
    """q at and next to +-(2^(32 dots - 1) - 1), the largest magnitudes a dot count may be used for, and small values."""
    for dots in (1, 2, 3):
        top = 2 ** (32 * dots - 1)
        values = [0, 1, -1, 127, 128, -128, -129, 255, 256, -255, -256, top - 1, -(top - 1), -top, top // 2, -(top // 2) - 1, top - 12345, -(top - 54321)]
        for m in sorted(set(cf.REAL_MODULI) | set(cf.CPLX_MODULI)):
            for v in values:
                w = v & (2 ** 96 - 1)
                st, ca = C.c_int32(), C.c_uint32()
                hm.hm_residue_raw(C.c_uint64(w & (2 ** 64 - 1)), C.c_uint32(w >> 64), dots, m, C.byref(st), C.byref(ca))
                assert ca.value == v % m, (dots, m, v)
                assert st.value == cf.signed_residue(v, m) or (m == 256 and (st.value - cf.signed_residue(v, m)) % 256 == 0), (dots, m, v)
                assert min(0, 128 - m) <= st.value <= 127


def test_f64_residues_below_2_pow_51(hm):
    """Three-instruction FP64 residue: exact for every |a| < 2^51, in the reference's stored range, also next to the ties."""
    rng = np.random.default_rng(29)
    top = 2 ** 51
    vals = [0, 1, -1, 127, 128, -128, -129, top - 1, -(top - 1), top - 2, -(top - 2)]
    vals += [int(v) for v in rng.integers(-top + 1, top, 4000)] + [int(v) for v in rng.integers(-70000, 70000, 4000)]
    for m in sorted(set(cf.REAL_MODULI) | set(cf.CPLX_MODULI)):
        near = [k * m + h + d for k in (-(top // m) + 1, -3, 0, 5, top // m - 2) for h in (m // 2, -(m // 2), 127, 128 - m) for d in (-1, 0, 1)]
        xs = [v for v in vals + near if abs(v) < top]
        a = np.array(xs, dtype=np.float64)
        assert [int(v) for v in a] == xs
        out = np.zeros(len(xs))
        hm.hm_residue_f64(_p(a), C.c_int64(len(xs)), C.c_uint32(m), 0, _p(out))
        want = [cf.signed_residue(v, m) for v in xs]
        got = [int(v) for v in out]
        if m == 256:
            assert all((g - w) % 256 == 0 and -128 <= g <= 127 for g, w in zip(got, want))
        else:
            assert got == want, m
        hm.hm_residue_f64(_p(a), C.c_int64(len(xs)), C.c_uint32(m), 1, _p(out))
        assert all((int(g) - v) % m == 0 and abs(g) <= m / 2 for g, v in zip(out, xs)), m


def test_reduce_small_is_exact_below_2_pow_20(hm):
    hm.hm_reduce_small_errors.restype = C.c_int64
    for m in sorted(set(cf.REAL_MODULI) | set(cf.CPLX_MODULI)):
        assert hm.hm_reduce_small_errors(C.c_uint32(m), C.c_uint32(1 << 20)) == 0, m


def test_frexp_exponents(hm):
    import math
    for tcode, dtype, minnorm in ((0, np.float64, 2.0**-1022), (2, np.float32, 2.0**-126), (4, np.float16, 0.0)):
        for v in [1.0, 0.5, 0.75, 3.0, 1e-5, 65504.0 if dtype == np.float16 else 1e30, np.finfo(dtype).tiny, np.finfo(dtype).tiny / 4, 0.0, 6e-8]:
            x = np.array([v], dtype=dtype)
            want = cf.column_exponent(abs(float(x[0])), 0, minnorm if dtype != np.float16 else 2.0**-126)
            got = hm.hm_frexp(tcode, _p(x))
            assert got == (cf.INT_MAX if want == cf.INT_MAX else -want)


def test_reduce_i32_and_limbs(hm):
    rng = np.random.default_rng(23)
    for m in cf.REAL_MODULI + cf.CPLX_MODULI:
        for v in [0, 1, -1, 2**31 - 1, -2**31, m, -m, 16384 * 131071] + [int(t) for t in rng.integers(-2**31, 2**31, 40)]:
            assert hm.hm_reduce_i32(C.c_int32(v), C.c_uint32(m)) == v % m
    for L in (1, 2, 3):
        bits = 63 * (L - 1) + 64
        for _ in range(200):
            base = int(rng.integers(-2**62, 2**62)) << int(rng.integers(0, max(1, bits - 64)))
            v, sh = int(rng.integers(-2**40, 2**40)), int(rng.integers(0, bits - 42))
            enc = np.zeros(L, np.uint64)
            t = base
            for l in range(L - 1):
                enc[l] = t & (2**63 - 1); t >>= 63
            enc[L - 1] = t & (2**64 - 1)
            out, words = np.zeros(L, np.uint64), np.zeros(3, np.uint64)
            hm.hm_limb_roundtrip(L, _p(enc), C.c_int64(v), C.c_uint32(sh), _p(out), _p(words))
            want = base + (v << sh)
            got = sum(int(out[l]) << (63 * l) for l in range(L - 1)) + ((int(out[L - 1]) - (2**64 if int(out[L - 1]) >= 2**63 else 0)) << (63 * (L - 1)))
            assert got == want


@pytest.mark.parametrize("table,moduli", [(0, cf.REAL_MODULI), (1, cf.CPLX_MODULI)])
def test_crt_lift(hm, table, moduli):
    rng = np.random.default_rng(24)
    for order in range(1, len(moduli) + 1):
        P = 1
        for m in moduli[:order]:
            P *= m
        vals = [0, 1, -1, P // 2 - 1, -(P // 2)] + [int(rng.integers(-2**62, 2**62)) * int(rng.integers(1, 2**62)) % P - P // 2 for _ in range(10)]
        for v in vals:
            # un-reduced residue sums, as the accumulators hold them
            res = np.array([(v % m) + m * int(rng.integers(0, 1000)) for m in moduli[:order]], np.uint32)
            words = np.zeros(3, np.uint64)
            hm.hm_crt_lift(table, order, _p(res), _p(words))
            got = sum(int(words[k]) << (64 * k) for k in range(3))
            got -= (1 << 192) if got >= (1 << 191) else 0
            assert got == v, (order, v)


def test_jacobi_stop_rule(hm):
    """When the host ends the Jacobi sweeps (host/jacobi_stop.hpp): sequences of (rotations, largest cosine) per sweep as
    the kernels report them, with the sweep after which the iteration must end."""
    def sweeps_run(cosines, rotations, tol):
        last = 0.0
        for k, (c, n) in enumerate(zip(cosines, rotations)):
            if hm.hm_jacobi_done(n, c * c, last, tol):
                return k + 1
            last = c * c
        return None
    # real FP64 2048 columns, eps 1e-12 (threshold eps / 16): quadratic from the third sweep on, 2 x (3.27e-7)^2 = 2.1e-13 <= 8 thresholds
    assert sweeps_run([1.17e-2, 4.24e-3, 4.08e-4, 3.27e-7, 6.25e-14], [2096107, 2094368, 1781819, 108880, 0], 6.25e-14) == 4
    # FP32 storage, eps 1e-5
    assert sweeps_run([1.58e-2, 2.38e-3, 4.54e-5, 6.25e-7], [184760, 116616, 1190, 0], 6.25e-7) == 3
    # complex FP64, eps 1e-12
    assert sweeps_run([8.70e-3, 2.62e-3, 9.31e-5, 5.59e-8, 6.25e-14], [2096128, 2095717, 1811563, 109586, 0], 6.25e-14) == 4
    # not yet contracting quadratically (constant above 16): no early end, the confirming sweep runs
    assert sweeps_run([1e-2, 5e-3, 1e-6, 1e-15], [1000, 900, 800, 0], 1e-14) == 4
    # contraction fine but the predicted cosines still above 8 thresholds
    assert hm.hm_jacobi_done(800, (1e-7) ** 2, (1e-4) ** 2, 1e-15) == 0        # constant 10, predicted 1e-13 > 8e-15
    assert hm.hm_jacobi_done(800, (1e-7) ** 2, (1e-4) ** 2, 2e-14) == 1        # 1e-13 <= 1.6e-13
    assert sweeps_run([1e-2, 1e-4, 1e-7, 1e-13, 1e-15], [1000, 900, 800, 10, 0], 1e-15) == 4
    # a sweep that met nothing above 8 thresholds ends the iteration even though it rotated
    assert hm.hm_jacobi_done(5, (7e-14) ** 2, 0.0, 1e-14) == 1
    assert hm.hm_jacobi_done(5, (9e-14) ** 2, 0.0, 1e-14) == 0
    # nothing rotated
    assert hm.hm_jacobi_done(0, 0.25, 0.0, 1e-14) == 1
    # first sweep never ends on the contraction rule (no sweep before it)
    assert hm.hm_jacobi_done(10, 1e-20, 0.0, 1e-14) == 0


def test_jacobi_output_settled_rule(hm):
    """The second way for the sweeps to end (host/jacobi_stop.hpp): the kept values moved by at most eps sigma_max / 4 during
    the sweep and the kept columns gained at most 1 / 32 of the squared norm left outside them."""
    def settled(before, after, kept, eps):
        a, b = np.ascontiguousarray(before, dtype=np.float64), np.ascontiguousarray(after, dtype=np.float64)
        return hm.hm_jacobi_settled(_p(a), _p(b), len(b), kept, eps)
    s = 10.0 ** (-np.arange(40) / 4.0)
    assert settled(s, s, 10, 1e-12) == 1
    assert settled(s, s, 40, 1e-12) == 0 and settled(s, s, 0, 1e-12) == 0          # nothing outside / nothing kept: the other rules decide
    moved = s.copy(); moved[3] += 0.2e-12                                            # a kept value moved by less than eps sigma_max / 4
    assert settled(s, moved, 10, 1e-12) == 1
    moved[3] += 0.2e-12
    assert settled(s, moved, 10, 1e-12) == 0
    # energy still flowing from the columns outside into the kept ones: the residual bound is still improving
    out = s.copy(); out[10:] *= 0.9                                                  # the outside lost 19 % of its squared norm
    assert settled(s, out, 10, 1e-3) == 0
    out = s.copy(); out[10:] *= 0.99                                                 # 2 %: below 1 / 32 of what is left
    assert settled(s, out, 10, 1e-3) == 1
    # the order of the columns does not matter, only the sorted values
    perm = np.random.default_rng(3).permutation(40)
    assert settled(s[perm], out[perm], 10, 1e-3) == 1
    # a flat floor that keeps mixing (its norms move among themselves, their sum stays) does not hold the end back
    floor = np.concatenate([s[:10], np.full(30, 1e-9)]); mixed = floor.copy(); mixed[10:] = 1e-9 * np.sqrt(np.linspace(0.5, 1.5, 30))
    assert abs((mixed[10:] ** 2).sum() - (floor[10:] ** 2).sum()) < 1e-30 and settled(floor, mixed, 10, 1e-12) == 1
    # one sweep early in the fast phase: this sweep moved the values by 2.4e-12 (above eps sigma_max / 4 = 2.5e-13) after 3.7e-8
    # in the sweep before: contraction 6.5e-5, the next move at that rate 1.6e-16 <= eps sigma_max / 4
    hm.hm_jacobi_settled_after.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_double, C.c_double]
    hm.hm_jacobi_settled_after.restype = C.c_int
    def after_move(before, after, kept, eps, last):
        a, b = np.ascontiguousarray(before, dtype=np.float64), np.ascontiguousarray(after, dtype=np.float64)
        return hm.hm_jacobi_settled_after(_p(a), _p(b), len(b), kept, eps, last)
    moved = s.copy(); moved[3] += 2.4e-12
    assert settled(s, moved, 10, 1e-12) == 0 and after_move(s, moved, 10, 1e-12, 0.0) == 0
    assert after_move(s, moved, 10, 1e-12, 3.7e-8) == 1
    assert after_move(s, moved, 10, 1e-12, 1e-10) == 0                               # contraction 1 / 42 only: not the fast phase
    moved = s.copy(); moved[3] += 4e-9
    assert after_move(s, moved, 10, 1e-12, 1e-6) == 0                                # fast (1 / 250), but the next move at that rate, 1.6e-11, is too large
    out = s.copy(); out[3] += 2.4e-12; out[10:] *= 0.9
    assert after_move(s, out, 10, 1e-12, 3.7e-8) == 0                                # the other condition still has to hold


def test_jacobi_head(hm):
    """The columns whose cosines the host watches (host/jacobi_stop.hpp): one past the last index among the K largest norms."""
    def head(norm, K):
        a = np.ascontiguousarray(norm, dtype=np.float64)
        return hm.hm_jacobi_head(_p(a), len(a), K)
    s = 2.0 ** -np.arange(12.0)
    assert head(s, 4) == 4 and head(s, 12) == 12 and head(s, 0) == 12 and head(s, 20) == 12
    t = s.copy(); t[[3, 9]] = t[[9, 3]]                       # the fourth largest sits at index 9
    assert head(t, 4) == 10 and head(t, 3) == 3
    assert head(np.ones(6), 2) == 6                           # ties: every column that could be handed out counts


def test_jacobi_columns_needed(hm):
    """Which prefix of the factor's columns the SVD works on (host/jacobi_stop.hpp): the trailing columns whose squared norms
    sum to at most eps nu_1 nu_K (a quarter of the 4 eps sigma_1 sigma_K the values found must confirm) are left out, never
    fewer than K columns kept.  The bound behind it, checked on an
    explicit matrix: dropping rows of R of squared Frobenius norm tau moves every singular value down, by at most
    tau / (2 sigma') (sigma' the value without them)."""
    rng = np.random.default_rng(11)
    def need(norm, K, eps):
        a = np.ascontiguousarray(norm, dtype=np.float64)
        return hm.hm_jacobi_columns_needed(_p(a), len(a), K, eps)
    floor = np.concatenate([10.0 ** -np.arange(8.0), np.full(100, 1e-9)])        # 8 graded columns over a floor of 100
    # K = 4: nu_1 = 1, nu_4 = 1e-3; eps = 1e-6 allows 1e-9: all of the floor (1e-16) and the columns below it
    t = need(floor, 4, 1e-6)
    assert 4 <= t <= 8 and (floor[t:] ** 2).sum() <= 1e-6 * 1.0 * 1e-3 < (floor[t - 1:] ** 2).sum()
    assert need(floor, 4, 1e-16) == 108                                          # nothing is small enough: 1e-19 < 1e-18
    assert need(floor, 4, 1.02e-12) == 8                                         # exactly the floor (100 x 1e-18 = 1e-16 <= 1.02e-15 ... and 1e-14 more is too much)
    assert need(floor, 108, 1.0) == 108 and need(floor, 0, 1.0) == 108           # every column wanted / no K: all
    assert need(np.full(20, 1.0), 5, 1.0) >= 5                                   # never fewer than K
    # the perturbation bound on an explicit factor: rows of R in pivot order, graded, the last 30 small
    R = rng.standard_normal((40, 60)) * np.concatenate([2.0 ** -np.arange(10.0), np.full(30, 1e-6)])[:, None]
    full = np.linalg.svd(R, compute_uv=False); cut = np.linalg.svd(R[:10], compute_uv=False); tau = (R[10:] ** 2).sum()
    assert np.all(full[:10] >= cut * (1 - 1e-15)) and np.all(full[:10] - cut <= tau / (2 * cut) * (1 + 1e-9))
    assert hm.hm_jacobi_truncation_holds(tau, cut[0], cut[9], tau / (4 * cut[0] * cut[9]) * 1.01) == 1
    assert hm.hm_jacobi_truncation_holds(tau, cut[0], cut[9], tau / (4 * cut[0] * cut[9]) * 0.99) == 0


def test_jacobi_columns_needed_spectral(hm):
    """The sharper cut (host/jacobi_stop.hpp): the largest eigenvalue of the Gram matrix of the columns left out is bounded by
    min(largest absolute row sum, Frobenius norm, trace) of every trailing block; a floor of many unrelated rows passes with
    a trace far above the budget of the values, as long as the trace stays within the budget of the residual."""
    rng = np.random.default_rng(12)
    hm.hm_jacobi_columns_needed_spectral.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_double, C.c_double, C.c_void_p, C.c_void_p]
    hm.hm_jacobi_columns_needed_spectral.restype = C.c_int
    hm.hm_jacobi_truncation_holds_spectral.argtypes = [C.c_double] * 6
    hm.hm_jacobi_truncation_holds_spectral.restype = C.c_int
    N, r, K, c0 = 400, 120, 20, 30
    scale = np.concatenate([2.0 ** -np.arange(40.0), np.full(80, 2.0 ** -40)])            # 40 graded rows over a floor of 80
    R = rng.standard_normal((r, N)) / np.sqrt(N) * scale[:, None]
    M = np.abs(R[c0:] @ R[c0:].T)
    def cut(value, residual):
        a = np.asfortranarray(M); tr, sp = C.c_double(), C.c_double()
        t = hm.hm_jacobi_columns_needed_spectral(a.ctypes.data_as(C.c_void_p), r, c0, K, value, residual, C.byref(tr), C.byref(sp))
        return t, tr.value, sp.value
    def bounds(t):
        B = M[t - c0:, t - c0:]
        return min(B.sum(1).max(), np.linalg.norm(B), np.trace(B)), np.trace(B), np.linalg.eigvalsh(R[t:] @ R[t:].T)[-1]
    floor_trace, floor_top = bounds(40)[1], bounds(40)[2]
    assert floor_top < floor_trace / 10                                                   # 80 unrelated rows: the trace overstates what moves a value
    # values may move by twice the floor's largest eigenvalue, the residual allows all of the floor: the cut takes the whole floor
    # (and what graded rows fit), where the trace rule alone would stop inside it
    t, tr, sp = cut(4 * floor_top, 2 * floor_trace)
    assert c0 <= t <= 40 and tr > 4 * floor_top
    b, trace, top = bounds(t)
    assert np.isclose(sp, b, rtol=1e-12) and np.isclose(tr, trace, rtol=1e-12) and top <= sp <= 4 * floor_top and tr <= 2 * floor_trace
    assert t == c0 or bounds(t - 1)[0] > 4 * floor_top or bounds(t - 1)[1] > 2 * floor_trace          # one more column would break a budget
    # a residual budget below the budget of the values changes nothing: then the trace is held to the budget of the values
    t2, tr2, _ = cut(4 * floor_top, 0.0)
    assert t2 > t and tr2 <= 4 * floor_top and (bounds(t2 - 1)[1] > 4 * floor_top)
    # nothing passes / everything in the window passes; never fewer than K columns kept
    assert cut(0.0, 1.0)[0] == r and cut(1e30, 1e30)[0] == c0
    a = np.asfortranarray(M); tr, sp = C.c_double(), C.c_double()
    assert hm.hm_jacobi_columns_needed_spectral(a.ctypes.data_as(C.c_void_p), r, c0, 50, 1e30, 1e30, C.byref(tr), C.byref(sp)) == 50
    # the test after the sweeps: eigenvalue bound within 4 eps sigma_1 sigma_K, and the trace within that or within 1 / 64 of what is outside
    holds = hm.hm_jacobi_truncation_holds_spectral
    assert holds(1e-3, 3.9e-6, 1.0, 1.0, 0.065, 1e-6) == 1 and holds(1e-3, 4.1e-6, 1.0, 1.0, 0.065, 1e-6) == 0
    assert holds(1e-3, 3.9e-6, 1.0, 1.0, 0.063, 1e-6) == 0 and holds(3.9e-6, 3.9e-6, 1.0, 1.0, 0.0, 1e-6) == 1


def test_jacobi_tail_rule(hm):
    """Which columns the sweeps leave alone (host/jacobi_stop.hpp): the longest trailing index range whose squared norms sum to
    at most 1 / 1024 of max(K-th largest squared norm, eps^2 sum), used only when it holds at least half of the columns.
    Whatever the singular values of that block are, they stay below 1 / 32 of the smallest value handed out (trace bound),
    checked here on an explicit matrix."""
    rng = np.random.default_rng(5)
    def top(norm, K, eps):
        a = np.ascontiguousarray(norm, dtype=np.float64)
        return hm.hm_jacobi_tail_start(_p(a), len(a), K, eps)
    # a few large columns in front of a broad floor: the floor is left alone once its sum is small enough
    assert top(np.concatenate([np.ones(8), np.full(100, 1e-3)]), 8, 0.0) == 8
    assert top(np.concatenate([np.ones(8), np.full(200, 2.0 ** -8)]), 8, 0.0) == 208           # 64 of the 200 would fit (64 / 2^16 = 1 / 1024): fewer than half of all
    assert top(np.concatenate([np.ones(8), np.full(100, 2.0 ** -8)]), 8, 0.0) == 108 - 64      # and here 64 are more than half of 108
    # graded norms: the tail starts where the remaining squared sum drops below nu^2 / 1024; with K close to r too few qualify
    g = 10.0 ** (-np.arange(64) / 8.0); t = top(g, 16, 0.0)
    assert 16 < t <= 32 and (g[t:] ** 2).sum() <= g[15] ** 2 / 1024 < (g[t - 1:] ** 2).sum()
    assert top(g, 40, 0.0) == 64
    # every column handed out, or none: nothing is left alone
    assert top(np.ones(5), 5, 0.0) == 5 and top(np.ones(5), 0, 0.0) == 5 and top(np.zeros(0), 3, 1e-3) == 0
    # unsorted norms: the range ends at the first column (from the back) that does not fit
    assert top(np.array([1.0, 1.0, 1e-4, 1.0, 1e-4, 1e-4, 1e-4, 1e-4]), 3, 0.0) == 4
    # the claim behind the rule, on a matrix whose last block is far from diagonal
    K, r = 6, 30
    B = rng.standard_normal((200, r)) * np.concatenate([np.ones(K), np.full(r - K, 0.0004)])
    Q, _ = np.linalg.qr(B[:, :K]); B[:, K:] -= Q @ (Q.T @ B[:, K:])              # leading columns orthogonal to the rest
    B[:, :K] = Q * np.linalg.norm(B[:, :K], axis=0)
    nrm = np.sqrt((B ** 2).sum(axis=0))
    assert top(nrm, K, 0.0) == K
    sv = np.linalg.svd(B, compute_uv=False)
    assert np.allclose(np.sort(sv[:K]), np.sort(nrm[:K]), rtol=1e-12) and sv[K] <= nrm[:K].min() / 32


def test_stop_rules_on_a_cluster_straddling_k(hm):
    """The loop of hyacinXGevd (host/tail.cpp) on the host, with a plain cyclic one-sided Jacobi in numpy in place of the
    kernels and the stop rules of host/jacobi_stop.hpp as compiled: a factor whose values 10 .. 14 are within 1e-3 of
    each other while K = 12 values are handed out, so that kept and discarded columns stay coupled long after the kept
    values have stopped moving.  Whatever sweep the rules end on, what is handed out must keep the library's promise: values
    within 10 eps of the largest, vectors orthonormal to sqrt(eps), residual of the basis within (10 eps)^2 |R|^2 of the
    optimal one.  (The orthogonality gate is the numpy twin of hykMaxCosine on the K largest columns.)"""
    rng = np.random.default_rng(17)
    n, r, K, eps = 48, 32, 12, 1e-8
    sv = np.concatenate([2.0 ** -np.arange(10.0), 1e-3 * (1 + 1e-3 * np.array([2.0, 1.0, 0.0, -1.0, -2.0])), 1e-5 * 2.0 ** -np.arange(17.0)])
    U, _ = np.linalg.qr(rng.standard_normal((n, r))); W, _ = np.linalg.qr(rng.standard_normal((r, r)))
    R = (U * sv) @ W.T                                          # n x r, singular values sv
    # columns graded as after a pivoted Cholesky: B = Q-less factor of R^T R with column pivoting stands in for the factor
    _, T, piv = __import__("scipy.linalg", fromlist=["qr"]).qr(R, mode="economic", pivoting=True)
    B = T.T.copy()                                              # r x r: column j = row j of the triangular factor; B^T B ~ P^T R^T R P
    tol = max(2.220446049250313e-16 * np.sqrt(r), eps / 16)

    def arr(v):
        return np.ascontiguousarray(v, dtype=np.float64)

    before = np.linalg.norm(B, axis=0)
    last = 0.0
    for sweep in range(60):
        head = hm.hm_jacobi_head(_p(arr(before)), r, K)
        rotations, worst = 0, 0.0
        for p in range(r - 1):
            for q in range(p + 1, r):
                a, b, g = B[:, p] @ B[:, p], B[:, q] @ B[:, q], B[:, p] @ B[:, q]
                if a * b > 0 and (p < head or q < head):
                    worst = max(worst, g * g / (a * b))
                if g * g > tol * tol * a * b and g != 0.0:
                    zeta = (b - a) / (2 * g); t = np.sign(zeta) / (abs(zeta) + np.hypot(1.0, zeta)) if zeta != 0 else 1.0
                    c = 1 / np.hypot(1.0, t); s = c * t
                    B[:, p], B[:, q] = c * B[:, p] - s * B[:, q], s * B[:, p] + c * B[:, q]
                    rotations += 1
        after = np.linalg.norm(B, axis=0)
        if hm.hm_jacobi_done(rotations, worst, last, tol):
            break
        if hm.hm_jacobi_settled(_p(arr(before)), _p(arr(after)), r, K, eps):
            top = np.argsort(-after)[:K]
            Vn = B[:, top] / after[top]
            defect = np.abs(Vn.T @ Vn - np.eye(K)).max()
            if defect <= np.sqrt(eps):
                break
        last, before = worst, after
    else:
        raise AssertionError("the rules never ended the sweeps")
    order = np.argsort(-after)[:K]
    S, V = after[order], B[:, order] / after[order]
    assert np.abs(S - sv[:K]).max() <= 10 * eps * sv[0]
    assert np.abs(V.T @ V - np.eye(K)).max() <= np.sqrt(eps)
    F = T.T                                                     # the factor the sweeps started from; the rotations act on its columns from the right
    resid2 = (F ** 2).sum() - ((V.T @ F) ** 2).sum()            # |F^T - F^T V V^T|_F^2 for orthonormal V: what the projection leaves
    excess = resid2 - (sv[K:] ** 2).sum()
    print("sweeps", sweep + 1, "excess residual", excess, "of", (sv ** 2).sum())
    assert excess <= (10 * eps) ** 2 * (sv ** 2).sum()
