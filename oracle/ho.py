"""ctypes front end of the CPU oracle (oracle/hyacin_oracle.c) plus the numpy
restatement of the floating-point tail of the reference.

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of bench.py; never by the library.

The C part covers the integer pipeline (src/fp_exponent.cu,
src/quantize_*.cu, src/hyacin_herk.cpp, src/limbs_*.cu, src/crt_*.cu,
src/fp_i63tp_dequantize.cu, src/hyacin_potrfp.cu).  The part below restates
src/gram_evd.cu:94-142 (tsvd), src/gram_id.cpp:28-51 (interp) and
src/lra.cpp:52-84,158-208 (fit drivers, check_answer) with numpy, using LAPACK
SVD / QR where the reference calls cuSOLVER: those vendor routines are outside
the reference tree, so that tail is compared by tolerance, never bit for bit.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("HYACIN_ORACLE_LIBRARY") or os.path.join(HERE, "libhyacin_oracle.so")   # (the variable: a build of the same source made elsewhere, e.g. with a sanitizer)

F64, F64C, F32, F32C, F16, F16C, DD, DDC = range(8)
INT_MAX = 2**31 - 1
INT_MIN = -(2**31)

NP_DTYPE = {F64: np.float64, F64C: np.complex128, F32: np.float32, F32C: np.complex64, F16: np.float16}


def build(force=False):
    if os.environ.get("HYACIN_ORACLE_LIBRARY"):
        return
    if force or not os.path.exists(LIB_PATH) or os.path.getmtime(LIB_PATH) < os.path.getmtime(os.path.join(HERE, "hyacin_oracle.c")):
        subprocess.check_call(["make", "-C", HERE, "-B", "libhyacin_oracle.so"], stdout=subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = C.CDLL(LIB_PATH)
        _lib.ho_dequantize_init.restype = C.c_int32
        _lib.ho_potrfp.restype = C.c_int32
        _lib.ho_table_count.restype = C.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def atype_of(A):
    """Precision enum of a numpy array; complex half is a float16 array with a trailing axis of 2."""
    if A.dtype == np.float64:
        return F64
    if A.dtype == np.complex128:
        return F64C
    if A.dtype == np.float32:
        return F32
    if A.dtype == np.complex64:
        return F32C
    if A.dtype == np.float16:
        return F16C if (A.ndim == 3 and A.shape[-1] == 2) else F16
    raise TypeError(A.dtype)


def colmajor(A):
    """Column-major contiguous copy; returns (array, lda). Complex half keeps its (re, im) pair innermost."""
    if A.dtype == np.float16 and A.ndim == 3:
        B = np.ascontiguousarray(np.transpose(A, (1, 0, 2)))  # [col][row][2]
        return B, A.shape[0]
    return np.asfortranarray(A), A.shape[0]


# ---------------------------------------------------------------- tables
def tables(which):
    n = lib().ho_table_count(which)
    arrs = [np.zeros(n, np.uint32) for _ in range(6)]
    lib().ho_table_basic(which, *[_p(a) for a in arrs])
    out = dict(zip(["mo", "range", "rem_e32", "rem_e63", "im", "im_inv"], arrs))
    out["prefix"] = {}
    for k in range(1, n + 1):
        minv = np.zeros(k, np.uint32)
        p = np.zeros(3, np.int64)
        pd = np.zeros(4 * k, np.int64)
        lib().ho_table_prefix(which, k, _p(minv), _p(p), _p(pd))
        out["prefix"][k] = (minv, p, pd)
    return out


# ---------------------------------------------------------------- planner
def herk_batch_init(eps, M, N, atype, corr=7):
    u, cP, lP, st = C.c_int32(), C.c_int32(), C.c_int32(), C.c_uint64()
    lib().ho_herk_batch_init(C.c_int32(corr), C.c_double(eps), C.c_uint64(M), C.c_int32(N), C.c_int(atype), C.byref(u), C.byref(cP), C.byref(lP), C.byref(st))
    return u.value, cP.value, lP.value, st.value


def gram_algorithm(alg, K, u, cplx, segmentK=8192, penalty=1.3):
    a = C.c_char(alg.encode())
    f, s = C.c_int32(), C.c_int32()
    lib().ho_gram_algorithm(C.byref(a), C.c_int32(K), C.c_int32(u), C.c_int32(cplx), C.c_int32(segmentK), C.c_double(penalty), C.byref(f), C.byref(s))
    return a.value.decode(), f.value, s.value


# ---------------------------------------------------------------- stages
def quantize_scale_batch(A, batches, segM, lastM, u):
    Af, lda = colmajor(A)
    N = A.shape[1]
    vexp = np.zeros((batches + 1) * N if batches > 0 else N, np.int32)
    lib().ho_quantize_scale_batch(C.c_int32(batches), C.c_int32(segM), C.c_int32(lastM), C.c_int32(N), C.c_int(atype_of(A)), _p(Af), C.c_int64(lda), C.c_int32(u), _p(vexp))
    return vexp


def vector_range(batches, N, u, vexp):
    segU = np.zeros(batches, np.int32)
    lib().ho_vector_range(C.c_int32(batches), C.c_int32(N), C.c_int32(u), _p(vexp), _p(segU))
    return segU


def n_panels(kind, order, cplx):
    if kind == "limbs":
        return order * (3 if cplx else 1)
    if cplx:
        return 2 * order if order <= 20 else 3 * order - 20
    return order


def quantize(kind, A, order, vexp, ldb=None):
    """int8 panels [panel][col][ldb] of quantize_limbs / quantize_crt."""
    Af, lda = colmajor(A)
    M, N = A.shape[0], A.shape[1]
    at = atype_of(A)
    ldb = ldb or M
    B = np.zeros((n_panels(kind, order, at & 1), N, ldb), np.int8)
    fn = lib().ho_quantize_limbs if kind == "limbs" else lib().ho_quantize_crt
    fn(C.c_int32(M), C.c_int32(N), C.c_int32(order), C.c_int(at), _p(Af), C.c_int64(lda), _p(np.ascontiguousarray(vexp[:N])), _p(B), C.c_int64(ldb))
    return B


def i8herk(kind, cplx, N, order, panels, beta, orderC, Cin=None):
    K = panels.shape[2]
    T = N * (N + 1) // 2
    Cout = np.zeros((1 + cplx) * orderC * T, np.uint64) if Cin is None else Cin.copy()
    fn = lib().ho_i8herk_limbs if kind == "limbs" else lib().ho_i8herk_crt
    fn(C.c_int(cplx), C.c_int32(N), C.c_int32(order), _p(np.ascontiguousarray(panels)), C.c_int32(K), C.c_int32(beta), C.c_int32(orderC), _p(Cout))
    return Cout


def reconstruct(cplx, residues, orderX, orderA, beta=0, Cin=None):
    """residues: uint8 [orderX][count] canonical."""
    count = residues.shape[1]
    out = np.zeros(orderA * count, np.uint64) if Cin is None else Cin.copy()
    lib().ho_reconstruct(C.c_int(cplx), C.c_int64(count), C.c_int(orderX), _p(np.ascontiguousarray(residues)), C.c_int(beta), C.c_int(orderA), _p(out))
    return out


def herk_batch(A, batches, segM, lastM, u, vexp, orderC, beta=0, Cin=None, alg="A", penalty=1.3, targetK=8192):
    Af, lda = colmajor(A)
    N = A.shape[1]
    at = atype_of(A)
    T = N * (N + 1) // 2
    Cout = np.zeros((1 + (at & 1)) * orderC * T, np.uint64) if Cin is None else Cin.copy()
    lib().ho_herk_batch(C.c_char(alg.encode()), C.c_double(penalty), C.c_int32(targetK), C.c_int32(batches), C.c_int32(segM), C.c_int32(lastM), C.c_int32(N),
                        C.c_int(at), _p(Af), C.c_int64(lda), C.c_int32(u), _p(vexp), C.c_int32(beta), C.c_int32(orderC), _p(Cout))
    return Cout


def dequantize_init(N, orderC, Cq, vexp, atype, corr=7, f64_capable=1):
    g, b = C.c_int(), C.c_int32()
    bits = lib().ho_dequantize_init(C.c_int32(corr), C.c_int32(f64_capable), C.c_int32(N), C.c_int32(orderC), _p(Cq), _p(vexp), C.c_int(atype), C.byref(g), C.byref(b))
    return g.value, b.value, bits


G_WIDTH = {F64: 1, F64C: 2, F32: 1, F32C: 2, DD: 2, DDC: 4}


def dequantize(N, orderC, Cq, vexp, gtype):
    """G as a raw array [N cols][N rows][width] (column-major, width = scalars per element)."""
    base = np.float32 if gtype in (F32, F32C) else np.float64
    G = np.zeros((N, N, G_WIDTH[gtype]), base)
    lib().ho_dequantize(C.c_int32(N), C.c_int32(orderC), _p(Cq), _p(vexp), C.c_int(gtype), _p(G), C.c_int64(N))
    return G


def g_to_complex(G, gtype):
    """Collapse the raw G layout to an ordinary (N, N) numpy matrix (hi + lo for double-double)."""
    Gt = np.transpose(G, (1, 0, 2)).astype(np.float64)
    if gtype in (F64, F32):
        return Gt[..., 0]
    if gtype in (F64C, F32C):
        return Gt[..., 0] + 1j * Gt[..., 1]
    if gtype == DD:
        return Gt[..., 0] + Gt[..., 1]
    return (Gt[..., 0] + Gt[..., 1]) + 1j * (Gt[..., 2] + Gt[..., 3])


def potrfp(G, gtype, eps, K):
    """In place on the raw G layout; F32 Grams are promoted by the caller. Returns (rank, jpiv)."""
    N = G.shape[0]
    assert G.dtype == np.float64
    jpiv = np.zeros(N, np.int32)
    r = lib().ho_potrfp(C.c_double(eps), C.c_int32(K), C.c_int32(N), C.c_int(gtype), _p(G), C.c_int64(N), _p(jpiv))
    return r, jpiv


# ---------------------------------------------------------------- 63-bit limbs <-> Python ints
def limbs_to_int(Cq, orderC, T, plane=0):
    """Exact integers of one complex plane (0 real, 1 imaginary) of the packed triangle."""
    base = plane * orderC * T
    out = []
    for e in range(T):
        v = 0
        for l in range(orderC):
            w = int(Cq[base + l * T + e])
            if l == orderC - 1 and w >= 2**63:
                w -= 2**64
            v += w << (63 * l)
        out.append(v)
    return out


def int_to_limbs(vals, orderC):
    """Unique encoding: lower limbs in [0, 2^63), top limb two's complement (internal.hpp:116-159)."""
    T = len(vals)
    out = np.zeros(orderC * T, np.uint64)
    for e, v in enumerate(vals):
        for l in range(orderC - 1):
            out[l * T + e] = v & (2**63 - 1)
            v >>= 63
        out[(orderC - 1) * T + e] = v & (2**64 - 1)
    return out


# ---------------------------------------------------------------- floating-point tail
STORAGE_REAL = {F64: np.float64, F64C: np.float64, F32: np.float32, F32C: np.float32, F16: np.float32, F16C: np.float32}


def upper_factor(Graw, gtype, rank, jpiv):
    """B = (R P^T)^H, N x rank: scatter_matcopy('U', jpiv), matcopy.cu:48-52; a double-double R is cut to its high word (matcopy.cu:17)."""
    N = Graw.shape[0]
    Gt = np.transpose(Graw, (1, 0, 2))
    if gtype in (F64, F32):
        R = Gt[..., 0]
    elif gtype in (F64C, F32C):
        R = Gt[..., 0] + 1j * Gt[..., 1]
    elif gtype == DD:
        R = Gt[..., 0]
    else:
        R = Gt[..., 0] + 1j * Gt[..., 2]
    R = np.triu(R[:rank, :])
    B = np.zeros((N, rank), R.dtype)
    B[jpiv - 1, :] = R.conj().T
    return B


def tsvd_tail(Graw, gtype, atype, eps, K, truncate=1):
    """gram_evd.cu:94-142: potrfp, SVD of the factor, energy rank cut. Returns (rank, S[K], V[N, rank])."""
    N = Graw.shape[0]
    real = STORAGE_REAL[atype]
    eps = min(max(abs(eps), float(np.finfo(real).eps)), 1.0)
    G64 = Graw.astype(np.float64)
    rank, jpiv = potrfp(G64, gtype, eps if truncate else 0.0, N)
    S = np.zeros(K, np.float64)
    if rank <= 0:
        return 0, S, np.zeros((N, 0))
    B = upper_factor(G64, gtype, rank, jpiv).astype(np.complex128 if (atype & 1) else np.float64)
    if real == np.float32:
        B = B.astype(np.complex64 if (atype & 1) else np.float32)
    U, sig, _ = np.linalg.svd(B, full_matrices=False)
    sig = sig.astype(np.float64)
    # find_srank_kernel (gram_evd.cu:44-70): keep i < K while the suffix energy exceeds eps^2 * total
    suffix = np.cumsum((sig ** 2)[::-1])[::-1]
    total = suffix[0]
    keep = [i for i in range(K) if (eps == 0.0) or (i < rank and eps * eps * total < suffix[i])]
    for i in keep:
        S[i] = sig[i]
    r = min(rank, len(keep))
    return r, S, U[:, :r]


def interp_tail(Graw, gtype, atype, eps, K):
    """gram_id.cpp:28-51: potrfp(eps, K), X = [I ; (R11^-1 R12)^H] scattered by pivot. Returns (rank, jpiv, X[N, rank])."""
    N = Graw.shape[0]
    real = STORAGE_REAL[atype]
    eps = min(max(abs(eps), float(np.finfo(real).eps)), 1.0)
    G64 = Graw.astype(np.float64)
    rank, jpiv = potrfp(G64, gtype, eps, K)
    if rank <= 0:
        return 0, jpiv, np.zeros((N, 0))
    Gt = np.transpose(G64, (1, 0, 2))
    if gtype in (F64, F32, DD):
        R = Gt[..., 0]
    elif gtype in (F64C, F32C):
        R = Gt[..., 0] + 1j * Gt[..., 1]
    else:
        R = Gt[..., 0] + 1j * Gt[..., 2]
    R = np.triu(R[:rank, :])
    X = np.zeros((N, rank), R.dtype)
    X[jpiv[:rank] - 1, :] = np.eye(rank)
    if rank < N:
        T = np.linalg.solve(R[:, :rank], R[:, rank:])
        X[jpiv[rank:] - 1, :] = T.conj().T
    return rank, jpiv, X


def check_norm(A, V):
    """lra.cpp:158-208: ||A - A Q Q^H||_F^2 with Q = orth(V); ||A||_F^2 when V has no columns."""
    A = np.asarray(A, dtype=np.complex128 if np.iscomplexobj(A) else np.float64)
    if V is None or V.shape[1] == 0:
        return float(np.linalg.norm(A) ** 2)
    Q, _ = np.linalg.qr(np.asarray(V, dtype=A.dtype))
    R = A - (A @ Q) @ Q.conj().T
    return float(np.linalg.norm(R) ** 2)


def fit_plan(M, N, eps, atype, corr=7, segK=8192):
    """lra.cpp:54-60: row slicing and bit plan of one fit."""
    batchIter = M if segK <= 0 else min(segK, M)
    batches = M // max(1, batchIter) + (1 if M % max(1, batchIter) else 0)
    lastM = M % max(1, batchIter) or batchIter
    u, cP, lP, stride = herk_batch_init(eps, M, N, atype, corr)
    return dict(batchIter=batchIter, batches=batches, lastM=lastM, u=u, cP=cP, lP=lP, stride=stride)


def gram_pipeline(A, eps, alg="A", corr=7, segK=8192, targetK=8192, penalty=1.3):
    """lra.cpp:57-79 up to the dequantized Gram. Returns dict with vexp, C, Gtype, G(raw)."""
    M, N = A.shape[0], A.shape[1]
    at = atype_of(A)
    pl = fit_plan(M, N, eps, at, corr, segK)
    vexp = quantize_scale_batch(A, pl["batches"], pl["batchIter"], pl["lastM"], pl["u"])
    Cq = herk_batch(A, pl["batches"], pl["batchIter"], pl["lastM"], pl["u"], vexp, pl["lP"], alg=alg, penalty=penalty, targetK=targetK)
    gtype, gbytes, bits = dequantize_init(N, pl["lP"], Cq, vexp, at, corr)
    G = dequantize(N, pl["lP"], Cq, vexp, gtype)
    return dict(plan=pl, vexp=vexp, C=Cq, gtype=gtype, gbytes=gbytes, bits=bits, G=G)


def tsvd_fit(A, eps, K, **kw):
    K = min(A.shape[1], K)
    g = gram_pipeline(A, eps, **kw)
    r, S, V = tsvd_tail(g["G"], g["gtype"], atype_of(A), eps, K)
    return r, S, V, g


def interpolate_fit(A, eps, K, **kw):
    K = min(A.shape[1], K)
    g = gram_pipeline(A, eps, **kw)
    r, jpiv, X = interp_tail(g["G"], g["gtype"], atype_of(A), eps, K)
    return r, jpiv, X, g
