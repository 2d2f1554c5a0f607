"""Shared helpers for the tests: seeded synthetic inputs and comparisons."""
import numpy as np

INT_MAX = 2**31 - 1


def rand_matrix(rng, M, N, kind, scale_spread=3.0):
    """kind: f64, f32, f16, c128, c64, c32h (complex half as float16 [M, N, 2])."""
    col = np.exp(rng.standard_normal(N) * scale_spread)
    re = rng.standard_normal((M, N)) * col
    im = rng.standard_normal((M, N)) * col
    if kind == "f64":
        return re
    if kind == "f32":
        return re.astype(np.float32)
    if kind == "f16":
        return np.clip(re, -6e4, 6e4).astype(np.float16)
    if kind == "c128":
        return re + 1j * im
    if kind == "c64":
        return (re + 1j * im).astype(np.complex64)
    if kind == "c32h":
        return np.clip(np.stack([re, im], axis=-1), -6e4, 6e4).astype(np.float16)
    raise ValueError(kind)


ALL_KINDS = ["f64", "f32", "f16", "c128", "c64", "c32h"]


def haar(rng, n, m, cplx=False):
    """n x m matrix with orthonormal columns, Haar distributed (QR of a Gaussian with the sign fix)."""
    g = rng.standard_normal((n, m)) + (1j * rng.standard_normal((n, m)) if cplx else 0)
    q, r = np.linalg.qr(g)
    d = np.diagonal(r)
    return q * (d / np.abs(d))


def as_complex(A):
    if A.ndim == 3:
        return A[..., 0].astype(np.float64) + 1j * A[..., 1].astype(np.float64)
    return A
