"""Closed forms the CPU oracle is pinned against (Python exact arithmetic).

TEST INFRASTRUCTURE ONLY.  Nothing here follows the reference's code: each
function states what the mathematics fixes, with Fractions / big integers, so
that a slip in the C restatement (a wrong shift, sign, index or a transposed
operand) cannot hide.
"""
from fractions import Fraction
import math

import numpy as np

INT_MAX = 2**31 - 1

REAL_MODULI = [256, 253, 251, 249, 247, 241, 239, 235, 233, 229, 227, 223, 217, 211, 199, 197, 193, 191, 181, 179, 173, 167, 163, 157]
CPLX_MODULI = [241, 233, 229, 221, 205, 197, 193, 181, 173, 157, 149, 137, 113, 109, 101, 97, 89, 73, 61, 53, 256, 253, 251, 249, 239]
CPLX_SPLIT = 20


def column_exponent(col_abs_max, u, min_normal):
    """vexp_j = u - (floor(log2 max) + 1); INT_MAX for a column whose maximum is below the smallest normal."""
    if not (col_abs_max >= min_normal):
        return INT_MAX
    m, e = math.frexp(float(col_abs_max))
    return u - e


def rne_scaled(x, expon):
    """round-half-even of x * 2^expon, exact (x is a finite binary float)."""
    if x == 0:
        return 0
    f = Fraction(float(x)) * (Fraction(2) ** expon)
    fl = f.numerator // f.denominator
    rem = f - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (fl & 1)):
        fl += 1
    return fl


def balanced_digits(q, order):
    """digits d_l in [-128, 127] with sum d_l 256^l == q (mod 256^order): repeated centred remainder."""
    out = []
    for _ in range(order):
        d = ((q + 128) % 256) - 128
        out.append(d)
        q = (q - d) // 256
    return out


def signed_residue(q, m):
    """q mod m stored in int8: residues above 127 wrap by -m (by -256 for m = 256)."""
    r = q % m
    return r - m if r > 127 else r


def sqrt_minus_one(m):
    """all roots of x^2 = -1 mod m"""
    return [x for x in range(m) if (x * x + 1) % m == 0]


def exact_gram(Qre, Qim=None):
    """C[y][x] = sum_k conj(q_ky) q_kx for y <= x with Python integers. Q*: lists of columns of ints."""
    N = len(Qre)
    re, im = {}, {}
    for x in range(N):
        for y in range(x + 1):
            if Qim is None:
                re[(y, x)] = sum(a * b for a, b in zip(Qre[y], Qre[x]))
            else:
                re[(y, x)] = sum(a * b + c * d for a, b, c, d in zip(Qre[y], Qre[x], Qim[y], Qim[x]))
                im[(y, x)] = sum(a * d - c * b for a, b, c, d in zip(Qre[y], Qre[x], Qim[y], Qim[x]))
    return re, im


def packed(tri, N):
    """dict[(y, x)] -> list in packed-triangle order y + x(x+1)/2."""
    out = [0] * (N * (N + 1) // 2)
    for (y, x), v in tri.items():
        out[y + x * (x + 1) // 2] = v
    return out


def crt_centered(residues, moduli):
    """the unique integer in [-P/2, P/2) with the given residues"""
    P = 1
    for m in moduli:
        P *= m
    v = 0
    for r, m in zip(residues, moduli):
        Pd = P // m
        v += r * Pd * pow(Pd % m, -1, m) if m > 1 else 0
    v %= P
    if 2 * v >= P:
        v -= P
    return v


def quantize_matrix(A, vexp):
    """Exact integer columns q[j][k] = RNE(A[k, j] 2^vexp_j); zero column for INT_MAX. Complex -> (re, im)."""
    M, N = A.shape[0], A.shape[1]
    cplx = np.iscomplexobj(A) or (A.ndim == 3)
    if A.ndim == 3:
        Ar, Ai = A[..., 0].astype(np.float64), A[..., 1].astype(np.float64)
    elif cplx:
        Ar, Ai = A.real.astype(np.float64), A.imag.astype(np.float64)
    else:
        Ar, Ai = A.astype(np.float64), None
    qre = [[0 if vexp[j] == INT_MAX else rne_scaled(Ar[k, j], int(vexp[j])) for k in range(M)] for j in range(N)]
    qim = None
    if cplx:
        qim = [[0 if vexp[j] == INT_MAX else rne_scaled(Ai[k, j], int(vexp[j])) for k in range(M)] for j in range(N)]
    return qre, qim


def herk_init(eps, globalM, N, mantissa, cplx, corr=7):
    """eps -> quantisation bits and limb count, from the definitions:
    u = number of binary digits after which 2^-u <= eps (eps = f 2^e, f in [1/2, 1): u = -e, +1 if f == 1/2),
    clamped to the mantissa; uc = clamp(u + corr, -1, 80); the Gram entry sum_k |q|^2 of nextpow2(M) terms of
    2(uc + cplx) bits plus sign needs 1 + 2(uc + cplx) + log2(M) bits, rounded up to 63-bit limbs."""
    f, e = math.frexp(abs(eps))
    u = min(max((1 if f == 0.5 else 0) - e, 0), mantissa)
    uc = max(-1, min(80, u + corr))
    Mp = 1
    while Mp < max(1, globalM):
        Mp *= 2
    lP = (63 + max(0, 2 * (uc + cplx)) + (Mp.bit_length() - 1)) // 63 if uc >= 0 else 0
    return uc, 1 + cplx, lP, N * (N + 1) // 2
