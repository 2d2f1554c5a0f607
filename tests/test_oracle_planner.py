"""Planner restatement (hyacin_herk.cpp:11-59) against known answers worked out by hand from the definitions."""
import math

import pytest

from oracle import closed_form as cf

F64, F64C, F32, F32C, F16, F16C = range(6)
MANT = {F64: 52, F64C: 52, F32: 23, F32C: 23, F16: 10, F16C: 10}

# (eps, globalM, N, type) -> (uc, cPanels, lPanels): the five benchmark configurations and the target shape
KNOWN_INIT = [
    ((1e-10, 4096, 256, F64), (40, 1, 2)),
    ((1e-5, 65536, 1024, F32), (23, 1, 1)),
    ((1e-12, 131072, 2048, F64C), (46, 2, 2)),
    ((1e-3, 262144, 4096, F16C), (16, 2, 1)),
    ((1e-8, 1048576, 4096, F64), (33, 1, 2)),
    ((1e-12, 131072, 2048, F64), (46, 1, 2)),
]


@pytest.mark.parametrize("args,want", KNOWN_INIT)
def test_herk_init_known(oracle, args, want):
    eps, M, N, t = args
    u, cP, lP, stride = oracle.herk_batch_init(eps, M, N, t)
    assert (u, cP, lP) == want and stride == N * (N + 1) // 2
    assert (u, cP, lP, stride) == cf.herk_init(eps, M, N, MANT[t], t & 1)


def test_herk_init_sweep(oracle):
    for t in range(6):
        for e in [1.0, 0.5, 0.25, 0.3, 1e-1, 1e-4, 2.0**-20, 3e-7, 1e-9, 1e-13, 1e-16, 1e-20, 1e-30, 0.0009765625]:
            for M in [1, 2, 3, 1000, 4096, 4097, 10**6, 2**31]:
                for corr in [0, 7, 16, -3, 40]:
                    assert oracle.herk_batch_init(e, M, 17, t, corr) == cf.herk_init(e, M, 17, MANT[t], t & 1, corr)


# (alg in, K, u (+complex already added), complex) -> (alg out, order, second)
KNOWN_ALG = [
    (("L", 4096, 40, 0), ("L", 6, 46)),
    (("A", 4096, 40, 0), ("C", 12, 4096)),          # 2*40+1+12 = 93 bits -> 12 moduli (94 bits), one spare bit
    (("A", 65536, 23, 0), ("C", 8, 65536)),         # 60 bits -> 8 moduli (63), 8192 << 3
    (("A", 131072, 47, 1), ("C", 15, 65536)),       # 108 bits -> 15 complex moduli (111), 8192 << 3
    (("L", 262144, 17, 1), ("L", 3, 22)),
    (("A", 262144, 17, 1), ("C", 7, 262144)),       # 48 bits -> 7 complex moduli (54), 8192 << 6 > K
    (("A", 1048576, 33, 0), ("C", 11, 1048576)),    # 80 bits -> 11 moduli (87), 8192 << 7
    (("A", 131072, 46, 0), ("C", 14, 131072)),      # 106 bits -> 14 moduli (110), 8192 << 4
    (("A", 1000, 7, 0), ("L", 1, 7)),
    (("A", 1000, 14, 0), ("L", 2, 14)),
    (("C", 1000, 90, 0), ("C", 0, 0)),              # 191 bits > 185: CRT cannot hold it
    (("A", 8192, 82, 1), ("C", 25, 8192)),          # 178 bits -> all 25 complex moduli
]


@pytest.mark.parametrize("args,want", KNOWN_ALG)
def test_gram_algorithm_known(oracle, args, want):
    alg, K, u, c = args
    assert oracle.gram_algorithm(alg, K, u, c) == want


def test_gram_algorithm_invariants(oracle):
    for c in (0, 1):
        moduli = cf.CPLX_MODULI if c else cf.REAL_MODULI
        for u in range(0, 82):
            for K in (1, 100, 8192, 100000, 2**20):
                alg, o, second = oracle.gram_algorithm("C", K, u, c)
                bits = 2 * u + 1 + math.ceil(math.log2(min(K, 8192)))
                P = 1
                for m in moduli[:o]:
                    P *= m
                if o:
                    assert P.bit_length() - 1 >= bits, "moduli must cover the chunk Gram"
                    if o > 1:
                        assert (P // moduli[o - 1]).bit_length() - 1 < bits, "one modulus fewer would not"
                    assert second % 128 == 0 or second == 8192 << (P.bit_length() - 1 - bits)
                alg, o, cap = oracle.gram_algorithm("L", K, u, c)
                assert alg == "L" and cap >= u and (o == 1 or [7, 14, 22, 30, 38, 46, 54, 62, 70, 78, 86, 94][o - 2] < u)
