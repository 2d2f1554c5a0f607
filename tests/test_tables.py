"""CRT constant tables: generated header == oracle's own derivation == number theory == the reference's header text."""
import os
import re
import subprocess
import sys

import numpy as np
import pytest

from oracle import closed_form as cf

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GEN = os.path.join(ROOT, "hyacinth_amd", "csrc", "gen_crt_tables.py")
HDR = os.path.join(ROOT, "hyacinth_amd", "csrc", "crt_tables.h")
REF = "/root/reference/include/crt_constants.hpp"


def test_header_is_up_to_date():
    out = subprocess.check_output([sys.executable, GEN], text=True)
    assert out == open(HDR).read()


def _prefix(moduli, n):
    P = 1
    for m in moduli[:n]:
        P *= m
    return P


@pytest.mark.parametrize("which,moduli", [(0, cf.REAL_MODULI), (1, cf.CPLX_MODULI)])
def test_oracle_tables_number_theory(oracle, which, moduli):
    t = oracle.tables(which)
    assert list(t["mo"]) == moduli
    for x, m in enumerate(moduli):
        assert t["rem_e32"][x] == (1 << 32) % m and t["rem_e63"][x] == (1 << 63) % m
        if which and x < cf.CPLX_SPLIT:
            assert (int(t["im"][x]) ** 2 + 1) % m == 0 and (2 * int(t["im"][x]) * int(t["im_inv"][x])) % m == 1
    for n in range(1, len(moduli) + 1):
        P = _prefix(moduli, n)
        assert t["range"][n - 1] == P.bit_length() - 1
        minv, p, pd = t["prefix"][n]
        assert sum(int(v) << (63 * k) for k, v in enumerate(p)) == P and all(0 <= int(v) < 2**63 for v in p)
        for x in range(n):
            Pd = P // moduli[x]
            assert sum(int(pd[4 * x + k]) << (55 * k) for k in range(4)) == Pd
            assert moduli[x] == 1 or (Pd * int(minv[x])) % moduli[x] == 1


def _parse_generated():
    txt = open(HDR).read()
    out = {}
    for name, body in re.findall(r"HYK_TABLE \w+ (\w+)(?:\[\d+\])+ = \{(.*?)\};", txt, re.S):
        out[name] = [int(v.rstrip("ul"), 0) for v in re.findall(r"0x[0-9a-f]+ull|\d+", body)]
    return out


@pytest.mark.parametrize("which,prefix,moduli", [(0, "hyk_crt_real", cf.REAL_MODULI), (1, "hyk_crt_cplx", cf.CPLX_MODULI)])
def test_generated_header_matches_oracle(oracle, which, prefix, moduli):
    g = _parse_generated()
    t = oracle.tables(which)
    n = len(moduli)
    assert g[prefix + "_mo"] == moduli and g[prefix + "_range"] == list(t["range"])
    for k in range(1, n + 1):
        P = _prefix(moduli, k)
        assert sum(g[prefix + "_P"][3 * (k - 1) + w] << (64 * w) for w in range(3)) == P
        for x in range(k):
            base = ((k - 1) * n + x) * 3
            assert sum(g[prefix + "_Pd"][base + w] << (64 * w) for w in range(3)) == P // moduli[x]
            assert g[prefix + "_minv"][(k - 1) * n + x] == t["prefix"][k][0][x]
    if which:
        assert g["hyk_crt_cplx_im"] == list(t["im"]) and g["hyk_crt_cplx_iminv"] == list(t["im_inv"])


@pytest.mark.skipif(not os.path.exists(REF), reason="reference tree not mounted")
@pytest.mark.parametrize("which,ns", [(0, "U8CRT"), (1, "U8CRT2M")])
def test_oracle_tables_match_reference_text(oracle, which, ns):
    txt = open(REF).read()
    block = txt[txt.index("namespace %s {" % ns):]
    block = block[:block.index("\n};\n")]
    t = oracle.tables(which)

    def arr(name, src):
        m = re.search(r"%s\[\d+\] =\s*\{(.*?)\};" % name, src, re.S)
        return [int(v) for v in re.findall(r"-?\d+", m.group(1).replace("ll", ""))]

    head = block[:block.index("template<>")]
    assert arr("range", head) == list(t["range"]) and arr("mo", head) == list(t["mo"])
    assert arr("rem_e32", head) == list(t["rem_e32"]) and arr("rem_e63", head) == list(t["rem_e63"])
    if which:
        assert arr("im", head) == list(t["im"]) and arr("im_inv", head) == list(t["im_inv"])
        assert int(re.search(r"len_2m_moduli = (\d+)", head).group(1)) == cf.CPLX_SPLIT
    structs = re.findall(r"struct Constants<(\d+)> \{(.*?)\n  \};", block, re.S)
    assert len(structs) == len(t["mo"])
    for n, body in structs:
        n = int(n)
        minv, p, pd = t["prefix"][n]
        assert arr("minv", body) == list(minv) and arr("p", body) == list(p) and arr("pd", body) == list(pd)
