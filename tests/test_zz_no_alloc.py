"""hykPotrfpStatic, the pivoted Cholesky that allocates nothing (its workspace is a device array built into the library),
against hykPotrfp with a caller-made workspace: same rank, same pivots, same factor, bit for bit, on two calls in a row,
the second on a smaller matrix (the built-in array still holds what the first call left there)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def spd(rng, N, r, cplx, dd):
    U = rng.standard_normal((N, N)) + (1j * rng.standard_normal((N, N)) if cplx else 0)
    U, _ = np.linalg.qr(U)
    sig = np.concatenate([10.0 ** (-np.arange(r) / 3.0), 1e-12 * np.ones(N - r)])
    Gm = (U * sig ** 2) @ U.conj().T
    Gt = ((Gm + Gm.conj().T) / 2).T
    step = 2 if dd else 1
    raw = np.zeros((N, N, step * (2 if cplx else 1)))
    raw[..., 0] = Gt.real
    if cplx:
        raw[..., step] = Gt.imag
    return raw


def run(L, static, raw, N, K, gtype, eps):
    from gpu_util import dev, zeros, ptr, stream, sync, host
    ldr = min(N, K + 1)
    Rt = zeros(N * ldr * raw.shape[2] * 8)
    jp, rk, dG = zeros(N * 4), zeros(4), dev(raw)
    if static:
        rc = L.hykPotrfpStatic(stream(), 256, eps, K, N, gtype, ptr(dG), N, ptr(Rt), ldr, ptr(jp), ptr(rk))
    else:
        ws = zeros(L.hykPotrfpWorkspaceBytes(N, gtype))
        rc = L.hykPotrfp(stream(), 256, eps, K, N, gtype, ptr(dG), N, ptr(Rt), ldr, ptr(jp), ptr(ws), ptr(rk))
    assert rc == 0
    sync()
    return int(host(rk, np.int32)[0]), host(jp, np.int32).copy(), host(Rt, np.uint64).copy()


@pytest.mark.parametrize("gtype", [0, 1, 6, 7])      # FP64, FP64 complex, double-double, double-double complex
def test_potrfp_static_matches_workspace_version(gtype):
    import hyacinth_amd as ha
    L = ha.lib()
    rng = np.random.default_rng(900 + gtype)
    cplx, dd = gtype & 1, gtype >= 6
    assert L.hykPotrfpStaticMaxN() == 8192
    for N, r, K in ((700, 80, 700), (150, 40, 33)):          # second call smaller: stale entries beyond N stay in the array
        raw = spd(rng, N, r, cplx, dd)
        want = run(L, False, raw, N, K, gtype, 1e-9)
        got = run(L, True, raw, N, K, gtype, 1e-9)
        assert want[0] > 0 and got[0] == want[0]
        assert np.array_equal(got[1], want[1])
        assert np.array_equal(got[2], want[2])


def test_potrfp_static_allocates_no_device_memory():
    """After a warm-up call (symbol lookup, kernel attribute), a hykPotrfpStatic call leaves the amount of free device memory
    exactly where it was, while the workspace version's caller had to allocate."""
    import torch
    import hyacinth_amd as ha
    from gpu_util import dev, zeros, ptr, stream, sync
    L = ha.lib()
    rng = np.random.default_rng(905)
    N, K, gtype = 600, 600, 6
    raw = spd(rng, N, 60, 0, True)
    Rt, jp, rk = zeros(N * N * raw.shape[2] * 8), zeros(N * 4), zeros(4)
    dG = [dev(raw) for _ in range(3)]                          # every buffer exists before the measurement starts
    assert L.hykPotrfpStatic(stream(), 256, 1e-9, K, N, gtype, ptr(dG[0]), N, ptr(Rt), N, ptr(jp), ptr(rk)) == 0
    sync()
    before = torch.cuda.mem_get_info()[0]
    for g in dG[1:]:
        assert L.hykPotrfpStatic(stream(), 256, 1e-9, K, N, gtype, ptr(g), N, ptr(Rt), N, ptr(jp), ptr(rk)) == 0
    sync()
    assert torch.cuda.mem_get_info()[0] == before


def test_potrfp_static_rejects_oversize():
    import hyacinth_amd as ha
    from gpu_util import zeros, ptr, stream
    L = ha.lib()
    N = L.hykPotrfpStaticMaxN() + 1
    tiny = zeros(64)
    # arguments are checked before anything is launched: no buffer is touched
    assert L.hykPotrfpStatic(stream(), 256, 1e-6, 4, N, 0, ptr(tiny), N, ptr(tiny), 5, ptr(tiny), ptr(tiny)) == -2
