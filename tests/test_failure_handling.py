"""What the library does when something it needs is not there: the call reports on stderr, launches nothing further,
returns 0 and records the failure for hykLastStatus().  The reference drops every status in release builds
(include/internal.hpp:232-236) and asserts in debug builds; a drop-in should at least not compute on null pointers."""
import ctypes as C

import numpy as np
import pytest

import hyacinth_amd as ha


def plain_handle():
    """A handle as a caller would fill it without hyacinCreate: defaults of src/utils.cpp:56-90, no device resources."""
    h = ha.Handle()
    h.GramMatrixAlgorithm = b"A"
    h.StrideBatchPerfPenalty = 1.3
    h.GramSegmentK, h.TCGemmTargetK, h.QuantizeBitCorrection, h.QRCPTruncateRank, h.JacobiSVDSweeps = 8192, 8192, 7, 1, 3
    h.DeviceSMs, h.DeviceIsF64Capable = 256, 1
    return h


def test_first_allocation_failing_stops_the_fit_before_any_device_work():
    """Runs without a GPU: the failure comes before the first HIP call, so nothing touches a device."""
    L = ha.lib()
    h = plain_handle()
    fake = C.c_void_p(0x1000)                       # never dereferenced: the fit stops at its first scratch block
    try:
        for fit in (L.hyacinTsvdFit, L.hyacinTsvdFitSegmentN, L.hyacinInterpolateFit):
            assert L.hykTestFailAllocation(1) == 0
            rank = fit(C.byref(h), 1e-6, b"N", 4096, 64, 16, fake, 4096, fake, fake, 64, 0, ha.F64)
            assert rank == 0 and L.hykLastStatus() == -4
    finally:
        L.hykTestFailAllocation(0)
    # a call that needs nothing starts with a clean status again
    assert L.hyacinTsvdFit(C.byref(h), 1e-6, b"N", 4096, 64, 0, fake, 4096, fake, fake, 64, 0, ha.F64) == 0
    assert L.hykLastStatus() == 0


@pytest.mark.gpu
@pytest.mark.parametrize("fit", ["hyacinTsvdFit", "hyacinInterpolateFit", "hyacinTsvdFitSegmentN"])
def test_any_allocation_failing_leaves_the_outputs_alone(fit):
    """The n-th scratch block of a fit fails, for every n the fit reaches: rank 0, status -4, S and V as they were, and the
    next call on the same handle works."""
    import torch
    from gpu_util import dev, ptr, host, sync
    L = ha.lib()
    rng = np.random.default_rng(91)
    M, N, K = 1500, 600 if fit == "hyacinTsvdFitSegmentN" else 96, 40
    A = rng.standard_normal((M, 30)) @ rng.standard_normal((30, N)) + 1e-9 * rng.standard_normal((M, N))
    dA = dev(np.ascontiguousarray(A.T))
    h = ha.create_handle(stream=torch.cuda.current_stream().cuda_stream)
    fn = getattr(L, fit)
    def run():
        S = dev(np.full(K, 7.0)) if fit != "hyacinInterpolateFit" else dev(np.full(N, 7, np.int32))
        V = dev(np.full((K, N), 7.0))
        rank = fn(C.byref(h), 1e-6, b"N", M, N, K, ptr(dA), M, ptr(S), ptr(V), N, 0, ha.F64)
        sync()
        return rank, host(S, np.int32 if fit == "hyacinInterpolateFit" else np.float64), host(V, np.float64)
    reached = 0
    try:
        for nth in range(1, 200):
            L.hykTestFailAllocation(nth)
            rank, S, V = run()
            if L.hykLastStatus() == 0:                  # the fit needs fewer than nth blocks: the hook is still armed
                assert rank > 0
                break
            reached = nth
            assert rank == 0 and L.hykLastStatus() == -4, (nth, rank, L.hykLastStatus())
            assert (V == 7.0).all(), nth                # the basis is written last
            if fit != "hyacinInterpolateFit":           # (the pivot vector is filled by the factorization itself, before the solve's blocks)
                assert (S == 7).all(), nth
        L.hykTestFailAllocation(0)
        assert reached >= 5
        rank, S, V = run()
        assert rank >= 30 and L.hykLastStatus() == 0
    finally:
        L.hykTestFailAllocation(0)                      # never leave the hook armed for the tests that follow
        ha.destroy_handle(h)


@pytest.mark.gpu
def test_a_jacobi_round_that_loses_its_partner_fails_the_fit():
    """hyacinXGevd with the split Jacobi rounds forced (from the host) into the case where one workgroup of a pair arrives and
    is never heard of again: the other gives up its bounded wait, nothing of the pair is stored, and the call ends with
    status -5, rank 0 and its outputs untouched; the next call works.  With the partner merely late, the fit gives the bits
    of the undisturbed one."""
    import torch
    from gpu_util import dev, ptr, host, sync, zeros
    from util import haar
    L = ha.lib()
    rng = np.random.default_rng(92)
    N = 512
    R = (2.0 ** (-np.arange(N) / 24.0))[:, None] * haar(rng, N, N, False).T
    G = np.ascontiguousarray((R.T @ R).T)
    h = ha.create_handle(stream=torch.cuda.current_stream().cuda_stream)
    def run():
        dG, S, X = dev(G), dev(np.full(N, 7.0)), dev(np.full((N, N), 7.0))
        rank = L.hyacinXGevd(C.byref(h), 1e-9, N, N, 0, ptr(X), N, ptr(S), 0, ptr(dG), N)
        sync()
        return rank, L.hykLastStatus(), host(S, np.float64).copy(), host(X, np.float64).copy()
    try:
        good = run()
        assert good[0] > N // 2 and good[1] == 0
        for mode in (1, 2):
            assert L.hykJacobiSetSplitTest(mode) == 0
            late = run()
            assert late[0] == good[0] and late[1] == 0 and np.array_equal(late[2], good[2]) and np.array_equal(late[3], good[3])
        assert L.hykJacobiSetSplitTest(3) == 0
        rank, status, S, X = run()
        assert rank == 0 and status == -5 and (S == 7.0).all() and (X == 7.0).all()
        L.hykJacobiSetSplitTest(0)
        again = run()
        assert again[0] == good[0] and again[1] == 0 and np.array_equal(again[2], good[2])
    finally:
        L.hykJacobiSetSplitTest(0)
        ha.destroy_handle(h)
