"""The C-ABI library loads without a GPU and exports every function the public headers declare."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared(header):
    txt = open(os.path.join(ROOT, "include", header)).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b(hyacin[A-Z_]\w*|hyk[A-Z]\w*)\s*\(", txt)))


def test_exports_match_headers():
    import hyacinth_amd as ha
    L = ha.lib()
    api, kern = declared("hyacin.h"), declared("hyacin_kernels.h")
    assert len(api) == 16
    assert sorted(ha.API_SYMBOLS) == api and sorted(ha.KERNEL_SYMBOLS) == kern
    for name in api + kern:
        assert hasattr(L, name), name


def test_handle_layout_and_host_planner():
    import ctypes as C
    import hyacinth_amd as ha
    from oracle import ho
    assert C.sizeof(ha.Handle) == 112 and ha.Handle.hipStream.offset == 56
    h = ha.Handle()
    h.QuantizeBitCorrection = 7
    for at, eps, M in ((0, 1e-10, 4096), (2, 1e-5, 65536), (1, 1e-12, 131072), (5, 1e-3, 262144), (0, 1e-8, 1048576)):
        assert ha.herk_batch_init(h, eps, M, 300, at) == ho.herk_batch_init(eps, M, 300, at, 7)
    # precision enum values are ABI
    assert (ha.F64, ha.F64C, ha.F32, ha.F32C, ha.F16, ha.F16C, ha.DD, ha.DDC, ha.TF, ha.TFC, ha.QF, ha.QFC) == tuple(range(12))


def test_every_kernel_entry_has_argument_types():
    """A ctypes call without argtypes passes Python ints as 32-bit C ints: a 64-bit leading dimension would arrive with
    undefined upper bits.  Every kernel-layer function therefore declares its arguments."""
    import hyacinth_amd as ha
    L = ha.lib()
    for name in ha.KERNEL_SYMBOLS:
        assert getattr(L, name).argtypes is not None, name
