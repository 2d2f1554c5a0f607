"""hyacinth_amd -- ctypes bindings of libhyacin.so, the MI355X-native implementation
of the Hyacin C API (include/hyacin.h) and of its thin HIP kernel layer
(include/hyacin_kernels.h).

Device memory is handed over as raw pointers; torch is only used by callers for
allocation (tensor.data_ptr()) and is imported here first so that the process
keeps a single HIP runtime.  Nothing here computes on the CPU: if the library is
missing the import fails.
"""
import ctypes as C
import os

try:  # one HIP runtime per process: let torch load its own first when it is installed
    import torch  # noqa: F401
except Exception:  # pragma: no cover
    torch = None

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("HYACIN_LIBRARY") or os.path.join(HERE, "libhyacin.so")   # override: another build of the same library

F64, F64C, F32, F32C, F16, F16C, DD, DDC, TF, TFC, QF, QFC = range(12)
GRAM_LIMBS, GRAM_CRT = 0, 1
INT_MAX = 2**31 - 1

API_SYMBOLS = [
    "hyacinCreate", "hyacinDestroy", "hyacinInterpolateFit", "hyacinTsvdFit", "hyacinTsvdFitSegmentN",
    "hyacinXherkBatchInit", "hyacinXherkBatch", "hyacinXquantizeScaleBatch", "hyacinXdequantizeInit",
    "hyacinXdequantize", "hyacinXGevd", "hyacinXGinterp", "hyacinCheckNorm", "hyacinAllReduce1Drow",
    "hyacinAllReduceVExp", "hyacinSync_TimerSegments",
]
KERNEL_SYMBOLS = [
    "hykColumnExponents", "hykSliceRange", "hykQuantizeLimbs", "hykQuantizeCrt", "hykZeroRows",
    "hykGramWorkspaceBytes", "hykGramWorkspaceClear", "hykGramCrt", "hykGramLimbs", "hykGramSetSlab",
    "hykGramProfile", "hykGramProfileRead", "hykMfmaCeiling", "hykGramRange", "hykDequantize", "hykPotrfpWorkspaceBytes", "hykPotrfp", "hykPotrfpLeftLooking", "hykPotrfpWanted", "hykMirrorLower", "hykPotrfpSetPlainLaunch", "hykPotrfpStaticMaxN", "hykPotrfpStatic", "hykFactorToB", "hykJacobiSweep", "hykJacobiSweepCarry", "hykJacobiSweepTop", "hykJacobiCarryBytes", "hykJacobiSetVariant", "hykJacobiSetSplitTest",
    "hykColumnNorms", "hykBasisOut", "hykValuesOut", "hykInterpSolve", "hykInterpOut", "hykMatcopy",
    "hykSumSquares", "hykMatmulCf16", "hykGemm", "hykOrthonormalize", "hykLastStatus", "hykTestFailAllocation", "hykColumnExponentsOp", "hykQuantizeLimbsOp", "hykQuantizeCrtOp",
    "hykQuantizeScaleBatchOp", "hykHerkBatchOp", "hykLastHerkPlan", "hykMaxCosine", "hykMaxDefect", "hykNewtonSchulzFactor",
]


class Handle(C.Structure):
    """hyacinHandle_t (include/hyacin.h)."""
    _fields_ = [
        ("GramMatrixAlgorithm", C.c_char),
        ("StrideBatchPerfPenalty", C.c_double),
        ("GramSegmentK", C.c_int32), ("TCGemmTargetK", C.c_int32),
        ("QuantizeBitCorrection", C.c_int32), ("QRCPTruncateRank", C.c_int32), ("JacobiSVDSweeps", C.c_int32),
        ("DeviceID", C.c_int32), ("DeviceSMs", C.c_int32), ("DeviceIsF64Capable", C.c_int32),
        ("HandleOwnedResource", C.c_uint32),
        ("hipStream", C.c_void_p), ("rocblasHandle", C.c_void_p), ("solverHandle", C.c_void_p), ("mempool", C.c_void_p),
        ("pinnedWorkspace", C.c_void_p), ("timer", C.c_void_p), ("logger", C.c_void_p),
    ]


class HerkPlan(C.Structure):
    """hykHerkPlan (include/hyacin_kernels.h)."""
    _fields_ = [("algorithm", C.c_int32), ("order", C.c_int32), ("chunkRows", C.c_int32), ("gramCalls", C.c_int32),
                ("quantizeCalls", C.c_int32), ("reserved", C.c_int32), ("rows", C.c_int64), ("int8Ops", C.c_double)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("libhyacin.so is not built: run `python -m hyacinth_amd.build` (needs hipcc)")
        L = C.CDLL(LIB_PATH)
        i32, i64, u64, dbl, vp, ch = C.c_int32, C.c_int64, C.c_uint64, C.c_double, C.c_void_p, C.c_char
        HP = C.POINTER(Handle)
        L.hyacinCreate.argtypes = [HP]; L.hyacinCreate.restype = None
        L.hyacinDestroy.argtypes = [HP]; L.hyacinDestroy.restype = None
        L.hyacinInterpolateFit.argtypes = [HP, dbl, ch, i32, i32, i32, vp, i32, vp, vp, i32, i64, C.c_int]; L.hyacinInterpolateFit.restype = i32
        for f in (L.hyacinTsvdFit, L.hyacinTsvdFitSegmentN):
            f.argtypes = [HP, dbl, ch, i32, i32, i32, vp, i32, vp, vp, i32, i64, C.c_int]; f.restype = i32
        L.hyacinXherkBatchInit.argtypes = [HP, dbl, u64, i32, C.c_int, C.POINTER(i32), C.POINTER(i32), C.POINTER(i32), C.POINTER(u64)]; L.hyacinXherkBatchInit.restype = None
        L.hyacinXherkBatch.argtypes = [HP, i32, i32, i32, i32, C.c_int, vp, i32, i32, vp, i32, i32, vp]; L.hyacinXherkBatch.restype = None
        L.hyacinXquantizeScaleBatch.argtypes = [HP, i32, i32, i32, i32, C.c_int, vp, i32, i32, vp]; L.hyacinXquantizeScaleBatch.restype = None
        L.hyacinXdequantizeInit.argtypes = [HP, i32, i32, vp, vp, C.c_int, C.POINTER(C.c_int), C.POINTER(i32)]; L.hyacinXdequantizeInit.restype = None
        L.hyacinXdequantize.argtypes = [HP, i32, i32, vp, vp, C.c_int, vp, i32]; L.hyacinXdequantize.restype = None
        L.hyacinXGevd.argtypes = [HP, dbl, i32, i32, C.c_int, vp, i32, vp, C.c_int, vp, i32]; L.hyacinXGevd.restype = i32
        L.hyacinXGinterp.argtypes = [HP, dbl, i32, i32, C.c_int, vp, i32, vp, C.c_int, vp, i32]; L.hyacinXGinterp.restype = i32
        L.hyacinCheckNorm.argtypes = [HP, ch, i32, i32, vp, i32, i32, vp, i32, C.c_int]; L.hyacinCheckNorm.restype = dbl
        L.hyacinSync_TimerSegments.argtypes = [HP, C.POINTER(dbl), i32]; L.hyacinSync_TimerSegments.restype = None
        # kernel layer
        L.hykColumnExponents.argtypes = [vp, i32, i32, i32, i32, i32, vp, i64, i32, vp]
        L.hykSliceRange.argtypes = [vp, i32, i32, i32, vp, vp]
        L.hykQuantizeLimbs.argtypes = [vp, i32, i32, i32, i32, vp, i64, vp, vp, i64]
        L.hykQuantizeCrt.argtypes = [vp, i32, i32, i32, i32, vp, i64, vp, vp, i64, i32]
        L.hykZeroRows.argtypes = [vp, vp, i64, i64, i32, i32]
        L.hykGramWorkspaceBytes.argtypes = [i32, i32, i32, i32]; L.hykGramWorkspaceBytes.restype = C.c_size_t
        L.hykGramWorkspaceClear.argtypes = [vp, vp, C.c_size_t]
        L.hykGramCrt.argtypes = [vp, i32, i32, i32, vp, i64, i32, i32, i32, vp, vp]
        L.hykGramLimbs.argtypes = [vp, i32, i32, i32, vp, i64, i32, i32, i32, vp, vp]
        L.hykGramSetSlab.argtypes = [i32]
        L.hykJacobiSetVariant.argtypes = [i32]
        L.hykJacobiSetSplitTest.argtypes = [i32]
        L.hykJacobiSweep.argtypes = [vp, i32, i32, i32, vp, dbl, vp]
        L.hykJacobiSweepCarry.argtypes = [vp, i32, i32, i32, vp, dbl, vp, vp]
        L.hykJacobiSweepTop.argtypes = [vp, i32, i32, i32, i32, i32, vp, dbl, vp, vp]
        L.hykJacobiCarryBytes.argtypes = [i32]; L.hykJacobiCarryBytes.restype = C.c_size_t
        L.hykGramProfile.argtypes = [i32]
        L.hykGramProfileRead.argtypes = [C.POINTER(dbl), C.POINTER(i32)]
        L.hykMfmaCeiling.argtypes = [vp, i32, i32, i32, C.POINTER(dbl), C.POINTER(dbl)]
        L.hykGramRange.argtypes = [vp, i32, i32, vp, vp, vp]
        L.hykDequantize.argtypes = [vp, i32, i32, vp, vp, i32, vp, i64]
        L.hykPotrfpWorkspaceBytes.argtypes = [i32, i32]; L.hykPotrfpWorkspaceBytes.restype = C.c_size_t
        L.hykPotrfp.argtypes = [vp, i32, dbl, i32, i32, i32, vp, i64, vp, i32, vp, vp, vp]
        L.hykPotrfpLeftLooking.argtypes = [vp, i32, dbl, i32, i32, i32, vp, i64, vp, i32, vp, vp, vp]
        L.hykPotrfpWanted.argtypes = [vp, i32, dbl, i32, i32, dbl, i32, i32, vp, i64, vp, i32, vp, vp, vp, vp]
        L.hykMirrorLower.argtypes = [vp, i32, i32, vp, i64]
        L.hykPotrfpSetPlainLaunch.argtypes = [i32]
        L.hykPotrfpStaticMaxN.argtypes = []; L.hykPotrfpStaticMaxN.restype = i32
        L.hykPotrfpStatic.argtypes = [vp, i32, dbl, i32, i32, i32, vp, i64, vp, i32, vp, vp]
        L.hykMatcopy.argtypes = [vp, ch, i64, i64, i32, vp, i64, i32, vp, i64]
        L.hykGemm.argtypes = [vp, ch, ch, i32, i32, i32, dbl, i32, vp, i64, vp, i64, dbl, vp, i64]
        L.hykMatmulCf16.argtypes = [vp, ch, i32, i32, i32, vp, i64, vp, i64, vp, i64]
        L.hykSumSquares.argtypes = [vp, i64, i64, vp, i64, vp]
        L.hykOrthonormalize.argtypes = [vp, i32, i32, i32, vp, i64, vp]
        L.hykColumnExponentsOp.argtypes = [vp, ch, i32, i32, i32, i32, i32, vp, i64, i32, vp]
        L.hykQuantizeLimbsOp.argtypes = [vp, ch, i32, i32, i32, i32, vp, i64, vp, vp, i64]
        L.hykQuantizeCrtOp.argtypes = [vp, ch, i32, i32, i32, i32, vp, i64, vp, vp, i64, i32]
        L.hykMaxCosine.argtypes = [vp, i32, i32, vp, i64, vp, vp]
        L.hykMaxDefect.argtypes = [vp, i32, i32, vp, i64, vp]
        L.hykNewtonSchulzFactor.argtypes = [vp, i32, i32, vp, i64]
        L.hykQuantizeScaleBatchOp.argtypes = [HP, ch, i32, i32, i32, i32, i32, vp, i64, i32, vp]; L.hykQuantizeScaleBatchOp.restype = None
        L.hykHerkBatchOp.argtypes = [HP, ch, i32, i32, i32, i32, i32, vp, i64, i32, vp, i32, i32, vp]; L.hykHerkBatchOp.restype = None
        L.hykLastHerkPlan.argtypes = [C.POINTER(HerkPlan)]
        L.hykLastStatus.argtypes = []
        L.hykTestFailAllocation.argtypes = [i32]
        L.hykFactorToB.argtypes = [vp, i32, i32, i32, vp, i32, i32, vp]
        L.hykColumnNorms.argtypes = [vp, i32, i32, i32, vp, vp]
        L.hykBasisOut.argtypes = [vp, i32, i32, i32, i32, vp, vp, vp, vp, i64]
        L.hykValuesOut.argtypes = [vp, i32, i32, vp, vp]
        L.hykInterpSolve.argtypes = [vp, i32, i32, i32, vp, i32, vp, vp, vp]
        L.hykInterpOut.argtypes = [vp, i32, i32, i32, vp, vp, vp, i64]
        _lib = L
    return _lib


def create_handle(stream=None, **fields):
    """Zero-initialised handle, optional borrowed stream, hyacinCreate(), then field overrides
    (e.g. GramMatrixAlgorithm=b'L')."""
    h = Handle()
    if stream is not None:
        h.hipStream = stream
    lib().hyacinCreate(C.byref(h))
    for k, v in fields.items():
        setattr(h, k, v)
    return h


def destroy_handle(h):
    lib().hyacinDestroy(C.byref(h))


def herk_batch_init(h, eps, M, N, atype):
    u, cP, lP, st = C.c_int32(), C.c_int32(), C.c_int32(), C.c_uint64()
    lib().hyacinXherkBatchInit(C.byref(h), eps, M, N, atype, C.byref(u), C.byref(cP), C.byref(lP), C.byref(st))
    return u.value, cP.value, lP.value, st.value
