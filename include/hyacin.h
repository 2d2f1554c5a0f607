/*
 * hyacin.h -- C API of the MI355X-native Hyacin Gram / low-rank-fit library.
 *
 * Drop-in for the reference's include/hyacin.h on one AMD GPU: same enum
 * values, same handle layout (every resource slot pointer-sized, in the same
 * order), same 16 entry points with the same argument meaning.  Resource types
 * are the HIP / rocBLAS ones; the reference's field names stay usable through
 * anonymous unions (cudaStream, cublasHandle, cusolverHandle).
 *
 * Every pointer named "device-pointer" is HBM memory reachable from the
 * handle's stream; every "host-pointer" is ordinary host memory.
 */
#pragma once
#include <stdint.h>
#include <hip/hip_runtime_api.h>

#ifdef __cplusplus
extern "C" {
#endif

/* reference: include/hyacin.h:11-18 (values are part of the ABI) */
typedef enum {
  HYACIN_F64 = 0, HYACIN_F64_COMPLEX = 1,
  HYACIN_F32 = 2, HYACIN_F32_COMPLEX = 3,
  HYACIN_F16 = 4, HYACIN_F16_COMPLEX = 5,
  HYACIN_DD = 6, HYACIN_DD_COMPLEX = 7,   /* double-double {hi, lo} */
  HYACIN_TF = 8, HYACIN_TF_COMPLEX = 9,   /* triple-float: never produced on an FP64-capable GPU */
  HYACIN_QF = 10, HYACIN_QF_COMPLEX = 11  /* quad-float:   never produced on an FP64-capable GPU */
} hyacinPrecision_t;

struct _rocblas_handle; /* rocblas_handle is a pointer to this */

/* reference: include/hyacin.h:20-53.  Zero-initialise, then hyacinCreate(). */
typedef struct {
  /* Performance parameters (env: HYACIN_GRAM_ALGORITHM 'A'|'L'|'C',
   * HYACIN_STRIDE_BATCH_PERF_PENALTY 1.3, HYACIN_GRAM_SEGMENT_K 8192,
   * HYACIN_TCGEMM_TARGET_K 8192) */
  char GramMatrixAlgorithm;
  double StrideBatchPerfPenalty;
  int32_t GramSegmentK, TCGemmTargetK;

  /* Spectral parameters (env: HYACIN_QUANTIZE_BITS_CORR 7,
   * HYACIN_QRCP_TRUNCATE_RANK 1, HYACIN_JACOBI_SVD_SWEEPS 3) */
  int32_t QuantizeBitCorrection, QRCPTruncateRank, JacobiSVDSweeps;

  /* Device parameters.  DeviceSMs holds the compute-unit count. */
  int32_t DeviceID, DeviceSMs, DeviceIsF64Capable;
  uint32_t HandleOwnedResource;
  union { hipStream_t hipStream; hipStream_t cudaStream; };
  union { struct _rocblas_handle* rocblasHandle; struct _rocblas_handle* cublasHandle; };
  /* rocSOLVER runs on the rocBLAS handle; the slot is kept for layout and may stay null. */
  union { void* solverHandle; void* cusolverHandle; };
  hipMemPool_t mempool;
  void* pinnedWorkspace, *timer, *logger;
} hyacinHandle_t;

/* reference: include/hyacin.h:59-61, src/utils.cpp:56-90 */
void hyacinCreate(hyacinHandle_t* handle);

/* reference: include/hyacin.h:63-65, src/utils.cpp:92-101 */
void hyacinDestroy(hyacinHandle_t* handle);

/* reference: include/hyacin.h:67-81, src/lra.cpp:18-50,210-220.
 * Interpolative decomposition op(A) ~= op(A)[:, jpvt[0:rank]-1] * V^H. Returns rank. */
int32_t hyacinInterpolateFit(
  const hyacinHandle_t* handle, double eps, char opA,
  int32_t M,          /* rows of op(A) */
  int32_t N,          /* cols of op(A), rows of V, length of jpvt */
  int32_t K,          /* cols of V */
  const void* A,      /* device-pointer */
  int32_t lda,
  int32_t* jpvt,      /* device-pointer, LAPACK 1-based */
  void* V,            /* device-pointer, only columns [0, rank) are written */
  int32_t ldv,
  int64_t globalM,    /* total rows if distributed; <= 0 means M */
  hyacinPrecision_t ComputeType);

/* reference: include/hyacin.h:83-97, src/lra.cpp:52-84,222-232.
 * Truncated SVD right basis V (N x rank) and singular values S (K reals of the
 * storage precision; entries >= rank are zero).  Returns rank.
 *
 * How the SVD of the Cholesky factor ends here (the reference hands the factor to the
 * vendor's gesvdj with handle->JacobiSVDSweeps as its sweep limit, src/gram_evd.cu:148-150):
 *  - the sweeps are plain round-robin Jacobi sweeps, each of which does less than a sweep of
 *    the vendor's blocked solver, so the limit is 5 * |JacobiSVDSweeps| of them: 15 with the
 *    default of 3; JacobiSVDSweeps == 0 (the reference's bidiagonalization backend) means a
 *    limit of 30.  They end earlier when a sweep finds no pair above the rotation threshold,
 *    or, with K below the rank of the factor, when the K values handed out have stopped
 *    moving and their vectors are orthogonal to sqrt(eps);
 *  - what is guaranteed for the result: S agrees with the singular values of op(A) to
 *    10 eps S[0] (eps clamped to the machine precision of the storage type), and the columns
 *    of V are orthonormal to max(sqrt(eps), rounding of the storage type) in every entry of
 *    V^H V - I, to max(eps, 1e-12) when all of the factor's columns are handed out (K >= rank
 *    of the factor), so that the projector V V^H is right to eps;
 *  - a failure (allocation, launch, workgroups that lost each other) returns rank 0 with S
 *    and V untouched; hykLastStatus() in hyacin_kernels.h tells which. */
int32_t hyacinTsvdFit(
  const hyacinHandle_t* handle, double eps, char opA,
  int32_t M, int32_t N, int32_t K,
  const void* A, int32_t lda,
  void* S, void* V, int32_t ldv,
  int64_t globalM, hyacinPrecision_t ComputeType);

/* reference: include/hyacin.h:99-113, src/lra.cpp:112-156,234-244.
 * Two-stage column-segmented variant; identical to hyacinTsvdFit when
 * floor(sqrt(N/K)) <= 1 or N < 512. */
int32_t hyacinTsvdFitSegmentN(
  const hyacinHandle_t* handle, double eps, char opA,
  int32_t M, int32_t N, int32_t K,
  const void* A, int32_t lda,
  void* S, void* V, int32_t ldv,
  int64_t globalM, hyacinPrecision_t ComputeType);

/* reference: include/hyacin.h:115-125, src/hyacin_herk.cpp:45-59.  Host-only planning. */
void hyacinXherkBatchInit(
  const hyacinHandle_t* handle, double eps, uint64_t M, int32_t N, hyacinPrecision_t Atype,
  int32_t* uA,        /* host-pointer: quantisation bits incl. correction */
  int32_t* cPanels,   /* host-pointer: 1 real, 2 complex */
  int32_t* lPanels,   /* host-pointer: 63-bit limbs per Gram entry */
  uint64_t* stride);  /* host-pointer: N(N+1)/2 */

/* reference: include/hyacin.h:127-141, src/hyacin_herk.cpp:386-407.
 * C (+)= Q^H Q exactly, Q = round(A * 2^vexp) column-wise.  C holds
 * cPanels*orderC planes of N(N+1)/2 uint64: packed upper triangle, index
 * y + x(x+1)/2 for y <= x, limbs of 63 bits (lower limbs in [0, 2^63), top limb
 * two's complement), real planes first, then imaginary. */
void hyacinXherkBatch(
  const hyacinHandle_t* handle, int32_t batches, int32_t segM, int32_t lastM, int32_t N,
  hyacinPrecision_t Atype,
  const void* A,       /* device-pointer, column-major */
  int32_t lda, int32_t u,
  const int32_t* vexp, /* device-pointer, (batches+1)*N */
  int32_t beta, int32_t orderC,
  uint64_t* C);        /* device-pointer */

/* reference: include/hyacin.h:143-154, src/fp_exponent.cu:53-65.
 * vexp[0:N) = per-column power-of-two scale, vexp[(1+b)*N + j] = scale of row slice b. */
void hyacinXquantizeScaleBatch(
  const hyacinHandle_t* handle, int32_t batches, int32_t segM, int32_t lastM, int32_t N,
  hyacinPrecision_t Atype,
  const void* A,       /* device-pointer */
  int32_t lda, int32_t uA,
  int32_t* vexp);      /* device-pointer */

/* reference: include/hyacin.h:156-165, src/fp_i63tp_dequantize.cu:29-54.  Synchronises the stream. */
void hyacinXdequantizeInit(
  const hyacinHandle_t* handle, int32_t N, int32_t orderC,
  const uint64_t* C,    /* device-pointer */
  const int32_t* vexp,  /* device-pointer */
  hyacinPrecision_t Atype,
  hyacinPrecision_t* Gtype, /* host-pointer */
  int32_t* gElemBytes);     /* host-pointer */

/* reference: include/hyacin.h:167-176, src/fp_i63tp_dequantize.cu:143-159 */
void hyacinXdequantize(
  const hyacinHandle_t* handle, int32_t N, int32_t orderC,
  const uint64_t* C,    /* device-pointer */
  const int32_t* vexp,  /* device-pointer */
  hyacinPrecision_t Gtype,
  void* G,              /* device-pointer, N x N column-major, full Hermitian */
  int32_t ldg);

/* reference: include/hyacin.h:178-190, src/gram_evd.cu:144-194.  G is destroyed. Returns rank. */
int32_t hyacinXGevd(
  const hyacinHandle_t* handle, double eps, int32_t N, int32_t K, hyacinPrecision_t Atype,
  void* X, int32_t ldx,
  void* S,              /* device-pointer */
  hyacinPrecision_t Gtype,
  void* G,              /* device-pointer */
  int32_t ldg);

/* reference: include/hyacin.h:192-204, src/gram_id.cpp:53-101.  G is destroyed. Returns rank. */
int32_t hyacinXGinterp(
  const hyacinHandle_t* handle, double eps, int32_t N, int32_t K, hyacinPrecision_t Atype,
  void* X,              /* device-pointer */
  int32_t ldx,
  int32_t* jpiv,        /* device-pointer */
  hyacinPrecision_t Gtype,
  void* G,              /* device-pointer */
  int32_t ldg);

/* reference: include/hyacin.h:206-217, src/lra.cpp:158-208,246-256.
 * Returns ||op(A) - op(A) Q Q^H||_F^2 with Q = orth(V[:, 0:rank]); ||op(A)||_F^2 if rank <= 0. */
double hyacinCheckNorm(
  const hyacinHandle_t* handle, char opA, int32_t M, int32_t N,
  const void* A,        /* device-pointer */
  int32_t lda, int32_t rank,
  const void* V,        /* device-pointer */
  int32_t ldv, hyacinPrecision_t ComputeType);

/* reference: include/hyacin.h:219-231, src/allreduce_1drow.cu:3-5 (the HYACIN_BUILD_NO_NCCL
 * stubs).  One GPU owns all rows, so both are no-ops. */
void hyacinAllReduce1Drow(const hyacinHandle_t* handle, int32_t Complex, int32_t orderA, uint64_t N, uint64_t* A);
void hyacinAllReduceVExp(const hyacinHandle_t* handle, uint64_t N, int32_t* vexp);

/* reference: include/hyacin.h:233-237, src/utils.cpp:116-141.  eventMs[i] holds a
 * request character 'D' / 'R' / 'C' on entry and the summed milliseconds on return. */
void hyacinSync_TimerSegments(const hyacinHandle_t* handle, double* eventMs, int32_t lenMs);

#ifdef __cplusplus
}
#endif
