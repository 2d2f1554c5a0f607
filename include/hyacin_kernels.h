/*
 * hyacin_kernels.h -- the thin C-ABI layer of hand-written HIP kernels under
 * the hyacin.h API.  Plain pointers and sizes only; every device pointer is HBM
 * memory, every function enqueues on the given stream and returns 0 on success,
 * a negative value for invalid arguments (-1, -2) or a failed launch (-3).
 * The host C++ of the library calls exactly these; tests bind them with ctypes.
 * Precision arguments take hyacinPrecision_t values.
 */
#pragma once
#include <stdint.h>
#include <stddef.h>
#include <hip/hip_runtime_api.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HYK_GRAM_LIMBS 0
#define HYK_GRAM_CRT 1

/* Per-column scales.  Replaces src/fp_exponent.cu:23-51 (init / per-slice exponent / min-reduce kernels).
 * vexp: (batches + 1) * N int32 = [global | slice 0 | slice 1 | ...]. lda in elements. */
int hykColumnExponents(hipStream_t stream, int32_t batches, int32_t segM, int32_t lastM, int32_t N, int32_t Atype, const void* A, int64_t lda, int32_t u, int32_t* vexp);

/* The same with the storage order of A as an argument: opA 'N' as above; 'T' / 'C': A is the stored N x M matrix with
 * op(A)[k, j] = A[j + k lda] (lda >= N), read in place.  Replaces the transposing copy of src/lra.cpp:63-69 +
 * src/matcopy.cu:36-43 followed by the kernels above. */
int hykColumnExponentsOp(hipStream_t stream, char opA, int32_t batches, int32_t segM, int32_t lastM, int32_t N, int32_t Atype, const void* A, int64_t lda, int32_t u, int32_t* vexp);

/* Bits needed per row slice.  Replaces internal::int8::vector_range, src/fp_exponent.cu:67-76. */
int hykSliceRange(hipStream_t stream, int32_t batches, int32_t N, int32_t u, const int32_t* vexp, int32_t* segU);

/* Limb panels.  Replaces internal::int8::quantize_limbs, src/quantize_limbs.cu:46-101.
 * B: panels of N columns x ldb rows int8, panel stride N * ldb; real orderA panels, complex 3 * orderA. */
int hykQuantizeLimbs(hipStream_t stream, int32_t M, int32_t N, int32_t orderA, int32_t Atype, const void* A, int64_t lda, const int32_t* vexp, int8_t* B, int64_t ldb);

/* CRT residue panels.  Replaces internal::int8::quantize_crt, src/quantize_crt_real.cu:63-112 and
 * src/quantize_crt_complex.cu:72-123.  maxBits: bound on the bit length of the quantized magnitudes (<= 0: unknown). */
int hykQuantizeCrt(hipStream_t stream, int32_t M, int32_t N, int32_t orderA, int32_t Atype, const void* A, int64_t lda, const int32_t* vexp, int8_t* B, int64_t ldb, int32_t maxBits);

/* The two quantizers reading op(A) from the stored N x M (conjugate) transpose when opA is 'T' / 'C' (A points at the
 * first of the M stored columns to quantize, lda >= N): a workgroup moves a tile through LDS, so the reads run along the
 * stored columns and the panel bytes still leave K-contiguous; 'C' conjugates on the way.  Same panels, bit for bit, as
 * a transposing copy followed by the column-major kernel (src/lra.cpp:63-69, src/matcopy.cu:36-43). */
int hykQuantizeLimbsOp(hipStream_t stream, char opA, int32_t M, int32_t N, int32_t orderA, int32_t Atype, const void* A, int64_t lda, const int32_t* vexp, int8_t* B, int64_t ldb);
int hykQuantizeCrtOp(hipStream_t stream, char opA, int32_t M, int32_t N, int32_t orderA, int32_t Atype, const void* A, int64_t lda, const int32_t* vexp, int8_t* B, int64_t ldb, int32_t maxBits);

/* Rows [row0, row1) of `cols` consecutive panel columns set to zero.  Replaces the cudaMemset2DAsync padding of
 * src/hyacin_herk.cpp:154,261,275. */
int hykZeroRows(hipStream_t stream, int8_t* B, int64_t ldb, int64_t cols, int32_t row0, int32_t row1);

/* Accumulator workspace of the Gram kernels: size, and clearing (the Gram calls expect it zero and leave it zero). */
size_t hykGramWorkspaceBytes(int32_t kind, int32_t Complex, int32_t N, int32_t orderA);
int hykGramWorkspaceClear(hipStream_t stream, void* workspace, size_t bytes);

/* C (+)= exact integer Gram of CRT residue panels (K rows, multiple of 128, padding rows zero).
 * Replaces i8herk_crt, src/hyacin_herk.cpp:163-281: int8 GEMMs + crt_diag_real / crt_rotate / crt_extra_* + reconstruct_*. */
int hykGramCrt(hipStream_t stream, int32_t Complex, int32_t N, int32_t orderA, const int8_t* panels, int64_t ldb, int32_t K, int32_t beta, int32_t orderC, uint64_t* C, void* workspace);

/* C (+)= exact integer Gram of limb panels.  Replaces i8herk_limbs, src/hyacin_herk.cpp:61-161: int8 GEMMs +
 * limbs_diag / limbs_cross_real / limbs_cross_imag. */
int hykGramLimbs(hipStream_t stream, int32_t Complex, int32_t N, int32_t orderA, const int8_t* panels, int64_t ldb, int32_t K, int32_t beta, int32_t orderC, uint64_t* C, void* workspace);

/* Measurement hooks (no counterpart in the reference): time every launch of the contraction kernel with HIP events on
 * its stream.  hykGramProfile(1) starts a fresh record, hykGramProfile(0) stops; Read waits for the recorded launches.
 * The record belongs to the calling host thread: it times that thread's launches only. */
int hykGramProfile(int32_t enable);
int hykGramProfileRead(double* totalMs, int32_t* launches);

/* Variant of the contraction kernel (tuning knob): 0 = operand slabs loaded straight from global memory into a ring of
 * LDS units with 128-byte rows (default); 2 = the same with 64-byte rows and four stages; 64 / 128 = staged through
 * registers with that many K bytes per LDS stage.  The setting is per host thread. */
int hykGramSetSlab(int32_t bk);

/* Measurement hook (no counterpart in the reference): int8 tera-ops per second that a register-only loop of
 * v_mfma_i32_32x32x32_i8 sustains on `blocks` workgroups of four wavefronts, with pseudo-random (random != 0) or all-zero
 * operands, and the shader clock in GHz it ran at.  The device lowers its clock under the power draw of busy matrix
 * cores, so this -- not the data-sheet peak -- is what a perfect contraction kernel could reach.  Synchronises the stream. */
int hykMfmaCeiling(hipStream_t stream, int32_t blocks, int32_t iters, int32_t random, double* teraOps, double* clockGHz);

/* Bit length of the dominant diagonal entry of the integer Gram.  Replaces gram_range_kernel, src/fp_i63tp_dequantize.cu:17-26. */
int hykGramRange(hipStream_t stream, int32_t N, int32_t orderC, const uint64_t* C, const int32_t* vexp, int32_t* out);

/* Packed integer Gram -> full Hermitian floating Gram.  Replaces triangle_unpack_dequantize_kernel, src/fp_i63tp_dequantize.cu:121-159. */
int hykDequantize(hipStream_t stream, int32_t N, int32_t orderC, const uint64_t* C, const int32_t* vexp, int32_t Gtype, void* G, int64_t ldg);

/* Pivoted Cholesky.  Replaces internal::Cholesky::potrfp, src/hyacin_potrfp.cu:119-343.
 * G: N x N (FP64 / FP64 complex / double-double / double-double complex), Hermitian with both triangles filled; it is
 * working storage: the strict upper triangle is overwritten (the reference overwrites G with the factor).
 * Rt: zero-initialised, column-wise factor Rt[c * ldr + k] = R[k, c] in the type of G, ldr >= min(N, K + 1).
 * jpiv: N 1-based pivots in the reference's swap order.  rankOut: device-visible int32 (pinned host memory); -1 when the
 * workgroups of the run lost each other (a bounded wait inside the kernel gave up).
 * hykPotrfp runs the blocked right-looking kernel (panels of 32 columns, 16 for complex matrices, one rank-32 or rank-16 update of the trailing matrix per
 * panel) for N <= 8192 when computeUnits >= ceil(N / 64), else the left-looking kernel, which hykPotrfpLeftLooking
 * always runs (it leaves G untouched).  Same pivots, same rank; factor entries equal to rounding. */
size_t hykPotrfpWorkspaceBytes(int32_t N, int32_t Gtype);
int hykPotrfp(hipStream_t stream, int32_t computeUnits, double eps, int32_t K, int32_t N, int32_t Gtype, void* G, int64_t ldg, void* Rt, int32_t ldr, int32_t* jpiv, void* workspace, int32_t* rankOut);
int hykPotrfpLeftLooking(hipStream_t stream, int32_t computeUnits, double eps, int32_t K, int32_t N, int32_t Gtype, void* G, int64_t ldg, void* Rt, int32_t ldr, int32_t* jpiv, void* workspace, int32_t* rankOut);
/* hykPotrfp for a caller that will use the `wanted` leading singular values of the factor only (the SVD tail with K < N;
 * no counterpart in the reference, whose factorization always runs to its eps rule, src/gram_evd.cu:105).  The rows never
 * computed are rows left out of G = R^H R: they take what is left of G (positive semidefinite, trace t) off it, which moves
 * a singular value by at most t / (2 sigma).  With b = cut nu_1 nu_w (the norms of rows 1 and w = wanted of the factor, which
 * are what steps 1 and w take off the trace of what is left): if t <= 32 b after
 * `wanted` steps (a floor right under the wanted values), the factorization also ends as soon as t <= b, one step later
 * at the earliest.  Otherwise it
 * runs to its eps rule as hykPotrfp does: the whole budget then stays with a caller that can bound the rows it leaves out
 * more sharply than by their trace.  nu_1 nu_w only estimates sigma_1 sigma_w: the caller has to test t against the values
 * it finds and, should the test fail, factor again without a cut (hykMirrorLower restores G for that: the factorization
 * changes the strict upper triangle only).  traceOut (device or pinned host memory, may be null): t when the factorization
 * ended if the second rule was in force (by whichever rule it then ended), else 0.  wanted <= 0, wanted >= N or cut == 0:
 * hykPotrfp.  The left-looking kernel (N > 8192, few compute units) ignores wanted / cut and reports 0. */
int hykPotrfpWanted(hipStream_t stream, int32_t computeUnits, double eps, int32_t K, int32_t wanted, double cut, int32_t N, int32_t Gtype, void* G, int64_t ldg, void* Rt, int32_t ldr, int32_t* jpiv, void* workspace, int32_t* rankOut, double* traceOut);
/* Process-wide launch mode of the two kernels above (no counterpart in the reference).  They are launched cooperatively by
 * default.  enable != 0: a grid that fits the device by the occupancy query is started with a plain launch.  For runs under
 * profilers whose kernel tracing does not get along with cooperative launches (rocprofv3 --kernel-trace: the process then
 * ends with a segmentation fault in the runtime's exit handler, after the trace has been written); hyacinCreate switches
 * it on when the environment variable HYACIN_PLAIN_LAUNCH is 1 / true.  The bounded waits inside the kernels make a grid
 * that is not resident after all end with rank -1 (status -5) instead of hanging.  A call whose cooperative launch the
 * runtime refuses (a second process on the device that has made cooperative launches of its own) takes the same plain
 * launch, whatever this setting. */
int hykPotrfpSetPlainLaunch(int32_t enable);

/* hykPotrfp for callers that may not call hipMalloc (serving loops, harnesses that forbid it).  No counterpart in the
 * reference.  The workspace of hykPotrfp (diagonal, position table, exchange records; 197 120 bytes) is a device array
 * built into the library, one copy per device, so the call allocates no device memory; inputs and outputs are the caller's
 * as in hykPotrfp.  N <= hykPotrfpStaticMaxN() (8192), larger N returns -2 with a message on stderr.  The first call on a
 * device looks the array's address up and sets a kernel attribute (which may load the code object): make one warm-up call
 * outside any region that must not block.  The launch is cooperative and therefore not meant for stream capture.  All calls
 * on one device share the array: calls that overlap on one device (two streams, two threads) race, and nothing detects it. */
int32_t hykPotrfpStaticMaxN(void);
int hykPotrfpStatic(hipStream_t stream, int32_t computeUnits, double eps, int32_t K, int32_t N, int32_t Gtype, void* G, int64_t ldg, void* Rt, int32_t ldr, int32_t* jpiv, int32_t* rankOut);

/* SVD tail.  Replaces the cuSOLVER gesvdj call and the copies around it, src/gram_evd.cu:110-137.
 * The factor B = (R P^T)^H is N x rank, column-major, complex interleaved, in the precision the reference runs its SVD in
 * (src/gram_evd.cu:96-98): Btype = HYK_F64 / HYK_F64C (0 / 1, doubles) for FP64 storage, HYK_F32 / HYK_F32C (2 / 3, floats)
 * for FP32 and FP16 storage.  With floats a thread keeps its rows and does the arithmetic on them in single precision;
 * the column products of a round are summed across threads in FP64 and every rotation is worked out in FP64. */
int hykFactorToB(hipStream_t stream, int32_t N, int32_t rank, int32_t Gtype, const void* Rt, int32_t ldr, int32_t Btype, void* B);
/* One sweep of one-sided Jacobi over the r columns of B (N x r of type Btype): every pair whose cosine exceeds
 * tol is rotated.  rotations: 16 bytes of device memory, zero before the call; afterwards rotations[0] = pairs rotated,
 * rotations[1] != 0 if a workgroup gave up waiting for its partner (split rounds of hykJacobiSweepCarry: B is then not to be
 * used) and the double at rotations + 2 = the largest squared cosine the sweep met (rotated or not). */
int hykJacobiSweep(hipStream_t stream, int32_t Btype, int32_t N, int32_t r, void* B, double tol, int32_t* rotations);
/* The same sweep with hykJacobiCarryBytes(r) bytes of device memory (16-byte aligned) for its rounds: the products inside a
 * column block travel through it from one round to the next instead of being summed again (ignored by the kernels of
 * variant 1), and it holds the words through which the two workgroups that share a block pair (real factors of up to 2048
 * rows, while the device holds them all at once) keep either from reading rows the other has already rotated.  The
 * memory needs no initialisation and holds nothing a later sweep relies on. */
size_t hykJacobiCarryBytes(int32_t r);
int hykJacobiSweepCarry(hipStream_t stream, int32_t Btype, int32_t N, int32_t r, void* B, double tol, int32_t* rotations, double* carry);
/* The same sweep with two index limits.  Pairs of two columns with index >= top are not rotated (block pairs wholly behind
 * `top` are skipped); the largest cosine is reported over the pairs with at least one column before `head` only (the pairs
 * whose convergence the caller waits for), while rotations[0] still counts every rotation.  head = top = r is the plain
 * sweep.  carry may be null. */
int hykJacobiSweepTop(hipStream_t stream, int32_t Btype, int32_t N, int32_t r, int32_t head, int32_t top, void* B, double tol, int32_t* rotations, double* carry);
/* Which kernel a sweep runs: 0 (default) one Gram matrix per round and workgroup, the steps of the round taken on it by
 * one wavefront; real factors in blocks of 8 columns, complex ones in blocks of 4, the rows of a factor in doubles in two
 * halves where N > 2048;
 * 1 one reduction and barrier per step; 2 as 0 with the narrower blocks that hold all rows at once (4 columns for real
 * factors, 2 for complex ones above 2048 rows).  All rotate by the same rule, and for equal block sizes they visit the
 * pairs in the same order; kept selectable so that tests cover every kernel.  The setting is per host thread. */
int hykJacobiSetVariant(int32_t variant);
/* Test hook (no counterpart in the reference) for the rounds that put two workgroups on a block pair: what they do when the
 * device does not start the partners together, forced from the host so that every kernel still ends normally.  0 (default)
 * nothing forced; 1 / 2 the workgroup of the second / first half of the rows arrives only when its partner has taken the
 * whole pair (and then leaves: the partner's result stands); 3 the second half's workgroup arrives and leaves without
 * reporting its loads, and the first gives up after 256 polls: nothing of the pair is stored, rotations[1] is set and
 * hyacinXGevd ends with status -5.  Per host thread. */
int hykJacobiSetSplitTest(int32_t mode);
int hykColumnNorms(hipStream_t stream, int32_t Btype, int32_t N, int32_t r, const void* B, double* sigma);

/* How far a set of columns is from orthogonal, from their Gram matrix (no counterpart in the reference, which takes what
 * gesvdj returns after its sweep budget, src/gram_evd.cu:9-42): G is n x n column-major of type Gtype (HYK_F64 / HYK_F64C /
 * HYK_F32 / HYK_F32C, complex interleaved), mark[p] != 0 selects the columns that count; *out (device, zero before the call) receives the largest
 * |G[p, q]|^2 / (G[p, p] G[q, q]) over the marked pairs p < q. */
int hykMaxCosine(hipStream_t stream, int32_t Gtype, int32_t n, const void* G, int64_t ldg, const int32_t* mark, double* out);
/* How far n columns are from orthonormal, from their Gram matrix (same types): *out (device, zero before the call) receives
 * the largest |G[p, q] - delta_pq|^2 over p <= q.  No counterpart in the reference. */
int hykMaxDefect(hipStream_t stream, int32_t Gtype, int32_t n, const void* G, int64_t ldg, double* out);
/* G <- (3 I - G) / 2 in place (same types): with G = V^H V, the factor T of the Newton-Schulz step V <- V T towards
 * orthonormal columns of the same span.  No counterpart in the reference. */
int hykNewtonSchulzFactor(hipStream_t stream, int32_t Gtype, int32_t n, void* G, int64_t ldg);
int hykBasisOut(hipStream_t stream, int32_t N, int32_t rank, int32_t Atype, int32_t Btype, const void* B, const double* sigma, const int32_t* order, void* X, int64_t ldx);
int hykValuesOut(hipStream_t stream, int32_t K, int32_t Atype, const double* S, void* out);

/* Interpolation tail.  Replaces cuBLAS trsm + scatter modes 'U' / 'I', src/gram_id.cpp:40-46, src/matcopy.cu:48-52.
 * hykInterpSolve: R11 (K x K) and T (K x (N - K)), FP64 or complex FP64, column-major with leading dimension K, are
 * written: the factor in pivot order and the solution of R11 T = R12 (blocked back substitution).  hykInterpOut scatters
 * the identity and conj(T) into X. */
int hykInterpSolve(hipStream_t stream, int32_t N, int32_t K, int32_t Gtype, const void* Rt, int32_t ldr, const int32_t* jpiv, double* R11, double* T);
int hykInterpOut(hipStream_t stream, int32_t N, int32_t K, int32_t Atype, const int32_t* jpiv, const double* Tt, void* X, int64_t ldx);

/* Converting copy / transpose.  Replaces scatter_matcopy modes 'A', 'T', 'C', src/matcopy.cu:23-44,58-96. */
int hykMatcopy(hipStream_t stream, char mode, int64_t M, int64_t N, int32_t srcType, const void* A, int64_t lda, int32_t dstType, void* B, int64_t ldb);

/* G[y, x] = conj(G[x, y]) for y < x (Gtype: FP64 or double-double, real or complex): writes the strict upper triangle of a
 * Hermitian matrix again from its lower one, which hykPotrfp leaves as it was.  No counterpart in the reference. */
int hykMirrorLower(hipStream_t stream, int32_t N, int32_t Gtype, void* G, int64_t ldg);

/* *out += sum of squares.  Replaces cublasDnrm2_64, src/lra.cpp:170,204. */
int hykSumSquares(hipStream_t stream, int64_t M, int64_t N, const double* A, int64_t lda, double* out);

/* Complex FP16 matrix product C = op(A) B on interleaved half pairs, FP32 accumulation, on the matrix cores
 * (v_mfma_f32_32x32x16_f16; the complex product is a real one of twice the depth, expanded in registers) when the
 * operands and leading dimensions are 16-byte aligned, else on the vector ALU.
 * Replaces internal::matmul_cf16_{cn,tn,nn}, src/matmul_fp16_complex.cu:21-89. opA: 'N', 'T' or 'C'. */
int hykMatmulCf16(hipStream_t stream, char opA, int32_t M, int32_t N, int32_t K, const void* A, int64_t lda, const void* B, int64_t ldb, void* C, int64_t ldc);

/* Real / complex matrix product C = op(A) B in the storage type (FP64, FP32, FP16 and complex FP64 / FP32), used by the
 * column-segmented fit and the residual check.  Replaces the cuBLAS gemm calls of src/lra.cpp:86-105,202-203.
 * alpha/beta are real scalars. opA 'N' | 'T' | 'C', opB 'N' | 'T' | 'C'.  FP16 and FP32 calls (real and complex) of the
 * form C = op(A) B (alpha 1, beta 0, opB 'N') with 16-byte aligned operands and leading dimensions run on the matrix cores
 * (v_mfma_f32_32x32x16_f16, v_mfma_f32_32x32x2_f32, FP32 accumulation); everything else on the vector ALU. */
int hykGemm(hipStream_t stream, char opA, char opB, int32_t M, int32_t N, int32_t K, double alpha, int32_t type, const void* A, int64_t lda, const void* B, int64_t ldb, double beta, void* C, int64_t ldc);

/* V (N x r, FP64 or complex FP64, interleaved) is overwritten by an orthonormal basis of its column space (one-sided
 * Jacobi rotations, then column normalisation).  Replaces the Q factor of cuSOLVER geqrf + orgqr/ungqr,
 * src/lra.cpp:176-191: the same subspace, a different basis of it.  work: r * sizeof(element) + 64 bytes. */
int hykOrthonormalize(hipStream_t stream, int32_t Complex, int32_t N, int32_t r, double* V, int64_t ldv, double* work);

/* hyacinXquantizeScaleBatch / hyacinXherkBatch (include/hyacin.h) with the storage order of A as an argument, as the
 * fits call them: opA 'N' column-major M x N, 'T' / 'C' the stored N x M (conjugate) transpose, lda >= N.  handle is a
 * const hyacinHandle_t*. */
void hykQuantizeScaleBatchOp(const void* handle, char opA, int32_t batches, int32_t segM, int32_t lastM, int32_t N, int32_t Atype, const void* A, int64_t lda, int32_t uA, int32_t* vexp);
void hykHerkBatchOp(const void* handle, char opA, int32_t batches, int32_t segM, int32_t lastM, int32_t N, int32_t Atype, const void* A, int64_t lda, int32_t u, const int32_t* vexp, int32_t beta, int32_t orderC, uint64_t* C);

/* What the last hyacinXherkBatch / hykHerkBatchOp of the calling thread planned and issued (no counterpart in the
 * reference, which prints the same facts through its logger): algorithm ('L' limbs / 'C' residues) and order of the last
 * bucket, rows per contraction call, calls issued, rows contracted, and the algorithmic int8 operations of all
 * contraction calls together (2 per multiply-add, upper triangle only). */
typedef struct { int32_t algorithm, order, chunkRows, gramCalls, quantizeCalls, reserved; int64_t rows; double int8Ops; } hykHerkPlan;
int hykLastHerkPlan(hykHerkPlan* out);

/* Status of the last outermost hyacin.h call made on the calling thread: 0, or the code of the first failure inside it
 * (a HIP error number, a negative kernel-layer return value, -4 a scratch allocation that failed, -5 a pivoted Cholesky
 * or a Jacobi round whose workgroups lost each other).  A failed call has launched nothing after the failure, returned 0 and written
 * neither S nor V (the pivot vector of an interpolation may already hold the pivots).  No counterpart in the reference, which drops every status in release builds (include/internal.hpp:232-236). */
int hykLastStatus(void);

/* Test hook (no counterpart in the reference): the nth scratch acquisition that the calling host thread makes from now on
 * fails as if the memory pool were exhausted; 0 switches the hook off.  Other threads' calls are not affected. */
int hykTestFailAllocation(int32_t nth);

#ifdef __cplusplus
}
#endif
