/*
 * tail.hip -- the small N x N tail after the pivoted Cholesky: SVD of the
 * Cholesky factor (truncated-SVD fit) and the triangular solve + scatter of the
 * interpolative decomposition.
 *
 * Replaces, in the reference, the cuSOLVER gesvdj / gesvd call and
 * find_srank_kernel of src/gram_evd.cu:44-142, the cuBLAS trsm of
 * src/gram_id.cpp:8-15,45 and the pivot-scatter modes of src/matcopy.cu:48-52.
 *
 * SVD: one-sided (Hestenes) Jacobi on B = (R P^T)^H, N x r, in FP64.  After the
 * pivoted Cholesky the columns of B are already graded, which is the
 * preconditioning under which a few sweeps reach machine precision (the
 * reference caps its Jacobi at 3 sweeps for the same reason).  Rounds follow
 * the round-robin tournament, so the r/2 column pairs of a round are disjoint:
 * one workgroup per pair, one launch per round.  Column j of the result has
 * norm sigma_j and direction u_j; the right basis of op(A) is V = U.
 *
 * R arrives column-wise: Rt[c * ldr + k] = R[k, c] for physical column c.
 */
#include <type_traits>
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include "hyk_common.h"
#include "hyacin_kernels.h"
#include "jacobi_rounds.h"

namespace {

/* B[c + k*N] = conj(R[k, c]) from the (possibly double-double) column-wise factor; WE doubles per element, WR per real part */
template <bool CPLX, typename XT>
__global__ void factor_to_b_kernel(int32_t N, int32_t rank, const double* __restrict__ Rt, int32_t ldr, int WE, int WR, XT* __restrict__ B) {
  const int c = blockIdx.x * T_THREADS + threadIdx.x, k = blockIdx.y; if (c >= N) { return; }
  const double* src = &Rt[((int64_t)c * ldr + k) * WE];
  if constexpr (CPLX) { B[2 * ((int64_t)c + (int64_t)k * N)] = (XT)src[0]; B[2 * ((int64_t)c + (int64_t)k * N) + 1] = (XT)-src[WR]; } else { B[(int64_t)c + (int64_t)k * N] = (XT)src[0]; }
}


template <bool CPLX, typename XT>
__global__ __launch_bounds__(T_THREADS) void column_norm_kernel(int32_t N, const XT* __restrict__ B, double* __restrict__ sigma) {
  __shared__ double scratch[T_THREADS / 64]; constexpr int W = CPLX ? 2 : 1;
  const XT* b = &B[(int64_t)blockIdx.x * N * W]; double s = 0.;
  for (int k = threadIdx.x; k < N * W; k += T_THREADS) { const double v = b[k]; s += v * v; }
  s = block_sum(s, scratch); if (threadIdx.x == 0) { sigma[blockIdx.x] = sqrt(s); }
}

template <typename T> __device__ __forceinline__ void store_real(T* p, double v);
template <> __device__ __forceinline__ void store_real<double>(double* p, double v) { *p = v; }
template <> __device__ __forceinline__ void store_real<float>(float* p, double v) { *p = (float)v; }
template <> __device__ __forceinline__ void store_real<__half>(__half* p, double v) { __half_raw r; r.data = static_cast<_Float16>(v); *p = r; }

/* X[:, j] = B[:, order[j]] / sigma[order[j]] converted to the storage type, j < rank */
template <typename T, bool CPLX, typename XT>
__global__ void basis_out_kernel(int32_t N, const XT* __restrict__ B, const double* __restrict__ sigma, const int32_t* __restrict__ order, T* __restrict__ X, int64_t ldx) {
  const int k = blockIdx.x * T_THREADS + threadIdx.x, j = blockIdx.y; if (k >= N) { return; }
  const int src = order[j]; const double s = sigma[src], inv = s > 0. ? 1. / s : 0.;
  if constexpr (CPLX) { const XT* b = &B[2 * ((int64_t)src * N + k)]; T* x = &X[2 * ((int64_t)j * ldx + k)]; store_real<T>(x, b[0] * inv); store_real<T>(x + 1, b[1] * inv); }
  else { store_real<T>(&X[(int64_t)j * ldx + k], B[(int64_t)src * N + k] * inv); }
}

/* column j <- column j / sigma_j in place (a zero column stays zero) */
__global__ void normalize_columns_kernel(int32_t N, int W, double* B, const double* sigma) {
  const int k = blockIdx.x * T_THREADS + threadIdx.x, j = blockIdx.y; if (k >= N * W) { return; }
  const double s = sigma[j]; B[(int64_t)j * N * W + k] *= (s > 0. ? 1. / s : 0.);
}

template <typename T> __global__ void values_out_kernel(int32_t K, const double* __restrict__ S, T* __restrict__ out) { const int i = blockIdx.x * T_THREADS + threadIdx.x; if (i < K) { store_real<T>(&out[i], S[i]); } }

/* R in pivot order, high words: R11[k + x K] = R[k, jpiv[x] - 1] for x < K (upper triangle, zero below), and the right-hand
 * sides T[k + (x - K) K] = R[k, jpiv[x] - 1] for x >= K */
template <bool CPLX>
__global__ void gather_factor_kernel(int32_t N, int32_t K, const double* __restrict__ Rt, int32_t ldr, int WE, int WR, const int32_t* __restrict__ jpiv, double* __restrict__ R11, double* __restrict__ T) {
  const int k = blockIdx.x * T_THREADS + threadIdx.x, x = blockIdx.y; if (k >= K) { return; }
  const double* src = &Rt[((int64_t)(jpiv[x] - 1) * ldr + k) * WE]; const bool low = k > x;
  double* dst = x < K ? &R11[((int64_t)k + (int64_t)x * K) * (CPLX ? 2 : 1)] : &T[((int64_t)k + (int64_t)(x - K) * K) * (CPLX ? 2 : 1)];
  dst[0] = low ? 0. : src[0]; if constexpr (CPLX) { dst[1] = low ? 0. : src[WR]; }
}

/* One block row of the blocked back substitution R11 T = R12: T[i0 .. i0+rows) <- R11[i0.., i0..]^-1 T[i0 .. i0+rows), the
 * rows below already eliminated from it by a matrix product.  One thread per right-hand side keeps its `rows` entries in
 * registers; the triangle sits in LDS (every thread reads the same entry: a broadcast). */
constexpr int SOLVE_ROWS = 32;
template <bool CPLX>
__global__ __launch_bounds__(T_THREADS) void block_solve_kernel(int32_t K, int32_t ncols, int32_t i0, int32_t rows, const double* __restrict__ R11, double* __restrict__ T) {
  constexpr int W = CPLX ? 2 : 1;
  __shared__ double tri[SOLVE_ROWS][SOLVE_ROWS][W];
  for (int e = threadIdx.x; e < SOLVE_ROWS * SOLVE_ROWS; e += T_THREADS) {
    const int i = e % SOLVE_ROWS, j = e / SOLVE_ROWS; const bool in = i < rows && j < rows;
    #pragma unroll
    for (int w = 0; w < W; ++w) { tri[i][j][w] = in ? R11[((int64_t)(i0 + i) + (int64_t)(i0 + j) * K) * W + w] : 0.; }
  }
  __syncthreads();
  const int col = blockIdx.x * T_THREADS + threadIdx.x; if (col >= ncols) { return; }
  double* t = &T[((int64_t)i0 + (int64_t)col * K) * W];
  double x[SOLVE_ROWS][W];
  #pragma unroll
  for (int i = 0; i < SOLVE_ROWS; ++i) {
    #pragma unroll
    for (int w = 0; w < W; ++w) { x[i][w] = i < rows ? t[i * W + w] : 0.; }
  }
  #pragma unroll
  for (int i = SOLVE_ROWS - 1; i >= 0; --i) {
    if (i < rows) {
      double sr = x[i][0], si = CPLX ? x[i][W - 1] : 0.;
      #pragma unroll
      for (int j = i + 1; j < SOLVE_ROWS; ++j) {
        if constexpr (CPLX) { sr -= tri[i][j][0] * x[j][0] - tri[i][j][1] * x[j][1]; si -= tri[i][j][0] * x[j][1] + tri[i][j][1] * x[j][0]; }
        else { sr -= tri[i][j][0] * x[j][0]; }
      }
      const double d = tri[i][i][0];   /* the diagonal of R is real */
      x[i][0] = sr / d; if constexpr (CPLX) { x[i][1] = si / d; }
    }
  }
  #pragma unroll
  for (int i = 0; i < SOLVE_ROWS; ++i) {
    if (i < rows) {
      #pragma unroll
      for (int w = 0; w < W; ++w) { t[i * W + w] = x[i][w]; }
    }
  }
}

/* X[jpiv[x]-1, y] = (x < K) ? (x == y) : conj(T[y, x-K]) for y < K (reference: scatter mode 'I', src/matcopy.cu:48-52); T is K x (N - K), column-major */
template <typename T, bool CPLX>
__global__ void interp_out_kernel(int32_t N, int32_t K, const int32_t* __restrict__ jpiv, const double* __restrict__ Tt, T* __restrict__ X, int64_t ldx) {
  const int y = blockIdx.x * T_THREADS + threadIdx.x, x = blockIdx.y; if (y >= K) { return; }
  const int64_t row = jpiv[x] - 1; double vr, vi = 0.;
  if (x < K) { vr = (x == y) ? 1. : 0.; } else { const double* t = &Tt[((int64_t)y + (int64_t)(x - K) * K) * (CPLX ? 2 : 1)]; vr = t[0]; if constexpr (CPLX) { vi = -t[1]; } }
  if constexpr (CPLX) { T* o = &X[2 * (row + (int64_t)y * ldx)]; store_real<T>(o, vr); store_real<T>(o + 1, vi); } else { store_real<T>(&X[row + (int64_t)y * ldx], vr); }
}

}  // namespace

/* Btype of the entry points below: HYK_F64 / HYK_F64C (0 / 1: B in doubles) or HYK_F32 / HYK_F32C (2 / 3: B in floats) */
static bool btype_ok(int32_t Btype) { return Btype >= HYK_F64 && Btype <= HYK_F32C; }

extern "C" int hykFactorToB(hipStream_t stream, int32_t N, int32_t rank, int32_t Gtype, const void* Rt, int32_t ldr, int32_t Btype, void* B) {
  if (N <= 0 || rank <= 0) { return 0; }
  const bool dd = (Gtype & ~1) == HYK_DD, cplx = Gtype & 1; const int WR = dd ? 2 : 1, WE = WR * (cplx ? 2 : 1);
  if (!btype_ok(Btype) || (Btype & 1) != (Gtype & 1)) { return -1; }
  dim3 grid((N + T_THREADS - 1) / T_THREADS, rank);
  if ((Btype & ~1) == HYK_F32) {
    if (cplx) { factor_to_b_kernel<true, float><<<grid, T_THREADS, 0, stream>>>(N, rank, (const double*)Rt, ldr, WE, WR, (float*)B); } else { factor_to_b_kernel<false, float><<<grid, T_THREADS, 0, stream>>>(N, rank, (const double*)Rt, ldr, WE, WR, (float*)B); }
  } else {
    if (cplx) { factor_to_b_kernel<true, double><<<grid, T_THREADS, 0, stream>>>(N, rank, (const double*)Rt, ldr, WE, WR, (double*)B); } else { factor_to_b_kernel<false, double><<<grid, T_THREADS, 0, stream>>>(N, rank, (const double*)Rt, ldr, WE, WR, (double*)B); }
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

/* one sweep = every pair of the r columns of B (N x r, FP64, complex interleaved) once; rotations counts the rotations applied */
static thread_local int g_splitTest = 0;   /* hykJacobiSetSplitTest */
static thread_local int g_jacobiVariant = 0;   /* 0: Gram-space rounds, 8-column blocks for real factors where they fit (default); 1: the step kernel everywhere; 2: Gram-space rounds, 4-column blocks */


extern "C" int hykJacobiSetSplitTest(int32_t mode) { if (mode < 0 || mode > 3) { return -1; } g_splitTest = mode; return 0; }

extern "C" int hykJacobiSetVariant(int32_t variant) { if (variant < 0 || variant > 2) { return -1; } g_jacobiVariant = variant; return 0; }

extern "C" size_t hykJacobiCarryBytes(int32_t r) { return r <= 0 ? 0 : carried_bytes(r) + pair_word_bytes(r); }

extern "C" int hykJacobiSweep(hipStream_t stream, int32_t Btype, int32_t N, int32_t r, void* B, double tol, int32_t* rotations) { return hykJacobiSweepTop(stream, Btype, N, r, r, r, B, tol, rotations, nullptr); }

extern "C" int hykJacobiSweepCarry(hipStream_t stream, int32_t Btype, int32_t N, int32_t r, void* B, double tol, int32_t* rotations, double* carry) { return hykJacobiSweepTop(stream, Btype, N, r, r, r, B, tol, rotations, carry); }

extern "C" int hykJacobiSweepTop(hipStream_t stream, int32_t Btype, int32_t N, int32_t r, int32_t head, int32_t top, void* B, double tol, int32_t* rotations, double* carry) {
  if (!btype_ok(Btype)) { return -1; }
  if ((Btype & ~1) == HYK_F32) { return hyk_jacobi_sweep_f32(stream, Btype & 1, N, r, head, top, (float*)B, tol, rotations, carry, g_jacobiVariant, g_splitTest); }
  return sweep_top<double>(stream, Btype & 1, N, r, head, top, (double*)B, tol, rotations, carry, g_jacobiVariant, g_splitTest);
}

extern "C" int hykColumnNorms(hipStream_t stream, int32_t Btype, int32_t N, int32_t r, const void* B, double* sigma) {
  if (N <= 0 || r <= 0) { return 0; }
  if (!btype_ok(Btype)) { return -1; }
  const bool Complex = Btype & 1;
  if ((Btype & ~1) == HYK_F32) { if (Complex) { column_norm_kernel<true, float><<<r, T_THREADS, 0, stream>>>(N, (const float*)B, sigma); } else { column_norm_kernel<false, float><<<r, T_THREADS, 0, stream>>>(N, (const float*)B, sigma); } }
  else if (Complex) { column_norm_kernel<true, double><<<r, T_THREADS, 0, stream>>>(N, (const double*)B, sigma); } else { column_norm_kernel<false, double><<<r, T_THREADS, 0, stream>>>(N, (const double*)B, sigma); }
  return 0;
}

/* the largest squared cosine among the marked columns, from their Gram matrix: G column-major n x n (complex interleaved),
 * mark[p] != 0 for the columns that count; out: one double, zero before the call, raised by an integer maximum on its bits */
/* DEFECT: the largest |G[p, q] - delta_pq|^2 over all p <= q instead (how far columns that should be orthonormal are from it; no marks) */
template <bool CPLX, typename GT, bool DEFECT = false>
__global__ __launch_bounds__(T_THREADS) void max_cosine_kernel(int32_t n, const GT* __restrict__ G, int64_t ldg, const int32_t* __restrict__ mark, double* __restrict__ out) {
  __shared__ double scratch[T_THREADS / 64]; constexpr int W = CPLX ? 2 : 1;
  const int q = blockIdx.x; double worst = 0.;
  if constexpr (DEFECT) {
    for (int p = threadIdx.x; p <= q; p += T_THREADS) {
      const GT* g = &G[((int64_t)p + (int64_t)q * ldg) * W]; const double g0 = (double)g[0] - (p == q ? 1. : 0.); double g2 = g0 * g0; if constexpr (CPLX) { const double g1 = g[1]; g2 = fma(g1, g1, g2); }
      worst = fmax(worst, g2);
    }
  } else if (mark[q]) {
    const double gqq = G[((int64_t)q + (int64_t)q * ldg) * W];
    for (int p = threadIdx.x; p < q; p += T_THREADS) {
      if (!mark[p]) { continue; }
      const GT* g = &G[((int64_t)p + (int64_t)q * ldg) * W]; const double g0 = g[0]; double g2 = g0 * g0; if constexpr (CPLX) { const double g1 = g[1]; g2 = fma(g1, g1, g2); }
      worst = fmax(worst, squared_cosine(g2, G[((int64_t)p + (int64_t)p * ldg) * W], gqq));
    }
  }
  for (int off = 32; off > 0; off >>= 1) { worst = fmax(worst, __shfl_xor(worst, off, 64)); }
  if ((threadIdx.x & 63) == 0) { scratch[threadIdx.x >> 6] = worst; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < T_THREADS / 64; ++w) { worst = fmax(worst, scratch[w]); }
    if (worst > 0.) { atomicMax(reinterpret_cast<unsigned long long*>(out), (unsigned long long)__double_as_longlong(worst)); }
  }
}

extern "C" int hykMaxCosine(hipStream_t stream, int32_t Gtype, int32_t n, const void* G, int64_t ldg, const int32_t* mark, double* out) {
  if (n <= 1) { return 0; }
  if (ldg < n || !btype_ok(Gtype)) { return -1; }
  const bool Complex = Gtype & 1;
  if ((Gtype & ~1) == HYK_F32) { if (Complex) { max_cosine_kernel<true, float><<<n, T_THREADS, 0, stream>>>(n, (const float*)G, ldg, mark, out); } else { max_cosine_kernel<false, float><<<n, T_THREADS, 0, stream>>>(n, (const float*)G, ldg, mark, out); } }
  else if (Complex) { max_cosine_kernel<true, double><<<n, T_THREADS, 0, stream>>>(n, (const double*)G, ldg, mark, out); } else { max_cosine_kernel<false, double><<<n, T_THREADS, 0, stream>>>(n, (const double*)G, ldg, mark, out); }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

/* G <- (3 I - G) / 2 in place: the factor of the Newton-Schulz step V <- V (3 I - V^H V) / 2 from the Gram matrix G = V^H V */
template <bool CPLX, typename GT>
__global__ __launch_bounds__(T_THREADS) void newton_schulz_factor_kernel(int32_t n, GT* __restrict__ G, int64_t ldg) {
  constexpr int W = CPLX ? 2 : 1; const int q = blockIdx.x;
  for (int p = threadIdx.x; p < n; p += T_THREADS) {
    GT* g = &G[((int64_t)p + (int64_t)q * ldg) * W];
    g[0] = (GT)((p == q ? 1.5 : 0.) - 0.5 * (double)g[0]); if constexpr (CPLX) { g[1] = (GT)(-0.5 * (double)g[1]); }
  }
}

extern "C" int hykNewtonSchulzFactor(hipStream_t stream, int32_t Gtype, int32_t n, void* G, int64_t ldg) {
  if (n <= 0) { return 0; }
  if (ldg < n || !btype_ok(Gtype)) { return -1; }
  const bool Complex = Gtype & 1;
  if ((Gtype & ~1) == HYK_F32) { if (Complex) { newton_schulz_factor_kernel<true, float><<<n, T_THREADS, 0, stream>>>(n, (float*)G, ldg); } else { newton_schulz_factor_kernel<false, float><<<n, T_THREADS, 0, stream>>>(n, (float*)G, ldg); } }
  else if (Complex) { newton_schulz_factor_kernel<true, double><<<n, T_THREADS, 0, stream>>>(n, (double*)G, ldg); } else { newton_schulz_factor_kernel<false, double><<<n, T_THREADS, 0, stream>>>(n, (double*)G, ldg); }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

extern "C" int hykMaxDefect(hipStream_t stream, int32_t Gtype, int32_t n, const void* G, int64_t ldg, double* out) {
  if (n <= 0) { return 0; }
  if (ldg < n || !btype_ok(Gtype)) { return -1; }
  const bool Complex = Gtype & 1;
  if ((Gtype & ~1) == HYK_F32) { if (Complex) { max_cosine_kernel<true, float, true><<<n, T_THREADS, 0, stream>>>(n, (const float*)G, ldg, nullptr, out); } else { max_cosine_kernel<false, float, true><<<n, T_THREADS, 0, stream>>>(n, (const float*)G, ldg, nullptr, out); } }
  else if (Complex) { max_cosine_kernel<true, double, true><<<n, T_THREADS, 0, stream>>>(n, (const double*)G, ldg, nullptr, out); } else { max_cosine_kernel<false, double, true><<<n, T_THREADS, 0, stream>>>(n, (const double*)G, ldg, nullptr, out); }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

template <typename XT>
static int basis_out(hipStream_t stream, int32_t N, int32_t rank, int32_t Atype, const XT* B, const double* sigma, const int32_t* order, void* X, int64_t ldx) {
  dim3 grid((N + T_THREADS - 1) / T_THREADS, rank);
  switch (Atype) {
    case HYK_F64: basis_out_kernel<double, false, XT><<<grid, T_THREADS, 0, stream>>>(N, B, sigma, order, (double*)X, ldx); break;
    case HYK_F32: basis_out_kernel<float, false, XT><<<grid, T_THREADS, 0, stream>>>(N, B, sigma, order, (float*)X, ldx); break;
    case HYK_F16: basis_out_kernel<__half, false, XT><<<grid, T_THREADS, 0, stream>>>(N, B, sigma, order, (__half*)X, ldx); break;
    case HYK_F64C: basis_out_kernel<double, true, XT><<<grid, T_THREADS, 0, stream>>>(N, B, sigma, order, (double*)X, ldx); break;
    case HYK_F32C: basis_out_kernel<float, true, XT><<<grid, T_THREADS, 0, stream>>>(N, B, sigma, order, (float*)X, ldx); break;
    case HYK_F16C: basis_out_kernel<__half, true, XT><<<grid, T_THREADS, 0, stream>>>(N, B, sigma, order, (__half*)X, ldx); break;
    default: return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

extern "C" int hykBasisOut(hipStream_t stream, int32_t N, int32_t rank, int32_t Atype, int32_t Btype, const void* B, const double* sigma, const int32_t* order, void* X, int64_t ldx) {
  if (N <= 0 || rank <= 0) { return 0; }
  if (!btype_ok(Btype) || (Btype & 1) != (Atype & 1)) { return -1; }
  return (Btype & ~1) == HYK_F32 ? basis_out<float>(stream, N, rank, Atype, (const float*)B, sigma, order, X, ldx) : basis_out<double>(stream, N, rank, Atype, (const double*)B, sigma, order, X, ldx);
}

extern "C" int hykValuesOut(hipStream_t stream, int32_t K, int32_t Atype, const double* S, void* out) {
  if (K <= 0) { return 0; }
  const int grid = (K + T_THREADS - 1) / T_THREADS;
  switch (Atype & ~1) {
    case HYK_F64: values_out_kernel<double><<<grid, T_THREADS, 0, stream>>>(K, S, (double*)out); break;
    case HYK_F32: values_out_kernel<float><<<grid, T_THREADS, 0, stream>>>(K, S, (float*)out); break;
    case HYK_F16: values_out_kernel<__half><<<grid, T_THREADS, 0, stream>>>(K, S, (__half*)out); break;
    default: return -1;
  }
  return 0;
}

/* interpolation: R11 (K x K) and T (K x (N - K)) are FP64 (complex: interleaved) column-major outputs with leading
 * dimension K; T returns the solution of R11 T = R12.  Blocked back substitution: from the last block of SOLVE_ROWS rows
 * upwards, the rows already solved are eliminated from the block by one matrix product, then the block is solved
 * against its own triangle. */
extern "C" int hykInterpSolve(hipStream_t stream, int32_t N, int32_t K, int32_t Gtype, const void* Rt, int32_t ldr, const int32_t* jpiv, double* R11, double* T) {
  if (N <= 0 || K <= 0 || K >= N) { return 0; }
  const bool dd = (Gtype & ~1) == HYK_DD, cplx = Gtype & 1; const int WR = dd ? 2 : 1, WE = WR * (cplx ? 2 : 1), W = cplx ? 2 : 1;
  dim3 grid((K + T_THREADS - 1) / T_THREADS, N); const int ncols = N - K, sgrid = (ncols + T_THREADS - 1) / T_THREADS;
  if (cplx) { gather_factor_kernel<true><<<grid, T_THREADS, 0, stream>>>(N, K, (const double*)Rt, ldr, WE, WR, jpiv, R11, T); }
  else { gather_factor_kernel<false><<<grid, T_THREADS, 0, stream>>>(N, K, (const double*)Rt, ldr, WE, WR, jpiv, R11, T); }
  for (int i0 = (K - 1) / SOLVE_ROWS * SOLVE_ROWS; i0 >= 0; i0 -= SOLVE_ROWS) {
    const int rows = K - i0 < SOLVE_ROWS ? K - i0 : SOLVE_ROWS, below = K - i0 - rows;
    if (below > 0) {   /* T[i0 .. i0+rows) -= R11[i0 .. i0+rows, i0+rows .. K) T[i0+rows .. K) */
      const int rc = hykGemm(stream, 'N', 'N', rows, ncols, below, -1.0, cplx ? HYK_F64C : HYK_F64, R11 + ((int64_t)i0 + (int64_t)(i0 + rows) * K) * W, K, T + (int64_t)(i0 + rows) * W, K, 1.0, T + (int64_t)i0 * W, K);
      if (rc != 0) { return rc; }
    }
    if (cplx) { block_solve_kernel<true><<<sgrid, T_THREADS, 0, stream>>>(K, ncols, i0, rows, R11, T); } else { block_solve_kernel<false><<<sgrid, T_THREADS, 0, stream>>>(K, ncols, i0, rows, R11, T); }
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

extern "C" int hykInterpOut(hipStream_t stream, int32_t N, int32_t K, int32_t Atype, const int32_t* jpiv, const double* Tt, void* X, int64_t ldx) {
  if (N <= 0 || K <= 0) { return 0; }
  dim3 grid((K + T_THREADS - 1) / T_THREADS, N);
  switch (Atype) {
    case HYK_F64: interp_out_kernel<double, false><<<grid, T_THREADS, 0, stream>>>(N, K, jpiv, Tt, (double*)X, ldx); break;
    case HYK_F32: interp_out_kernel<float, false><<<grid, T_THREADS, 0, stream>>>(N, K, jpiv, Tt, (float*)X, ldx); break;
    case HYK_F16: interp_out_kernel<__half, false><<<grid, T_THREADS, 0, stream>>>(N, K, jpiv, Tt, (__half*)X, ldx); break;
    case HYK_F64C: interp_out_kernel<double, true><<<grid, T_THREADS, 0, stream>>>(N, K, jpiv, Tt, (double*)X, ldx); break;
    case HYK_F32C: interp_out_kernel<float, true><<<grid, T_THREADS, 0, stream>>>(N, K, jpiv, Tt, (float*)X, ldx); break;
    case HYK_F16C: interp_out_kernel<__half, true><<<grid, T_THREADS, 0, stream>>>(N, K, jpiv, Tt, (__half*)X, ldx); break;
    default: return -1;
  }
  return 0;
}

/* Orthonormal basis of the column space by one-sided Jacobi: V W = U Sigma; the columns are rotated until mutually
 * orthogonal, then normalised in place (a zero column stays zero and drops out of the projector).
 * work: at least 64 + 8 r bytes of device memory. */
extern "C" int hykOrthonormalize(hipStream_t stream, int32_t Complex, int32_t N, int32_t r, double* V, int64_t ldv, double* work) {
  if (N <= 0 || r <= 0) { return 0; }
  if (ldv != N) { return -1; }
  int32_t* counter = reinterpret_cast<int32_t*>(work); double* sigma = work + 8;
  for (int sweep = 0; sweep < 40 && r > 1; ++sweep) {
    if (hykGramWorkspaceClear(stream, counter, 64) != 0) { return -3; }
    if (hykJacobiSweep(stream, Complex, N, r, V, 2.220446049250313e-16 * sqrt((double)N), counter) != 0) { return -3; }
    struct { int32_t rotations, pad; double cosine2; } seen = { 0, 0, 0. }; const double level = 8. * 2.220446049250313e-16 * sqrt((double)N);
    if (hipMemcpyAsync(&seen, counter, sizeof(seen), hipMemcpyDeviceToHost, stream) != hipSuccess || hipStreamSynchronize(stream) != hipSuccess) { return -3; }
    if (seen.pad != 0) { return -5; }   /* a split round gave up (hykJacobiSweep passes no carry memory, so this cannot be set here; kept with the layout) */
    if (seen.rotations == 0 || seen.cosine2 <= level * level) { break; }
  }
  if (hykColumnNorms(stream, Complex, N, r, V, sigma) != 0) { return -3; }
  const int W = Complex ? 2 : 1; dim3 grid((N * W + T_THREADS - 1) / T_THREADS, r);
  normalize_columns_kernel<<<grid, T_THREADS, 0, stream>>>(N, W, V, sigma);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
