/*
 * matcopy.hip -- type-converting copy / transpose / conjugate-transpose between
 * the six storage types, and a sum of squares.
 *
 * Replaces the modes 'A', 'T', 'C' of the reference's scatter_matcopy
 * (src/matcopy.cu:23-44, 58-96) and the cuBLAS nrm2 calls of
 * src/lra.cpp:170,204.  B (M x N, ld ldb) = op(A): mode 'A' copies A (M x N),
 * modes 'T' / 'C' read A as N x M.  Transposes go through a 32 x 33 LDS tile so
 * that both the read and the write are coalesced.
 */
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include "hyk_common.h"
#include "hyacin_kernels.h"

namespace {

template <int T> struct El;
template <> struct El<HYK_F64> { using S = double; static constexpr int n = 1; };
template <> struct El<HYK_F32> { using S = float; static constexpr int n = 1; };
template <> struct El<HYK_F16> { using S = __half; static constexpr int n = 1; };
template <> struct El<HYK_F64C> { using S = double; static constexpr int n = 2; };
template <> struct El<HYK_F32C> { using S = float; static constexpr int n = 2; };
template <> struct El<HYK_F16C> { using S = __half; static constexpr int n = 2; };

__device__ __forceinline__ double to_d(double v) { return v; }
__device__ __forceinline__ double to_d(float v) { return (double)v; }
__device__ __forceinline__ double to_d(__half v) { return (double)__half2float(v); }
__device__ __forceinline__ void from_d(double* p, double v) { *p = v; }
__device__ __forceinline__ void from_d(float* p, double v) { *p = (float)v; }
__device__ __forceinline__ void from_d(__half* p, double v) { __half_raw r; r.data = static_cast<_Float16>(v); *p = r; }

template <int SRC, int DST>
__global__ __launch_bounds__(256) void copy_kernel(int64_t M, int64_t N, const typename El<SRC>::S* __restrict__ A, int64_t lda, typename El<DST>::S* __restrict__ B, int64_t ldb) {
  const int64_t y = (int64_t)blockIdx.x * 256 + threadIdx.x, x = blockIdx.y; if (y >= M) { return; }
  constexpr int n = El<SRC>::n;
  #pragma unroll
  for (int c = 0; c < n; ++c) { from_d(&B[(y + x * ldb) * n + c], to_d(A[(y + x * lda) * n + c])); }
}

template <int SRC, int DST, bool CONJ>
__global__ __launch_bounds__(256) void transpose_kernel(int64_t M, int64_t N, const typename El<SRC>::S* __restrict__ A, int64_t lda, typename El<DST>::S* __restrict__ B, int64_t ldb) {
  constexpr int n = El<SRC>::n; __shared__ double tile[32][33][n];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5; const int64_t m0 = (int64_t)blockIdx.x * 32, n0 = (int64_t)blockIdx.y * 32;
  /* A is N x M: element (col-of-B, row-of-B) = A[nIdx + mIdx * lda] */
  for (int r = ty; r < 32; r += 8) { const int64_t mi = m0 + r, ni = n0 + tx; if (mi < M && ni < N) { for (int c = 0; c < n; ++c) { tile[r][tx][c] = to_d(A[(ni + mi * lda) * n + c]); } } }
  __syncthreads();
  for (int r = ty; r < 32; r += 8) { const int64_t ni = n0 + r, mi = m0 + tx; if (mi < M && ni < N) { for (int c = 0; c < n; ++c) { double v = tile[tx][r][c]; if (CONJ && c == 1) { v = -v; } from_d(&B[(mi + ni * ldb) * n + c], v); } } }
}

__global__ __launch_bounds__(256) void sumsq_kernel(int64_t M, int64_t N, const double* __restrict__ A, int64_t lda, double* __restrict__ out) {
  __shared__ double part[4]; double s = 0.;
  for (int64_t x = blockIdx.y; x < N; x += gridDim.y) for (int64_t y = (int64_t)blockIdx.x * 256 + threadIdx.x; y < M; y += (int64_t)gridDim.x * 256) { const double v = A[y + x * lda]; s += v * v; }
  for (int off = 32; off > 0; off >>= 1) { s += __shfl_xor(s, off, 64); }
  if ((threadIdx.x & 63) == 0) { part[threadIdx.x >> 6] = s; } __syncthreads();
  if (threadIdx.x == 0) { atomicAdd(out, part[0] + part[1] + part[2] + part[3]); }
}

template <int SRC, int DST> int run(hipStream_t stream, char mode, int64_t M, int64_t N, const void* A, int64_t lda, void* B, int64_t ldb) {
  using SA = typename El<SRC>::S; using SB = typename El<DST>::S;
  if (mode == 'A') { dim3 grid((uint32_t)((M + 255) / 256), (uint32_t)N); copy_kernel<SRC, DST><<<grid, 256, 0, stream>>>(M, N, (const SA*)A, lda, (SB*)B, ldb); }
  else { dim3 grid((uint32_t)((M + 31) / 32), (uint32_t)((N + 31) / 32));
    if (mode == 'C') { transpose_kernel<SRC, DST, true><<<grid, 256, 0, stream>>>(M, N, (const SA*)A, lda, (SB*)B, ldb); } else { transpose_kernel<SRC, DST, false><<<grid, 256, 0, stream>>>(M, N, (const SA*)A, lda, (SB*)B, ldb); } }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

template <int SRC> int run_dst(hipStream_t stream, char mode, int64_t M, int64_t N, int32_t dst, const void* A, int64_t lda, void* B, int64_t ldb) {
  constexpr int cp = SRC & 1;
  switch (dst) {
    case HYK_F64 + cp: return run<SRC, HYK_F64 + cp>(stream, mode, M, N, A, lda, B, ldb);
    case HYK_F32 + cp: return run<SRC, HYK_F32 + cp>(stream, mode, M, N, A, lda, B, ldb);
    case HYK_F16 + cp: return run<SRC, HYK_F16 + cp>(stream, mode, M, N, A, lda, B, ldb);
    default: return -1;
  }
}

}  // namespace

extern "C" int hykMatcopy(hipStream_t stream, char mode, int64_t M, int64_t N, int32_t srcType, const void* A, int64_t lda, int32_t dstType, void* B, int64_t ldb) {
  if (M <= 0 || N <= 0) { return 0; }
  if (mode == 't') { mode = 'T'; } if (mode == 'c') { mode = 'C'; } if (mode != 'T' && mode != 'C') { mode = 'A'; }
  if (N > 65535 * 32 || (mode == 'A' && N > 65535)) { return -1; }
  switch (srcType) {
    case HYK_F64: return run_dst<HYK_F64>(stream, mode, M, N, dstType, A, lda, B, ldb);
    case HYK_F32: return run_dst<HYK_F32>(stream, mode, M, N, dstType, A, lda, B, ldb);
    case HYK_F16: return run_dst<HYK_F16>(stream, mode, M, N, dstType, A, lda, B, ldb);
    case HYK_F64C: return run_dst<HYK_F64C>(stream, mode, M, N, dstType, A, lda, B, ldb);
    case HYK_F32C: return run_dst<HYK_F32C>(stream, mode, M, N, dstType, A, lda, B, ldb);
    case HYK_F16C: return run_dst<HYK_F16C>(stream, mode, M, N, dstType, A, lda, B, ldb);
    default: return -1;
  }
}

/* G[y, x] = conj(G[x, y]) for y < x: the strict upper triangle of a Hermitian matrix written again from its lower one.
 * W doubles per real or imaginary part (1: FP64, 2: double-double).  A thread per entry, adjacent threads along y. */
template <int W, bool CPLX>
__global__ __launch_bounds__(256) void mirror_lower_kernel(int32_t N, double* __restrict__ G, int64_t ldg) {
  constexpr int WE = W * (CPLX ? 2 : 1);
  const int y = (int)(blockIdx.x * 256 + threadIdx.x), x = (int)blockIdx.y;
  if (y >= x || x >= N) { return; }
  const double* src = &G[((int64_t)x + (int64_t)y * ldg) * WE]; double* dst = &G[((int64_t)y + (int64_t)x * ldg) * WE];
  #pragma unroll
  for (int w = 0; w < WE; ++w) { dst[w] = (CPLX && w >= W) ? -src[w] : src[w]; }
}

extern "C" int hykMirrorLower(hipStream_t stream, int32_t N, int32_t Gtype, void* G, int64_t ldg) {
  if (N <= 1) { return 0; }
  if (!G || ldg < N || N > 65535) { return -1; }
  dim3 grid((uint32_t)((N + 255) / 256), (uint32_t)N);
  switch (Gtype) {
    case HYK_F64: mirror_lower_kernel<1, false><<<grid, 256, 0, stream>>>(N, (double*)G, ldg); break;
    case HYK_F64C: mirror_lower_kernel<1, true><<<grid, 256, 0, stream>>>(N, (double*)G, ldg); break;
    case HYK_DD: mirror_lower_kernel<2, false><<<grid, 256, 0, stream>>>(N, (double*)G, ldg); break;
    case HYK_DDC: mirror_lower_kernel<2, true><<<grid, 256, 0, stream>>>(N, (double*)G, ldg); break;
    default: return -1;
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

/* *out += sum of squares of the M x N FP64 matrix (a complex matrix is passed as 2M x N) */
extern "C" int hykSumSquares(hipStream_t stream, int64_t M, int64_t N, const double* A, int64_t lda, double* out) {
  if (M <= 0 || N <= 0) { return 0; }
  dim3 grid((uint32_t)((M + 255) / 256 < 64 ? (M + 255) / 256 : 64), (uint32_t)(N < 256 ? N : 256));
  sumsq_kernel<<<grid, 256, 0, stream>>>(M, N, A, lda, out); return hipGetLastError() == hipSuccess ? 0 : -3;
}
