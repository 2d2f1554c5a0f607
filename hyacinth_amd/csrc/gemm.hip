/*
 * gemm.hip -- C = alpha op(A) op(B) + beta C for the stage products of the
 * column-segmented fit and for the residual check, in the six storage types.
 *
 * Replaces the cuBLAS Dgemm / Zgemm / GemmEx calls of the reference's
 * src/lra.cpp:86-105,202-203 and the planar-split complex-half product of
 * src/matmul_fp16_complex.cu:21-89 (there: two real FP16 GEMMs on a planar
 * copy; here: the interleaved operands are multiplied directly with FP32
 * accumulation, which is at least as accurate as the reference's FP16
 * accumulation).  FP64 types accumulate in FP64, FP32 / FP16 types in FP32.
 * LDS-tiled 64 x 64 x 16, 256 threads, a 4 x 4 register tile per thread.
 */
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include "hyk_common.h"
#include "hyacin_kernels.h"

namespace {

constexpr int GT = 64, GK = 16;

template <typename S> struct AccOf { using T = float; };
template <> struct AccOf<double> { using T = double; };

template <typename S> __device__ __forceinline__ typename AccOf<S>::T ld(const S* p) { return (typename AccOf<S>::T)(*p); }
template <> __device__ __forceinline__ float ld<__half>(const __half* p) { return __half2float(*p); }
template <typename S, typename A> __device__ __forceinline__ void st(S* p, A v) { *p = (S)v; }
template <> __device__ __forceinline__ void st<__half, float>(__half* p, float v) { *p = __float2half(v); }

/* element (r, c) of op(X), X stored column-major with leading dimension ld; op 'N', 'T' or 'C' */
template <typename S, bool CPLX>
__device__ __forceinline__ void fetch(const S* X, int64_t ld_, char op, int64_t r, int64_t c, bool ok, typename AccOf<S>::T& re, typename AccOf<S>::T& im) {
  re = 0; im = 0; if (!ok) { return; }
  const int64_t idx = (op == 'N') ? (r + c * ld_) : (c + r * ld_);
  if constexpr (CPLX) { re = ld<S>(&X[2 * idx]); im = ld<S>(&X[2 * idx + 1]); if (op == 'C') { im = -im; } } else { re = ld<S>(&X[idx]); }
}

template <typename S, bool CPLX>
__global__ __launch_bounds__(256) void gemm_kernel(char opA, char opB, int32_t M, int32_t N, int32_t K, double alpha, const S* __restrict__ A, int64_t lda, const S* __restrict__ B, int64_t ldb, double beta, S* __restrict__ C, int64_t ldc) {
  using Acc = typename AccOf<S>::T; constexpr int W = CPLX ? 2 : 1;
  __shared__ Acc sa[GK][GT + 1][W], sb[GK][GT + 1][W];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4; const int64_t m0 = (int64_t)blockIdx.x * GT, n0 = (int64_t)blockIdx.y * GT;
  Acc cr[4][4], ci[4][4];
  #pragma unroll
  for (int i = 0; i < 4; ++i) {
    #pragma unroll
    for (int j = 0; j < 4; ++j) { cr[i][j] = 0; ci[i][j] = 0; }
  }
  for (int k0 = 0; k0 < K; k0 += GK) {
    #pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int p = tid + r * 256;
      { const int i = (opA == 'N') ? (p & 63) : (p >> 4), kk = (opA == 'N') ? (p >> 6) : (p & 15); Acc re, im; fetch<S, CPLX>(A, lda, opA, m0 + i, k0 + kk, (m0 + i) < M && (k0 + kk) < K, re, im); sa[kk][i][0] = re; if constexpr (CPLX) { sa[kk][i][1] = im; } }
      { const int j = (opB == 'N') ? (p >> 4) : (p & 63), kk = (opB == 'N') ? (p & 15) : (p >> 6); Acc re, im; fetch<S, CPLX>(B, ldb, opB, k0 + kk, n0 + j, (n0 + j) < N && (k0 + kk) < K, re, im); sb[kk][j][0] = re; if constexpr (CPLX) { sb[kk][j][1] = im; } }
    }
    __syncthreads();
    #pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      Acc ar[4], ai[4], br[4], bi[4];
      #pragma unroll
      for (int i = 0; i < 4; ++i) { ar[i] = sa[kk][tx + 16 * i][0]; if constexpr (CPLX) { ai[i] = sa[kk][tx + 16 * i][1]; } br[i] = sb[kk][ty + 16 * i][0]; if constexpr (CPLX) { bi[i] = sb[kk][ty + 16 * i][1]; } }
      #pragma unroll
      for (int i = 0; i < 4; ++i) {
        #pragma unroll
        for (int j = 0; j < 4; ++j) {
          if constexpr (CPLX) { cr[i][j] += ar[i] * br[j] - ai[i] * bi[j]; ci[i][j] += ar[i] * bi[j] + ai[i] * br[j]; } else { cr[i][j] += ar[i] * br[j]; }
        }
      }
    }
    __syncthreads();
  }
  #pragma unroll
  for (int i = 0; i < 4; ++i) {
    #pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t m = m0 + tx + 16 * i, n = n0 + ty + 16 * j; if (m >= M || n >= N) { continue; }
      S* c = &C[(m + n * ldc) * W];
      if constexpr (CPLX) {
        Acc orr = 0, oi = 0; if (beta != 0.) { orr = ld<S>(c); oi = ld<S>(c + 1); }
        st<S, Acc>(c, (Acc)alpha * cr[i][j] + (Acc)beta * orr); st<S, Acc>(c + 1, (Acc)alpha * ci[i][j] + (Acc)beta * oi);
      } else { Acc o = 0; if (beta != 0.) { o = ld<S>(c); } st<S, Acc>(c, (Acc)alpha * cr[i][j] + (Acc)beta * o); }
    }
  }
}

template <typename S, bool CPLX> int run(hipStream_t stream, char opA, char opB, int32_t M, int32_t N, int32_t K, double alpha, const void* A, int64_t lda, const void* B, int64_t ldb, double beta, void* C, int64_t ldc) {
  dim3 grid((M + GT - 1) / GT, (N + GT - 1) / GT);
  gemm_kernel<S, CPLX><<<grid, 256, 0, stream>>>(opA, opB, M, N, K, alpha, (const S*)A, lda, (const S*)B, ldb, beta, (S*)C, ldc);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

char norm_op(char c) { return (c == 't' || c == 'T') ? 'T' : ((c == 'c' || c == 'C') ? 'C' : 'N'); }

}  // namespace

extern "C" int hykGemm(hipStream_t stream, char opA, char opB, int32_t M, int32_t N, int32_t K, double alpha, int32_t type, const void* A, int64_t lda, const void* B, int64_t ldb, double beta, void* C, int64_t ldc) {
  if (M <= 0 || N <= 0) { return 0; }
  if (K < 0 || (N + GT - 1) / GT > 65535) { return -1; }
  opA = norm_op(opA); opB = norm_op(opB);
  switch (type) {
    case HYK_F64: return run<double, false>(stream, opA, opB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
    case HYK_F32: return run<float, false>(stream, opA, opB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
    case HYK_F16: return run<__half, false>(stream, opA, opB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
    case HYK_F64C: return run<double, true>(stream, opA, opB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
    case HYK_F32C: return run<float, true>(stream, opA, opB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
    case HYK_F16C: return run<__half, true>(stream, opA, opB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
    default: return -1;
  }
}

extern "C" int hykMatmulCf16(hipStream_t stream, char opA, int32_t M, int32_t N, int32_t K, const void* A, int64_t lda, const void* B, int64_t ldb, void* C, int64_t ldc) {
  return hykGemm(stream, opA, 'N', M, N, K, 1.0, HYK_F16C, A, lda, B, ldb, 0.0, C, ldc);
}
