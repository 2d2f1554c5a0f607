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
 * General kernel: LDS-tiled 64 x 64 x 16, 256 threads, a 4 x 4 register tile per thread (vector ALU).  The FP16 and FP32
 * products C = op(A) B, the shape of matmul_cf16_{cn,tn,nn} and of the stage products of the segmented fit, run on the
 * matrix cores (the two kernels below).
 */
#include <type_traits>
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
  typedef double d4_t __attribute__((ext_vector_type(4)));
  [[maybe_unused]] d4_t mr[2][2], mi[2][2];   /* FP64: accumulators of the matrix-core blocks, [block of n][block of m] */
  #pragma unroll
  for (int i = 0; i < 2; ++i) {
    #pragma unroll
    for (int j = 0; j < 2; ++j) { mr[i][j] = d4_t{ 0., 0., 0., 0. }; mi[i][j] = d4_t{ 0., 0., 0., 0. }; }
  }
  for (int k0 = 0; k0 < K; k0 += GK) {
    #pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int p = tid + r * 256;
      { const int i = (opA == 'N') ? (p & 63) : (p >> 4), kk = (opA == 'N') ? (p >> 6) : (p & 15); Acc re, im; fetch<S, CPLX>(A, lda, opA, m0 + i, k0 + kk, (m0 + i) < M && (k0 + kk) < K, re, im); sa[kk][i][0] = re; if constexpr (CPLX) { sa[kk][i][1] = im; } }
      { const int j = (opB == 'N') ? (p >> 4) : (p & 63), kk = (opB == 'N') ? (p & 15) : (p >> 6); Acc re, im; fetch<S, CPLX>(B, ldb, opB, k0 + kk, n0 + j, (n0 + j) < N && (k0 + kk) < K, re, im); sb[kk][j][0] = re; if constexpr (CPLX) { sb[kk][j][1] = im; } }
    }
    __syncthreads();
    if constexpr (std::is_same<S, double>::value) {
      /* FP64 on the matrix cores: v_mfma_f64_16x16x4_f64, a wavefront takes a 32 x 32 quarter of the tile as 2 x 2 blocks.
       * The instruction's row operand is B (lane: column n = lane % 16 of the block, k = lane / 16) and its column operand
       * op(A) (row m = lane % 16, k = lane / 16), so that a lane ends up with entries C[m, lane / 16 + 4 r] (the FP64 blocks interleave their rows over the four register pairs): lanes 0-15
       * store 16 adjacent rows m.  Complex products as four real ones (the negated imaginary part makes -Ai Bi). */
      const int lane = tid & 63, wave = tid >> 6, l16 = lane & 15, lk = lane >> 4, mb = (wave & 1) * 32, nb = (wave >> 1) * 32;
      #pragma unroll
      for (int k4 = 0; k4 < GK / 4; ++k4) {
        const int kk = 4 * k4 + lk;
        double ar[2], ai[2], br[2], bi[2];
        #pragma unroll
        for (int b = 0; b < 2; ++b) { ar[b] = sa[kk][mb + 16 * b + l16][0]; br[b] = sb[kk][nb + 16 * b + l16][0]; if constexpr (CPLX) { ai[b] = sa[kk][mb + 16 * b + l16][1]; bi[b] = sb[kk][nb + 16 * b + l16][1]; } }
        #pragma unroll
        for (int bn = 0; bn < 2; ++bn) {
          #pragma unroll
          for (int bm = 0; bm < 2; ++bm) {
            mr[bn][bm] = __builtin_amdgcn_mfma_f64_16x16x4f64(br[bn], ar[bm], mr[bn][bm], 0, 0, 0);
            if constexpr (CPLX) {
              mr[bn][bm] = __builtin_amdgcn_mfma_f64_16x16x4f64(-bi[bn], ai[bm], mr[bn][bm], 0, 0, 0);
              mi[bn][bm] = __builtin_amdgcn_mfma_f64_16x16x4f64(bi[bn], ar[bm], mi[bn][bm], 0, 0, 0);
              mi[bn][bm] = __builtin_amdgcn_mfma_f64_16x16x4f64(br[bn], ai[bm], mi[bn][bm], 0, 0, 0);
            }
          }
        }
      }
      __syncthreads();
      continue;
    }
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
  if constexpr (std::is_same<S, double>::value) {
    const int lane = tid & 63, wave = tid >> 6, l16 = lane & 15, lk = lane >> 4, mb = (wave & 1) * 32, nb = (wave >> 1) * 32;
    #pragma unroll
    for (int bn = 0; bn < 2; ++bn) {
      #pragma unroll
      for (int bm = 0; bm < 2; ++bm) {
        #pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int64_t m = m0 + mb + 16 * bm + l16, n = n0 + nb + 16 * bn + lk + 4 * r; if (m >= M || n >= N) { continue; }
          double* c = reinterpret_cast<double*>(&C[(m + n * ldc) * W]);
          if constexpr (CPLX) { double orr = 0., oi = 0.; if (beta != 0.) { orr = c[0]; oi = c[1]; } c[0] = alpha * mr[bn][bm][r] + beta * orr; c[1] = alpha * mi[bn][bm][r] + beta * oi; }
          else { double o = 0.; if (beta != 0.) { o = c[0]; } c[0] = alpha * mr[bn][bm][r] + beta * o; }
        }
      }
    }
    return;
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

/* ------------------------------------------------------------------ FP16 products on the matrix cores
 * C = op(A) B for real and complex FP16 (interleaved), FP32 accumulation, `v_mfma_f32_32x32x16_f16`.
 *
 * Complex as a real product of twice the depth: with k' = 2 k + s, B seen as a real (2 K) x N matrix is exactly its
 * interleaved storage (B'[2k] = Br, B'[2k+1] = Bi), and op(A) expands to A're[m][2k] = Ar, [2k+1] = -Ai for the real part
 * of C and A'im[m][2k] = Ai, [2k+1] = Ar for the imaginary part.  Both expansions are made in registers from the same
 * 16 bytes (four complex numbers) a lane reads from LDS: a sign flip of the upper halves, and a 16-bit rotation of every
 * word (the conjugate for op 'C' moves the sign flip).  No planar copy of either operand is made (the reference builds
 * [Ar; -+Ai] and [-Bi; Br; Bi] in memory, src/matmul_fp16_complex.cu:4-14).
 *
 * Workgroup = 4 wavefronts (2 x 2), tile 128 rows of op(A) x 128 columns of B, wavefront 64 x 64 = 2 x 2 MFMA blocks (x 2
 * accumulator sets when complex).  The contraction advances in slabs of 128 bytes per row (32 complex or 64 real
 * numbers = four MFMA steps), double-buffered in LDS, next slab prefetched into registers during the MFMAs.  LDS rows are
 * 128 bytes with XOR-swizzled 16-byte slots, so the fragment reads are bank-conflict-free.  The MFMA's row operand is B
 * and its column operand op(A): a lane then owns one row m of C and stores run along the contiguous index.
 * Needs 16-byte aligned operands and leading dimensions; other calls take the vector-ALU kernel above. */
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
constexpr int HT = 128, HROW = 128, HTILE = HT * HROW;

__device__ __forceinline__ int h_swz(int row) { return ((row ^ (row >> 3)) & 1) | (row & 6); }

/* 16 bytes of tile row `q`, piece `p`, from a matrix whose contraction index runs along memory (B, or A under op 'T' / 'C') */
template <int E>
__device__ __forceinline__ uint4 load_piece_contiguous(const char* X, int64_t ldx, int64_t q, int64_t Q, int64_t k, int64_t K) {
  constexpr int PE = 16 / E; uint4 v = make_uint4(0u, 0u, 0u, 0u);
  if (q >= Q || k >= K) { return v; }
  const char* src = X + (k + q * ldx) * E;
  if (k + PE <= K) { return *reinterpret_cast<const uint4*>(src); }
  uint16_t h[8] = { 0, 0, 0, 0, 0, 0, 0, 0 };
  for (int i = 0; i < (int)(K - k) * (E / 2); ++i) { h[i] = reinterpret_cast<const uint16_t*>(src)[i]; }
  v.x = h[0] | ((uint32_t)h[1] << 16); v.y = h[2] | ((uint32_t)h[3] << 16); v.z = h[4] | ((uint32_t)h[5] << 16); v.w = h[6] | ((uint32_t)h[7] << 16);
  return v;
}
/* the same piece of op(A) = A (rows run along memory): PE strided elements */
template <int E>
__device__ __forceinline__ uint4 load_piece_strided(const char* X, int64_t ldx, int64_t q, int64_t Q, int64_t k, int64_t K) {
  constexpr int PE = 16 / E; uint32_t w[4] = { 0u, 0u, 0u, 0u };
  if (q < Q) {
    #pragma unroll
    for (int i = 0; i < PE; ++i) {
      if (k + i < K) {
        const char* src = X + (q + (k + i) * ldx) * E;
        if constexpr (E == 8) { const uint2 v = *reinterpret_cast<const uint2*>(src); w[2 * i] = v.x; w[2 * i + 1] = v.y; }
        else if constexpr (E == 4) { w[i] = *reinterpret_cast<const uint32_t*>(src); } else { w[i >> 1] |= (uint32_t)*reinterpret_cast<const uint16_t*>(src) << (16 * (i & 1)); }
      }
    }
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

template <bool CPLX, int OPA>   /* OPA: 0 'N', 1 'T', 2 'C' */
__global__ __launch_bounds__(256) void gemm_f16_mfma_kernel(int32_t M, int32_t N, int32_t K, const char* __restrict__ A, int64_t lda, const char* __restrict__ B, int64_t ldb, char* __restrict__ C, int64_t ldc) {
  constexpr int E = CPLX ? 4 : 2, PE = 16 / E, KS = HROW / E;   /* bytes per element, elements per 16-byte piece, elements per slab */
  __shared__ __attribute__((aligned(16))) char lds[2][2][HTILE];  /* [buffer][A | B][row * 128 + slot * 16] */
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave & 1, wn = wave >> 1;
  const int64_t m0 = (int64_t)blockIdx.x * HT, n0 = (int64_t)blockIdx.y * HT;
  uint4 ra[4], rb[4];
  auto fetch = [&](int64_t k0) {
    #pragma unroll
    for (int r = 0; r < 4; ++r) {
      if constexpr (OPA == 0) { const int row = tid & 127, p = (tid >> 7) + 2 * r; ra[r] = load_piece_strided<E>(A, lda, m0 + row, M, k0 + p * PE, K); }
      else { const int row = (tid >> 3) + 32 * r, p = tid & 7; ra[r] = load_piece_contiguous<E>(A, lda, m0 + row, M, k0 + p * PE, K); }
      { const int row = (tid >> 3) + 32 * r, p = tid & 7; rb[r] = load_piece_contiguous<E>(B, ldb, n0 + row, N, k0 + p * PE, K); }
    }
  };
  auto park = [&](int buf) {
    #pragma unroll
    for (int r = 0; r < 4; ++r) {
      { const int row = OPA == 0 ? (tid & 127) : (tid >> 3) + 32 * r, p = OPA == 0 ? (tid >> 7) + 2 * r : (tid & 7);
        *reinterpret_cast<uint4*>(&lds[buf][0][row * HROW + ((p ^ h_swz(row)) << 4)]) = ra[r]; }
      { const int row = (tid >> 3) + 32 * r, p = tid & 7; *reinterpret_cast<uint4*>(&lds[buf][1][row * HROW + ((p ^ h_swz(row)) << 4)]) = rb[r]; }
    }
  };
  constexpr int SETS = CPLX ? 2 : 1;
  float16_t acc[SETS][2][2];   /* [re | im][block of n][block of m] */
  #pragma unroll
  for (int s = 0; s < SETS; ++s) {
    #pragma unroll
    for (int i = 0; i < 2; ++i) {
      #pragma unroll
      for (int j = 0; j < 2; ++j) {
        #pragma unroll
        for (int e = 0; e < 16; ++e) { acc[s][i][j][e] = 0.f; }
      }
    }
  }
  const int slabs = (K + KS - 1) / KS;
  const int rowM = (wm * 64 + (lane & 31)) * HROW, rowN = (wn * 64 + (lane & 31)) * HROW, sw = h_swz(lane & 31), hi = lane >> 5;
  if (slabs > 0) { fetch(0); park(0); }
  __syncthreads();
  for (int it = 0; it < slabs; ++it) {
    const int buf = it & 1;
    if (it + 1 < slabs) { fetch((int64_t)(it + 1) * KS); }
    #pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int slot = ((2 * s + hi) ^ sw) << 4;
      uint4 fm[2], fn[2];
      #pragma unroll
      for (int b = 0; b < 2; ++b) {
        fm[b] = *reinterpret_cast<const uint4*>(&lds[buf][0][rowM + b * 32 * HROW + slot]);
        fn[b] = *reinterpret_cast<const uint4*>(&lds[buf][1][rowN + b * 32 * HROW + slot]);
      }
      #pragma unroll
      for (int j = 0; j < 2; ++j) {
        if constexpr (CPLX) {
          /* word = Ar | Ai << 16.  Real part of C: (Ar, -Ai), conjugated A: (Ar, Ai).  Imaginary part: (Ai, Ar), conjugated: (-Ai, Ar). */
          const uint32_t w[4] = { fm[j].x, fm[j].y, fm[j].z, fm[j].w }; uint32_t wr[4], wi[4];
          #pragma unroll
          for (int q = 0; q < 4; ++q) {
            wr[q] = OPA == 2 ? w[q] : (w[q] ^ 0x80000000u);
            const uint32_t rot = __builtin_amdgcn_alignbit(w[q], w[q], 16); wi[q] = OPA == 2 ? (rot ^ 0x00008000u) : rot;
          }
          const uint4 ure = make_uint4(wr[0], wr[1], wr[2], wr[3]), uim = make_uint4(wi[0], wi[1], wi[2], wi[3]);
          #pragma unroll
          for (int i = 0; i < 2; ++i) {
            acc[0][i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, fn[i]), __builtin_bit_cast(half8_t, ure), acc[0][i][j], 0, 0, 0);
            acc[1][i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, fn[i]), __builtin_bit_cast(half8_t, uim), acc[1][i][j], 0, 0, 0);
          }
        } else {
          #pragma unroll
          for (int i = 0; i < 2; ++i) { acc[0][i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, fn[i]), __builtin_bit_cast(half8_t, fm[j]), acc[0][i][j], 0, 0, 0); }
        }
      }
    }
    if (it + 1 < slabs) { park(buf ^ 1); }   /* the other buffer was last read before the previous barrier */
    __syncthreads();
  }
  /* lane: row m of the block; register e: column n = 8 (e / 4) + 4 (lane / 32) + e % 4 of the block */
  #pragma unroll
  for (int i = 0; i < 2; ++i) {
    #pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t m = m0 + wm * 64 + j * 32 + (lane & 31); if (m >= M) { continue; }
      #pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int64_t n = n0 + wn * 64 + i * 32 + ((e >> 2) << 3) + (hi << 2) + (e & 3); if (n >= N) { continue; }
        char* dst = C + (m + n * ldc) * E;
        if constexpr (CPLX) { *reinterpret_cast<__half2*>(dst) = __floats2half2_rn(acc[0][i][j][e], acc[1][i][j][e]); }
        else { *reinterpret_cast<__half*>(dst) = __float2half(acc[0][i][j][e]); }
      }
    }
  }
}

/* ------------------------------------------------------------------ FP32 products on the matrix cores
 * The same tiling with `v_mfma_f32_32x32x2_f32` (C = op(A) B, real and complex FP32, FP32 accumulation): the stage products
 * of the column-segmented fit for FP32 storage (reference: the GemmEx calls of src/lra.cpp:90-93,102-105).  A 16-byte piece
 * of an LDS row holds four consecutive contraction indices (two complex numbers); the lanes 0..31 take the even pieces and
 * the lanes 32..63 the odd ones, and the four MFMA steps of a piece use its four floats in turn: both operands follow the
 * same assignment, so every index is contracted once.  Complex as a real product of twice the depth, as above: B's
 * interleaved storage is the real (2 K) x N operand, op(A) expands to (Ar, -Ai) / (Ai, Ar) (conjugated: (Ar, Ai) /
 * (-Ai, Ar)) in registers. */
template <bool CPLX, int OPA>   /* OPA: 0 'N', 1 'T', 2 'C' */
__global__ __launch_bounds__(256) void gemm_f32_mfma_kernel(int32_t M, int32_t N, int32_t K, const char* __restrict__ A, int64_t lda, const char* __restrict__ B, int64_t ldb, char* __restrict__ C, int64_t ldc) {
  constexpr int E = CPLX ? 8 : 4, PE = 16 / E, KS = HROW / E;
  __shared__ __attribute__((aligned(16))) char lds[2][2][HTILE];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave & 1, wn = wave >> 1;
  const int64_t m0 = (int64_t)blockIdx.x * HT, n0 = (int64_t)blockIdx.y * HT;
  uint4 ra[4], rb[4];
  auto fetch = [&](int64_t k0) {
    #pragma unroll
    for (int r = 0; r < 4; ++r) {
      if constexpr (OPA == 0) { const int row = tid & 127, p = (tid >> 7) + 2 * r; ra[r] = load_piece_strided<E>(A, lda, m0 + row, M, k0 + p * PE, K); }
      else { const int row = (tid >> 3) + 32 * r, p = tid & 7; ra[r] = load_piece_contiguous<E>(A, lda, m0 + row, M, k0 + p * PE, K); }
      { const int row = (tid >> 3) + 32 * r, p = tid & 7; rb[r] = load_piece_contiguous<E>(B, ldb, n0 + row, N, k0 + p * PE, K); }
    }
  };
  auto park = [&](int buf) {
    #pragma unroll
    for (int r = 0; r < 4; ++r) {
      { const int row = OPA == 0 ? (tid & 127) : (tid >> 3) + 32 * r, p = OPA == 0 ? (tid >> 7) + 2 * r : (tid & 7);
        *reinterpret_cast<uint4*>(&lds[buf][0][row * HROW + ((p ^ h_swz(row)) << 4)]) = ra[r]; }
      { const int row = (tid >> 3) + 32 * r, p = tid & 7; *reinterpret_cast<uint4*>(&lds[buf][1][row * HROW + ((p ^ h_swz(row)) << 4)]) = rb[r]; }
    }
  };
  constexpr int SETS = CPLX ? 2 : 1;
  float16_t acc[SETS][2][2];   /* [re | im][block of n][block of m] */
  #pragma unroll
  for (int s = 0; s < SETS; ++s) {
    #pragma unroll
    for (int i = 0; i < 2; ++i) {
      #pragma unroll
      for (int j = 0; j < 2; ++j) {
        #pragma unroll
        for (int e = 0; e < 16; ++e) { acc[s][i][j][e] = 0.f; }
      }
    }
  }
  const int slabs = (K + KS - 1) / KS;
  const int rowM = (wm * 64 + (lane & 31)) * HROW, rowN = (wn * 64 + (lane & 31)) * HROW, sw = h_swz(lane & 31), hi = lane >> 5;
  if (slabs > 0) { fetch(0); park(0); }
  __syncthreads();
  for (int it = 0; it < slabs; ++it) {
    const int buf = it & 1;
    if (it + 1 < slabs) { fetch((int64_t)(it + 1) * KS); }
    #pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int slot = ((2 * s + hi) ^ sw) << 4;
      float4 fm[2], fn[2];
      #pragma unroll
      for (int b = 0; b < 2; ++b) {
        fm[b] = *reinterpret_cast<const float4*>(&lds[buf][0][rowM + b * 32 * HROW + slot]);
        fn[b] = *reinterpret_cast<const float4*>(&lds[buf][1][rowN + b * 32 * HROW + slot]);
      }
      #pragma unroll
      for (int j = 0; j < 2; ++j) {
        const float a[4] = { fm[j].x, fm[j].y, fm[j].z, fm[j].w };
        float are[4], aim[4];
        if constexpr (CPLX) {   /* a = (Ar0, Ai0, Ar1, Ai1) */
          are[0] = a[0]; are[1] = OPA == 2 ? a[1] : -a[1]; are[2] = a[2]; are[3] = OPA == 2 ? a[3] : -a[3];
          aim[0] = OPA == 2 ? -a[1] : a[1]; aim[1] = a[0]; aim[2] = OPA == 2 ? -a[3] : a[3]; aim[3] = a[2];
        } else { are[0] = a[0]; are[1] = a[1]; are[2] = a[2]; are[3] = a[3]; aim[0] = aim[1] = aim[2] = aim[3] = 0.f; }
        #pragma unroll
        for (int i = 0; i < 2; ++i) {
          const float b[4] = { fn[i].x, fn[i].y, fn[i].z, fn[i].w };
          #pragma unroll
          for (int e = 0; e < 4; ++e) {
            acc[0][i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[e], are[e], acc[0][i][j], 0, 0, 0);
            if constexpr (CPLX) { acc[1][i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[e], aim[e], acc[1][i][j], 0, 0, 0); }
          }
        }
      }
    }
    if (it + 1 < slabs) { park(buf ^ 1); }
    __syncthreads();
  }
  /* lane: row m of the block; register e: column n = 8 (e / 4) + 4 (lane / 32) + e % 4 of the block */
  #pragma unroll
  for (int i = 0; i < 2; ++i) {
    #pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t m = m0 + wm * 64 + j * 32 + (lane & 31); if (m >= M) { continue; }
      #pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int64_t n = n0 + wn * 64 + i * 32 + ((e >> 2) << 3) + (hi << 2) + (e & 3); if (n >= N) { continue; }
        char* dst = C + (m + n * ldc) * E;
        if constexpr (CPLX) { *reinterpret_cast<float2*>(dst) = make_float2(acc[0][i][j][e], acc[1][i][j][e]); }
        else { *reinterpret_cast<float*>(dst) = acc[0][i][j][e]; }
      }
    }
  }
}

template <bool CPLX> int run_f32_mfma(hipStream_t stream, char opA, int32_t M, int32_t N, int32_t K, const void* A, int64_t lda, const void* B, int64_t ldb, void* C, int64_t ldc) {
  dim3 grid((M + HT - 1) / HT, (N + HT - 1) / HT); const char* a = (const char*)A; const char* b = (const char*)B; char* c = (char*)C;
  if (opA == 'N') { gemm_f32_mfma_kernel<CPLX, 0><<<grid, 256, 0, stream>>>(M, N, K, a, lda, b, ldb, c, ldc); }
  else if (opA == 'T' || !CPLX) { gemm_f32_mfma_kernel<CPLX, 1><<<grid, 256, 0, stream>>>(M, N, K, a, lda, b, ldb, c, ldc); }
  else { gemm_f32_mfma_kernel<CPLX, 2><<<grid, 256, 0, stream>>>(M, N, K, a, lda, b, ldb, c, ldc); }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

template <bool CPLX> int run_f16_mfma(hipStream_t stream, char opA, int32_t M, int32_t N, int32_t K, const void* A, int64_t lda, const void* B, int64_t ldb, void* C, int64_t ldc) {
  dim3 grid((M + HT - 1) / HT, (N + HT - 1) / HT); const char* a = (const char*)A; const char* b = (const char*)B; char* c = (char*)C;
  if (opA == 'N') { gemm_f16_mfma_kernel<CPLX, 0><<<grid, 256, 0, stream>>>(M, N, K, a, lda, b, ldb, c, ldc); }
  else if (opA == 'T' || !CPLX) { gemm_f16_mfma_kernel<CPLX, 1><<<grid, 256, 0, stream>>>(M, N, K, a, lda, b, ldb, c, ldc); }
  else { gemm_f16_mfma_kernel<CPLX, 2><<<grid, 256, 0, stream>>>(M, N, K, a, lda, b, ldb, c, ldc); }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

/* the matrix-core kernels cover C = op(A) B (alpha 1, beta 0, B as stored) on 16-byte aligned operands, FP16 and FP32 storage */
bool mfma_applies(char opB, double alpha, double beta, int32_t type, const void* A, int64_t lda, const void* B, int64_t ldb, const void* C, int32_t N) {
  if ((type != HYK_F16 && type != HYK_F16C && type != HYK_F32 && type != HYK_F32C) || opB != 'N' || alpha != 1.0 || beta != 0.0 || (N + HT - 1) / HT > 65535) { return false; }
  const int64_t e = type == HYK_F16C ? 4 : (type == HYK_F16 ? 2 : (type == HYK_F32 ? 4 : 8));
  return ((uintptr_t)A % 16 == 0) && ((uintptr_t)B % 16 == 0) && ((uintptr_t)C % e == 0) && (lda * e) % 16 == 0 && (ldb * e) % 16 == 0;
}

char norm_op(char c) { return (c == 't' || c == 'T') ? 'T' : ((c == 'c' || c == 'C') ? 'C' : 'N'); }

}  // namespace

extern "C" int hykGemm(hipStream_t stream, char opA, char opB, int32_t M, int32_t N, int32_t K, double alpha, int32_t type, const void* A, int64_t lda, const void* B, int64_t ldb, double beta, void* C, int64_t ldc) {
  if (M <= 0 || N <= 0) { return 0; }
  if (K < 0 || (N + GT - 1) / GT > 65535) { return -1; }
  opA = norm_op(opA); opB = norm_op(opB);
  if (K > 0 && mfma_applies(opB, alpha, beta, type, A, lda, B, ldb, C, N)) {
    switch (type) {
      case HYK_F16C: return run_f16_mfma<true>(stream, opA, M, N, K, A, lda, B, ldb, C, ldc);
      case HYK_F16: return run_f16_mfma<false>(stream, opA, M, N, K, A, lda, B, ldb, C, ldc);
      case HYK_F32C: return run_f32_mfma<true>(stream, opA, M, N, K, A, lda, B, ldb, C, ldc);
      default: return run_f32_mfma<false>(stream, opA, M, N, K, A, lda, B, ldb, C, ldc);
    }
  }
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
