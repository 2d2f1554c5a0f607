/*
 * exponent.hip -- per-column power-of-two scales (HBM-bound, one read of A).
 *
 * Replaces the reference's src/fp_exponent.cu: for every row slice b and
 * column j, mexp[b][j] = u - frexp_exponent(max_k max(|re|, |im|)) (INT_MAX for
 * a slice column whose maximum is zero or sub-normal), vexp[j] = min_b
 * mexp[b][j]; and the per-slice bit range segU[b] = u + max_j(vexp[j] -
 * mexp[b][j]).  The maximum is taken on the IEEE bit patterns with the sign
 * cleared, which orders non-negative floats like their values.
 *
 * Layout: A column-major with leading dimension lda (elements); vexp holds
 * (batches + 1) * N int32: [global | slice 0 | slice 1 | ...].
 * One 256-thread workgroup per (slice, column); 16-byte loads when the slice
 * start is 16-byte aligned, element loads otherwise.
 */
#include <hip/hip_runtime.h>
#include "hyk_common.h"
#include "hyacin_kernels.h"

namespace {

constexpr int EXP_THREADS = 256;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <typename U> __device__ __forceinline__ U wave_max(U v) {
  for (int off = 32; off > 0; off >>= 1) { U o = __shfl_xor(v, off, 64); v = o > v ? o : v; }
  return v;
}

/* SCALAR: uint64 (f64), uint32 (f32), uint16 (f16); a complex element is two scalars */
template <typename SCALAR>
__global__ __launch_bounds__(EXP_THREADS) void column_exponent_kernel(int32_t segM, int32_t lastM, int32_t comps, const SCALAR* __restrict__ A, int64_t lda_scalars, int32_t u, int32_t N, int32_t* __restrict__ mexp) {
  const int32_t b = blockIdx.x, j = blockIdx.y;
  const int64_t rows = (b + 1 == (int32_t)gridDim.x) ? lastM : segM, count = rows * comps;
  const SCALAR* col = A + (int64_t)b * segM * comps + (int64_t)j * lda_scalars;
  constexpr SCALAR ABS = (SCALAR)(~(SCALAR)0) >> 1;
  constexpr int VEC = 16 / sizeof(SCALAR);
  SCALAR mx = 0;
  if ((((uintptr_t)col) & 15u) == 0) {
    const int64_t nvec = count / VEC; const u32x4* v = reinterpret_cast<const u32x4*>(col);
    for (int64_t i = threadIdx.x; i < nvec; i += EXP_THREADS) {
      const u32x4 w = __builtin_nontemporal_load(&v[i]);
      if constexpr (sizeof(SCALAR) == 8) {
        uint64_t a = (((uint64_t)w.y << 32) | w.x) & ABS, c = (((uint64_t)w.w << 32) | w.z) & ABS; a = a > c ? a : c; mx = a > mx ? a : mx;
      } else if constexpr (sizeof(SCALAR) == 4) {
        uint32_t a = w.x & ABS, c = w.y & ABS, d = w.z & ABS, e = w.w & ABS; a = a > c ? a : c; d = d > e ? d : e; a = a > d ? a : d; mx = a > mx ? a : mx;
      } else {
        uint32_t ws[4] = { w.x, w.y, w.z, w.w };
        #pragma unroll
        for (int t = 0; t < 4; ++t) { SCALAR a = (SCALAR)(ws[t] & 0x7fffu), c = (SCALAR)((ws[t] >> 16) & 0x7fffu); a = a > c ? a : c; mx = a > mx ? a : mx; }
      }
    }
    for (int64_t i = nvec * VEC + threadIdx.x; i < count; i += EXP_THREADS) { SCALAR a = col[i] & ABS; mx = a > mx ? a : mx; }
  } else {
    for (int64_t i = threadIdx.x; i < count; i += EXP_THREADS) { SCALAR a = col[i] & ABS; mx = a > mx ? a : mx; }
  }
  __shared__ SCALAR part[EXP_THREADS / 64];
  mx = wave_max(mx);
  if ((threadIdx.x & 63) == 0) { part[threadIdx.x >> 6] = mx; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < EXP_THREADS / 64; ++w) { mx = part[w] > mx ? part[w] : mx; }
    int32_t e;
    if constexpr (sizeof(SCALAR) == 8) { e = hyk::frexp_exp_f64(mx); } else if constexpr (sizeof(SCALAR) == 4) { e = hyk::frexp_exp_f32(mx); } else { e = hyk::frexp_exp_f16(mx); }
    mexp[(int64_t)b * N + j] = (e == HYK_INT_MAX) ? HYK_INT_MAX : (u - e);
  }
}

/* A stored as its transpose: the N x M matrix S with op(A)[k, j] = S[j + k lda] (a conjugate changes no magnitude), rows of
 * op(A) contiguous in memory.  A thread owns 16 bytes' worth of adjacent columns and walks down EXP_T_ROWS rows of one row
 * slice, so every load instruction of a wavefront covers 1 KB of one stored row; the per-chunk results meet in mexp (filled
 * with INT_MAX before) through an integer minimum: u - e is smallest where the magnitude is largest.  Replaces the
 * transposing copy of src/lra.cpp:63-69 followed by src/fp_exponent.cu:23-51. */
constexpr int EXP_T_ROWS = 64;    /* rows per workgroup: a multiple of this, chosen on the host so that the launch still has a few thousand workgroups */
template <typename SCALAR>
__global__ __launch_bounds__(EXP_THREADS) void column_exponent_transposed_kernel(int32_t segM, int32_t lastM, int32_t comps, const SCALAR* __restrict__ S, int64_t lda_scalars, int32_t u, int32_t N, int32_t* __restrict__ mexp, int32_t rowsPerBlock) {
  constexpr int VEC = 16 / sizeof(SCALAR); constexpr SCALAR ABS = (SCALAR)(~(SCALAR)0) >> 1;
  const int32_t b = blockIdx.y; const int64_t rows = (b + 1 == (int32_t)gridDim.y) ? lastM : segM;
  const int64_t r0 = (int64_t)blockIdx.x * rowsPerBlock; if (r0 >= rows) { return; }
  const int64_t r1 = r0 + rowsPerBlock < rows ? r0 + rowsPerBlock : rows, width = (int64_t)N * comps;
  const int64_t c0 = ((int64_t)blockIdx.z * EXP_THREADS + threadIdx.x) * VEC; if (c0 >= width) { return; }
  const SCALAR* base = S + ((int64_t)b * segM + r0) * lda_scalars + c0;
  SCALAR mx[VEC];
  #pragma unroll
  for (int i = 0; i < VEC; ++i) { mx[i] = 0; }
  const bool vec = c0 + VEC <= width && (((uintptr_t)base) & 15u) == 0 && ((lda_scalars * (int64_t)sizeof(SCALAR)) & 15) == 0;
  if (vec) {
    #pragma unroll 8
    for (int64_t r = 0; r < r1 - r0; ++r) {
      const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(base + r * lda_scalars));
      SCALAR v[VEC];
      if constexpr (sizeof(SCALAR) == 8) { v[0] = ((uint64_t)w.y << 32) | w.x; v[1] = ((uint64_t)w.w << 32) | w.z; }
      else if constexpr (sizeof(SCALAR) == 4) { v[0] = w.x; v[1] = w.y; v[2] = w.z; v[3] = w.w; }
      else { const uint32_t ws[4] = { w.x, w.y, w.z, w.w };
        #pragma unroll
        for (int t = 0; t < 4; ++t) { v[2 * t] = (SCALAR)(ws[t] & 0xffffu); v[2 * t + 1] = (SCALAR)(ws[t] >> 16); } }
      #pragma unroll
      for (int i = 0; i < VEC; ++i) { const SCALAR a = v[i] & ABS; mx[i] = a > mx[i] ? a : mx[i]; }
    }
  } else {
    for (int64_t r = 0; r < r1 - r0; ++r) {
      #pragma unroll
      for (int i = 0; i < VEC; ++i) { if (c0 + i < width) { const SCALAR a = base[r * lda_scalars + i] & ABS; mx[i] = a > mx[i] ? a : mx[i]; } }
    }
  }
  #pragma unroll
  for (int i = 0; i < VEC; i += 1) {
    if (c0 + i >= width) { break; }
    if (comps == 2 && (i & 1)) { continue; }          /* the pair (re, im) is judged at its real part's turn */
    SCALAR m = mx[i]; if (comps == 2 && i + 1 < VEC) { m = mx[i + 1] > m ? mx[i + 1] : m; }
    int32_t e;
    if constexpr (sizeof(SCALAR) == 8) { e = hyk::frexp_exp_f64(m); } else if constexpr (sizeof(SCALAR) == 4) { e = hyk::frexp_exp_f32(m); } else { e = hyk::frexp_exp_f16(m); }
    if (e != HYK_INT_MAX) { atomicMin(&mexp[(int64_t)b * N + (c0 + i) / comps], u - e); }
  }
}

__global__ void exponent_fill_kernel(int32_t N, int32_t* __restrict__ vexp) { int32_t i = blockIdx.x * blockDim.x + threadIdx.x; if (i < N) { vexp[i] = HYK_INT_MAX; } }

__global__ void exponent_min_kernel(int32_t N, int32_t batches, int32_t* __restrict__ vexp) {
  int32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < N) { int32_t m = HYK_INT_MAX; for (int32_t b = 0; b < batches; ++b) { int32_t v = vexp[(int64_t)(1 + b) * N + i]; m = v < m ? v : m; } vexp[i] = m; }
}

__global__ __launch_bounds__(EXP_THREADS) void slice_range_kernel(int32_t N, int32_t u, const int32_t* __restrict__ vexp, int32_t* __restrict__ segU) {
  const int32_t* mexp = &vexp[(int64_t)(1 + blockIdx.x) * N]; int32_t t = HYK_INT_MIN;
  for (int32_t i = threadIdx.x; i < N; i += EXP_THREADS) { int32_t e = mexp[i]; if (e < HYK_INT_MAX) { int32_t d = vexp[i] - e; t = d > t ? d : t; } }
  __shared__ int32_t part[EXP_THREADS / 64];
  t = wave_max(t);
  if ((threadIdx.x & 63) == 0) { part[threadIdx.x >> 6] = t; }
  __syncthreads();
  if (threadIdx.x == 0) { for (int w = 1; w < EXP_THREADS / 64; ++w) { t = part[w] > t ? part[w] : t; } segU[blockIdx.x] = (t == HYK_INT_MIN) ? HYK_INT_MIN : (u + t); }
}

/* bit length of the dominant diagonal entry (reference: src/fp_i63tp_dequantize.cu:6-26) */
__device__ __forceinline__ int32_t limb_bitlen(int orderC, const uint64_t* c, int64_t stride) {
  int32_t e = 64 - __clzll((long long)c[0]);
  if (orderC > 1) { int32_t n = 127 - __clzll((long long)c[stride]); e = 63 < n ? n : e; }
  if (orderC > 2) { int32_t n = 190 - __clzll((long long)c[2 * stride]); e = 126 < n ? n : e; }
  return e;
}

__global__ __launch_bounds__(EXP_THREADS) void gram_range_kernel(int32_t N, int32_t orderC, const uint64_t* __restrict__ C, int64_t strideC, const int32_t* __restrict__ vexp, int32_t* __restrict__ out) {
  int32_t bx = HYK_INT_MIN, by = 0;
  for (int32_t i = threadIdx.x; i < N; i += EXP_THREADS) {
    int32_t ex = vexp[i];
    if (ex < HYK_INT_MAX) {
      int32_t e = limb_bitlen(orderC, &C[((uint64_t)i * ((uint64_t)i + 3ull)) >> 1], strideC), k = e - (ex + ex);
      if (k == bx) { by = e > by ? e : by; } else if (bx < k) { bx = k; by = e; }
    }
  }
  __shared__ int32_t px[EXP_THREADS], py[EXP_THREADS];
  px[threadIdx.x] = bx; py[threadIdx.x] = by; __syncthreads();
  for (int s = EXP_THREADS / 2; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) {
      int32_t ox = px[threadIdx.x + s], oy = py[threadIdx.x + s];
      if (ox == px[threadIdx.x]) { py[threadIdx.x] = oy > py[threadIdx.x] ? oy : py[threadIdx.x]; } else if (px[threadIdx.x] < ox) { px[threadIdx.x] = ox; py[threadIdx.x] = oy; }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) { *out = py[0]; }
}

}  // namespace

extern "C" int hykColumnExponentsOp(hipStream_t stream, char opA, int32_t batches, int32_t segM, int32_t lastM, int32_t N, int32_t Atype, const void* A, int64_t lda, int32_t u, int32_t* vexp) {
  if (N <= 0) { return 0; }
  if (Atype < HYK_F64 || Atype > HYK_F16C) { return -1; }
  if (batches <= 0 || u < 0) { exponent_fill_kernel<<<(N + 255) / 256, 256, 0, stream>>>(N, vexp); return 0; }
  if (N > 65535 || batches > 65535 || segM <= 0 || lastM <= 0 || lastM > segM) { return -2; }
  const int32_t comps = 1 + (Atype & 1);
  const bool transposed = opA == 'T' || opA == 't' || opA == 'C' || opA == 'c';
  if (!transposed) {
    dim3 grid((uint32_t)batches, (uint32_t)N);
    switch (Atype & ~1) {
      case HYK_F64: column_exponent_kernel<uint64_t><<<grid, EXP_THREADS, 0, stream>>>(segM, lastM, comps, (const uint64_t*)A, lda * comps, u, N, &vexp[N]); break;
      case HYK_F32: column_exponent_kernel<uint32_t><<<grid, EXP_THREADS, 0, stream>>>(segM, lastM, comps, (const uint32_t*)A, lda * comps, u, N, &vexp[N]); break;
      default: column_exponent_kernel<uint16_t><<<grid, EXP_THREADS, 0, stream>>>(segM, lastM, comps, (const uint16_t*)A, lda * comps, u, N, &vexp[N]); break;
    }
  } else {
    const int64_t cells = (int64_t)batches * N; exponent_fill_kernel<<<(uint32_t)((cells + 255) / 256), 256, 0, stream>>>((int32_t)cells, &vexp[N]);
    const int scalarBytes = (Atype & ~1) == HYK_F64 ? 8 : ((Atype & ~1) == HYK_F32 ? 4 : 2); const int64_t perBlock = (int64_t)EXP_THREADS * (16 / scalarBytes);
    const int64_t across = ((int64_t)N * comps + perBlock - 1) / perBlock, at64 = (int64_t)((segM + EXP_T_ROWS - 1) / EXP_T_ROWS) * batches * across;
    const int32_t rowsPerBlock = EXP_T_ROWS * (int32_t)std::min<int64_t>(16, std::max<int64_t>(1, at64 / 4096));   /* fewer atomic minima per column while 4096 workgroups remain */
    dim3 grid((uint32_t)((segM + rowsPerBlock - 1) / rowsPerBlock), (uint32_t)batches, (uint32_t)across);
    switch (Atype & ~1) {
      case HYK_F64: column_exponent_transposed_kernel<uint64_t><<<grid, EXP_THREADS, 0, stream>>>(segM, lastM, comps, (const uint64_t*)A, lda * comps, u, N, &vexp[N], rowsPerBlock); break;
      case HYK_F32: column_exponent_transposed_kernel<uint32_t><<<grid, EXP_THREADS, 0, stream>>>(segM, lastM, comps, (const uint32_t*)A, lda * comps, u, N, &vexp[N], rowsPerBlock); break;
      default: column_exponent_transposed_kernel<uint16_t><<<grid, EXP_THREADS, 0, stream>>>(segM, lastM, comps, (const uint16_t*)A, lda * comps, u, N, &vexp[N], rowsPerBlock); break;
    }
  }
  exponent_min_kernel<<<(N + 255) / 256, 256, 0, stream>>>(N, batches, vexp);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

extern "C" int hykColumnExponents(hipStream_t stream, int32_t batches, int32_t segM, int32_t lastM, int32_t N, int32_t Atype, const void* A, int64_t lda, int32_t u, int32_t* vexp) {
  return hykColumnExponentsOp(stream, 'N', batches, segM, lastM, N, Atype, A, lda, u, vexp);
}

extern "C" int hykSliceRange(hipStream_t stream, int32_t batches, int32_t N, int32_t u, const int32_t* vexp, int32_t* segU) {
  if (batches <= 0 || N <= 0) { return 0; }
  slice_range_kernel<<<batches, EXP_THREADS, 0, stream>>>(N, u, vexp, segU); return 0;
}

extern "C" int hykGramRange(hipStream_t stream, int32_t N, int32_t orderC, const uint64_t* C, const int32_t* vexp, int32_t* out) {
  if (N <= 0 || orderC < 1 || orderC > 3) { return -1; }
  const int64_t strideC = ((int64_t)N * N + N) / 2;
  gram_range_kernel<<<1, EXP_THREADS, 0, stream>>>(N, orderC, C, strideC, vexp, out); return 0;
}
