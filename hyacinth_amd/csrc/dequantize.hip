/*
 * dequantize.hip -- packed-triangle 63-bit-limb integer Gram -> full Hermitian
 * floating-point Gram (HBM-bound, O(N^2)).
 *
 * Replaces the reference's triangle_unpack_dequantize_kernel
 * (src/fp_i63tp_dequantize.cu:56-129): G[y, x] = value(C[y, x]) * 2^-(vexp[x] +
 * vexp[y]) for y <= x, G[x, y] = conj(G[y, x]); zero when either column's scale
 * is INT_MAX.  Output types: FP32, FP64, double-double {hi, lo}, each real or
 * complex ({re, im} of the real type).  The FP64 conversion is the chained
 * (top * 2^63 + hi32) + lo32 of the reference; the double-double one is exact up
 * to the 106-bit mantissa via error-free transforms (compile without FP
 * contraction).
 */
#include <type_traits>
#include <hip/hip_runtime.h>
#include "hyk_common.h"
#include "hyk_dd.h"
#include "hyacin_kernels.h"

namespace {

using hyk::dd_t;

__device__ __forceinline__ dd_t conv_i64_dd(uint64_t i) { return dd_t{ ldexp((double)(int32_t)(i >> 32), 32), (double)(uint32_t)i }; }

__device__ __forceinline__ double conv_f64(int L, const uint64_t* a, int32_t e) {
  double res = (double)(int64_t)a[L - 1];
  if (L > 2) { dd_t i = conv_i64_dd(a[1]); res = (ldexp(res, 63) + i.x) + i.y; }
  if (L > 1) { dd_t i = conv_i64_dd(a[0]); res = (ldexp(res, 63) + i.x) + i.y; }
  return ldexp(res, e);
}

__device__ __forceinline__ dd_t conv_dd(int L, const uint64_t* a, int32_t e) {
  dd_t res = hyk::dd_renorm(conv_i64_dd(a[L - 1]));
  if (L > 2) { res = hyk::dd_add(dd_t{ ldexp(res.x, 63), ldexp(res.y, 63) }, hyk::dd_renorm(conv_i64_dd(a[1]))); }
  if (L > 1) { res = hyk::dd_add(dd_t{ ldexp(res.x, 63), ldexp(res.y, 63) }, hyk::dd_renorm(conv_i64_dd(a[0]))); }
  return dd_t{ ldexp(res.x, e), ldexp(res.y, e) };
}

/* One element of G: W scalars of type T ({re}, {re, im}, {hi, lo} or {re hi, re lo, im hi, im lo}), stored in one piece. */
template <typename T, int W> struct alignas(sizeof(T) * W > 16 ? 16 : sizeof(T) * W) Elem { T v[W]; };

/* KIND: 0 FP32, 1 FP64, 2 double-double.  A workgroup takes one 32 x 32 tile (tile row <= tile column) of the upper
 * triangle: thread (y, x) reads the limbs of C[y, x] (entries of a column are adjacent in the packed triangle, so 32
 * threads read 256 adjacent bytes per limb), converts, stores G[y, x] (adjacent in y) and parks the value in LDS; after the
 * barrier the tile is read across and its conjugate stored to the lower triangle as G[x, y], adjacent in x: both triangles
 * leave in full lines (a thread per entry writing its own mirror image puts every element of the lower triangle into a
 * line of its own).  Entries on the diagonal are written by the second pass (conjugated: the imaginary part of a
 * diagonal entry is -0 where the integer is 0, as with the reference's order of its two stores,
 * src/fp_i63tp_dequantize.cu:121-129). */
constexpr int DQ_TILE = 32;
template <int KIND, int CPLX>
__global__ __launch_bounds__(256) void dequantize_kernel(int32_t N, int32_t L, const uint64_t* __restrict__ C, int64_t strideC, const int32_t* __restrict__ vexp, void* __restrict__ Gv, int64_t ldg) {
  using T = std::conditional_t<KIND == 0, float, double>;
  constexpr int W = (KIND == 2 ? 2 : 1) * (CPLX ? 2 : 1);
  using E = Elem<T, W>;
  /* workgroup b takes tile (row ty <= column tx) with b = ty + tx (tx + 1) / 2: only tiles on or above the diagonal are launched */
  int tx = (int)((sqrtf(8.f * (float)blockIdx.x + 1.f) - 1.f) * 0.5f);
  while ((uint32_t)(tx + 1) * (uint32_t)(tx + 2) / 2u <= blockIdx.x) { ++tx; }
  while ((uint32_t)tx * (uint32_t)(tx + 1) / 2u > blockIdx.x) { --tx; }
  const int ty = (int)(blockIdx.x - (uint32_t)tx * (uint32_t)(tx + 1) / 2u);
  __shared__ E tile[DQ_TILE][DQ_TILE + 1];   /* [x][y], one element of padding per row */
  const int y0 = ty * DQ_TILE, x0 = tx * DQ_TILE, ti = threadIdx.x % DQ_TILE, tj = threadIdx.x / DQ_TILE;
  E* G = reinterpret_cast<E*>(Gv);
  {
    const int y = y0 + ti; const int32_t ey = y < N ? vexp[y] : 0;
    #pragma unroll
    for (int p = 0; p < DQ_TILE / 8; ++p) {
      const int xl = tj + 8 * p, x = x0 + xl;
      if (x >= N || y > x) { continue; }
      const int32_t ex = vexp[x]; const bool zero = (ex == HYK_INT_MAX || ey == HYK_INT_MAX); const int32_t e = zero ? 0 : -(ex + ey);
      uint64_t re[3] = { 0, 0, 0 }, im[3] = { 0, 0, 0 }; const uint64_t* src = &C[hyk::tri_index(y, x)];
      for (int l = 0; l < L; ++l) { re[l] = src[l * strideC]; if (CPLX) { im[l] = src[(L + l) * strideC]; } }
      E out;
      if constexpr (KIND == 2) {
        const dd_t z{ 0., 0. }, vr = zero ? z : conv_dd(L, re, e), vi = (zero || !CPLX) ? z : conv_dd(L, im, e);
        out.v[0] = vr.x; out.v[1] = vr.y; if constexpr (CPLX) { out.v[2] = vi.x; out.v[3] = vi.y; }
      } else if constexpr (KIND == 1) {
        out.v[0] = zero ? 0. : conv_f64(L, re, e); if constexpr (CPLX) { out.v[1] = zero ? 0. : conv_f64(L, im, e); }
      } else {
        out.v[0] = zero ? 0.f : (float)conv_f64(L, re, e); if constexpr (CPLX) { out.v[1] = zero ? 0.f : (float)conv_f64(L, im, e); }
      }
      tile[xl][ti] = out;
      if (y < x) { G[(int64_t)y + (int64_t)x * ldg] = out; }
    }
  }
  __syncthreads();
  {
    const int x = x0 + ti;
    #pragma unroll
    for (int p = 0; p < DQ_TILE / 8; ++p) {
      const int yl = tj + 8 * p, y = y0 + yl;
      if (x >= N || y > x) { continue; }
      E out = tile[ti][yl];
      if constexpr (CPLX) {
        #pragma unroll
        for (int w = W / 2; w < W; ++w) { out.v[w] = -out.v[w]; }
      }
      G[(int64_t)x + (int64_t)y * ldg] = out;
    }
  }
}

}  // namespace

extern "C" int hykDequantize(hipStream_t stream, int32_t N, int32_t orderC, const uint64_t* C, const int32_t* vexp, int32_t Gtype, void* G, int64_t ldg) {
  if (N <= 0) { return 0; }
  if (orderC < 1 || orderC > 3 || N > 65535 || ldg < N) { return -1; }
  const int64_t strideC = ((int64_t)N * N + N) / 2; const uint32_t tiles = (uint32_t)((N + DQ_TILE - 1) / DQ_TILE); dim3 grid(tiles * (tiles + 1) / 2);
  switch (Gtype) {
    case HYK_F32: dequantize_kernel<0, 0><<<grid, 256, 0, stream>>>(N, orderC, C, strideC, vexp, G, ldg); break;
    case HYK_F32C: dequantize_kernel<0, 1><<<grid, 256, 0, stream>>>(N, orderC, C, strideC, vexp, G, ldg); break;
    case HYK_F64: dequantize_kernel<1, 0><<<grid, 256, 0, stream>>>(N, orderC, C, strideC, vexp, G, ldg); break;
    case HYK_F64C: dequantize_kernel<1, 1><<<grid, 256, 0, stream>>>(N, orderC, C, strideC, vexp, G, ldg); break;
    case HYK_DD: dequantize_kernel<2, 0><<<grid, 256, 0, stream>>>(N, orderC, C, strideC, vexp, G, ldg); break;
    case HYK_DDC: dequantize_kernel<2, 1><<<grid, 256, 0, stream>>>(N, orderC, C, strideC, vexp, G, ldg); break;
    default: return -1;  /* triple-float / quad-float Grams are only chosen on GPUs without fast FP64 */
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
