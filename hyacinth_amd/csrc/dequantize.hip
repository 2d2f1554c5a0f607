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

/* KIND: 0 FP32, 1 FP64, 2 double-double */
template <int KIND, int CPLX>
__global__ __launch_bounds__(256) void dequantize_kernel(int32_t N, int32_t L, const uint64_t* __restrict__ C, int64_t strideC, const int32_t* __restrict__ vexp, void* __restrict__ Gv, int64_t ldg) {
  const int64_t y = (int64_t)blockIdx.x * 256 + threadIdx.x, x = blockIdx.y;
  if (y > x) { return; }
  const int32_t ex = vexp[x], ey = vexp[y]; const bool zero = (ex == HYK_INT_MAX || ey == HYK_INT_MAX); const int32_t e = zero ? 0 : -(ex + ey);
  uint64_t re[3] = { 0, 0, 0 }, im[3] = { 0, 0, 0 }; const uint64_t* src = &C[hyk::tri_index(y, x)];
  for (int l = 0; l < L; ++l) { re[l] = src[l * strideC]; if (CPLX) { im[l] = src[(L + l) * strideC]; } }
  const int64_t up = y + x * ldg, lo = x + y * ldg;
  if constexpr (KIND == 2) {
    dd_t z{ 0., 0. }, vr = zero ? z : conv_dd(L, re, e), vi = (zero || !CPLX) ? z : conv_dd(L, im, e); double* g = reinterpret_cast<double*>(Gv);
    if constexpr (CPLX) { double4* g4 = reinterpret_cast<double4*>(Gv); g4[up] = make_double4(vr.x, vr.y, vi.x, vi.y); g4[lo] = make_double4(vr.x, vr.y, -vi.x, -vi.y); }
    else { double2* g2 = reinterpret_cast<double2*>(g); g2[up] = make_double2(vr.x, vr.y); g2[lo] = make_double2(vr.x, vr.y); }
  } else if constexpr (KIND == 1) {
    const double vr = zero ? 0. : conv_f64(L, re, e), vi = (zero || !CPLX) ? 0. : conv_f64(L, im, e);
    if constexpr (CPLX) { double2* g2 = reinterpret_cast<double2*>(Gv); g2[up] = make_double2(vr, vi); g2[lo] = make_double2(vr, -vi); }
    else { double* g = reinterpret_cast<double*>(Gv); g[up] = vr; g[lo] = vr; }
  } else {
    const float vr = zero ? 0.f : (float)conv_f64(L, re, e), vi = (zero || !CPLX) ? 0.f : (float)conv_f64(L, im, e);
    if constexpr (CPLX) { float2* g2 = reinterpret_cast<float2*>(Gv); g2[up] = make_float2(vr, vi); g2[lo] = make_float2(vr, -vi); }
    else { float* g = reinterpret_cast<float*>(Gv); g[up] = vr; g[lo] = vr; }
  }
}

}  // namespace

extern "C" int hykDequantize(hipStream_t stream, int32_t N, int32_t orderC, const uint64_t* C, const int32_t* vexp, int32_t Gtype, void* G, int64_t ldg) {
  if (N <= 0) { return 0; }
  if (orderC < 1 || orderC > 3 || N > 65535 || ldg < N) { return -1; }
  const int64_t strideC = ((int64_t)N * N + N) / 2; dim3 grid((uint32_t)((N + 255) / 256), (uint32_t)N);
  switch (Gtype) {
    case HYK_F32: dequantize_kernel<0, 0><<<grid, 256, 0, stream>>>(N, orderC, C, strideC, vexp, G, ldg); break;
    case HYK_F32C: dequantize_kernel<0, 1><<<grid, 256, 0, stream>>>(N, orderC, C, strideC, vexp, G, ldg); break;
    case HYK_F64: dequantize_kernel<1, 0><<<grid, 256, 0, stream>>>(N, orderC, C, strideC, vexp, G, ldg); break;
    case HYK_F64C: dequantize_kernel<1, 1><<<grid, 256, 0, stream>>>(N, orderC, C, strideC, vexp, G, ldg); break;
    case HYK_DD: dequantize_kernel<2, 0><<<grid, 256, 0, stream>>>(N, orderC, C, strideC, vexp, G, ldg); break;
    case HYK_DDC: dequantize_kernel<2, 1><<<grid, 256, 0, stream>>>(N, orderC, C, strideC, vexp, G, ldg); break;
    default: return -1;  /* triple-float / quad-float Grams are only chosen on GPUs without fast FP64 */
  }
  return 0;
}
