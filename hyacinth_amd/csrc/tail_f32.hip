/*
 * tail_f32.hip -- the one-sided Jacobi rounds of jacobi_rounds.h instantiated for a factor held in floats: the SVD tail of
 * FP32 and FP16 storage (the reference runs gesvdj in single precision there, src/gram_evd.cu:96-98,114-130).  A
 * translation unit of its own, so that the two sets of kernel instantiations compile side by side.
 */
#include "jacobi_rounds.h"

int hyk_jacobi_sweep_f32(hipStream_t stream, int32_t Complex, int32_t N, int32_t r, int32_t head, int32_t top, float* B, double tol, int32_t* rotations, double* carry, int variant, int splitTest) {
  return sweep_top<float>(stream, Complex, N, r, head, top, B, tol, rotations, carry, variant, splitTest);
}
