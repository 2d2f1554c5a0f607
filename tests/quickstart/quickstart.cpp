/*
 * The reference's quick start (README.md:109-167: complex FP64, hyacinTsvdFitSegmentN + hyacinCheckNorm +
 * hyacinSync_TimerSegments) with the application-owned stream of its "Reuse your application's CUDA resources"
 * section (README.md:183-196), compiled as C++ against include/hyacin.h and linked to libhyacin.so: what a caller
 * of the reference writes, with the CUDA runtime calls spelled as their HIP namesakes.  The handle fields keep the
 * reference's names (cudaStream, cublasHandle, cusolverHandle).  The matrix is a sum of two rank-one terms, so the
 * fit must return rank 2 and a basis that captures it.  Prints one line; tests/test_quickstart.py reads it.
 */
#include <hyacin.h>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

struct cplx { double x, y; };   /* cuDoubleComplex: interleaved real and imaginary part */

static void check_hip(hipError_t status) {
  if (status != hipSuccess) {
    std::fprintf(stderr, "%s\n", hipGetErrorString(status));
    std::exit(EXIT_FAILURE);
  }
}

int main() {
  constexpr int M = 512, N = 128, K = N;
  constexpr double eps = 1e-10;
  check_hip(hipSetDevice(0));

  // This example matrix has a low-dimensional right subspace.
  std::vector<cplx> A(size_t(M) * N);
  for (int j = 0; j < N; ++j)
    for (int i = 0; i < M; ++i)
      A[i + size_t(j) * M] = cplx{ (1. + .01 * i) * (1. + .02 * j), std::sin(.1 * i) * std::cos(.2 * j) };

  cplx *d_A = nullptr, *d_V = nullptr;
  double* d_S = nullptr;
  check_hip(hipMalloc(reinterpret_cast<void**>(&d_A), A.size() * sizeof(*d_A)));
  check_hip(hipMalloc(reinterpret_cast<void**>(&d_V), size_t(N) * K * sizeof(*d_V)));
  check_hip(hipMalloc(reinterpret_cast<void**>(&d_S), K * sizeof(*d_S)));
  check_hip(hipMemcpy(d_A, A.data(), A.size() * sizeof(*d_A), hipMemcpyHostToDevice));

  // stream belongs to the application; the vendor-library slots stay null (this library needs neither).
  hipStream_t stream = nullptr;
  check_hip(hipStreamCreate(&stream));
  hyacinHandle_t handle{};
  handle.cudaStream = stream;
  handle.cublasHandle = nullptr;
  handle.cusolverHandle = nullptr;
  hyacinCreate(&handle);
  if (handle.cudaStream != stream || handle.hipStream != stream) { std::fprintf(stderr, "hyacinCreate replaced the supplied stream\n"); return EXIT_FAILURE; }

  const int rank = hyacinTsvdFitSegmentN(
    &handle, eps, 'N', M, N, K,
    d_A, M, d_S, d_V, N, M, HYACIN_F64_COMPLEX);

  const double norm2 = hyacinCheckNorm(
    &handle, 'N', M, N, d_A, M, 0, nullptr, 0, HYACIN_F64_COMPLEX);
  const double residual2 = hyacinCheckNorm(
    &handle, 'N', M, N, d_A, M, rank, d_V, N, HYACIN_F64_COMPLEX);
  const double relative_error = norm2 > 0. ? std::sqrt(residual2 / norm2) : 0.;

  hyacinSync_TimerSegments(&handle, nullptr, 0);
  std::vector<cplx> V(size_t(N) * (rank > 0 ? rank : 0));
  std::vector<double> S(K);
  if (rank > 0)
    check_hip(hipMemcpy(V.data(), d_V, V.size() * sizeof(*d_V), hipMemcpyDeviceToHost));
  check_hip(hipMemcpy(S.data(), d_S, K * sizeof(double), hipMemcpyDeviceToHost));
  // the basis is orthonormal: largest deviation of V^H V from the identity
  double defect = 0.;
  for (int a = 0; a < rank; ++a)
    for (int b = 0; b < rank; ++b) {
      double re = 0., im = 0.;
      for (int i = 0; i < N; ++i) { const cplx p = V[i + size_t(a) * N], q = V[i + size_t(b) * N]; re += p.x * q.x + p.y * q.y; im += p.x * q.y - p.y * q.x; }
      defect = std::fmax(defect, std::fmax(std::fabs(re - (a == b ? 1. : 0.)), std::fabs(im)));
    }
  std::printf("rank = %d, relative projection error = %.3e, orthonormality defect = %.3e, S0 = %.15e, S1 = %.15e, S2 = %.15e\n",
              rank, relative_error, defect, S[0], S[1], S[2]);

  hyacinDestroy(&handle);
  check_hip(hipStreamDestroy(stream));   // still the application's: hyacinDestroy leaves borrowed resources alone
  check_hip(hipFree(d_S));
  check_hip(hipFree(d_V));
  check_hip(hipFree(d_A));
  return 0;
}
