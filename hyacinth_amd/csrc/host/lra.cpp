/*
 * lra.cpp -- the fit drivers of the public API: hyacinTsvdFit, hyacinTsvdFitSegmentN,
 * hyacinInterpolateFit, hyacinCheckNorm.
 *
 * Mirrors the reference's src/lra.cpp: interp_dispatcher (:18-50), svd_dispatcher (:52-84), an_gemm
 * (:86-110), svd_segN_dispatcher (:112-156), check_answer (:158-208) and the precision switches (:210-256).
 * The stage order is the reference's: column scales -> exact integer Gram -> dequantize -> factorize.
 */
#include <numeric>
#include <cfloat>
#include "common.hpp"

namespace {

struct Slices { int32_t batchIter, batches, lastM; };
Slices slice_rows(const hyacinHandle_t* h, int32_t M) {
  Slices s; s.batchIter = h->GramSegmentK <= 0 ? M : std::min(h->GramSegmentK, M);
  const int32_t d = std::max(1, s.batchIter), q = M / d, r = M % d; s.batches = q + (0 < r ? 1 : 0); s.lastM = 0 < r ? r : s.batchIter; return s;
}

char norm_op(char c) { return c == 't' ? 'T' : (c == 'c' ? 'C' : c); }

/* stages shared by both fits: returns the dequantized Gram (caller frees through the Scratch) */
struct GramResult { hyacinPrecision_t Gtype; int32_t gElemBytes; };

template <typename Tail>
int32_t fit_common(const hyacinHandle_t* h, double eps, char opA, int32_t M, int32_t N, int Atype, const void* A, int32_t lda, int64_t globalM, Tail&& tail) {
  const Slices sl = slice_rows(h, M); opA = norm_op(opA); hipStream_t s = h->hipStream;
  int32_t u = 0, cPanels = 1, lPanels = 1; uint64_t strideC = 0;
  hyacinXherkBatchInit(h, eps, (uint64_t)globalM, N, (hyacinPrecision_t)Atype, &u, &cPanels, &lPanels, &strideC);
  hyh::Scratch vexp(h, sizeof(int32_t) * (size_t)(sl.batches + 1) * (size_t)N), C(h, sizeof(uint64_t) * (size_t)cPanels * (size_t)std::max(1, lPanels) * (size_t)strideC);
  if (!hyh::ok()) { return 0; }
  /* opA = 'T' / 'C': the exponent and quantization kernels read the stored N x M matrix directly (the reference makes a
   * transposed copy first, src/lra.cpp:63-69) */
  hyh::quantize_scale_batch(h, opA, sl.batches, sl.batchIter, sl.lastM, N, Atype, A, lda, u, vexp.as<int32_t>());
  hyacinAllReduceVExp(h, (uint64_t)N, vexp.as<int32_t>());
  hyh::herk_batch(h, opA, sl.batches, sl.batchIter, sl.lastM, N, Atype, A, lda, u, vexp.as<int32_t>(), 0, lPanels, C.as<uint64_t>());
  hyacinAllReduce1Drow(h, cPanels, lPanels, strideC, C.as<uint64_t>());
  if (lPanels <= 0 || !hyh::ok()) { return 0; }   /* u < 0: nothing was quantized */
  hyacinPrecision_t Gtype = HYACIN_F64; int32_t gBytes = 8;
  hyacinXdequantizeInit(h, N, lPanels, C.as<uint64_t>(), vexp.as<int32_t>(), (hyacinPrecision_t)Atype, &Gtype, &gBytes);
  if (!hyh::ok()) { return 0; }
  hyh::Scratch G(h, (size_t)N * (size_t)N * (size_t)gBytes);
  if (!hyh::ok()) { return 0; }
  hyacinXdequantize(h, N, lPanels, C.as<uint64_t>(), vexp.as<int32_t>(), Gtype, G.p, N);
  if (!hyh::ok()) { return 0; }
  const int32_t rank = tail(Gtype, G.p);
  return hyh::ok() ? rank : 0;
}

int32_t svd_fit(const hyacinHandle_t* h, double eps, char opA, int32_t M, int32_t N, int32_t K, int Atype, const void* A, int32_t lda, void* S, void* V, int32_t ldv, int64_t globalM) {
  K = std::min(N, K); if (K <= 0) { return 0; }
  return fit_common(h, eps, opA, M, N, Atype, A, lda, globalM, [&](hyacinPrecision_t Gtype, void* G) { return hyacinXGevd(h, eps, N, K, (hyacinPrecision_t)Atype, V, ldv, S, Gtype, G, N); });
}

int32_t interp_fit(const hyacinHandle_t* h, double eps, char opA, int32_t M, int32_t N, int32_t K, int Atype, const void* A, int32_t lda, int32_t* jpvt, void* V, int32_t ldv, int64_t globalM) {
  K = std::min(N, K); if (K <= 0) { return 0; }
  return fit_common(h, eps, opA, M, N, Atype, A, lda, globalM, [&](hyacinPrecision_t Gtype, void* G) { return hyacinXGinterp(h, eps, N, K, (hyacinPrecision_t)Atype, V, ldv, jpvt, Gtype, G, N); });
}

const char* at(const void* p, int64_t elems, int Atype) { return (const char*)p + elems * hyh::elem_bytes(Atype); }
char* at(void* p, int64_t elems, int Atype) { return (char*)p + elems * hyh::elem_bytes(Atype); }

/* reference: svd_segN_dispatcher, src/lra.cpp:112-156 */
int32_t svd_fit_segmented(const hyacinHandle_t* h, double eps, char opA, int32_t M, int32_t N, int32_t K, int Atype, const void* A, int32_t lda, void* S, void* V, int32_t ldv, int64_t globalM) {
  K = std::min(N, K); if (K <= 0) { return 0; }
  const int32_t segments = 512 <= N ? (int32_t)std::floor(std::sqrt((double)N / (double)K)) : 1;
  if (segments <= 1) { return svd_fit(h, eps, opA, M, N, K, Atype, A, lda, S, V, ldv, globalM); }
  eps *= std::sqrt(0.5); opA = norm_op(opA); const bool transA = opA == 'T' || opA == 'C'; hipStream_t s = h->hipStream;
  const int32_t q = N / segments, r = N % segments, N1 = q + (0 < r ? 1 : 0); const size_t eb = (size_t)hyh::elem_bytes(Atype), v1Stride = (size_t)N1 * N1;
  const size_t sBytes = (size_t)(eb / (1 + (Atype & 1)));
  hyh::Scratch V1(h, v1Stride * segments * eb), S1(h, (size_t)N1 * sBytes);
  if (!hyh::ok()) { return 0; }
  std::vector<int32_t> ranks; int64_t locA = 0;
  for (int32_t i = 0; i < segments; ++i) {
    const int32_t cols = q + (i < r ? 1 : 0);
    ranks.push_back(svd_fit(h, eps, opA, M, cols, cols, Atype, at(A, locA, Atype), lda, S1.p, at(V1.p, (int64_t)(i * v1Stride), Atype), N1, globalM));
    locA += transA ? cols : (int64_t)cols * lda;
    if (!hyh::ok()) { return 0; }
  }
  const int32_t N2 = std::accumulate(ranks.begin(), ranks.end(), 0); if (N2 <= 0) { return 0; }
  int32_t rank;
  hyh::Scratch V2(h, (size_t)N2 * std::min(N2, K) * eb);
  { hyh::Scratch A2(h, (size_t)M * N2 * eb); locA = 0; int64_t locA2 = 0;
    if (!hyh::ok()) { return 0; }
    hyh::timer_mark(h, hyh::Segment::dist_kernel);
    if (0 < M) for (int32_t i = 0; i < segments; ++i) {
      const int32_t cols = q + (i < r ? 1 : 0);
      HYH_KERNEL(hykGemm(s, opA, 'N', M, ranks[i], cols, 1.0, Atype, at(A, locA, Atype), lda, at(V1.p, (int64_t)(i * v1Stride), Atype), N1, 0.0, at(A2.p, locA2, Atype), M));
      locA += transA ? cols : (int64_t)cols * lda; locA2 += (int64_t)ranks[i] * M;
    }
    K = std::min(N2, K);
    rank = svd_fit(h, eps, 'N', M, N2, K, Atype, A2.p, M, S, V2.p, N2, globalM);
  }
  hyh::timer_mark(h, hyh::Segment::rep_kernel);
  int32_t row = 0, rowV = 0;
  for (int32_t i = 0; i < segments; ++i) {
    const int32_t cols = q + (i < r ? 1 : 0);
    if (rank > 0 && ranks[i] > 0) { HYH_KERNEL(hykGemm(s, 'N', 'N', cols, rank, ranks[i], 1.0, Atype, at(V1.p, (int64_t)(i * v1Stride), Atype), N1, at(V2.p, rowV, Atype), N2, 0.0, at(V, row, Atype), ldv)); }
    else if (rank > 0) { HYH_KERNEL(hykGemm(s, 'N', 'N', cols, rank, 0, 0.0, Atype, V1.p, N1, V2.p, N2, 0.0, at(V, row, Atype), ldv)); }
    row += cols; rowV += ranks[i];
  }
  return hyh::ok() ? rank : 0;
}

/* reference: check_answer, src/lra.cpp:158-208 */
double check_norm(const hyacinHandle_t* h, char opA, int32_t M, int32_t N, int32_t rank, int Atype, const void* V, int32_t ldv, const void* A, int32_t lda) {
  if (M <= 0 || N <= 0) { return 0.; }
  hyh::timer_mark(h, hyh::Segment::untimed);
  opA = norm_op(opA); const bool transA = opA == 'T' || opA == 'C'; const int Complex = Atype & 1, wide = HYACIN_F64 + Complex; const int32_t block = 2048;
  const size_t eb = (size_t)8 * (1 + Complex); hipStream_t s = h->hipStream; const char mode = transA ? opA : 'A';
  hyh::Scratch acc(h, 64); if (!hyh::ok()) { return 0.; } HYH_KERNEL(hykGramWorkspaceClear(s, acc.p, 64));
  if (rank <= 0) {
    hyh::Scratch matA(h, (size_t)block * block * eb);
    if (!hyh::ok()) { return 0.; }
    for (int32_t i = 0; i < M; i += block) { const int32_t rows = std::min(M - i, block);
      for (int32_t j = 0; j < N; j += block) { const int32_t cols = std::min(N - j, block);
        const void* src = transA ? at(A, (int64_t)j + (int64_t)i * lda, Atype) : at(A, (int64_t)i + (int64_t)j * lda, Atype);
        HYH_KERNEL(hykMatcopy(s, mode, rows, cols, Atype, src, lda, wide, matA.p, rows));
        HYH_KERNEL(hykSumSquares(s, (int64_t)rows * (1 + Complex), cols, matA.as<double>(), (int64_t)rows * (1 + Complex), acc.as<double>()));
      } }
  } else {
    rank = std::min(rank, N);
    hyh::Scratch Q(h, (size_t)N * rank * eb), work(h, (size_t)rank * 16 + 64);
    if (!hyh::ok()) { return 0.; }
    HYH_KERNEL(hykMatcopy(s, 'A', N, rank, Atype, V, ldv, wide, Q.p, N));
    HYH_KERNEL(hykOrthonormalize(s, Complex, N, rank, Q.as<double>(), N, work.as<double>()));
    hyh::Scratch matA(h, (size_t)block * N * eb), matU(h, (size_t)block * rank * eb);
    if (!hyh::ok()) { return 0.; }
    for (int32_t i = 0; i < M; i += block) { const int32_t rows = std::min(M - i, block);
      const void* src = transA ? at(A, (int64_t)i * lda, Atype) : at(A, (int64_t)i, Atype);
      HYH_KERNEL(hykMatcopy(s, mode, rows, N, Atype, src, lda, wide, matA.p, rows));
      HYH_KERNEL(hykGemm(s, 'N', 'N', rows, rank, N, 1.0, wide, matA.p, rows, Q.p, N, 0.0, matU.p, block));
      HYH_KERNEL(hykGemm(s, 'N', 'C', rows, N, rank, -1.0, wide, matU.p, block, Q.p, N, 1.0, matA.p, rows));
      HYH_KERNEL(hykSumSquares(s, (int64_t)rows * (1 + Complex), N, matA.as<double>(), (int64_t)rows * (1 + Complex), acc.as<double>()));
    }
  }
  double err = 0.; HYH_CHECK(hipMemcpyAsync(&err, acc.p, sizeof(double), hipMemcpyDeviceToHost, s)); HYH_CHECK(hipStreamSynchronize(s));
  return hyh::ok() ? err : 0.;
}

}  // namespace

extern "C" int32_t hyacinInterpolateFit(const hyacinHandle_t* handle, double eps, char opA, int32_t M, int32_t N, int32_t K, const void* A, int32_t lda, int32_t* jpvt, void* V, int32_t ldv, int64_t globalM, hyacinPrecision_t ComputeType) {
  hyh::ApiScope scope;
  if ((int)ComputeType < 0 || (int)ComputeType > HYACIN_F16_COMPLEX) { return 0; }
  return interp_fit(handle, eps, opA, M, N, K, (int)ComputeType, A, lda, jpvt, V, ldv, globalM <= 0 ? (int64_t)M : globalM);
}

extern "C" int32_t hyacinTsvdFit(const hyacinHandle_t* handle, double eps, char opA, int32_t M, int32_t N, int32_t K, const void* A, int32_t lda, void* S, void* V, int32_t ldv, int64_t globalM, hyacinPrecision_t ComputeType) {
  hyh::ApiScope scope;
  if ((int)ComputeType < 0 || (int)ComputeType > HYACIN_F16_COMPLEX) { return 0; }
  return svd_fit(handle, eps, opA, M, N, K, (int)ComputeType, A, lda, S, V, ldv, globalM <= 0 ? (int64_t)M : globalM);
}

extern "C" int32_t hyacinTsvdFitSegmentN(const hyacinHandle_t* handle, double eps, char opA, int32_t M, int32_t N, int32_t K, const void* A, int32_t lda, void* S, void* V, int32_t ldv, int64_t globalM, hyacinPrecision_t ComputeType) {
  hyh::ApiScope scope;
  if ((int)ComputeType < 0 || (int)ComputeType > HYACIN_F16_COMPLEX) { return 0; }
  return svd_fit_segmented(handle, eps, opA, M, N, K, (int)ComputeType, A, lda, S, V, ldv, globalM <= 0 ? (int64_t)M : globalM);
}

extern "C" double hyacinCheckNorm(const hyacinHandle_t* handle, char opA, int32_t M, int32_t N, const void* A, int32_t lda, int32_t rank, const void* V, int32_t ldv, hyacinPrecision_t ComputeType) {
  hyh::ApiScope scope;
  if ((int)ComputeType < 0 || (int)ComputeType > HYACIN_F16_COMPLEX) { return 0.; }
  return check_norm(handle, opA, M, N, rank, (int)ComputeType, V, ldv, A, lda);
}
