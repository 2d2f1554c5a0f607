/*
 * herk.cpp -- planning and orchestration of the quantized Gram build:
 * hyacinXherkBatchInit, hyacinXquantizeScaleBatch, hyacinXherkBatch,
 * hyacinXdequantizeInit, hyacinXdequantize.
 *
 * Mirrors the reference's src/hyacin_herk.cpp (gram_algorithm :11-43, hyacinXherkBatchInit :45-59,
 * herk_dispatcher :283-310, herk_batch_dispatcher :312-384, hyacinXherkBatch :386-407), the host parts
 * of src/fp_exponent.cu:45-65 and src/fp_i63tp_dequantize.cu:29-54,143-159.
 *
 * What is kept exactly: every planning decision (bits from eps, limb count, limbs-vs-CRT choice, number
 * of limbs / moduli, per-slice precision buckets), because they fix the quantized panels and the range
 * of the integer Gram.  What is free, because the integer Gram is an exact sum over rows: how many rows
 * go into one contraction call.  Row chunks here never exceed the reference's CRT chunk length (which
 * bounds |partial Gram| < P/2) and are additionally capped so that the int8 panels of one chunk stay
 * below a fixed workspace budget.
 */
#include "common.hpp"
#include "../crt_tables.h"

namespace {

constexpr int32_t kLimbCapacity[12] = { 7, 14, 22, 30, 38, 46, 54, 62, 70, 78, 86, 94 };   /* bits held by 1..12 balanced base-256 digits */
constexpr size_t kPanelBudget = (size_t)8 << 30;   /* bytes of int8 panels per contraction call */

int32_t first_at_least(const uint16_t* table, int32_t count, int32_t v) { int32_t i = 0; while (i < count && (int32_t)table[i] < v) { ++i; } return i; }

}  // namespace

hyh::GramPlan hyh::gram_algorithm(char alg, int32_t K, int32_t u, int32_t Complex, int32_t segmentK, double batchPenalty) {
  u = std::max(0, u); K = std::max(1, K);
  const int32_t kk = 0 < segmentK ? std::min(K, segmentK) : K;
  const int32_t crtBits = (2 * u + 1) + (int32_t)std::ceil(std::log2((double)kk));
  const uint16_t* range = Complex ? hyk_crt_cplx_range : hyk_crt_real_range; const int32_t count = Complex ? HYK_CRT_CPLX_COUNT : HYK_CRT_REAL_COUNT;
  const int32_t alignedK = (K + 127) & ~127;
  auto crt_plan = [&]() { const int32_t o = 1 + first_at_least(range, count, crtBits); const int32_t rows = segmentK << ((int32_t)range[o - 1] - crtBits); return hyh::GramPlan{ 'C', o, std::min(alignedK, rows) }; };
  const bool forceC = (alg == 'C' || alg == 'c'), forceL = (alg == 'L' || alg == 'l');
  if (forceC) { return crtBits <= (int32_t)range[count - 1] ? crt_plan() : hyh::GramPlan{ 'C', 0, 0 }; }
  int32_t oL = 1; while (oL <= 12 && kLimbCapacity[oL - 1] < u) { ++oL; }
  if (!forceL && 2 < oL && crtBits <= (int32_t)range[count - 1]) {
    /* cost in units of one N x N x K int8 GEMM: limbs o/2 triangular + o(o-1)/2 cross (+ o^2 complex); CRT one triangular
     * GEMM per modulus (real) or one full GEMM per rotating modulus plus 1.5 per extra modulus (complex) */
    const double costL = batchPenalty * oL * 0.5 + (double)((uint32_t)(oL * (oL - 1)) >> 1) + (Complex ? (double)(oL * oL) : 0.);
    const hyh::GramPlan c = crt_plan();
    const double costC = Complex ? batchPenalty * ((double)c.order + 0.5 * std::max(0, c.order - HYK_CRT_CPLX_SPLIT)) : batchPenalty * c.order * 0.5;
    if (costC < costL) { return c; }
  }
  return hyh::GramPlan{ 'L', oL, kLimbCapacity[std::min(oL, 12) - 1] };
}

extern "C" void hyacinXherkBatchInit(const hyacinHandle_t* handle, double eps, uint64_t M, int32_t N, hyacinPrecision_t Atype, int32_t* uA, int32_t* cPanels, int32_t* lPanels, uint64_t* stride) {
  hyh::ApiScope scope;
  if (stride) { const uint64_t n = (uint64_t)std::max(0, N); *stride = (n * n + n) >> 1; }
  if (!uA && !cPanels && !lPanels) { return; }
  static const int32_t mantissa[12] = { 52, 52, 23, 23, 10, 10, 105, 105, 71, 71, 95, 95 };
  if ((int)Atype < 0 || (int)Atype > 11) { return; }
  uint64_t Mp = 1; while (Mp < M && Mp < ((uint64_t)1 << 63)) { Mp <<= 1; }   /* next power of two >= M */
  int e; const double f = std::frexp(std::fabs(eps), &e);
  const int32_t u = std::min(std::max((int32_t)(f == 0.5) - e, 0), mantissa[(int)Atype]);
  const int32_t Complex = (int)Atype & 1, uc = std::max(-1, std::min(80, handle->QuantizeBitCorrection + u));
  if (uA) { *uA = uc; } if (cPanels) { *cPanels = 1 + Complex; }
  if (lPanels) { *lPanels = 0 <= uc ? (63 + std::max(0, 2 * (uc + Complex)) + (int32_t)std::ceil(std::log2((double)Mp))) / 63 : 0; }
}

void hyh::quantize_scale_batch(const hyacinHandle_t* handle, char op, int32_t batches, int32_t segM, int32_t lastM, int32_t N, int Atype, const void* A, int64_t lda, int32_t uA, int32_t* vexp) {
  if (N <= 0 || Atype > HYACIN_F16_COMPLEX) { return; }
  hyh::timer_mark(handle, hyh::Segment::dist_kernel);
  HYH_KERNEL(hykColumnExponentsOp(handle->hipStream, op, batches, segM, lastM, N, (int32_t)Atype, A, lda, uA, vexp));
}

extern "C" void hyacinXquantizeScaleBatch(const hyacinHandle_t* handle, int32_t batches, int32_t segM, int32_t lastM, int32_t N, hyacinPrecision_t Atype, const void* A, int32_t lda, int32_t uA, int32_t* vexp) {
  hyh::ApiScope scope;
  hyh::quantize_scale_batch(handle, 'N', batches, segM, lastM, N, (int)Atype, A, lda, uA, vexp);
}

namespace {

/* op: 'N' A is column-major M x N; 'T' / 'C' A is the stored N x M (conjugate) transpose, op(A)[k, j] = (conj) A[j + k lda] */
struct Ctx { const hyacinHandle_t* h; hipStream_t s; char op; int32_t N, Atype, Complex, u; const char* A; int64_t lda; const int32_t* vexp; int32_t beta, orderC; uint64_t* C; };

const void* row_ptr(const Ctx& c, int64_t row) { return c.A + row * (c.op == 'N' ? 1 : c.lda) * (int64_t)hyh::elem_bytes(c.Atype); }

int32_t crt_panels(int32_t order, int32_t Complex) { return Complex ? 2 * order + std::max(0, order - HYK_CRT_CPLX_SPLIT) : order; }

/* Leading dimension of the panel rows for a capacity of `cap` K-bytes: a row length that is a multiple of 4096 bytes gets
 * 256 more, so that the rows of a tile (one cache line each per K slab) do not all fall on the same few cache sets and
 * memory channels. */
int64_t panel_ld(int64_t cap) { return cap + ((cap % 4096 == 0) ? 256 : 0); }

/* a list of row runs [first, first + count) of A, quantized back to back into one compact panel set and contracted */
struct Run { int64_t first; int32_t count; };

/* what the last hyacinXherkBatch of this thread did (hykLastHerkPlan) */
thread_local hykHerkPlan g_plan;
void note_quantize() { ++g_plan.quantizeCalls; }
void note_gram(const Ctx& c, char alg, int32_t order, int32_t chunkRows, int32_t rows) {
  /* algorithmic int8 operations (2 per multiply-add, triangle only) of one contraction over `rows` rows */
  const double M = rows, N = c.N; double ops;
  if (alg == 'C') { ops = c.Complex ? std::min(order, HYK_CRT_CPLX_SPLIT) * 2. * M * N * N + std::max(order - HYK_CRT_CPLX_SPLIT, 0) * (M * N * (N + 1.) + 2. * M * N * N) : order * M * N * (N + 1.); }
  else { ops = order * M * N * (N + 1.) + (double)order * (order - 1) * M * N * N + (c.Complex ? (double)order * order * 2. * M * N * N : 0.); }
  g_plan.algorithm = alg; g_plan.order = order; g_plan.chunkRows = chunkRows; ++g_plan.gramCalls; g_plan.rows += rows; g_plan.int8Ops += ops;
}

void log_gemm(const Ctx& c, const char* kind, int32_t K, int32_t order) {
  if (c.h->logger) { std::fprintf((FILE*)c.h->logger, "I8I32-GEMM-%s [algo=TN,%s] [M=N=%d] [K=%d] [Order=%d]\n", c.Complex ? "COMPLEX" : "REAL", kind, (c.N + 63) & ~63, K, order); }
}

void limb_bucket(Ctx& c, const std::vector<Run>& runs, int32_t order) {
  int64_t rows = 0; for (const Run& r : runs) { rows += r.count; } if (rows <= 0) { return; }
  const int32_t groups = c.Complex ? 3 : 1; const int64_t rowBytes = (int64_t)c.N * order * groups;
  int64_t cap = std::max<int64_t>(8192, (int64_t)(kPanelBudget / (size_t)rowBytes) / 128 * 128); cap = std::min<int64_t>(cap, (rows + 127) / 128 * 128);
  const size_t wsBytes = hykGramWorkspaceBytes(HYK_GRAM_LIMBS, c.Complex, c.N, order);
  const int64_t ld = panel_ld(cap);
  hyh::Scratch W(c.h, (size_t)ld * (size_t)rowBytes), ws(c.h, wsBytes);
  if (!hyh::ok()) { return; }
  HYH_KERNEL(hykGramWorkspaceClear(c.s, ws.p, wsBytes));
  int32_t filled = 0;
  auto flush = [&]() {
    if (filled <= 0) { return; } const int32_t K = hyh::round_up(filled, 128);
    HYH_KERNEL(hykZeroRows(c.s, W.as<int8_t>(), ld, (int64_t)c.N * order * groups, filled, K));
    HYH_KERNEL(hykGramLimbs(c.s, c.Complex, c.N, order, W.as<int8_t>(), ld, K, c.beta, c.orderC, c.C, ws.p)); c.beta = 1; log_gemm(c, "limbs", K, order); note_gram(c, 'L', order, (int32_t)cap, filled); filled = 0;
  };
  for (const Run& r : runs) {
    int64_t first = r.first; int32_t left = r.count;
    while (left > 0) {
      const int32_t take = (int32_t)std::min<int64_t>(left, cap - filled);
      HYH_KERNEL(hykQuantizeLimbsOp(c.s, c.op, take, c.N, order, c.Atype, row_ptr(c, first), c.lda, c.vexp, W.as<int8_t>() + filled, ld)); note_quantize();
      filled += take; first += take; left -= take; if (filled == cap) { flush(); }
    }
  }
  flush();
}

void crt_bucket(Ctx& c, const std::vector<Run>& runs, int32_t order, int32_t chunkRows, int32_t maxBits) {
  int64_t rows = 0; for (const Run& r : runs) { rows += r.count; } if (rows <= 0 || order <= 0) { return; }
  const int32_t panels = crt_panels(order, c.Complex); const int64_t rowBytes = (int64_t)c.N * panels;
  int64_t cap = std::max<int64_t>(8192, (int64_t)(kPanelBudget / (size_t)rowBytes) / 128 * 128);
  cap = std::min<int64_t>(cap, std::max(128, chunkRows / 128 * 128)); cap = std::min<int64_t>(cap, (rows + 127) / 128 * 128);
  const size_t wsBytes = hykGramWorkspaceBytes(HYK_GRAM_CRT, c.Complex, c.N, order);
  const int64_t ld = panel_ld(cap);
  hyh::Scratch W(c.h, (size_t)ld * (size_t)rowBytes), ws(c.h, wsBytes);
  if (!hyh::ok()) { return; }
  HYH_KERNEL(hykGramWorkspaceClear(c.s, ws.p, wsBytes));
  int32_t filled = 0;
  auto flush = [&]() {
    if (filled <= 0) { return; } const int32_t K = hyh::round_up(filled, 128);
    HYH_KERNEL(hykZeroRows(c.s, W.as<int8_t>(), ld, (int64_t)c.N * panels, filled, K));
    HYH_KERNEL(hykGramCrt(c.s, c.Complex, c.N, order, W.as<int8_t>(), ld, K, c.beta, c.orderC, c.C, ws.p)); c.beta = 1; log_gemm(c, "crt", K, order); note_gram(c, 'C', order, (int32_t)cap, filled); filled = 0;
  };
  for (const Run& r : runs) {
    int64_t first = r.first; int32_t left = r.count;
    while (left > 0) {
      const int32_t take = (int32_t)std::min<int64_t>(left, cap - filled);
      HYH_KERNEL(hykQuantizeCrtOp(c.s, c.op, take, c.N, order, c.Atype, row_ptr(c, first), c.lda, c.vexp, W.as<int8_t>() + filled, ld, maxBits)); note_quantize();
      filled += take; first += take; left -= take; if (filled == cap) { flush(); }
    }
  }
  flush();
}

void zero_gram(const Ctx& c) {
  const size_t bytes = (size_t)c.N * (size_t)(c.N + 1) / 2 * (size_t)c.orderC * (c.Complex ? 2 : 1) * 8;
  HYH_KERNEL(hykGramWorkspaceClear(c.s, c.C, bytes));
}

/* reference: herk_dispatcher, src/hyacin_herk.cpp:283-310 */
void herk_single(Ctx& c, int32_t M) {
  if (M <= 0 || c.u < 0) { if (c.beta == 0) { zero_gram(c); } return; }
  const hyh::GramPlan p = hyh::gram_algorithm(c.h->GramMatrixAlgorithm, M, c.u + c.Complex, c.Complex, c.h->TCGemmTargetK, c.h->StrideBatchPerfPenalty);
  std::vector<Run> runs{ Run{ 0, M } };
  if (p.alg == 'L') { limb_bucket(c, runs, p.order); } else { crt_bucket(c, runs, p.order, p.second, c.u + 1); }
}

/* reference: herk_batch_dispatcher, src/hyacin_herk.cpp:312-384 */
void herk_sliced(Ctx& c, int32_t batches, int32_t segM, int32_t lastM) {
  const int32_t uCeil = c.Complex + c.u, M = (batches - 1) * segM + lastM;
  std::vector<int32_t> segU((size_t)batches);
  { hyh::Scratch d(c.h, sizeof(int32_t) * (size_t)batches);
    HYH_KERNEL(hykSliceRange(c.s, batches, c.N, c.u + c.Complex, c.vexp, d.as<int32_t>()));
    if (hyh::ok()) { HYH_CHECK(hipMemcpyAsync(segU.data(), d.p, sizeof(int32_t) * (size_t)batches, hipMemcpyDeviceToHost, c.s)); } HYH_CHECK(hipStreamSynchronize(c.s)); }
  if (!hyh::ok()) { return; }
  /* precision levels at which the limb path wins: slices whose own bit range fits level i are contracted with that few limbs */
  std::vector<hyh::GramPlan> limbLevels; int32_t uFloor = c.Complex;
  while (uFloor <= uCeil) {
    const hyh::GramPlan p = hyh::gram_algorithm(c.h->GramMatrixAlgorithm, M, uFloor, c.Complex, c.h->TCGemmTargetK, c.h->StrideBatchPerfPenalty);
    if (p.alg == 'L') { uFloor = 1 + p.second; limbLevels.push_back(p); } else { uFloor = 1 + uCeil; }
  }
  const int32_t nLevels = (int32_t)limbLevels.size(); std::vector<int32_t> bucketOf((size_t)batches, -1), bucketRows((size_t)nLevels + 1, 0);
  for (int32_t i = 0; i < batches; ++i) {
    if (segU[i] < 0) { continue; }   /* all-zero slice */
    int32_t b = 0; while (b < nLevels && segU[i] > limbLevels[b].second) { ++b; }
    bucketOf[i] = b; bucketRows[b] += (i + 1 == batches) ? lastM : segM;
  }
  const hyh::GramPlan ceil = hyh::gram_algorithm(c.h->GramMatrixAlgorithm, bucketRows[nLevels], uCeil, c.Complex, c.h->TCGemmTargetK, c.h->StrideBatchPerfPenalty);
  auto runs_of = [&](int32_t b) {
    std::vector<Run> runs; int32_t i = 0;
    while (i < batches) {
      if (bucketOf[i] != b) { ++i; continue; }
      int32_t j = i; while (j < batches && bucketOf[j] == b) { ++j; }
      const int64_t first = (int64_t)i * segM, end = std::min<int64_t>(M, (int64_t)j * segM); runs.push_back(Run{ first, (int32_t)(end - first) }); i = j;
    }
    return runs;
  };
  bool any = false;
  for (int32_t b = 0; b < nLevels; ++b) if (bucketRows[b] > 0) { limb_bucket(c, runs_of(b), limbLevels[b].order); any = true; }
  if (bucketRows[nLevels] > 0) {
    if (ceil.alg == 'L') { limb_bucket(c, runs_of(nLevels), ceil.order); } else { crt_bucket(c, runs_of(nLevels), ceil.order, ceil.second, c.u + 1); }
    any = true;
  }
  if (!any && c.beta == 0) { zero_gram(c); }
}

}  // namespace

void hyh::herk_batch(const hyacinHandle_t* handle, char op, int32_t batches, int32_t segM, int32_t lastM, int32_t N, int Atype, const void* A, int64_t lda, int32_t u, const int32_t* vexp, int32_t beta, int32_t orderC, uint64_t* C) {
  if (N <= 0 || orderC <= 0 || Atype < 0 || Atype > HYACIN_F16_COMPLEX) { return; }
  hyh::timer_mark(handle, hyh::Segment::dist_kernel);
  g_plan = hykHerkPlan{};
  Ctx c{ handle, handle->hipStream, (op == 'T' || op == 'C') ? op : 'N', N, (int32_t)Atype, (int32_t)Atype & 1, u, (const char*)A, lda, vexp, beta, orderC, C };
  if (batches <= 1) { herk_single(c, lastM); } else { herk_sliced(c, batches, segM, lastM); }
}

extern "C" void hyacinXherkBatch(const hyacinHandle_t* handle, int32_t batches, int32_t segM, int32_t lastM, int32_t N, hyacinPrecision_t Atype, const void* A, int32_t lda, int32_t u, const int32_t* vexp, int32_t beta, int32_t orderC, uint64_t* C) {
  hyh::ApiScope scope;
  hyh::herk_batch(handle, 'N', batches, segM, lastM, N, (int)Atype, A, lda, u, vexp, beta, orderC, C);
}

/* the two stage functions above with the storage order of A as an argument (the reference transposes first, src/lra.cpp:63-69) */
extern "C" void hykQuantizeScaleBatchOp(const void* handle, char opA, int32_t batches, int32_t segM, int32_t lastM, int32_t N, int32_t Atype, const void* A, int64_t lda, int32_t uA, int32_t* vexp) {
  hyh::ApiScope scope; const char op = (opA == 'T' || opA == 't') ? 'T' : ((opA == 'C' || opA == 'c') ? 'C' : 'N');
  hyh::quantize_scale_batch((const hyacinHandle_t*)handle, op, batches, segM, lastM, N, Atype, A, lda, uA, vexp);
}
extern "C" void hykHerkBatchOp(const void* handle, char opA, int32_t batches, int32_t segM, int32_t lastM, int32_t N, int32_t Atype, const void* A, int64_t lda, int32_t u, const int32_t* vexp, int32_t beta, int32_t orderC, uint64_t* C) {
  hyh::ApiScope scope; const char op = (opA == 'T' || opA == 't') ? 'T' : ((opA == 'C' || opA == 'c') ? 'C' : 'N');
  hyh::herk_batch((const hyacinHandle_t*)handle, op, batches, segM, lastM, N, Atype, A, lda, u, vexp, beta, orderC, C);
}
extern "C" int hykLastHerkPlan(hykHerkPlan* out) { if (!out) { return -1; } *out = g_plan; return 0; }

extern "C" void hyacinXdequantizeInit(const hyacinHandle_t* handle, int32_t N, int32_t orderC, const uint64_t* C, const int32_t* vexp, hyacinPrecision_t Atype, hyacinPrecision_t* Gtype, int32_t* gElemBytes) {
  hyh::ApiScope scope;
  if (N <= 0 && (Gtype != nullptr || gElemBytes != nullptr)) { return; }
  hyh::timer_mark(handle, hyh::Segment::rep_kernel);
  int32_t* word = (int32_t*)handle->pinnedWorkspace; if (!word) { hyh::fail(-1, "hyacinXdequantizeInit", "the handle has no pinned word (hyacinCreate not called?)", __FILE__, __LINE__); return; } *word = 0;
  if (N > 0 && orderC >= 1 && orderC <= 3) { HYH_KERNEL(hykGramRange(handle->hipStream, N, orderC, C, vexp, word)); }
  HYH_CHECK(hipStreamSynchronize(handle->hipStream));
  /* significant bits of the Gram = bit length of the dominant diagonal entry minus the 2 x correction bits of head-room */
  const int32_t bits = *word - 2 * handle->QuantizeBitCorrection;
  int g = bits <= 23 ? HYACIN_F32_COMPLEX : (bits <= 52 ? HYACIN_F64_COMPLEX : ((bits <= 71 && !handle->DeviceIsF64Capable) ? HYACIN_TF_COMPLEX : ((bits <= 95 && !handle->DeviceIsF64Capable) ? HYACIN_QF_COMPLEX : HYACIN_DD_COMPLEX)));
  if (!((int)Atype & 1)) { g &= ~1; }
  if (Gtype) { *Gtype = (hyacinPrecision_t)g; } if (gElemBytes) { *gElemBytes = hyh::elem_bytes(g); }
}

extern "C" void hyacinXdequantize(const hyacinHandle_t* handle, int32_t N, int32_t orderC, const uint64_t* C, const int32_t* vexp, hyacinPrecision_t Gtype, void* G, int32_t ldg) {
  hyh::ApiScope scope;
  if (N <= 0) { return; }
  hyh::timer_mark(handle, hyh::Segment::rep_kernel);
  HYH_KERNEL(hykDequantize(handle->hipStream, N, orderC, C, vexp, (int32_t)Gtype, G, ldg));
}
