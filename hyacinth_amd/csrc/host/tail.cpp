/*
 * tail.cpp -- hyacinXGevd (truncated SVD from the Gram matrix) and hyacinXGinterp
 * (interpolative decomposition from the Gram matrix).
 *
 * Mirrors the reference's src/gram_evd.cu:94-194 (tsvd, find_srank_kernel, hyacinXGevd) and
 * src/gram_id.cpp:28-101 (interp, hyacinXGinterp).  The factorization itself runs in the HIP kernels of
 * potrfp.hip and tail.hip; no vendor solver is involved.  Differences that are visible to a caller:
 *  - an FP32 Gram is widened to FP64 before the Cholesky (the reference factors it in FP32);
 *  - the SVD runs on a factor in doubles for FP64 storage and in floats for FP32 / FP16 storage, as the reference's does;
 *    every rotation is worked out in FP64 either way;
 *  - the Jacobi iteration stops as soon as a sweep applies no rotation, or leaves only cosines that the quadratic
 *    contraction measured over the last two sweeps puts within 8 thresholds, or once the values that are handed out have
 *    stopped moving and their columns are orthogonal to sqrt(eps); a sweep here is one plain round-robin pass over all
 *    column pairs, which does less work than a sweep of the vendor's blocked solver, so the cap is 5 x |JacobiSVDSweeps|
 *    plain sweeps (15 by default); JacobiSVDSweeps == 0 (the reference's "bidiagonalization backend") caps at 30.
 * G is working storage, as in the reference (which overwrites it with the factor): the Cholesky keeps the trailing matrix
 * in its strict upper triangle.  An FP32 Gram is factored from a widened copy and stays as it was.
 */
#include <numeric>
#include <cfloat>
#include "common.hpp"
#include "jacobi_stop.hpp"

namespace {

double storage_eps(int Atype) { return (Atype == HYACIN_F64 || Atype == HYACIN_F64_COMPLEX) ? DBL_EPSILON : (double)FLT_EPSILON; }
int factor_type(int Gtype) { const int c = Gtype & 1; return ((Gtype & ~1) == HYACIN_DD ? HYACIN_DD : HYACIN_F64) + c; }

struct Factor {
  hyh::Scratch widened, Rt, work; void* G; int64_t ldg; int type; int32_t ldr; size_t rtBytes;
  Factor(const hyacinHandle_t* h, int32_t N, int32_t Kmax, int Gtype, void* Gin, int64_t ldgIn)
    : widened(h, ((Gtype & ~1) == HYACIN_F32) ? (size_t)N * N * 8 * (1 + (Gtype & 1)) : 0),
      Rt(h, (size_t)N * (size_t)std::min(N, Kmax + 1) * (size_t)hyh::elem_bytes(factor_type(Gtype))),
      work(h, hykPotrfpWorkspaceBytes(N, factor_type(Gtype))) {
    type = factor_type(Gtype); ldr = std::min(N, Kmax + 1); rtBytes = (size_t)N * ldr * hyh::elem_bytes(type); G = Gin; ldg = ldgIn;
    if (!hyh::ok()) { return; }
    if (widened.p) { HYH_KERNEL(hykMatcopy(h->hipStream, 'A', N, N, Gtype, Gin, ldgIn, HYACIN_F64 + (Gtype & 1), widened.p, N)); G = widened.p; ldg = N; }
    HYH_KERNEL(hykGramWorkspaceClear(h->hipStream, Rt.p, rtBytes));
  }
};

const char* type_tag(int t) { switch (t) { case HYACIN_F64: return "FP64"; case HYACIN_F64_COMPLEX: return "FP64-COMPLEX"; case HYACIN_DD: return "FP128-DD"; default: return "FP128-DD-COMPLEX"; } }

/* wanted / cut / left: hykPotrfpWanted (the factorization may end early for a caller that uses `wanted` values only; *left is
 * then the trace of what it did not factor) */
int32_t run_potrfp(const hyacinHandle_t* h, Factor& f, double eps, int32_t K, int32_t N, int32_t* jpiv, int32_t wanted = 0, double cut = 0., double* left = nullptr) {
  int32_t* word = (int32_t*)h->pinnedWorkspace; if (!word) { hyh::fail(-1, "pivoted Cholesky", "the handle has no pinned word (hyacinCreate not called?)", __FILE__, __LINE__); }
  if (!hyh::ok()) { return 0; }
  double* trace = reinterpret_cast<double*>(word + 2);   /* the pinned block is 64 bytes */
  *word = 0; *trace = 0.;
  HYH_KERNEL(hykPotrfpWanted(h->hipStream, h->DeviceSMs, eps, K, wanted, cut, N, f.type, f.G, f.ldg, f.Rt.p, f.ldr, jpiv, f.work.p, word, trace));
  HYH_CHECK(hipStreamSynchronize(h->hipStream));
  if (!hyh::ok()) { return 0; }
  int32_t rank = *word; if (left) { *left = *trace; }
  if (rank < 0) {   /* the workgroups lost each other (a bounded wait inside the kernel gave up): no basis rather than a wrong one */
    hyh::fail(-5, "pivoted Cholesky", "a workgroup gave up waiting for the others; no factor was produced", __FILE__, __LINE__);
    return 0;
  }
  if (h->logger) { std::fprintf((FILE*)h->logger, "POTRFP-%s [eps=%.1le] [N=%d] [K=%d] [Cholesky-rank=%d]\n", type_tag(f.type), eps, N, K, rank); }
  return rank;
}

}  // namespace

extern "C" int32_t hyacinXGevd(const hyacinHandle_t* handle, double eps, int32_t N, int32_t K, hyacinPrecision_t Atype, void* X, int32_t ldx, void* S, hyacinPrecision_t Gtype, void* G, int32_t ldg) {
  hyh::ApiScope scope;
  if (N <= 0) { return 0; }
  K = K <= 0 ? N : std::min(N, K);
  if ((int)Atype < 0 || (int)Atype > HYACIN_F16_COMPLEX || ((int)Atype & 1) != ((int)Gtype & 1)) { return 0; }
  const int gbase = (int)Gtype & ~1; if (gbase != HYACIN_F64 && gbase != HYACIN_F32 && gbase != HYACIN_DD) { return 0; }
  hipStream_t s = handle->hipStream; hyh::timer_mark(handle, hyh::Segment::rep_kernel);
  const int32_t lrqr = handle->QRCPTruncateRank, jac = std::abs(handle->JacobiSVDSweeps), bid = std::abs(std::min(0, handle->JacobiSVDSweeps));
  const int32_t sweeps = lrqr ? jac : bid;   /* FP64-capable device: the same rule for every storage type (src/gram_evd.cu:148-150) */
  const int Complex = (int)Atype & 1; const double machineEps = storage_eps((int)Atype);
  eps = std::min(std::max(std::fabs(eps), machineEps), 1.);

  hyh::Scratch jpiv(handle, sizeof(int32_t) * (size_t)N);
  int32_t rank = 0;
  /* First with a factorization that may end early (hykPotrfpWanted: K values are wanted, and a floor right under them is
   * not worth its rows); if the values found then say that what was not factored weighs too much, once more in full. */
  for (int attempt = 0; attempt < 2; ++attempt) {
    bool again = false;
    Factor f(handle, N, N, (int)Gtype, G, ldg);
    if (attempt > 0 && !f.widened.p) { HYH_KERNEL(hykMirrorLower(s, N, f.type, f.G, f.ldg)); }   /* the first factorization has used the strict upper triangle of G */
    const bool mayEndEarly = attempt == 0 && lrqr && K < N;
    double unfactored = 0.;
    rank = run_potrfp(handle, f, lrqr ? eps : 0., N, N, jpiv.as<int32_t>(), mayEndEarly ? K : 0, mayEndEarly ? hyh::kTruncationGuess * hyh::kTruncationBudget * eps : 0., &unfactored);
    if (rank <= 0 || !hyh::ok()) { return 0; }
    if (handle->logger && unfactored > 0.) { std::fprintf((FILE*)handle->logger, "POTRFP: ended after %d columns, what is left of G has trace %.2le\n", rank, unfactored); }
    /* B = (R P^T)^H, N x rank, in the precision of the output storage type: doubles for FP64, floats for FP32 and FP16
     * (reference: src/gram_evd.cu:96-98) */
    const bool wideB = (int)Atype == HYACIN_F64 || (int)Atype == HYACIN_F64_COMPLEX; const int Btype = (wideB ? HYACIN_F64 : HYACIN_F32) + Complex;
    hyh::Scratch B(handle, (size_t)N * rank * (wideB ? 8 : 4) * (1 + Complex)), sigma(handle, sizeof(double) * (size_t)rank), counter(handle, 64), carry(handle, hykJacobiCarryBytes(rank));
    if (!hyh::ok()) { return 0; }
    HYH_KERNEL(hykFactorToB(s, N, rank, f.type, f.Rt.p, f.ldr, Btype, B.p));
    const int32_t maxSweeps = sweeps > 0 ? 5 * sweeps : 30; int32_t used = 0;
    /* A pair is rotated while its cosine exceeds the storage precision, but never below sqrt(N) FP64 roundings: that is
     * what the dot product of two columns of length N carries as noise (the threshold of LAPACK's xGESVJ); rotating
     * below it costs sweeps and leaves the orthogonality where it was.  Nor below a sixteenth of the accuracy asked for:
     * cosines of that size move a singular value by less than eps / 2 of the largest one. */
    const double rotateAbove = std::max(std::max(machineEps, std::sqrt((double)N) * 2.220446049250313e-16), eps / 16.);
    std::vector<double> before((size_t)rank), after, sig;
    auto fetch_norms = [&](std::vector<double>& v, int32_t cols) {
      v.resize((size_t)cols);
      HYH_KERNEL(hykColumnNorms(s, Btype, N, cols, B.p, sigma.as<double>()));
      HYH_CHECK(hipMemcpyAsync(v.data(), sigma.p, sizeof(double) * (size_t)cols, hipMemcpyDeviceToHost, s));
    };
    /* The sweeps may end on the values alone (jacobi_output_settled), which settle with the square of what the vectors still
     * lack: singular values 2 % apart leave their vectors several per cent away from orthogonal when the values have long
     * stopped moving.  What is handed out as singular vectors is held to sqrt(eps) in every entry of V^H V - I: the
     * projector V V^H is then right to eps.
     * (The scratch for that -- a Gram matrix, two copies of the vectors, their order, the result word -- is taken once, before
     * the sweeps: whether a sweep ends "settled" depends on the data, and an allocation in the middle of the loop would make
     * the calls that can fail depend on it too; needed only when fewer values are handed out than the factor has columns.) */
    const bool mayCheck = K < rank && rank > 1;
    const size_t elemB = (size_t)(wideB ? 8 : 4) * (1 + Complex);
    hyh::Scratch gram(handle, mayCheck ? (size_t)rank * rank * elemB : 0), dOut(handle, mayCheck ? 64 : 0);
    hyh::Scratch polishA(handle, mayCheck ? (size_t)N * K * elemB : 0), polishB(handle, mayCheck ? (size_t)N * K * elemB : 0), dPolishOrder(handle, mayCheck ? sizeof(int32_t) * (size_t)K : 0);
    if (!hyh::ok()) { return 0; }
    const double orthogonalTo = std::sqrt(eps), tightTo = std::max(eps, 64. * (wideB ? 2.220446049250313e-16 : 1.1920928955078125e-07));
    int32_t cols = rank; double dropped2 = 0., droppedSpectral = 0.;
    /* rank cut (reference: find_srank_kernel, src/gram_evd.cu:44-70): with the values in descending order (`order`), keep i < K
     * while sum_{j>=i} sigma_j^2 > eps^2 sum_j sigma_j^2; the columns left out of the sweeps count with what they weigh (the sum
     * over all values is the trace of G either way).  Returns how many are kept. */
    auto rank_cut = [&](const std::vector<double>& value, std::vector<int32_t>& order) -> int32_t {
      const int32_t n = (int32_t)value.size(); order.resize((size_t)n); std::iota(order.begin(), order.end(), 0);
      std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return value[(size_t)a] > value[(size_t)b]; });
      std::vector<double> suffix((size_t)n + 1, dropped2); for (int32_t i = n - 1; i >= 0; --i) { const double v = value[(size_t)order[(size_t)i]]; suffix[(size_t)i] = std::fma(v, v, suffix[(size_t)i + 1]); }
      const double resid = eps * eps * suffix[0]; int32_t kept = 0;
      for (int32_t i = 0; i < K && i < n; ++i) { if (resid < suffix[(size_t)i]) { ++kept; } }
      return kept;
    };
    /* Once the values have settled, the vectors that will be handed out (the rank cut applied to the norms as they are) are
     * normalised into a copy V and every entry of V^H V - I is measured.  Within sqrt(eps): done.  Short of that by a
     * cluster of values that K cuts through (the sweeps bring its vectors apart slowly, and which basis of the cluster's
     * span is handed out is immaterial): V is made orthonormal directly, V <- V (3 I - V^H V) / 2 (the Newton-Schulz step
     * towards the orthonormal factor of V's polar decomposition: same span, so the same projection residual; a defect d
     * becomes about d^2 per step), measured again after each step.  sqrt(eps) is what is needed for the sweeps to end; the
     * steps (three at most) go on to eps, or to the rounding of the copy's type, while they gain: the reference's vectors,
     * a product of rotations, are orthonormal to rounding whatever state its sweeps end in.  It has to be exactly the vectors that are
     * handed out: a vector made orthogonal to one that is then dropped would carry a share of that direction and lose as
     * much of its own.  Returns 0: not orthogonal, the sweeps go on; 1: orthogonal as the columns are; 2: the first
     * `polishedCols` columns of `polished` are what is handed out, in the order `polishOrder`. */
    void* polished = nullptr; int32_t polishedCols = 0; std::vector<int32_t> polishOrder;
    auto orthonormal = [&](const std::vector<double>& norm, int32_t ncols) -> int {
      const int32_t k = rank_cut(std::vector<double>(norm.begin(), norm.begin() + ncols), polishOrder); if (k < 2 || !polishA.p) { return 1; }
      HYH_CHECK(hipMemcpyAsync(dPolishOrder.p, polishOrder.data(), sizeof(int32_t) * (size_t)k, hipMemcpyHostToDevice, s));
      void* cur = polishA.p; void* nxt = polishB.p;
      HYH_KERNEL(hykBasisOut(s, N, k, Btype, Btype, B.p, sigma.as<double>(), dPolishOrder.as<int32_t>(), cur, N));   /* sigma holds the norms of the sweep just finished */
      double defect = 1., before_ = 2.; int steps = 0;
      for (;; ++steps) {
        double defect2 = 1.;
        HYH_KERNEL(hykGramWorkspaceClear(s, dOut.p, 64));
        HYH_KERNEL(hykGemm(s, 'C', 'N', k, k, N, 1., Btype, cur, N, cur, N, 0., gram.p, k));
        HYH_KERNEL(hykMaxDefect(s, Btype, k, gram.p, k, dOut.as<double>()));   /* the diagonal included: a step leaves the norms off by about d^2 too */
        HYH_CHECK(hipMemcpyAsync(&defect2, dOut.p, sizeof(double), hipMemcpyDeviceToHost, s)); HYH_CHECK(hipStreamSynchronize(s));
        if (!hyh::ok()) { return 0; }
        defect = std::sqrt(defect2);
        if (handle->logger) { std::fprintf((FILE*)handle->logger, "GESVJ sweep %d: the %d vectors to be handed out%s: largest entry of V^H V - I %.2le (needed: %.2le, aimed at: %.2le)\n", used, k, steps ? " after an orthonormalisation step" : "", defect, orthogonalTo, tightTo); }
        if (defect <= tightTo || steps == 3 || defect > 0.25 || defect > 0.25 * before_) { break; }   /* there, or out of steps, or too far for the step to converge, or no longer gaining */
        before_ = defect;
        HYH_KERNEL(hykNewtonSchulzFactor(s, Btype, k, gram.p, k));
        HYH_KERNEL(hykGemm(s, 'N', 'N', N, k, k, 1., Btype, cur, N, gram.p, k, 0., nxt, N));
        std::swap(cur, nxt);
      }
      if (!hyh::ok() || defect > orthogonalTo) { return 0; }
      if (steps == 0) { return 1; }
      polished = cur; polishedCols = k; return 2;
    };
    /* Only the K largest values and their vectors are handed out.  Leaving the last rows of the Cholesky factor (the last
     * columns of B) out of the SVD takes a positive semidefinite matrix of trace tau (the sum of their squared norms) off
     * G: every eigenvalue moves down by at most tau, a singular value by at most tau / (2 sigma'), sigma' being the value
     * found without them.  The columns of a noise floor under the values that are wanted are not worth their rotations:
     * the prefix is picked from the column norms (choose_cut below), and what the sweeps then find must confirm it
     * (jacobi_truncation_holds_spectral with the values themselves), or columns are taken back in. */
    /* The cut for given budgets: the longest tail [t, rank), t >= atLeast, that passes the trace rule or the sharper rule
     * (jacobi_columns_needed_spectral: what moves a value is the largest eigenvalue of the Gram matrix of the columns left
     * out, which for the rows of a noise floor is a small part of their trace).  The Gram matrix is formed once, for the
     * window [c0, rank) of columns that can pass at all under the first (largest) budgets: squared norm (a diagonal entry,
     * below the largest eigenvalue) within the budget of the values, trace within the budget of the residual. */
    std::vector<double> allNorms, absGram; int32_t c0 = rank;
    auto choose_cut = [&](double valueBudget, double residualBudget, int32_t atLeast) {
      int32_t t = rank; double sum = unfactored;   /* trace rule; what the Cholesky left unfactored counts as rows left out, with its trace as the bound of its largest eigenvalue */
      while (t > atLeast && sum + allNorms[(size_t)(t - 1)] * allNorms[(size_t)(t - 1)] <= valueBudget) { sum += allNorms[(size_t)(t - 1)] * allNorms[(size_t)(t - 1)]; --t; }
      cols = t; bool sharper = false;
      if (!absGram.empty() && c0 < cols) {
        const hyh::JacobiCut cut = hyh::jacobi_columns_needed_spectral(absGram, rank, c0, atLeast, (valueBudget - unfactored) / 1.01, residualBudget - unfactored);   /* 1 %: the products are rounded */
        if (cut.cols < cols) { cols = cut.cols; droppedSpectral = 1.01 * cut.spectral + unfactored; sharper = true; }
      }
      dropped2 = unfactored; for (int32_t j = rank - 1; j >= cols; --j) { dropped2 = std::fma(allNorms[(size_t)j], allNorms[(size_t)j], dropped2); }
      if (!sharper) { droppedSpectral = dropped2; }   /* the trace bounds the largest eigenvalue */
      if (handle->logger && cols < rank) { std::fprintf((FILE*)handle->logger, "GESVJ: the last %d of %d columns (squared norms %.2le in all, largest eigenvalue of their Gram matrix at most %.2le) are left out of the sweeps\n", rank - cols, rank, dropped2, droppedSpectral); }
    };
    dropped2 = droppedSpectral = unfactored;
    if (K < rank && rank > 1) {
      fetch_norms(allNorms, rank); HYH_CHECK(hipStreamSynchronize(s)); if (!hyh::ok()) { return 0; }
      std::vector<double> v(allNorms); std::nth_element(v.begin(), v.begin() + (K - 1), v.end(), std::greater<double>());
      const double nuK = v[(size_t)(K - 1)], nu1 = *std::max_element(allNorms.begin(), allNorms.end()), valueGuess = hyh::kTruncationGuess * hyh::kTruncationBudget * eps * nu1 * nuK;
      double outside = 0.; for (size_t j = (size_t)K; j < v.size(); ++j) { outside = std::fma(v[j], v[j], outside); }   /* the squared norms beyond the K largest */
      const double residualGuess = outside / 256.;
      { double suffix = 0.; while (c0 > K) { const double w = allNorms[(size_t)(c0 - 1)] * allNorms[(size_t)(c0 - 1)]; if (w > valueGuess || suffix + w > std::max(valueGuess, residualGuess)) { break; } suffix += w; --c0; } }
      if (c0 < hyh::jacobi_columns_needed(allNorms, K, eps) && gram.p) {   /* the sharper rule can reach further than the trace rule */
        const int32_t d = rank - c0; const size_t elem = (size_t)(wideB ? 8 : 4) * (1 + Complex);
        HYH_KERNEL(hykGemm(s, 'C', 'N', d, d, N, 1., Btype, (const char*)B.p + (size_t)c0 * N * elem, N, (const char*)B.p + (size_t)c0 * N * elem, N, 0., gram.p, d));
        std::vector<char> raw((size_t)d * d * elem); absGram.resize((size_t)d * d);
        HYH_CHECK(hipMemcpyAsync(raw.data(), gram.p, raw.size(), hipMemcpyDeviceToHost, s)); HYH_CHECK(hipStreamSynchronize(s)); if (!hyh::ok()) { return 0; }
        for (size_t i = 0; i < absGram.size(); ++i) {
          double re, im = 0.;
          if (wideB) { const double* q = reinterpret_cast<const double*>(raw.data()) + i * (1 + Complex); re = q[0]; if (Complex) { im = q[1]; } }
          else { const float* q = reinterpret_cast<const float*>(raw.data()) + i * (1 + Complex); re = q[0]; if (Complex) { im = q[1]; } }
          absGram[i] = Complex ? std::hypot(re, im) : std::fabs(re);
        }
      }
      choose_cut(valueGuess, residualGuess, K);
      before.assign(allNorms.begin(), allNorms.begin() + cols);
    }
    bool recut = false;
    for (;;) {
      double lastCosine2 = 0., lastMoved = 0.;
      const bool watchOutput = K < cols;   /* with every column handed out only the cosines can end the sweeps */
      for (int32_t sw = 0; sw < maxSweeps && cols > 1; ++sw) {
        const int32_t top = watchOutput ? hyh::jacobi_tail_start(before, K, eps) : cols;   /* a broad floor of small columns is left alone */
        HYH_KERNEL(hykGramWorkspaceClear(s, counter.p, 64));
        const int32_t headCols = watchOutput ? std::min(top, hyh::jacobi_head(before, K)) : cols;   /* cosines are watched on the pairs that involve a column that can be handed out */
        HYH_KERNEL(hykJacobiSweepTop(s, Btype, N, cols, headCols, top, B.p, rotateAbove, counter.as<int32_t>(), carry.as<double>())); ++used;
        if (watchOutput) { fetch_norms(after, cols); }
        struct { int32_t rotations, pad; double cosine2; } seen = { 0, 0, 0. };
        HYH_CHECK(hipMemcpyAsync(&seen, counter.p, sizeof(seen), hipMemcpyDeviceToHost, s)); HYH_CHECK(hipStreamSynchronize(s));
        if (!hyh::ok()) { return 0; }
        if (seen.pad != 0) { hyh::fail(-5, "Jacobi sweep", "a workgroup gave up waiting for the partner it shares a block pair with; no basis was produced", __FILE__, __LINE__); return 0; }
        if (handle->logger) { std::fprintf((FILE*)handle->logger, "GESVJ sweep %d: %d rotations, largest cosine %.2le among pairs with a column before %d%s\n", used, seen.rotations, std::sqrt(seen.cosine2), headCols, top < cols ? " (floor of small columns left alone)" : ""); }
        if (hyh::jacobi_sweeps_done(seen.rotations, seen.cosine2, lastCosine2, rotateAbove)) { break; }
        if (watchOutput) {
          double moved[3] = { 0., 0., 0. }; const bool settled = hyh::jacobi_output_settled(before, after, K, eps, moved, lastMoved); lastMoved = moved[0];
          if (handle->logger) { std::fprintf((FILE*)handle->logger, "GESVJ sweep %d: the %d values handed out moved by at most %.2le, their columns gained %.2le of %.2le outside%s\n", used, K, moved[0], moved[1], moved[2], settled ? ": settled" : ""); }
          if (settled) {
            const int state = orthonormal(after, cols); if (!hyh::ok()) { return 0; }
            if (state != 0) { break; }
          }
        }
        lastCosine2 = seen.cosine2; before.swap(after);
      }
      fetch_norms(sig, cols); HYH_CHECK(hipStreamSynchronize(s));
      if (!hyh::ok()) { return 0; }
      if (cols == rank && unfactored == 0.) { break; }
      std::vector<double> top(sig); std::nth_element(top.begin(), top.begin() + (K - 1), top.end(), std::greater<double>());
      const double sigmaK = top[(size_t)(K - 1)], sigma1 = *std::max_element(sig.begin(), sig.end());
      double outside2 = 0.; for (size_t j = (size_t)K; j < top.size(); ++j) { outside2 = std::fma(top[j], top[j], outside2); }   /* the squared values that are not handed out */
      if (hyh::jacobi_truncation_holds_spectral(dropped2, droppedSpectral, sigma1, sigmaK, outside2, eps)) { break; }
      /* The guess from the column norms left out too much.  The first time, the cut is made again with half of the budget
       * that the values found allow (the columns taken back in are the unrotated ones next to the cut; the others stay as the
       * sweeps left them); should that fail too, the sweeps go on with all columns. */
      if (unfactored > 0. && !hyh::jacobi_truncation_holds_spectral(unfactored, unfactored, sigma1, sigmaK, outside2, eps)) { again = true; break; }   /* no cut of the rows at hand can make up for the rows that were never factored */
      polished = nullptr; polishedCols = 0;   /* (it held columns of a cut that did not stand) */
      const int32_t had = cols;
      if (!recut) { recut = true; choose_cut(0.5 * hyh::kTruncationBudget * eps * sigma1 * sigmaK, outside2 / 128., had); } else { cols = rank; dropped2 = droppedSpectral = unfactored; }
      if (cols <= had) { cols = rank; dropped2 = droppedSpectral = unfactored; }
      if (handle->logger) { std::fprintf((FILE*)handle->logger, "GESVJ: value %d is %.2le: the %d columns left out weigh too much, the sweeps go on with %d of %d\n", K, sigmaK, rank - had, cols, rank); }
      fetch_norms(before, cols); HYH_CHECK(hipStreamSynchronize(s)); if (!hyh::ok()) { return 0; }
    }
    if (again) {
      if (handle->logger) { std::fprintf((FILE*)handle->logger, "GESVJ: what the Cholesky left unfactored (%.2le) weighs too much against the values found: factoring again, in full\n", unfactored); }
      continue;
    }
    std::vector<int32_t> order; const int32_t kept = rank_cut(sig, order);
    std::vector<double> Sout((size_t)K, 0.); for (int32_t i = 0; i < kept; ++i) { Sout[(size_t)i] = sig[(size_t)order[(size_t)i]]; }
    const int32_t svdRank = kept; rank = std::min(rank, kept);
    hyh::Scratch dS(handle, sizeof(double) * (size_t)K), dOrder(handle, sizeof(int32_t) * (size_t)std::max(1, rank));
    if (!hyh::ok()) { return 0; }
    HYH_CHECK(hipMemcpyAsync(dS.p, Sout.data(), sizeof(double) * (size_t)K, hipMemcpyHostToDevice, s));
    if (rank > 0) { HYH_CHECK(hipMemcpyAsync(dOrder.p, order.data(), sizeof(int32_t) * (size_t)rank, hipMemcpyHostToDevice, s)); }
    HYH_KERNEL(hykValuesOut(s, K, (int32_t)Atype, dS.as<double>(), S));
    if (polished && !(rank == polishedCols && std::equal(order.begin(), order.begin() + rank, polishOrder.begin()))) { polished = nullptr; }   /* (the norms are those of the sweep the copy was made after, so cut and order agree) */
    if (rank > 0 && polished) { HYH_KERNEL(hykMatcopy(s, 'A', N, rank, Btype, polished, N, (int32_t)Atype, X, ldx)); }
    else if (rank > 0) { HYH_KERNEL(hykBasisOut(s, N, rank, (int32_t)Atype, Btype, B.p, sigma.as<double>(), dOrder.as<int32_t>(), X, ldx)); }
    HYH_CHECK(hipStreamSynchronize(s));   /* Sout / order are host temporaries */
    if (!hyh::ok()) { return 0; }
    if (handle->logger) { std::fprintf((FILE*)handle->logger, "GESVJ-%s [eps=%.1le] [M=%d] [N=%d] [K=%d] [sweeps=%d] [SVD-rank=%d]\n", wideB ? (Complex ? "FP64-COMPLEX" : "FP64") : (Complex ? "FP32-COMPLEX" : "FP32"), eps, N, rank, K, used, svdRank); }
    break;
  }
  return hyh::ok() ? rank : 0;
}

extern "C" int32_t hyacinXGinterp(const hyacinHandle_t* handle, double eps, int32_t N, int32_t K, hyacinPrecision_t Atype, void* X, int32_t ldx, int32_t* jpiv, hyacinPrecision_t Gtype, void* G, int32_t ldg) {
  hyh::ApiScope scope;
  if (N <= 0) { return 0; }
  K = K <= 0 ? N : std::min(N, K);
  if ((int)Atype < 0 || (int)Atype > HYACIN_F16_COMPLEX || ((int)Atype & 1) != ((int)Gtype & 1)) { return 0; }
  const int gbase = (int)Gtype & ~1; if (gbase != HYACIN_F64 && gbase != HYACIN_F32 && gbase != HYACIN_DD) { return 0; }
  hipStream_t s = handle->hipStream; hyh::timer_mark(handle, hyh::Segment::rep_kernel);
  const int Complex = (int)Atype & 1; eps = std::min(std::max(std::fabs(eps), storage_eps((int)Atype)), 1.);
  Factor f(handle, N, K, (int)Gtype, G, ldg);
  /* The factorization counts a single remaining column in (src/hyacin_potrfp.cu:271), so K = N - 1 can come back as N; the
   * reference then writes N columns into an X that the caller sized for K (src/gram_id.cpp:41).  Never more than K here. */
  const int32_t rank = std::min(K, run_potrfp(handle, f, eps, K, N, jpiv));
  if (rank <= 0 || !hyh::ok()) { return 0; }
  if (rank >= N) { HYH_KERNEL(hykInterpOut(s, N, N, (int32_t)Atype, jpiv, nullptr, X, ldx)); return hyh::ok() ? N : 0; }
  hyh::Scratch Rp(handle, (size_t)rank * rank * 8 * (1 + Complex)), Tt(handle, (size_t)rank * (N - rank) * 8 * (1 + Complex));
  if (!hyh::ok()) { return 0; }
  HYH_KERNEL(hykInterpSolve(s, N, rank, f.type, f.Rt.p, f.ldr, jpiv, Rp.as<double>(), Tt.as<double>()));
  HYH_KERNEL(hykInterpOut(s, N, rank, (int32_t)Atype, jpiv, Tt.as<double>(), X, ldx));
  if (handle->logger) { std::fprintf((FILE*)handle->logger, "TRSM-LEFT-%s [M=%d] [N=%d]\n", Complex ? "FP64-COMPLEX" : "FP64", rank, N - rank); }
  return hyh::ok() ? rank : 0;
}
