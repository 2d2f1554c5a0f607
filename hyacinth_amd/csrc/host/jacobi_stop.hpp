/*
 * jacobi_stop.hpp -- when the Jacobi sweeps of the SVD tail are done (host arithmetic only).
 *
 * The sweep kernels report how many pairs they rotated and the largest squared cosine they met.  The reference leaves the
 * iteration to cuSOLVER gesvdj with a fixed sweep budget (src/gram_evd.cu:9-42); here the host decides after every sweep.
 */
#pragma once
#include <algorithm>
#include <cmath>
#include <functional>
#include <vector>

namespace hyh {

/* rotations, cosine2: what the sweep just finished reported; lastCosine2: the largest squared cosine of the sweep before
 * it (0 for the first sweep); rotateAbove: the cosine below which a pair is left alone.
 * Done when nothing was rotated, or when every cosine the sweep met was within 8 thresholds (rotating such pairs moves the
 * other cosines by products of two of them, so a further sweep would only confirm), or when the quadratic phase makes the
 * confirming sweep superfluous: c_k / c_{k-1}^2 measures the constant of the contraction as it is on this matrix (clusters
 * of singular values make it larger); if it is at most 16 and, applied once more, puts the cosines this sweep has left
 * behind (constant x c_k^2) within the same 8 thresholds, the columns are there already. */
inline bool jacobi_sweeps_done(int rotations, double cosine2, double lastCosine2, double rotateAbove) {
  if (rotations == 0 || cosine2 <= 64. * rotateAbove * rotateAbove) { return true; }
  if (lastCosine2 > 0. && cosine2 > 0.) {
    const double contraction = std::max(1., std::sqrt(cosine2) / lastCosine2);
    if (contraction <= 16. && contraction * cosine2 <= 8. * rotateAbove) { return true; }
  }
  return false;
}

/* A second way for the sweeps to end: what is handed out has stopped moving.
 * Only the `kept` largest singular values and their vectors leave the library (K of them at most, and none below the rank
 * cut), the values to an absolute accuracy of a few eps sigma_max and the vectors through the projection residual
 * |A - A V V^H|, whose square is at most the sum of the squared norms of the columns that are not handed out, whatever
 * state those are in (the columns of B stay an orthogonal transform of the factor).  A cyclic sweep changes a column's squared
 * norm by the sum of the eigenvalue shifts of its 2 x 2 rotations, which is, to first order, how far that norm still is from
 * its singular value squared.  So the iteration may end after a sweep in which
 *   (i)  no kept value moved by more than eps sigma_max / 4, and
 *   (ii) the kept columns gained at most 1 / 32 of what is left outside them (the residual bound has stopped improving).
 * (i) also counts as met one sweep early when the iteration is visibly in its fast phase: lastMoved is what the kept values
 * moved by in the sweep before (0: unknown); if this sweep's move is at most 1 / 64 of it and, shrunk once more by no more
 * than the same ratio (the method contracts faster from sweep to sweep there, so this overstates the next move: by two
 * orders of magnitude where it was watched), stays within the same eps sigma_max / 4, the sweep that would only confirm it
 * is not run: the values are already as far from their
 * limits as that next move.
 * A noise floor of hundreds of nearly equal small columns, which a cyclic Jacobi method needs ten and more sweeps to resolve
 * and which is never handed out, then no longer decides when the sweeps end.  With nothing left outside (kept = all columns
 * and a zero cut) rule (ii) never holds and the rules above decide alone.
 * before / after: the column norms (not squared) at the start and at the end of the sweep, in the same column order.
 * seen (optional): { largest move of a kept value, what the kept columns gained, what is left outside } for the log. */
inline bool jacobi_output_settled(const std::vector<double>& before, const std::vector<double>& after, int kept, double eps, double* seen = nullptr, double lastMoved = 0.) {
  const size_t r = after.size(); if (before.size() != r || r == 0 || kept <= 0 || (size_t)kept >= r) { return false; }
  std::vector<double> a(before), b(after);
  std::sort(a.begin(), a.end(), std::greater<double>()); std::sort(b.begin(), b.end(), std::greater<double>());
  double moved = 0.; for (int i = 0; i < kept; ++i) { moved = std::max(moved, std::fabs(b[(size_t)i] - a[(size_t)i])); }
  double outsideBefore = 0., outsideAfter = 0.;   /* summed from the small end: no cancellation against the large values */
  for (size_t i = r; i-- > (size_t)kept;) { outsideBefore += a[i] * a[i]; outsideAfter += b[i] * b[i]; }
  const double gained = outsideBefore - outsideAfter;
  if (seen) { seen[0] = moved; seen[1] = gained; seen[2] = outsideAfter; }
  const bool still = moved <= 0.25 * eps * b[0] || (lastMoved > 0. && moved <= lastMoved / 64. && moved * (moved / lastMoved) <= 0.25 * eps * b[0]);
  return still && gained <= outsideAfter / 32.;
}

/* The columns whose pairs the caller waits for: one past the last index among the `kept` largest column norms.  Pairs of two
 * columns from there on are never handed out; what their cosines are says nothing about the vectors that are. */
inline int jacobi_head(const std::vector<double>& norm, int kept) {
  const int r = (int)norm.size(); if (kept <= 0 || kept >= r) { return r; }
  std::vector<double> v(norm); std::nth_element(v.begin(), v.begin() + (kept - 1), v.end(), std::greater<double>());
  const double nu = v[(size_t)(kept - 1)]; int head = 0;
  for (int i = 0; i < r; ++i) { if (norm[(size_t)i] >= nu) { head = i + 1; } }
  return head;
}

/* How many leading columns of B (rows of the Cholesky factor, in pivot order) the SVD needs when only the K largest values
 * and their vectors are handed out.  G = R^H R is the sum over the rows of R of their outer products, so leaving the rows
 * from t on out of the SVD takes a positive semidefinite matrix of trace tau_t = sum_{j >= t} |row j|^2 off G: no eigenvalue
 * moves up and none moves down by more than tau_t, hence 0 <= sigma_i - sigma'_i <= tau_t / (sigma_i + sigma'_i) <=
 * tau_t / (2 sigma'_i) for the values sigma' of the truncated factor.  With tau_t <= 4 eps sigma'_1 sigma'_K every value that
 * is handed out is within 2 eps sigma_1 of the true one (a fifth of the 10 eps sigma_1 the values are held to; the bound is
 * attained only when all the weight left out lies along the K-th vector), and the residual |A - A V V^H|^2, which depends on
 * the span of V alone, grows by at most tau_t (V spans the leading subspace of G - E with E positive semidefinite of trace
 * tau_t: tr((I - P) G) = tr((I - P)(G - E)) + tr((I - P) E) <= the optimum for G + tau_t).
 * jacobi_columns_needed guesses t from the column norms (largest norm for sigma_1, K-th largest norm for sigma_K, a quarter
 * of the bound for the guess: the norms of the columns are not the singular values; the K-th largest norm was 3.8 times the
 * K-th value on a dense spectrum with neighbours 1.8 % apart, which the quarter just covers; half the share takes twice the
 * rows of a broad floor back in, whose sweeps cost far more than an occasional second cut); jacobi_truncation_holds is the test with the values the sweeps
 * have found, and the caller takes columns back in when it fails.  A noise floor under the wanted
 * values, which costs a cyclic Jacobi method the most sweeps, and the graded columns beneath it are what this leaves out:
 * the work of a sweep goes with the square of the columns it takes. */
constexpr double kTruncationBudget = 4.;   /* tau_t <= kTruncationBudget eps sigma'_1 sigma'_K */
constexpr double kTruncationGuess = 0.25;  /* the share of it that the guess from the column norms may use */
inline int jacobi_columns_needed(const std::vector<double>& norm, int K, double eps) {
  const int r = (int)norm.size(); if (K < 1 || K >= r) { return r; }
  std::vector<double> v(norm); std::nth_element(v.begin(), v.begin() + (K - 1), v.end(), std::greater<double>());
  const double nuK = v[(size_t)(K - 1)], nu1 = *std::max_element(norm.begin(), norm.end()), bound = kTruncationGuess * kTruncationBudget * eps * nu1 * nuK;
  double sum = 0.; int t = r;
  while (t > K && sum + norm[(size_t)(t - 1)] * norm[(size_t)(t - 1)] <= bound) { sum += norm[(size_t)(t - 1)] * norm[(size_t)(t - 1)]; --t; }
  return t;
}
inline bool jacobi_truncation_holds(double dropped2, double sigma1, double sigmaK, double eps) { return dropped2 <= kTruncationBudget * eps * sigma1 * sigmaK; }

/* The same cut with the sharper of the two bounds.  What moves a singular value is the largest eigenvalue of what is taken off
 * G, not its trace (Weyl): 0 <= sigma_i^2 - sigma'_i^2 <= |E|_2, and |E|_2 = |R_d|_2^2 is the largest eigenvalue of the Gram
 * matrix M = B_d^H B_d of the columns left out.  For the rows of a noise floor (hundreds of rows of about equal norm pointing
 * in unrelated directions) that is a small fraction of the trace: d rows of squared norm w weigh d w, their largest
 * eigenvalue is about w (1 + sqrt(d / N))^2.  M is small (d x d) and cheap to form; its largest eigenvalue is bounded from
 * above by min(largest absolute row sum, Frobenius norm, trace), all three taken on the trailing block [t, r) for every t
 * in one pass from the back.  The residual |A - A V V^H|^2 still grows by up to the trace, so the trace must stay either
 * within the same budget as |E|_2 (the rule above, which needs nothing else) or within 1 / 64 of the squared residual itself
 * (the squared values that are not handed out): a residual 0.8 % larger.
 *
 * absGram: |M[i][j]| for the columns c0 .. r - 1 of B, d x d with d = r - c0, column-major; valueBudget bounds |E|_2,
 * residualBudget the trace where it exceeds valueBudget.  Returns the smallest t >= max(c0, K) whose trailing block passes
 * (r when none does); trace / spectral: the two figures of that block, for the test after the sweeps. */
struct JacobiCut { int cols; double trace, spectral; };
inline JacobiCut jacobi_columns_needed_spectral(const std::vector<double>& absGram, int r, int c0, int K, double valueBudget, double residualBudget) {
  JacobiCut cut{ r, 0., 0. }; const int d = r - c0; if (d <= 0 || absGram.size() < (size_t)d * (size_t)d) { return cut; }
  std::vector<double> rowSum((size_t)d, 0.); double frob2 = 0., trace = 0.;
  for (int t = r - 1; t >= std::max(c0, K); --t) {
    const int i = t - c0; double own = 0.;
    for (int j = i; j < d; ++j) { const double a = absGram[(size_t)i + (size_t)j * (size_t)d]; own += a; if (j > i) { rowSum[(size_t)j] += a; frob2 += 2. * a * a; } else { frob2 += a * a; trace += a; } }
    rowSum[(size_t)i] = own;
    double gersh = 0.; for (int j = i; j < d; ++j) { gersh = std::max(gersh, rowSum[(size_t)j]); }
    const double spectral = std::min(std::min(gersh, std::sqrt(frob2)), trace);
    if (!(spectral <= valueBudget && (trace <= valueBudget || trace <= residualBudget))) { break; }
    cut.cols = t; cut.trace = trace; cut.spectral = spectral;
  }
  return cut;
}
/* the test with the values found: sigma1, sigmaK as above, outside2 = the sum of the squared values found that are not handed out */
inline bool jacobi_truncation_holds_spectral(double trace, double spectral, double sigma1, double sigmaK, double outside2, double eps) {
  const double budget = kTruncationBudget * eps * sigma1 * sigmaK;
  return spectral <= budget && (trace <= budget || trace <= outside2 / 64.);
}

/* Columns a sweep may leave alone.  Let nu be the K-th largest column norm and b = max(nu^2, eps^2 sum of all squared norms).
 * The tail is the longest index range [top, r) whose squared norms sum to at most b / 1024; it is used only when it holds
 * at least half of the columns (a few large columns in front of a broad floor of small ones: a low-rank matrix plus noise),
 * else top = r.  Pairs of two tail columns are then never rotated.  Once the columns before `top` are orthogonal to all
 * others, the singular values are their norms together with the values of the tail block, and those are at most
 * sqrt(trace of its Gram matrix) <= max(nu, eps |B|_F) / 32, below everything that is handed out; the tail's share of
 * sum sigma^2 is the sum of its squared norms in whatever basis.  What rotations inside the tail would have removed from the
 * rows of a column p in front decays linearly, by about (tail sum) / |p|^2 per sweep: at most 1 / 1024 for the K columns
 * that are handed out.  norm: the r column norms (not squared) as they are now. */
inline int jacobi_tail_start(const std::vector<double>& norm, int K, double eps) {
  const int r = (int)norm.size(); if (r == 0 || K < 1 || K >= r) { return r; }
  double total = 0.; for (int i = r - 1; i >= 0; --i) { total += norm[(size_t)i] * norm[(size_t)i]; }
  std::vector<double> v(norm); std::nth_element(v.begin(), v.begin() + (K - 1), v.end(), std::greater<double>());
  const double nu2 = v[(size_t)(K - 1)] * v[(size_t)(K - 1)], bound = std::max(nu2, eps * eps * total) / 1024.;
  double sum = 0.; int t = r; while (t > 0 && sum + norm[(size_t)(t - 1)] * norm[(size_t)(t - 1)] <= bound) { sum += norm[(size_t)(t - 1)] * norm[(size_t)(t - 1)]; --t; }
  return 2 * t <= r ? t : r;
}

}  // namespace hyh
