/*
 * jacobi_stop.hpp -- when the Jacobi sweeps of the SVD tail are done (host arithmetic only).
 *
 * The sweep kernels report how many pairs they rotated and the largest squared cosine they met.  The reference leaves the
 * iteration to cuSOLVER gesvdj with a fixed sweep budget (src/gram_evd.cu:9-42); here the host decides after every sweep.
 */
#pragma once
#include <algorithm>
#include <cmath>

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

}  // namespace hyh
