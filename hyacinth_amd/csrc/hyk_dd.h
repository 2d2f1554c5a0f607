/*
 * hyk_dd.h -- double-double arithmetic (a value is hi + lo with |lo| <= ulp(hi)/2).
 *
 * Used by the dequantizer and the pivoted Cholesky whenever the integer Gram
 * needs more than 52 bits (reference: the double2 overloads of
 * include/internal.hpp:181-214 and src/hyacin_potrfp.cu:5-63).  The error-free
 * transforms below are only exact without FP contraction and without fast-math:
 * every translation unit that includes this header is compiled with
 * -ffp-contract=off.
 */
#pragma once
#include "hyk_common.h"
#include <math.h>

namespace hyk {

struct dd_t { double x, y; };

HYK_HD void two_sum(double a, double b, double& s, double& e) { s = a + b; double bb = s - a; e = (a - (s - bb)) + (b - bb); }
HYK_HD dd_t dd_renorm(dd_t a) { double s = a.x + a.y; return dd_t{ s, a.y - (s - a.x) }; }   /* requires |a.x| >= |a.y| */
HYK_HD dd_t dd_neg(dd_t a) { return dd_t{ -a.x, -a.y }; }
HYK_HD dd_t dd_add(dd_t a, dd_t b) { double s, e; two_sum(a.x, b.x, s, e); return dd_renorm(dd_t{ s, e + (a.y + b.y) }); }
HYK_HD dd_t dd_sub(dd_t a, dd_t b) { return dd_add(a, dd_neg(b)); }
HYK_HD dd_t dd_mul(dd_t a, dd_t b) { double p = a.x * b.x, e = fma(a.x, b.x, -p); e += fma(a.x, b.y, a.y * b.x); return dd_renorm(dd_t{ p, e }); }
HYK_HD dd_t dd_mul_d(dd_t a, double b) { double p = a.x * b, e = fma(a.x, b, -p); e += a.y * b; return dd_renorm(dd_t{ p, e }); }
HYK_HD dd_t dd_sqr(dd_t a) { double p = a.x * a.x, e = fma(a.x, a.x, -p); e += 2.0 * (a.x * a.y); return dd_renorm(dd_t{ p, e }); }
HYK_HD bool dd_less(dd_t a, dd_t b) { return a.x < b.x || (a.x == b.x && a.y < b.y); }

/* r = 1/sqrt(a) to double-double accuracy (two Newton steps r <- r (3 - a r^2) / 2 from the FP64 seed); a > 0 */
HYK_HD dd_t dd_rsqrt(dd_t a) {
  dd_t r{ 1.0 / sqrt(a.x), 0.0 };
  for (int it = 0; it < 2; ++it) {
    dd_t h = dd_sub(dd_t{ 3.0, 0.0 }, dd_mul(a, dd_sqr(r)));
    r = dd_mul(r, dd_t{ 0.5 * h.x, 0.5 * h.y });
  }
  return r;
}

}  // namespace hyk
