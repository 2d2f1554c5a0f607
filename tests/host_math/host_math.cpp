/* Host build of the integer device helpers (hyk_common.h) so their arithmetic can be checked on a CPU
 * against the oracle before any kernel runs: rounding, balanced digits, residues, limb encoding. */
#include <cstring>
#include "hyk_common.h"
#include "crt_tables.h"
#include "host/jacobi_stop.hpp"

using namespace hyk;

static Dec dec_of(int type, const void* p, int64_t i, int part) {
  switch (type & ~1) {
    case HYK_F64: { uint64_t b; std::memcpy(&b, (const char*)p + (i * (1 + (type & 1)) + part) * 8, 8); return decompose_f64(b); }
    case HYK_F32: { uint32_t b; std::memcpy(&b, (const char*)p + (i * (1 + (type & 1)) + part) * 4, 4); return decompose_f32(b); }
    default: { uint16_t b; std::memcpy(&b, (const char*)p + (i * (1 + (type & 1)) + part) * 2, 2); return decompose_f16(b); }
  }
}

extern "C" {

/* out[i] = {lo64, hi32 sign-extended to 64} of RNE(x_i 2^expon) */
void hm_round(int type, const void* x, int64_t n, int32_t expon, int64_t* out) {
  for (int64_t i = 0; i < n; ++i) { I96 q = round_scaled(dec_of(type, x, i, 0), expon); out[2 * i] = (int64_t)q.lo; out[2 * i + 1] = (int64_t)(int32_t)q.hi; }
}

void hm_digits(int type, const void* x, int64_t n, int32_t expon, int order, int8_t* out) {
  for (int64_t i = 0; i < n; ++i) {
    I96 q = round_scaled(dec_of(type, x, i, 0), expon); uint32_t carry = 0;
    for (int l = 0; l < order; ++l) { uint32_t t = i96_byte(q, l) + carry; out[i * order + l] = (int8_t)(t & 0xffu); carry = (t >> 8) + ((t >> 7) & 1u); }
  }
}

void hm_residues(int cplxTable, int dots, int type, const void* x, int64_t n, int32_t expon, int order, int8_t* out) {
  for (int64_t i = 0; i < n; ++i) {
    I96 q = round_scaled(dec_of(type, x, i, 0), expon);
    for (int m = 0; m < order; ++m) {
      DotMod k = make_dotmod(cplxTable ? hyk_crt_cplx_mo[m] : hyk_crt_real_mo[m]);
      int32_t r = dots == 1 ? stored_residue_dot<1>(q, k) : dots == 2 ? stored_residue_dot<2>(q, k) : stored_residue_dot<3>(q, k);
      out[i * order + m] = (int8_t)r;
    }
  }
}

/* stored residue and canonical residue of the 96-bit two's complement {lo, hi} for one modulus */
void hm_residue_raw(uint64_t lo, uint32_t hi, int dots, uint32_t m, int32_t* stored, uint32_t* canonical) {
  I96 q; q.lo = lo; q.hi = hi; DotMod k = make_dotmod(m);
  *stored = dots == 1 ? stored_residue_dot<1>(q, k) : dots == 2 ? stored_residue_dot<2>(q, k) : stored_residue_dot<3>(q, k);
  *canonical = dots == 1 ? residue_dot<1>(q, k, 0u) : dots == 2 ? residue_dot<2>(q, k, 0u) : residue_dot<3>(q, k, 0u);
}

/* FP64 residue path: out[i] = representative of a_i mod m in the stored range (mode 0) or the symmetric one (mode 1) */
void hm_residue_f64(const double* a, int64_t n, uint32_t m, int mode, double* out) {
  F64Mod k = make_f64mod(m, mode ? 0.0 : stored_delta(m));
  for (int64_t i = 0; i < n; ++i) { out[i] = residue_f64(a[i], k); }
}

/* number of t in [0, limit) with reduce_small(t) != t mod m */
int64_t hm_reduce_small_errors(uint32_t m, uint32_t limit) {
  DotMod k = make_dotmod(m); int64_t bad = 0;
  for (uint32_t t = 0; t < limit; ++t) { bad += (reduce_small(t, k) != t % m); }
  return bad;
}

int32_t hm_frexp(int type, const void* x) {
  switch (type & ~1) {
    case HYK_F64: { uint64_t b; std::memcpy(&b, x, 8); return frexp_exp_f64(b & 0x7fffffffffffffffull); }
    case HYK_F32: { uint32_t b; std::memcpy(&b, x, 4); return frexp_exp_f32(b & 0x7fffffffu); }
    default: { uint16_t b; std::memcpy(&b, x, 2); return frexp_exp_f16(b & 0x7fffu); }
  }
}

/* limbs (L x 1, stride 1) -> 192-bit -> (+ v << sh) -> limbs */
void hm_limb_roundtrip(int L, const uint64_t* in, int64_t v, uint32_t sh, uint64_t* out, uint64_t* words) {
  I192 a = limbs_to_i192(L, in, 1); i192_add_shifted_i64(a, v, sh); i192_to_limbs(a, L, out, 1); words[0] = a.w[0]; words[1] = a.w[1]; words[2] = a.w[2];
}

int32_t hm_reduce_i32(int32_t v, uint32_t m) { return (int32_t)reduce_i32(v, m, (uint32_t)(0x100000000ull / m), (uint32_t)(0x100000000ull % m)); }

/* centred CRT lift as in the reconstruction kernel; residues canonical; returns three 64-bit words */
void hm_crt_lift(int cplxTable, int order, const uint32_t* residues, uint64_t* words) {
  I192 a; a.w[0] = a.w[1] = a.w[2] = 0;
  for (int x = 0; x < order; ++x) {
    const uint32_t m = cplxTable ? hyk_crt_cplx_mo[x] : hyk_crt_real_mo[x], d = (uint32_t)(0x100000000ull / m);
    const uint32_t minv = cplxTable ? hyk_crt_cplx_minv[order - 1][x] : hyk_crt_real_minv[order - 1][x];
    const uint32_t tt = reduce_u32(reduce_u32(residues[x], m, d) * minv, m, d);
    I192 pd; for (int k = 0; k < 3; ++k) { pd.w[k] = cplxTable ? hyk_crt_cplx_Pd[order - 1][x][k] : hyk_crt_real_Pd[order - 1][x][k]; }
    if (i192_is_neg(a)) { i192_add(a, i192_mul_small(pd, tt)); } else { i192_add(a, i192_neg(i192_mul_small(pd, m - tt))); }
  }
  I192 P; for (int k = 0; k < 3; ++k) { P.w[k] = cplxTable ? hyk_crt_cplx_P[order - 1][k] : hyk_crt_real_P[order - 1][k]; }
  if (i192_is_neg(a)) { i192_add(a, P); }
  I192 twice = a; i192_add(twice, a); I192 diff = twice; i192_add(diff, i192_neg(P));
  if (!i192_is_neg(diff)) { i192_add(a, i192_neg(P)); }
  words[0] = a.w[0]; words[1] = a.w[1]; words[2] = a.w[2];
}

/* the host's rule for ending the Jacobi sweeps of the SVD tail */
int hm_jacobi_done(int rotations, double cosine2, double lastCosine2, double rotateAbove) { return hyh::jacobi_sweeps_done(rotations, cosine2, lastCosine2, rotateAbove) ? 1 : 0; }
/* ... and for ending them when what is handed out has settled */
int hm_jacobi_tail_start(const double* norm, int r, int K, double eps) { return hyh::jacobi_tail_start(std::vector<double>(norm, norm + r), K, eps); }
int hm_jacobi_settled(const double* before, const double* after, int r, int kept, double eps) { return hyh::jacobi_output_settled(std::vector<double>(before, before + r), std::vector<double>(after, after + r), kept, eps) ? 1 : 0; }
int hm_jacobi_settled_after(const double* before, const double* after, int r, int kept, double eps, double lastMoved) { return hyh::jacobi_output_settled(std::vector<double>(before, before + r), std::vector<double>(after, after + r), kept, eps, nullptr, lastMoved) ? 1 : 0; }
int hm_jacobi_columns_needed(const double* norm, int r, int K, double eps) { return hyh::jacobi_columns_needed(std::vector<double>(norm, norm + r), K, eps); }
int hm_jacobi_truncation_holds(double dropped2, double sigma1, double sigmaK, double eps) { return hyh::jacobi_truncation_holds(dropped2, sigma1, sigmaK, eps) ? 1 : 0; }
int hm_jacobi_columns_needed_spectral(const double* absGram, int r, int c0, int K, double valueBudget, double residualBudget, double* traceOut, double* spectralOut) {
  const size_t d = (size_t)(r - c0); const hyh::JacobiCut c = hyh::jacobi_columns_needed_spectral(std::vector<double>(absGram, absGram + d * d), r, c0, K, valueBudget, residualBudget);
  *traceOut = c.trace; *spectralOut = c.spectral; return c.cols;
}
int hm_jacobi_truncation_holds_spectral(double trace, double spectral, double sigma1, double sigmaK, double outside2, double eps) { return hyh::jacobi_truncation_holds_spectral(trace, spectral, sigma1, sigmaK, outside2, eps) ? 1 : 0; }
int hm_jacobi_head(const double* norm, int r, int kept) { return hyh::jacobi_head(std::vector<double>(norm, norm + r), kept); }

}
