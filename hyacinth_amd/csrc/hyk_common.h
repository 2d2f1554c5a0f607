/*
 * hyk_common.h -- integer building blocks shared by the HIP kernels.
 *
 * Everything here is exact integer arithmetic whose results are fixed by the
 * mathematics (and therefore equal to the reference's, whatever instruction
 * sequence produced them there):
 *   - fixed-point rounding  q = RNE(x * 2^e) of a binary float to a 96-bit
 *     two's-complement integer (reference: src/quantize_limbs.cu:14-27),
 *   - balanced base-256 digits (src/quantize_limbs.cu:29-44),
 *   - q mod m for the CRT moduli (src/quantize_crt_real.cu:30-35),
 *   - 192-bit accumulators and the 63-bit-limb encoding of the integer Gram
 *     (include/internal.hpp:116-159).
 * The functions are HYK_HD so a host compiler can run them too.
 */
#pragma once
#include <stdint.h>

#if defined(__HIPCC__) || defined(__HIP__)
#include <hip/hip_runtime.h>
#define HYK_HD __host__ __device__ __forceinline__
#else
#define HYK_HD static inline
#endif

#define HYK_INT_MAX 2147483647
#define HYK_INT_MIN (-2147483647 - 1)

/* precision enum values of include/hyacin.h */
enum { HYK_F64 = 0, HYK_F64C = 1, HYK_F32 = 2, HYK_F32C = 3, HYK_F16 = 4, HYK_F16C = 5, HYK_DD = 6, HYK_DDC = 7 };

namespace hyk {

/* ---------------------------------------------------------------- decomposed floats */
/* value = (-1)^neg * mant * 2^e2, mant < 2^53 */
struct Dec { uint64_t mant; int32_t e2; uint32_t neg; };

HYK_HD Dec decompose_f64(uint64_t bits) {
  Dec d; uint32_t E = (uint32_t)(bits >> 52) & 0x7ffu; uint64_t frac = bits & 0x000fffffffffffffull;
  d.neg = (uint32_t)(bits >> 63); d.mant = E ? (frac | 0x0010000000000000ull) : frac; d.e2 = (int32_t)(E ? E : 1u) - 1075; return d;
}
HYK_HD Dec decompose_f32(uint32_t bits) {
  Dec d; uint32_t E = (bits >> 23) & 0xffu, frac = bits & 0x007fffffu;
  d.neg = bits >> 31; d.mant = E ? (frac | 0x00800000u) : frac; d.e2 = (int32_t)(E ? E : 1u) - 150; return d;
}
HYK_HD Dec decompose_f16(uint32_t bits) {
  Dec d; uint32_t E = (bits >> 10) & 0x1fu, frac = bits & 0x3ffu;
  d.neg = (bits >> 15) & 1u; d.mant = E ? (frac | 0x400u) : frac; d.e2 = (int32_t)(E ? E : 1u) - 25; return d;
}

/* frexp exponent of |x| (x = f 2^e, f in [1/2, 1)) for a normal-or-larger value, HYK_INT_MAX below the
 * smallest normal of the storage type (reference: src/fp_exponent.cu:20-21; half is widened to float there,
 * so every non-zero half counts as normal) */
HYK_HD int32_t frexp_exp_f64(uint64_t absbits) { uint32_t E = (uint32_t)(absbits >> 52); return E ? (int32_t)E - 1022 : HYK_INT_MAX; }
HYK_HD int32_t frexp_exp_f32(uint32_t absbits) { uint32_t E = absbits >> 23; return E ? (int32_t)E - 126 : HYK_INT_MAX; }
HYK_HD int32_t frexp_exp_f16(uint32_t absbits) {
  if (!absbits) { return HYK_INT_MAX; } uint32_t E = absbits >> 10, frac = absbits & 0x3ffu;
  if (E) { return (int32_t)E - 14; }
  int32_t top = 31 - __builtin_clz(frac); /* subnormal half: value = frac 2^-24 */ return top - 24 + 1;
}

/* ---------------------------------------------------------------- 96-bit integers */
/* two's complement, little endian: value = lo + hi * 2^64 (hi sign-extended from 32 bits) */
struct I96 { uint64_t lo; uint32_t hi; };

HYK_HD I96 i96_neg(I96 a) { I96 r; r.lo = ~a.lo + 1ull; r.hi = ~a.hi + (uint32_t)(r.lo == 0ull); return r; }
HYK_HD I96 i96_add(I96 a, I96 b) { I96 r; r.lo = a.lo + b.lo; r.hi = a.hi + b.hi + (uint32_t)(r.lo < a.lo); return r; }

/* q = RNE(mant * 2^(e2 + expon)) with sign; |q| must stay below 2^95 (the planner keeps it below 2^82) */
HYK_HD I96 round_scaled(Dec d, int32_t expon) {
  I96 q; q.lo = 0ull; q.hi = 0u; if (!d.mant) { return q; }
  int64_t sh = (int64_t)d.e2 + (int64_t)expon;
  if (sh >= 0) {
    /* exact: the planner keeps |q| below 2^82, anything that would not fit 95 bits is cut at the top */
    const uint32_t s = sh > 95 ? 95u : (uint32_t)sh;
    if (s == 0u) { q.lo = d.mant; } else if (s < 64u) { q.lo = d.mant << s; q.hi = (uint32_t)(d.mant >> (64u - s)); } else { q.hi = (uint32_t)(d.mant << (s - 64u)); }
  } else {
    uint64_t r = (uint64_t)(-sh);
    if (r <= 54ull) {
      uint64_t fl = d.mant >> r, rem = d.mant & ((1ull << r) - 1ull), half = 1ull << (r - 1ull);
      q.lo = fl + (uint64_t)((rem > half) || (rem == half && (fl & 1ull)));
    }
  }
  return d.neg ? i96_neg(q) : q;
}

/* ---------------------------------------------------------------- modular reduction */
HYK_HD constexpr uint32_t pow2_mod(uint32_t k, uint32_t m) { uint32_t r = 1u % m; for (uint32_t i = 0; i < k; ++i) { r = (r * 2u) % m; } return r; }
HYK_HD uint32_t umulhi32(uint32_t a, uint32_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __umulhi(a, b);
#else
  return (uint32_t)(((uint64_t)a * b) >> 32);
#endif
}

/* canonical x mod m for any 32-bit x */
HYK_HD uint32_t reduce_u32(uint32_t x, uint32_t m, uint32_t d) { x -= umulhi32(x, d) * m; uint32_t y = x - m; return y < x ? y : x; }
/* canonical residue of a signed 32-bit value */
HYK_HD uint32_t reduce_i32(int32_t v, uint32_t m, uint32_t d, uint32_t c32) {
  uint32_t r = reduce_u32((uint32_t)v, m, d); if (v < 0) { r = (r >= c32) ? (r - c32) : (r + m - c32); } return r;
}

/* ---------------------------------------------------------------- residues through byte dot products
 * For a modulus m <= 256 every power 2^(8 i) mod m fits a byte, so the residue of a multi-byte non-negative integer is
 * the dot product of its bytes with those constants, reduced once more.  A signed q is first biased by 2^(32 DOTS - 1)
 * (a flip of the top bit of its DOTS-dword two's complement), which makes it non-negative; the bias and the centring of
 * the stored value are folded into one constant addend. */
struct DotMod { uint32_t m; uint32_t cv[3]; float inv, halfInv; uint32_t bias[3]; };   /* bias[d - 1] = -2^(32 d - 1) mod m */

HYK_HD constexpr uint32_t pack_pow2(uint32_t first, uint32_t m) {
  return pow2_mod(first, m) | (pow2_mod(first + 8, m) << 8) | (pow2_mod(first + 16, m) << 16) | (pow2_mod(first + 24, m) << 24);
}
HYK_HD constexpr DotMod make_dotmod(uint32_t m) {
  return DotMod{ m, { pack_pow2(0, m), pack_pow2(32, m), pack_pow2(64, m) }, 1.0f / (float)m, 0.5f / (float)m,
                 { (m - pow2_mod(31, m)) % m, (m - pow2_mod(63, m)) % m, (m - pow2_mod(95, m)) % m } };
}

/* sum of the four byte products + c */
HYK_HD uint32_t udot4(uint32_t a, uint32_t b, uint32_t c) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_udot4(a, b, c, false);
#else
  for (int i = 0; i < 4; ++i) { c += ((a >> (8 * i)) & 0xffu) * ((b >> (8 * i)) & 0xffu); } return c;
#endif
}

/* canonical t mod m for t < 2^20: the quotient comes from one float multiply-add; the half-unit offset keeps the product
 * at least 1/(2m) away from an integer, far more than the rounding error for t < 2^22, so truncation gives floor(t / m) */
HYK_HD uint32_t reduce_small(uint32_t t, const DotMod& k) {
  const uint32_t q = (uint32_t)((float)t * k.inv + k.halfInv); return t - q * k.m;
}

/* canonical (q + addend) mod m of a signed q with |q| < 2^(32 DOTS - 1); addend < 2^10 */
template <int DOTS> HYK_HD uint32_t residue_dot(I96 q, const DotMod& k, uint32_t addend) {
  const uint32_t w0 = (uint32_t)q.lo, w1 = (uint32_t)(q.lo >> 32), w2 = q.hi;
  uint32_t t = udot4(DOTS == 1 ? (w0 ^ 0x80000000u) : w0, k.cv[0], k.bias[DOTS - 1] + addend);
  if (DOTS > 1) { t = udot4(DOTS == 2 ? (w1 ^ 0x80000000u) : w1, k.cv[1], t); }
  if (DOTS > 2) { t = udot4(w2 ^ 0x80000000u, k.cv[2], t); }
  return reduce_small(t, k);
}

/* The int8 the reference stores for a canonical residue r: r itself up to 127, r - m above.  For any t congruent to r,
 * ((t + c) mod m) - c with c = max(m - 128, 0) is that value: it lies in [-c, m - 1 - c] = [128 - m, 127] (m > 128). */
HYK_HD constexpr uint32_t stored_centre(uint32_t m) { return m > 128u ? m - 128u : 0u; }
template <int DOTS> HYK_HD int32_t stored_residue_dot(I96 q, const DotMod& k) {
  return (int32_t)residue_dot<DOTS>(q, k, stored_centre(k.m)) - (int32_t)stored_centre(k.m);
}

/* ---------------------------------------------------------------- residues in double precision
 * For |a| < 2^51 the integer a is exact in a double and  a - m * rint((a - delta) / m)  is the representative of a mod m
 * in [delta - (m-1)/2, delta + (m-1)/2]: the quotient is computed with an error below 2^-10 while (a - delta) / m stays at
 * least 1/(2m) >= 2^-9 away from a rounding tie (m odd, or m = 256 with a half-integer delta), so rint never picks the
 * wrong neighbour, and the final multiply-add is exact.  Three full-rate FP64 instructions per residue. */
struct F64Mod { double inv, tieShift, negM; };   /* 1/m, -delta/m, -m */
HYK_HD constexpr double stored_delta(uint32_t m) { return (m > 128u ? 128.0 - (double)m : 0.0) + ((double)m - 1.0) * 0.5; }  /* range [128 - m, 127] or [0, m - 1] */
HYK_HD constexpr F64Mod make_f64mod(uint32_t m, double delta) { return F64Mod{ 1.0 / (double)m, -delta / (double)m, -(double)m }; }
HYK_HD double residue_f64(double a, const F64Mod& k) {
  const double quot = __builtin_rint(__builtin_fma(a, k.inv, k.tieShift));
  return __builtin_fma(k.negM, quot, a);
}

/* residue stored in int8: values above 127 wrap by -m (reference: src/quantize_crt_real.cu:33) */
HYK_HD int8_t residue_to_i8(uint32_t r, uint32_t m) { return (int8_t)(r > 127u ? r - m : r); }

/* ---------------------------------------------------------------- balanced base-256 digits */
/* byte l (0..11) of the two's-complement integer */
HYK_HD uint32_t i96_byte(I96 q, int l) { return l < 8 ? (uint32_t)(q.lo >> (8 * l)) & 0xffu : (q.hi >> (8 * (l - 8))) & 0xffu; }

/* ---------------------------------------------------------------- 192-bit accumulators */
struct I192 { uint64_t w[3]; };

HYK_HD uint64_t umulhi64(uint64_t a, uint64_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __umul64hi(a, b);
#else
  return (uint64_t)(((unsigned __int128)a * b) >> 64);
#endif
}

HYK_HD void i192_add(I192& a, const I192& b) {
  uint64_t s0 = a.w[0] + b.w[0], c0 = (uint64_t)(s0 < a.w[0]);
  uint64_t s1 = a.w[1] + b.w[1], c1 = (uint64_t)(s1 < a.w[1]); uint64_t s1c = s1 + c0; c1 += (uint64_t)(s1c < s1);
  a.w[0] = s0; a.w[1] = s1c; a.w[2] = a.w[2] + b.w[2] + c1;
}
HYK_HD I192 i192_neg(const I192& a) { I192 r; r.w[0] = ~a.w[0]; r.w[1] = ~a.w[1]; r.w[2] = ~a.w[2]; I192 one; one.w[0] = 1; one.w[1] = 0; one.w[2] = 0; i192_add(r, one); return r; }
HYK_HD bool i192_is_neg(const I192& a) { return (a.w[2] >> 63) != 0; }
/* non-negative b times small non-negative s (s < 2^32) */
HYK_HD I192 i192_mul_small(const I192& b, uint64_t s) {
  I192 r; r.w[0] = b.w[0] * s; uint64_t h0 = umulhi64(b.w[0], s); uint64_t l1 = b.w[1] * s, h1 = umulhi64(b.w[1], s);
  r.w[1] = l1 + h0; uint64_t c = (uint64_t)(r.w[1] < l1); r.w[2] = b.w[2] * s + h1 + c; return r;
}
/* a += v * 2^sh for a signed 64-bit v, 0 <= sh < 128 */
HYK_HD void i192_add_shifted_i64(I192& a, int64_t v, uint32_t sh) {
  uint64_t ext = (uint64_t)(v >> 63); I192 t; t.w[0] = (uint64_t)v; t.w[1] = ext; t.w[2] = ext;
  uint32_t ws = sh >> 6, bs = sh & 63u; I192 s;
  for (int i = 2; i >= 0; --i) {
    uint64_t hi = (i - (int)ws >= 0) ? t.w[i - ws] : 0ull, lo = (i - (int)ws - 1 >= 0) ? t.w[i - ws - 1] : 0ull;
    s.w[i] = bs ? ((hi << bs) | (lo >> (64u - bs))) : hi;
  }
  i192_add(a, s);
}

/* 63-bit-limb encoding (lower limbs in [0, 2^63), top limb two's complement) <-> 192-bit two's complement */
HYK_HD I192 limbs_to_i192(int L, const uint64_t* c, int64_t stride) {
  I192 r; const uint64_t M63 = 0x7fffffffffffffffull;
  if (L == 1) { uint64_t a = c[0]; uint64_t ext = (uint64_t)((int64_t)a >> 63); r.w[0] = a; r.w[1] = ext; r.w[2] = ext; }
  else if (L == 2) { uint64_t a0 = c[0] & M63, a1 = c[stride]; uint64_t ext = (uint64_t)((int64_t)a1 >> 63);
    r.w[0] = a0 | (a1 << 63); r.w[1] = (a1 >> 1) | (ext << 63); r.w[2] = ext; }
  else { uint64_t a0 = c[0] & M63, a1 = c[stride] & M63, a2 = c[2 * stride]; uint64_t ext = (uint64_t)((int64_t)a2 >> 63);
    r.w[0] = a0 | (a1 << 63); r.w[1] = (a1 >> 1) | (a2 << 62); r.w[2] = (a2 >> 2) | (ext << 62); }
  return r;
}
HYK_HD void i192_to_limbs(const I192& v, int L, uint64_t* c, int64_t stride) {
  const uint64_t M63 = 0x7fffffffffffffffull;
  if (L == 1) { c[0] = v.w[0]; }
  else if (L == 2) { c[0] = v.w[0] & M63; c[stride] = (v.w[0] >> 63) | (v.w[1] << 1); }
  else { c[0] = v.w[0] & M63; c[stride] = ((v.w[0] >> 63) | (v.w[1] << 1)) & M63; c[2 * stride] = (v.w[1] >> 62) | (v.w[2] << 2); }
}

HYK_HD int64_t tri_index(int64_t y, int64_t x) { return y + ((x * (x + 1)) >> 1); }

}  // namespace hyk
