/*
 * hyacin_oracle.c -- CPU restatement of the reference's quantized Gram path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing the library ships may call into this
 * file: it exists so that tests, the smoke check and the CPU-baseline leg of
 * the benchmark have an independent answer to compare the GPU against.
 *
 * Each function restates one piece of the reference (QxGbM/hyacinth) and
 * cites the file:line it follows.  The restatement keeps the reference's
 * arithmetic step by step (95-bit rounding, balanced base-256 digits, 3-word
 * modular split, Barrett / mulx reductions, 63-bit-limb add_shifted, the
 * sign-balanced CRT reconstruction); only the GPU launch structure is
 * replaced by loops.  What pins it: tests/test_oracle_*.py compare every
 * integer function with Python big-integer closed forms (exact rational
 * rounding, q mod m, sum(d_l 256^l), Q^H Q, CRT uniqueness), and the floating
 * point tail with numpy/scipy factorizations.
 *
 * Build: see oracle/Makefile (plain gcc, -ffp-contract=off so the error-free
 * transforms of the double-double code stay exact).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <limits.h>
#include <float.h>
#include <stdio.h>

#define HO_F64 0
#define HO_F64_COMPLEX 1
#define HO_F32 2
#define HO_F32_COMPLEX 3
#define HO_F16 4
#define HO_F16_COMPLEX 5
#define HO_DD 6
#define HO_DD_COMPLEX 7

typedef unsigned __int128 u128;
typedef __int128 i128;

static const uint64_t I63 = 0x7fffffffffffffffull;

/* ------------------------------------------------------------------ */
/* CRT tables: moduli are the reference's data (crt_constants.hpp:7,  */
/* :269-270); the derived constants are recomputed here with a small  */
/* 256-bit integer, following crt_constants.py:29-44,58-106.          */
/* ------------------------------------------------------------------ */
#define NREAL 24
#define NCPLX 25
#define NROT 20
static const uint32_t MO_REAL[NREAL] = { 256, 253, 251, 249, 247, 241, 239, 235, 233, 229, 227, 223, 217, 211, 199, 197, 193, 191, 181, 179, 173, 167, 163, 157 };
static const uint32_t MO_CPLX[NCPLX] = { 241, 233, 229, 221, 205, 197, 193, 181, 173, 157, 149, 137, 113, 109, 101, 97, 89, 73, 61, 53, 256, 253, 251, 249, 239 };
static const uint32_t IM_CPLX[NCPLX] = { 64, 89, 107, 21, 32, 14, 81, 19, 80, 28, 44, 37, 15, 33, 10, 22, 34, 27, 11, 23, 0, 0, 0, 0, 0 };

typedef struct { uint64_t w[4]; } big_t;
static big_t big_one(void) { big_t b = { { 1, 0, 0, 0 } }; return b; }
static big_t big_mul_small(big_t a, uint32_t m) { u128 c = 0; for (int i = 0; i < 4; ++i) { c += (u128)a.w[i] * m; a.w[i] = (uint64_t)c; c >>= 64; } return a; }
static big_t big_div_small(big_t a, uint32_t m, uint32_t* rem) { u128 r = 0; for (int i = 3; i >= 0; --i) { u128 cur = (r << 64) | a.w[i]; a.w[i] = (uint64_t)(cur / m); r = cur % m; } if (rem) { *rem = (uint32_t)r; } return a; }
static int big_bits(big_t a) { for (int i = 3; i >= 0; --i) if (a.w[i]) { return 64 * i + 64 - __builtin_clzll(a.w[i]); } return 0; }
static uint64_t big_extract(big_t a, int pos, int len) { /* bits [pos, pos+len) */
  uint64_t r = 0; for (int b = 0; b < len; ++b) { int p = pos + b; if (p < 256 && ((a.w[p >> 6] >> (p & 63)) & 1)) { r |= (uint64_t)1 << b; } } return r; }

typedef struct {
  int count, rot;
  uint32_t mo[NCPLX], range[NCPLX], rem_e32[NCPLX], rem_e63[NCPLX], im[NCPLX], im_inv[NCPLX];
  uint32_t minv[NCPLX + 1][NCPLX];   /* [n][x], n = number of moduli in use */
  int64_t p[NCPLX + 1][3];           /* P in 63-bit limbs */
  int64_t pd[NCPLX + 1][NCPLX * 4];  /* P/m_x in 55-bit limbs */
} crt_table_t;

static crt_table_t TAB_REAL, TAB_CPLX;
static int tables_ready = 0;

static uint32_t inv_mod(uint32_t a, uint32_t m) { if (m == 1) { return 0; } a %= m; for (uint32_t x = 1; x < m; ++x) if ((a * x) % m == 1) { return x; } return 0; }
static uint32_t pow2_mod(int e, uint32_t m) { uint32_t r = 1 % m; for (int i = 0; i < e; ++i) { r = (r * 2) % m; } return r; }

static void build_table(crt_table_t* t, const uint32_t* mo, const uint32_t* im, int count, int rot) {
  memset(t, 0, sizeof(*t)); t->count = count; t->rot = rot;
  for (int x = 0; x < count; ++x) {
    t->mo[x] = mo[x]; t->rem_e32[x] = pow2_mod(32, mo[x]); t->rem_e63[x] = pow2_mod(63, mo[x]);
    t->im[x] = im ? im[x] : 0; t->im_inv[x] = (im && im[x]) ? inv_mod(2 * im[x], mo[x]) : 0;
  }
  for (int n = 1; n <= count; ++n) {
    big_t P = big_one(); for (int x = 0; x < n; ++x) { P = big_mul_small(P, mo[x]); }
    t->range[n - 1] = (uint32_t)(big_bits(P) - 1);
    for (int k = 0; k < 3; ++k) { t->p[n][k] = (int64_t)big_extract(P, 63 * k, 63); }
    for (int x = 0; x < n; ++x) {
      uint32_t rem; big_t Pd = big_div_small(P, mo[x], &rem), tmp; uint32_t pdm; tmp = big_div_small(Pd, mo[x], &pdm); (void)tmp;
      t->minv[n][x] = inv_mod(pdm, mo[x]);
      for (int k = 0; k < 4; ++k) { t->pd[n][4 * x + k] = (int64_t)big_extract(Pd, 55 * k, 55); }
    }
  }
}

static void ensure_tables(void) {
  if (!tables_ready) { build_table(&TAB_REAL, MO_REAL, NULL, NREAL, 0); build_table(&TAB_CPLX, MO_CPLX, IM_CPLX, NCPLX, NROT); tables_ready = 1; }
}

/* table accessors for the tests: which = 0 real, 1 complex */
int ho_table_count(int which) { ensure_tables(); return which ? NCPLX : NREAL; }
void ho_table_basic(int which, uint32_t* mo, uint32_t* range, uint32_t* rem_e32, uint32_t* rem_e63, uint32_t* im, uint32_t* im_inv) {
  ensure_tables(); const crt_table_t* t = which ? &TAB_CPLX : &TAB_REAL;
  for (int x = 0; x < t->count; ++x) { mo[x] = t->mo[x]; range[x] = t->range[x]; rem_e32[x] = t->rem_e32[x]; rem_e63[x] = t->rem_e63[x]; im[x] = t->im[x]; im_inv[x] = t->im_inv[x]; }
}
void ho_table_prefix(int which, int n, uint32_t* minv, int64_t* p, int64_t* pd) {
  ensure_tables(); const crt_table_t* t = which ? &TAB_CPLX : &TAB_REAL;
  for (int x = 0; x < n; ++x) { minv[x] = t->minv[n][x]; } for (int k = 0; k < 3; ++k) { p[k] = t->p[n][k]; } for (int k = 0; k < 4 * n; ++k) { pd[k] = t->pd[n][k]; }
}

/* ------------------------------------------------------------------ */
/* Planner (src/hyacin_herk.cpp:11-59)                                 */
/* ------------------------------------------------------------------ */
static const int32_t LIMBS_U_LIST[12] = { 7, 14, 22, 30, 38, 46, 54, 62, 70, 78, 86, 94 };
static int lower_bound_u32(const uint32_t* a, int n, int32_t v) { int i = 0; while (i < n && (int32_t)a[i] < v) { ++i; } return i; }
static int lower_bound_i32(const int32_t* a, int n, int32_t v) { int i = 0; while (i < n && a[i] < v) { ++i; } return i; }

/* src/hyacin_herk.cpp:11-43.  Returns (first, second) and updates *alg. */
void ho_gram_algorithm(char* alg, int32_t K, int32_t u, int32_t Complex, int32_t segmentK, double batch_penalty, int32_t* first, int32_t* second) {
  ensure_tables();
  const int32_t alignmentK = 127;
  u = u > 0 ? u : 0; K = K > 1 ? K : 1;
  int32_t kk = (0 < segmentK) ? (K < segmentK ? K : segmentK) : K;
  int32_t crt_bits = (u + u + 1) + (int32_t)ceil(log2((double)kk));
  int is_c = (*alg == 'C' || *alg == 'c'), is_l = (*alg == 'L' || *alg == 'l');
  const crt_table_t* t = Complex ? &TAB_CPLX : &TAB_REAL; int cnt = t->count;
  int32_t algnK = (K + alignmentK) & (~alignmentK);
  if (is_c) {
    *alg = 'C';
    if (crt_bits <= (int32_t)t->range[cnt - 1]) {
      int32_t o = 1 + lower_bound_u32(t->range, cnt, crt_bits), seg32 = segmentK << (t->range[o - 1] - crt_bits);
      *first = o; *second = algnK < seg32 ? algnK : seg32;
    } else { *first = 0; *second = 0; }
    return;
  }
  int32_t o_l = 1 + lower_bound_i32(LIMBS_U_LIST, 12, u);
  if (!is_l && 2 < o_l) {
    double cost_limbs = (batch_penalty * (double)o_l * 0.5) + (double)(((uint32_t)(o_l * (o_l - 1))) >> 1) + (double)(Complex ? o_l * o_l : 0);
    if (crt_bits <= (int32_t)t->range[cnt - 1]) {
      int32_t o = 1 + lower_bound_u32(t->range, cnt, crt_bits);
      double cost_crt = Complex ? batch_penalty * ((double)o + (double)((o - NROT) > 0 ? (o - NROT) : 0) * 0.5) : batch_penalty * (double)o * 0.5;
      if (cost_crt < cost_limbs) { int32_t seg32 = segmentK << (t->range[o - 1] - crt_bits); *alg = 'C'; *first = o; *second = algnK < seg32 ? algnK : seg32; return; }
    }
  }
  *alg = 'L'; *first = o_l; *second = LIMBS_U_LIST[(o_l > 12 ? 12 : o_l) - 1];
}

static const int32_t TYPE_MANTISSA[12] = { 52, 52, 23, 23, 10, 10, 105, 105, 71, 71, 95, 95 };
static int type_is_complex(int t) { return t & 1; }

/* src/hyacin_herk.cpp:45-59 */
void ho_herk_batch_init(int32_t corr, double eps, uint64_t M, int32_t N, int Atype, int32_t* uA, int32_t* cPanels, int32_t* lPanels, uint64_t* stride) {
  if (stride) { uint64_t n = (uint64_t)(N > 0 ? N : 0); *stride = (n * n + n) >> 1; }
  if (1 < M) { --M; M |= M >> 1; M |= M >> 2; M |= M >> 4; M |= M >> 8; M |= M >> 16; M |= M >> 32; ++M; } else { M = 1; }
  int exp_eps; double frac = frexp(fabs(eps), &exp_eps);
  int32_t u = (int32_t)(frac == 0.5) - exp_eps; if (u < 0) { u = 0; } if (u > TYPE_MANTISSA[Atype]) { u = TYPE_MANTISSA[Atype]; }
  int32_t Complex = type_is_complex(Atype), uc = corr + u; if (uc > 80) { uc = 80; } if (uc < -1) { uc = -1; }
  if (uA) { *uA = uc; } if (cPanels) { *cPanels = 1 + Complex; }
  if (lPanels) { int32_t b = (uc + Complex) * 2; if (b < 0) { b = 0; } *lPanels = (0 <= uc) ? ((63 + b + (int32_t)ceil(log2((double)M))) / 63) : 0; }
}

/* ------------------------------------------------------------------ */
/* Element access                                                      */
/* ------------------------------------------------------------------ */
static float half_to_float(uint16_t h) {
  uint32_t s = (uint32_t)(h >> 15) << 31, e = (h >> 10) & 0x1f, m = h & 0x3ff, bits;
  if (e == 0) { if (m == 0) { bits = s; } else { int sh = 0; while (!(m & 0x400)) { m <<= 1; ++sh; } m &= 0x3ff; bits = s | ((uint32_t)(127 - 15 - sh + 1) << 23) | (m << 13); } }
  else if (e == 31) { bits = s | 0x7f800000u | (m << 13); } else { bits = s | ((e + 112) << 23) | (m << 13); }
  float f; memcpy(&f, &bits, 4); return f;
}

/* real and imaginary part of element (k, j) widened to double; the flag says
 * whether the storage type is double (else float arithmetic in the reference) */
static void load_elem(int Atype, const void* A, int64_t idx, double* re, double* im) {
  switch (Atype) {
    case HO_F64: *re = ((const double*)A)[idx]; *im = 0.; break;
    case HO_F64_COMPLEX: *re = ((const double*)A)[2 * idx]; *im = ((const double*)A)[2 * idx + 1]; break;
    case HO_F32: *re = ((const float*)A)[idx]; *im = 0.; break;
    case HO_F32_COMPLEX: *re = ((const float*)A)[2 * idx]; *im = ((const float*)A)[2 * idx + 1]; break;
    case HO_F16: *re = half_to_float(((const uint16_t*)A)[idx]); *im = 0.; break;
    case HO_F16_COMPLEX: *re = half_to_float(((const uint16_t*)A)[2 * idx]); *im = half_to_float(((const uint16_t*)A)[2 * idx + 1]); break;
    default: *re = *im = 0.;
  }
}

/* ------------------------------------------------------------------ */
/* fp_exponent (src/fp_exponent.cu:20-76)                              */
/* ------------------------------------------------------------------ */
static int32_t float_frexp(double a, int is_double) { /* fp_exponent.cu:20-21 */
  if (is_double ? (a < DBL_MIN) : ((float)a < FLT_MIN)) { return INT_MAX; }
  int x; frexp(a, &x); return x;
}

/* fp_exponent.cu:45-51.  vexp has (batches + 1) * N entries. */
void ho_quantize_scale_batch(int32_t batches, int32_t segM, int32_t lastM, int32_t N, int Atype, const void* A, int64_t lda, int32_t u, int32_t* vexp) {
  if (N <= 0) { return; }
  if (batches <= 0 || u < 0) { for (int32_t j = 0; j < N; ++j) { vexp[j] = INT_MAX; } return; }
  int is_double = (Atype == HO_F64 || Atype == HO_F64_COMPLEX);
  #pragma omp parallel for collapse(2) schedule(static)
  for (int32_t b = 0; b < batches; ++b) for (int32_t j = 0; j < N; ++j) {
    int32_t M = (b + 1 == batches) ? lastM : segM; double mx = 0.;
    for (int32_t i = 0; i < M; ++i) { double re, im; load_elem(Atype, A, (int64_t)b * segM + i + (int64_t)j * lda, &re, &im); re = fabs(re); im = fabs(im); mx = fmax(mx, fmax(re, im)); }
    int32_t e = float_frexp(mx, is_double); vexp[(int64_t)(1 + b) * N + j] = (e == INT_MAX) ? INT_MAX : (u - e);
  }
  for (int32_t j = 0; j < N; ++j) { int32_t m = vexp[(int64_t)N + j]; for (int32_t b = 1; b < batches; ++b) { int32_t v = vexp[(int64_t)(1 + b) * N + j]; m = v < m ? v : m; } vexp[j] = m; }
}

/* fp_exponent.cu:67-76 */
void ho_vector_range(int32_t batches, int32_t N, int32_t u, const int32_t* vexp, int32_t* segU) {
  for (int32_t b = 0; b < batches; ++b) {
    int32_t t = INT_MIN; const int32_t* mexp = &vexp[(int64_t)(1 + b) * N];
    for (int32_t i = 0; i < N; ++i) { int32_t e = mexp[i]; if (e < INT_MAX) { int32_t d = vexp[i] - e; t = d > t ? d : t; } }
    segU[b] = (t == INT_MIN) ? INT_MIN : (u + t);
  }
}

/* ------------------------------------------------------------------ */
/* 95-bit rounding (src/quantize_limbs.cu:14-27)                       */
/* ------------------------------------------------------------------ */
static void round_i95(double x, int is_double, int32_t expon, uint64_t* lo, uint32_t* hi) {
  if (x == 0.) { *lo = 0; *hi = 0; return; } /* ilogb(0) = INT_MIN: on the GPU the shifts clamp and produce 0 */
  int64_t ie = (int64_t)ilogb(x) + (int64_t)expon - 62; uint32_t e = (uint32_t)(ie > 0 ? ie : 0);
  uint64_t i;
  if (is_double) { i = (uint64_t)llrint(scalbn(x, expon - (int32_t)e)); } else { i = (uint64_t)llrintf(scalbnf((float)x, expon - (int32_t)e)); }
  *lo = (i << e) & I63; *hi = ((-(uint32_t)(i >> 63)) << (1u + e)) | (uint32_t)(i >> (63u - e));
}

/* ------------------------------------------------------------------ */
/* quantize_limbs (src/quantize_limbs.cu:29-58)                        */
/* ------------------------------------------------------------------ */
static int8_t* quantize_i8_limbs(int order, uint64_t lo, uint32_t hi, int8_t* A, int64_t strideA) {
  uint32_t a = 0;
  for (int l = 0; l < order; ++l) {
    uint8_t byte;
    if (l < 7) { byte = (uint8_t)(lo >> (8 * l)); } else if (l == 7) { byte = (uint8_t)((hi << 7) | (uint32_t)(lo >> 56)); } else { byte = (uint8_t)(hi >> (1 + 8 * (l - 8))); }
    if (l == 0) { a = byte; } else { a = (a >> 8) + ((a >> 7) & 1u) + byte; }
    *A = (int8_t)a; A += strideA;
  }
  return A;
}

void ho_quantize_limbs(int32_t M, int32_t N, int32_t orderA, int Atype, const void* A, int64_t lda, const int32_t* vexp, int8_t* B, int64_t ldb) {
  int Complex = type_is_complex(Atype), is_double = (Atype == HO_F64 || Atype == HO_F64_COMPLEX); int64_t strideB = (int64_t)N * ldb;
  if (orderA < 1 || orderA > 12) { return; }
  #pragma omp parallel for schedule(static)
  for (int32_t j = 0; j < N; ++j) {
    int32_t expon = vexp[j];
    for (int32_t i = 0; i < M; ++i) {
      int8_t* b = &B[(int64_t)j * ldb + i];
      if (expon == INT_MAX) { for (int l = 0; l < orderA * (Complex ? 3 : 1); ++l) { b[l * strideB] = 0; } continue; }
      double re, im; load_elem(Atype, A, i + (int64_t)j * lda, &re, &im);
      if (Complex) {
        uint64_t rl_lo, im_lo; uint32_t rl_hi, im_hi; round_i95(re, is_double, expon, &rl_lo, &rl_hi); round_i95(im, is_double, expon, &im_lo, &im_hi);
        uint64_t lo = rl_lo + im_lo; uint32_t hi = rl_hi + im_hi + (uint32_t)(lo >> 63); lo &= I63;
        b = quantize_i8_limbs(orderA, lo, hi, b, strideB); b = quantize_i8_limbs(orderA, rl_lo, rl_hi, b, strideB); quantize_i8_limbs(orderA, im_lo, im_hi, b, strideB);
      } else { uint64_t lo; uint32_t hi; round_i95(re, is_double, expon, &lo, &hi); quantize_i8_limbs(orderA, lo, hi, b, strideB); }
    }
  }
}

/* ------------------------------------------------------------------ */
/* Modular helpers (include/internal.hpp:161-179)                      */
/* ------------------------------------------------------------------ */
static uint32_t barrett_reduc(uint32_t DIV, uint32_t x) {
  if (!DIV) { return 0; }
  uint32_t d = (uint32_t)(0x100000000ull / (uint64_t)DIV), minus_div = (uint32_t)(-(int32_t)DIV);
  x += (uint32_t)(((uint64_t)x * d) >> 32) * minus_div; uint32_t y = minus_div + x; return y < x ? y : x;
}
static uint32_t mulx_reduc(int sign, uint32_t MUL, uint32_t DIV, uint32_t x) {
  if (!(MUL && DIV)) { return 0; }
  uint32_t mul = MUL % DIV, mul_r16 = (mul << 16) % DIV, mul_x;
  mul_x = (mul_r16 * (x >> 16)) + (mul * (x & 0xffffu));
  if (sign) { uint32_t mul_r32 = ((DIV - mul_r16) << 16) % DIV; return mul_x + ((-(x >> 31)) & mul_r32); }
  return mul_x;
}
static int8_t to_i8(uint32_t r, uint32_t m) { return (int8_t)(r + ((127u < r) ? (uint32_t)(-(int32_t)m) : 0u)); }

/* ------------------------------------------------------------------ */
/* quantize_crt real (src/quantize_crt_real.cu:15-67)                  */
/* quantize_crt complex (src/quantize_crt_complex.cu:15-77)            */
/* ------------------------------------------------------------------ */
typedef struct { uint32_t x, y, z; } u3_t;
static u3_t round_i95_u3(double v, int is_double, int32_t expon) {
  uint64_t lo; uint32_t hi; round_i95(v, is_double, expon, &lo, &hi);
  u3_t r = { (uint32_t)lo, (uint32_t)(lo >> 32) & 0x7fffffffu, hi }; return r;
}

void ho_quantize_crt(int32_t M, int32_t N, int32_t orderA, int Atype, const void* A, int64_t lda, const int32_t* vexp, int8_t* B, int64_t ldb) {
  ensure_tables();
  int Complex = type_is_complex(Atype), is_double = (Atype == HO_F64 || Atype == HO_F64_COMPLEX); int64_t strideB = (int64_t)N * ldb;
  const crt_table_t* t = Complex ? &TAB_CPLX : &TAB_REAL; if (orderA < 1 || orderA > t->count) { return; }
  int cols = Complex ? (orderA <= NROT ? orderA * 2 : orderA * 3 - NROT) : orderA;
  #pragma omp parallel for schedule(static)
  for (int32_t j = 0; j < N; ++j) {
    int32_t expon = vexp[j];
    for (int32_t i = 0; i < M; ++i) {
      int8_t* b = &B[(int64_t)j * ldb + i];
      if (expon == INT_MAX) { for (int l = 0; l < cols; ++l) { b[l * strideB] = 0; } continue; }
      double re, im; load_elem(Atype, A, i + (int64_t)j * lda, &re, &im);
      u3_t rl = round_i95_u3(re, is_double, expon), ig = round_i95_u3(im, is_double, expon);
      for (int x = 0; x < orderA; ++x) {
        uint32_t MO = t->mo[x], R32 = t->rem_e32[x], R63 = t->rem_e63[x];
        uint32_t r = mulx_reduc(0, 1, MO, rl.x) + mulx_reduc(0, R32, MO, rl.y) + mulx_reduc(1, R63, MO, rl.z);
        if (!Complex) { r = barrett_reduc(MO, r); *b = to_i8(r, MO); b += strideB; continue; }
        uint32_t ii = mulx_reduc(0, 1, MO, ig.x) + mulx_reduc(0, R32, MO, ig.y) + mulx_reduc(1, R63, MO, ig.z);
        if (x < NROT) {
          uint32_t IM = t->im[x];
          uint32_t p = barrett_reduc(MO, r + mulx_reduc(0, MO - IM, MO, ii)), q = barrett_reduc(MO, r + mulx_reduc(0, IM, MO, ii));
          *b = to_i8(p, MO); b += strideB; *b = to_i8(q, MO); b += strideB;
        } else {
          r = barrett_reduc(MO, r); ii = barrett_reduc(MO, ii); uint32_t s = r + ii, s2 = s - MO; s = s2 < s ? s2 : s;
          *b = to_i8(s, MO); b += strideB; *b = to_i8(r, MO); b += strideB; *b = to_i8(ii, MO); b += strideB;
        }
      }
    }
  }
}

/* ------------------------------------------------------------------ */
/* int8 GEMM with int32 accumulation, "TN": W[i + j*ldw] = sum_k       */
/* A[k + i*lda] * B[k + j*ldb]  (cuBLAS call sites hyacin_herk.cpp:65, */
/* 99-107).  upper != 0 computes only i <= j.                          */
/* ------------------------------------------------------------------ */
static int32_t dot_i8(const int8_t* a, const int8_t* b, int32_t K) { int32_t s = 0; for (int32_t k = 0; k < K; ++k) { s += (int32_t)a[k] * (int32_t)b[k]; } return s; }
static void gemm_tn_i8(int upper, int32_t Mo, int32_t No, int32_t K, const int8_t* A, int64_t lda, const int8_t* B, int64_t ldb, int32_t* W, int64_t ldw) {
  #pragma omp parallel for schedule(dynamic, 8)
  for (int32_t j = 0; j < No; ++j) { int32_t iend = upper ? (j + 1 < Mo ? j + 1 : Mo) : Mo; for (int32_t i = 0; i < iend; ++i) { W[i + j * ldw] = dot_i8(&A[i * lda], &B[j * ldb], K); } }
}

/* the K-chunk schedule of hyacin_herk.cpp:62-92,111-138 (limbs: tail in one piece if rem <= 130816)
 * and :163-189 (CRT: tail in one piece if rem <= 65536); calls fn(k0, klen, first) per chunk */
typedef void (*chunk_fn)(void* ctx, int32_t k0, int32_t klen, int first);
static void k_chunks(int32_t K, int crt_rule, chunk_fn fn, void* ctx) {
  const int32_t iter_k = 130816, iter_h = 65536;
  if (K <= iter_k) { fn(ctx, 0, K, 1); return; }
  int32_t rem_k = K % iter_k; rem_k = rem_k < iter_h ? (rem_k + iter_k) : rem_k; int32_t range_k = K - rem_k;
  for (int32_t k = 0; k < range_k; k += iter_k) { fn(ctx, k, iter_k, k == 0); }
  if (rem_k <= (crt_rule ? iter_h : iter_k)) { fn(ctx, range_k, rem_k, range_k == 0); }
  else { fn(ctx, range_k, iter_h, range_k == 0); fn(ctx, range_k + iter_h, rem_k - iter_h, 0); }
}

/* ------------------------------------------------------------------ */
/* 63-bit-limb integers (include/internal.hpp:116-159)                 */
/* ------------------------------------------------------------------ */
static void add_shifted(int L, uint64_t* a, uint32_t expon, int64_t i) {
  uint64_t ui = (uint64_t)i, sign = -(ui >> 63);
  if (L == 1) { if (expon == 0) { a[0] += ui; } else if (expon <= 63) { a[0] += ui << expon; } return; }
  if (L == 2) {
    if (expon == 0) { a[0] += ui & I63; a[1] += sign + (a[0] >> 63); a[0] &= I63; }
    else if (expon == 63) { a[1] += ui; }
    else if (expon < 63) { uint64_t q0 = ui << expon, q1 = (sign << (1 + expon)) | (ui >> (63 - expon)); a[0] += q0 & I63; a[1] += q1 + (a[0] >> 63); a[0] &= I63; }
    else if (expon <= 126) { a[1] += ui << (expon - 63); }
    return;
  }
  if (expon == 0) { a[0] += ui & I63; a[1] += (sign & I63) + (a[0] >> 63); a[0] &= I63; a[2] += sign + (a[1] >> 63); a[1] &= I63; }
  else if (expon == 63) { a[1] += ui & I63; a[2] += sign + (a[1] >> 63); a[1] &= I63; }
  else if (expon == 126) { a[2] += ui; }
  else if (expon < 63) { uint64_t q0 = ui << expon, q1 = (sign << (1 + expon)) | (ui >> (63 - expon)); a[0] += q0 & I63; a[1] += (q1 & I63) + (a[0] >> 63); a[0] &= I63; a[2] += sign + (a[1] >> 63); a[1] &= I63; }
  else if (expon < 126) { uint32_t ls = expon - 63; uint64_t q0 = ui << ls, q1 = (sign << (1 + ls)) | (ui >> (126 - expon)); a[1] += q0 & I63; a[2] += q1 + (a[1] >> 63); a[1] &= I63; }
  else if (expon <= 189) { a[2] += ui << (expon - 126); }
}

static int64_t tri_index(int64_t y, int64_t x) { return y + ((x + 1) * x) / 2; }

/* ------------------------------------------------------------------ */
/* limb Gram: i8herk_limbs (src/hyacin_herk.cpp:140-161) with the      */
/* accumulate kernels of limbs_diag.cu:4-41, limbs_cross_real.cu:4-42, */
/* limbs_cross_imag.cu:4-46                                            */
/* ------------------------------------------------------------------ */
typedef struct { int32_t N, algnN, K, orderA, orderC, beta, sft, mode; const int8_t* A, *AT; uint64_t* C; int32_t* W; int64_t strideC; } limb_ctx_t;

static void load_c(int L, const uint64_t* C, int64_t stride, uint64_t* a) { for (int l = 0; l < L; ++l) { a[l] = C[l * stride]; } }
static void store_c(int L, uint64_t* C, int64_t stride, const uint64_t* a) { for (int l = 0; l < L; ++l) { C[l * stride] = a[l]; } }

static void limb_diag_chunk(void* vctx, int32_t k0, int32_t klen, int first) {
  limb_ctx_t* c = (limb_ctx_t*)vctx; int64_t strideA = (int64_t)c->N * c->K, strideW = (int64_t)c->algnN * c->algnN; int beta = first ? c->beta : 1;
  for (int l = 0; l < c->orderA; ++l) { gemm_tn_i8(1, c->N, c->N, klen, &c->A[l * strideA + k0], c->K, &c->A[l * strideA + k0], c->K, &c->W[l * strideW], c->algnN); }
  #pragma omp parallel for schedule(dynamic, 8)
  for (int32_t x = 0; x < c->N; ++x) for (int32_t y = 0; y <= x; ++y) {
    uint64_t a[3] = { 0, 0, 0 }; uint64_t* Cp = &c->C[tri_index(y, x)]; if (beta) { load_c(c->orderC, Cp, c->strideC, a); }
    for (int l = 0; l < c->orderA; ++l) { add_shifted(c->orderC, a, 16u * l, (int64_t)c->W[y + (int64_t)x * c->algnN + l * strideW]); }
    store_c(c->orderC, Cp, c->strideC, a);
  }
}

static void limb_cross_chunk(void* vctx, int32_t k0, int32_t klen, int first) {
  limb_ctx_t* c = (limb_ctx_t*)vctx; int64_t strideX = (int64_t)c->algnN * c->N; int beta = first ? c->beta : 1;
  /* W = AT^T [A_0 .. A_{orderA-1}]: algnN x (N*orderA), ld algnN */
  gemm_tn_i8(0, c->N, c->N * c->orderA, klen, &c->AT[k0], c->K, &c->A[k0], c->K, c->W, c->algnN);
  #pragma omp parallel for schedule(dynamic, 8)
  for (int32_t x = 0; x < c->N; ++x) for (int32_t y = 0; y <= x; ++y) {
    uint64_t* Cp = &c->C[tri_index(y, x)];
    if (c->mode == 'R') {
      uint64_t a[3] = { 0, 0, 0 }; if (beta) { load_c(c->orderC, Cp, c->strideC, a); }
      for (int l = 0; l < c->orderA; ++l) { add_shifted(c->orderC, a, (uint32_t)(c->sft + 8 * l), (int64_t)c->W[y + (int64_t)x * c->algnN + l * strideX]); }
      for (int l = 0; l < c->orderA; ++l) { add_shifted(c->orderC, a, (uint32_t)(c->sft + 8 * l), (int64_t)c->W[x + (int64_t)y * c->algnN + l * strideX]); }
      store_c(c->orderC, Cp, c->strideC, a);
    } else {
      uint64_t r[3] = { 0, 0, 0 }, im[3] = { 0, 0, 0 }; uint64_t* Ci = Cp + c->orderC * c->strideC;
      load_c(c->orderC, Cp, c->strideC, r); if (beta) { load_c(c->orderC, Ci, c->strideC, im); }
      for (int l = 0; l < c->orderA; ++l) { int32_t X = c->W[y + (int64_t)x * c->algnN + l * strideX]; add_shifted(c->orderC, r, (uint32_t)(c->sft + 8 * l), -(int64_t)X); add_shifted(c->orderC, im, (uint32_t)(c->sft + 8 * l), (int64_t)X); }
      for (int l = 0; l < c->orderA; ++l) { int32_t X = c->W[x + (int64_t)y * c->algnN + l * strideX]; add_shifted(c->orderC, r, (uint32_t)(c->sft + 8 * l), -(int64_t)X); add_shifted(c->orderC, im, (uint32_t)(c->sft + 8 * l), -(int64_t)X); }
      store_c(c->orderC, Cp, c->strideC, r); store_c(c->orderC, Ci, c->strideC, im);
    }
  }
}

/* A: int8 panels, ld K (rows already zero-padded to K), real: orderA panels; complex: 3*orderA */
static void i8herk_limbs(int Complex, int32_t N, int32_t orderA, const int8_t* A, int32_t K, int32_t beta, int32_t orderC, uint64_t* C) {
  int32_t algnN = (N + 63) & ~63; int64_t strideA = (int64_t)N * K;
  limb_ctx_t c; memset(&c, 0, sizeof(c)); c.N = N; c.algnN = algnN; c.K = K; c.orderA = orderA; c.orderC = orderC; c.C = C; c.strideC = ((int64_t)N * N + N) / 2;
  int64_t wlen = (int64_t)algnN * algnN * orderA; int64_t wlen2 = (int64_t)algnN * N * orderA; if (wlen2 > wlen) { wlen = wlen2; }
  c.W = (int32_t*)calloc((size_t)wlen, sizeof(int32_t));
  c.A = A; c.beta = beta; k_chunks(K, 0, limb_diag_chunk, &c);
  for (int32_t i = 1; i < orderA; ++i) { c.mode = 'R'; c.sft = i << 3; c.orderA = i; c.AT = &A[i * strideA]; c.A = A; c.beta = 1; k_chunks(K, 0, limb_cross_chunk, &c); }
  if (Complex) {
    const int8_t* R = &A[(int64_t)orderA * strideA], *I = &A[2 * (int64_t)orderA * strideA];
    for (int32_t i = 0; i < orderA; ++i) { c.mode = 'I'; c.sft = i << 3; c.orderA = orderA; c.AT = &R[i * strideA]; c.A = I; c.beta = beta || (0 < i); k_chunks(K, 0, limb_cross_chunk, &c); }
  }
  free(c.W);
}

/* ------------------------------------------------------------------ */
/* CRT Gram: i8herk_crt (src/hyacin_herk.cpp:163-281) with             */
/* crt_diag_real.cu:4-29, crt_rotate.cu:4-46, crt_extra_real.cu:4-22,  */
/* crt_extra_imag.cu:4-46 and the reconstruction of                    */
/* crt_reconstruct_real.cu:4-92 / crt_reconstruct_complex.cu:4-93      */
/* ------------------------------------------------------------------ */
typedef struct { int32_t N, algnN, K, orderA, phase; const int8_t* A; uint8_t* B; int32_t* W; int64_t strideB; } crt_ctx_t;
/* B: byte residues, plane x at B[x*strideB ..]; complex: real planes [0, o), imaginary planes [o, 2o) */

static void crt_real_chunk(void* vctx, int32_t k0, int32_t klen, int first) {
  crt_ctx_t* c = (crt_ctx_t*)vctx; int64_t strideA = (int64_t)c->N * c->K, strideW = (int64_t)c->algnN * c->algnN;
  for (int x = 0; x < c->orderA; ++x) { gemm_tn_i8(1, c->N, c->N, klen, &c->A[x * strideA + k0], c->K, &c->A[x * strideA + k0], c->K, &c->W[x * strideW], c->algnN); }
  #pragma omp parallel for schedule(dynamic, 8)
  for (int32_t x = 0; x < c->N; ++x) for (int32_t y = 0; y <= x; ++y) for (int m = 0; m < c->orderA; ++m) {
    uint32_t mo = TAB_REAL.mo[m]; uint8_t* b = &c->B[m * c->strideB + tri_index(y, x)]; uint32_t a = first ? 0u : *b;
    *b = (uint8_t)barrett_reduc(mo, a + mulx_reduc(1, 1, mo, (uint32_t)c->W[y + (int64_t)x * c->algnN + m * strideW]));
  }
}

static void crt_rotate_chunk(void* vctx, int32_t k0, int32_t klen, int first) {
  crt_ctx_t* c = (crt_ctx_t*)vctx; int64_t strideA = (int64_t)c->N * c->K, strideW = (int64_t)c->algnN * c->algnN; int len = c->orderA < NROT ? c->orderA : NROT;
  for (int x = 0; x < len; ++x) { gemm_tn_i8(0, c->N, c->N, klen, &c->A[(2 * x) * strideA + k0], c->K, &c->A[(2 * x + 1) * strideA + k0], c->K, &c->W[x * strideW], c->algnN); }
  #pragma omp parallel for schedule(dynamic, 8)
  for (int32_t x = 0; x < c->N; ++x) for (int32_t y = 0; y <= x; ++y) for (int m = 0; m < len; ++m) {
    uint32_t mo = TAB_CPLX.mo[m], minv = TAB_CPLX.im_inv[m], inv2 = (mo + 1) / 2;
    uint8_t* br = &c->B[m * c->strideB + tri_index(y, x)], *bi = br + c->orderA * c->strideB; uint32_t r = first ? 0u : *br, i = first ? 0u : *bi;
    uint32_t p = (uint32_t)c->W[y + (int64_t)x * c->algnN + m * strideW], q = (uint32_t)c->W[x + (int64_t)y * c->algnN + m * strideW];
    *br = (uint8_t)barrett_reduc(mo, r + mulx_reduc(1, inv2, mo, p) + mulx_reduc(1, inv2, mo, q));
    *bi = (uint8_t)barrett_reduc(mo, i + mulx_reduc(1, minv, mo, p) + mulx_reduc(1, mo - minv, mo, q));
  }
}

static void crt_extra_chunk(void* vctx, int32_t k0, int32_t klen, int first) {
  crt_ctx_t* c = (crt_ctx_t*)vctx; int64_t strideA = (int64_t)c->N * c->K, strideW = (int64_t)c->algnN * c->algnN; int len = c->orderA - NROT;
  const int8_t* Ae = &c->A[(int64_t)strideA * NROT * 2];
  if (c->phase == 'R') {
    for (int x = 0; x < len; ++x) { gemm_tn_i8(1, c->N, c->N, klen, &Ae[(3 * x) * strideA + k0], c->K, &Ae[(3 * x) * strideA + k0], c->K, &c->W[x * strideW], c->algnN); }
    #pragma omp parallel for schedule(dynamic, 8)
    for (int32_t x = 0; x < c->N; ++x) for (int32_t y = 0; y <= x; ++y) for (int m = 0; m < len; ++m) {
      uint32_t mo = TAB_CPLX.mo[NROT + m]; uint8_t* b = &c->B[(NROT + m) * c->strideB + tri_index(y, x)]; uint32_t a = first ? 0u : *b;
      *b = (uint8_t)barrett_reduc(mo, a + mulx_reduc(1, 1, mo, (uint32_t)c->W[y + (int64_t)x * c->algnN + m * strideW]));
    }
  } else {
    /* crt_cextra<'I'> is called with A advanced by one panel (hyacin_herk.cpp:265): A = real part, next panel = imaginary part */
    for (int x = 0; x < len; ++x) { gemm_tn_i8(0, c->N, c->N, klen, &Ae[(3 * x + 1) * strideA + k0], c->K, &Ae[(3 * x + 2) * strideA + k0], c->K, &c->W[x * strideW], c->algnN); }
    #pragma omp parallel for schedule(dynamic, 8)
    for (int32_t x = 0; x < c->N; ++x) for (int32_t y = 0; y <= x; ++y) for (int m = 0; m < len; ++m) {
      uint32_t mo = TAB_CPLX.mo[NROT + m], mul = mo - 1;
      uint8_t* br = &c->B[(NROT + m) * c->strideB + tri_index(y, x)], *bi = br + c->orderA * c->strideB; uint32_t r = *br, i = first ? 0u : *bi;
      uint32_t a0 = (uint32_t)c->W[y + (int64_t)x * c->algnN + m * strideW], a1 = (uint32_t)c->W[x + (int64_t)y * c->algnN + m * strideW];
      r = barrett_reduc(mo, r + mulx_reduc(1, mul, mo, a0)); i = barrett_reduc(mo, i + mulx_reduc(1, 1, mo, a0));
      r = barrett_reduc(mo, r + mulx_reduc(1, mul, mo, a1)); i = barrett_reduc(mo, i + mulx_reduc(1, mul, mo, a1));
      *br = (uint8_t)r; *bi = (uint8_t)i;
    }
  }
}

/* crt_reconstruct_real.cu:4-92 for one entry; res[x] canonical residues */
static void reconstruct_entry(const crt_table_t* t, int orderX, const uint8_t* res, int64_t stride_res, int beta, int orderA, uint64_t* out, int64_t stride_out) {
  const int64_t* p = t->p[orderX]; int orderP = (0 < p[0]) + (0 < p[1]) + (0 < p[2]), orderAcc = orderA < orderP ? orderP : orderA;
  uint64_t a[3] = { 0, 0, 0 }, neg[3];
  for (int x = 0; x < orderX; ++x) {
    uint32_t mo = t->mo[x], mask_sign = (uint32_t)(a[orderAcc - 1] >> 63) + 0xffffffffu;
    int32_t s = (int32_t)(barrett_reduc(mo, mulx_reduc(0, t->minv[orderX][x], mo, (uint32_t)res[x * stride_res])) - (mo & mask_sign));
    for (int k = 0; k < 4; ++k) { int64_t pd = t->pd[orderX][4 * x + k]; if (pd) { add_shifted(orderAcc, a, 55u * k, pd * (int64_t)s); } }
  }
  for (int k = 0; k < orderAcc; ++k) { neg[k] = a[k]; }
  if (a[orderAcc - 1] >> 63) { for (int k = 0; k < 3; ++k) if (p[k]) { add_shifted(orderAcc, a, 63u * k, p[k]); } }
  else { for (int k = 0; k < 3; ++k) if (p[k]) { add_shifted(orderAcc, neg, 63u * k, -p[k]); } }
  uint64_t sum = a[0] + neg[0]; for (int k = 1; k < orderAcc; ++k) { sum = (sum >> 63) + a[k] + neg[k]; }
  if (!(sum >> 63)) { for (int k = 0; k < orderAcc; ++k) { a[k] = neg[k]; } }
  if (beta) { for (int k = 0; k < orderA; ++k) { add_shifted(orderAcc, a, 63u * k, (int64_t)out[k * stride_out]); } }
  if (0 < orderA && orderA < orderAcc) { a[orderA - 1] |= a[orderAcc - 1] & 0x8000000000000000ull; }
  for (int k = 0; k < orderA; ++k) { out[k * stride_out] = a[k]; }
}

static void i8herk_crt(int Complex, int32_t N, int32_t orderA, const int8_t* A, int32_t K, int32_t beta, int32_t orderC, uint64_t* C) {
  ensure_tables();
  int32_t algnN = (N + 63) & ~63; int64_t strideB = ((int64_t)N * N + N) / 2;
  crt_ctx_t c; memset(&c, 0, sizeof(c)); c.N = N; c.algnN = algnN; c.K = K; c.orderA = orderA; c.A = A; c.strideB = strideB;
  int wl = Complex ? (orderA > NROT ? orderA : NROT) : orderA;
  c.W = (int32_t*)calloc((size_t)algnN * algnN * wl, sizeof(int32_t)); c.B = (uint8_t*)calloc((size_t)strideB * orderA * (Complex ? 2 : 1), 1);
  if (Complex) {
    k_chunks(K, 1, crt_rotate_chunk, &c);
    if (NROT < orderA) { c.phase = 'R'; k_chunks(K, 1, crt_extra_chunk, &c); c.phase = 'I'; k_chunks(K, 1, crt_extra_chunk, &c); }
    #pragma omp parallel for schedule(static)
    for (int64_t e = 0; e < strideB; ++e) for (int z = 0; z < 2; ++z)
    { reconstruct_entry(&TAB_CPLX, orderA, &c.B[z * orderA * strideB + e], strideB, beta, orderC, &C[z * orderC * strideB + e], strideB); }
  } else {
    k_chunks(K, 1, crt_real_chunk, &c);
    #pragma omp parallel for schedule(static)
    for (int64_t e = 0; e < strideB; ++e) { reconstruct_entry(&TAB_REAL, orderA, &c.B[e], strideB, beta, orderC, &C[e], strideB); }
  }
  free(c.W); free(c.B);
}

/* stand-alone entry points so tests can drive each stage on given int8 panels */
void ho_i8herk_limbs(int Complex, int32_t N, int32_t orderA, const int8_t* A, int32_t K, int32_t beta, int32_t orderC, uint64_t* C) { i8herk_limbs(Complex, N, orderA, A, K, beta, orderC, C); }
void ho_i8herk_crt(int Complex, int32_t N, int32_t orderA, const int8_t* A, int32_t K, int32_t beta, int32_t orderC, uint64_t* C) { i8herk_crt(Complex, N, orderA, A, K, beta, orderC, C); }
void ho_reconstruct(int Complex, int64_t count, int orderX, const uint8_t* res, int beta, int orderA, uint64_t* out) {
  ensure_tables(); for (int64_t e = 0; e < count; ++e) { reconstruct_entry(Complex ? &TAB_CPLX : &TAB_REAL, orderX, &res[e], count, beta, orderA, &out[e], count); }
}

/* ------------------------------------------------------------------ */
/* herk_dispatcher / herk_batch_dispatcher (hyacin_herk.cpp:283-384)   */
/* ------------------------------------------------------------------ */
typedef struct { char alg; double penalty; int32_t targetK; } plan_cfg_t;
static int elem_size(int Atype) { static const int s[6] = { 8, 16, 4, 8, 2, 4 }; return s[Atype]; }
static const void* elem_ptr(int Atype, const void* A, int64_t idx) { return (const char*)A + idx * elem_size(Atype); }
static int64_t c_len(int32_t N, int32_t orderC, int Complex) { return (((int64_t)N * N + N) / 2) * orderC * (Complex ? 2 : 1); }

static void herk_dispatcher(const plan_cfg_t* cfg, int32_t M, int32_t N, int Atype, const void* A, int64_t lda, int32_t u, const int32_t* vexp, int32_t beta, int32_t orderC, uint64_t* C) {
  int Complex = type_is_complex(Atype);
  if ((M <= 0 || u < 0) && beta == 0) { memset(C, 0, (size_t)c_len(N, orderC, Complex) * 8); return; }
  char alg = cfg->alg; int32_t orderA, second; ho_gram_algorithm(&alg, M, u + Complex, Complex, cfg->targetK, cfg->penalty, &orderA, &second);
  int32_t algnM = (M + 127) & ~127;
  if (alg == 'L') {
    int64_t strideA = (int64_t)algnM * N * orderA; int8_t* W = (int8_t*)calloc((size_t)(strideA * (Complex ? 3 : 1)), 1);
    ho_quantize_limbs(M, N, orderA, Atype, A, lda, vexp, W, algnM);
    i8herk_limbs(Complex, N, orderA, W, algnM, beta, orderC, C); free(W);
  } else {
    int32_t segM = second; int64_t panels = Complex ? (orderA * 2 + (orderA > NROT ? orderA - NROT : 0)) : orderA;
    int8_t* W = (int8_t*)malloc((size_t)((int64_t)segM * N * panels));
    for (int32_t y = 0; y < M; y += segM) {
      int32_t rows = (M - y) < segM ? (M - y) : segM; memset(W, 0, (size_t)((int64_t)segM * N * panels));
      ho_quantize_crt(rows, N, orderA, Atype, elem_ptr(Atype, A, y), lda, vexp, W, segM);
      i8herk_crt(Complex, N, orderA, W, segM, beta, orderC, C); beta = 1;
    }
    free(W);
  }
}

typedef struct { int32_t first, second; } pair_t;

static void herk_batch_dispatcher(const plan_cfg_t* cfg, int32_t batches, int32_t segM, int32_t lastM, int32_t N, int Atype, const void* A, int64_t lda, int32_t u, const int32_t* vexp, int32_t beta, int32_t orderC, uint64_t* C) {
  int Complex = type_is_complex(Atype);
  int32_t* segU = (int32_t*)malloc(sizeof(int32_t) * batches); ho_vector_range(batches, N, u + Complex, vexp, segU);
  int32_t u_floor = Complex, u_ceil = Complex + u, M = (batches - 1) * segM + lastM; pair_t limb_batches[16]; int nlb = 0;
  while (u_floor <= u_ceil) {
    char algo = cfg->alg; pair_t p; ho_gram_algorithm(&algo, M, u_floor, Complex, cfg->targetK, cfg->penalty, &p.first, &p.second);
    if (algo == 'L') { u_floor = 1 + p.second; limb_batches[nlb++] = p; } else { u_floor = 1 + u_ceil; }
  }
  int32_t* batchRows = (int32_t*)calloc(nlb + 2, sizeof(int32_t));
  for (int32_t i = 0; i < batches; ++i) {
    int32_t uc = segU[i]; if (0 <= uc) { int idx = 0; while (idx < nlb && !(uc <= limb_batches[idx].second)) { ++idx; } batchRows[idx] += (i + 1 == batches) ? lastM : segM; segU[i] = idx; } else { segU[i] = -1; }
  }
  int32_t ceil_batch_rows = batchRows[nlb]; char algo = cfg->alg; pair_t ceil_batch;
  ho_gram_algorithm(&algo, ceil_batch_rows, u_ceil, Complex, cfg->targetK, cfg->penalty, &ceil_batch.first, &ceil_batch.second);
  int n_limb_batches = nlb; if (algo == 'L') { limb_batches[n_limb_batches++] = ceil_batch; }
  for (int b = 0; b < n_limb_batches; ++b) if (0 < batchRows[b]) {
    int32_t orderA = limb_batches[b].first, algnM = (batchRows[b] + 127) & ~127; int64_t strideA = (int64_t)algnM * N * orderA;
    int8_t* W = (int8_t*)calloc((size_t)(strideA * (Complex ? 3 : 1)), 1); int32_t rowsW = 0, i = 0;
    while (i < batches && segU[i] != b) { ++i; }
    while (i < batches) {
      int32_t i_end = i; while (i_end < batches && segU[i_end] == b) { ++i_end; }
      int32_t rowsA = i * segM, rows = (M < i_end * segM ? M : i_end * segM) - rowsA;
      ho_quantize_limbs(rows, N, orderA, Atype, elem_ptr(Atype, A, rowsA), lda, vexp, &W[rowsW], algnM);
      rowsW += rows; i = i_end; while (i < batches && segU[i] != b) { ++i; }
    }
    i8herk_limbs(Complex, N, orderA, W, algnM, beta, orderC, C); beta = 1; free(W);
  }
  if (algo == 'C' && 0 < ceil_batch_rows) {
    /* the gather/flush loop of hyacin_herk.cpp:357-383: rows of the ceil bucket are packed into W and the CRT
     * Gram is flushed every algnM rows; the integer result equals one flush per algnM consecutive packed rows */
    int32_t orderA = ceil_batch.first, algnM = ceil_batch.second; int64_t panels = Complex ? (orderA * 2 + (orderA > NROT ? orderA - NROT : 0)) : orderA;
    int8_t* W = (int8_t*)calloc((size_t)((int64_t)algnM * N * panels), 1); int32_t rowsW = 0;
    for (int32_t i = 0; i < batches; ++i) if (segU[i] == n_limb_batches) {
      int32_t rowsA = i * segM, rows = (i + 1 == batches) ? lastM : segM;
      while (0 < rows) {
        int32_t take = (algnM - rowsW) < rows ? (algnM - rowsW) : rows;
        ho_quantize_crt(take, N, orderA, Atype, elem_ptr(Atype, A, rowsA), lda, vexp, &W[rowsW], algnM);
        rowsW += take; rowsA += take; rows -= take;
        if (rowsW == algnM) { i8herk_crt(Complex, N, orderA, W, algnM, beta, orderC, C); beta = 1; rowsW = 0; memset(W, 0, (size_t)((int64_t)algnM * N * panels)); }
      }
    }
    if (0 < rowsW) { i8herk_crt(Complex, N, orderA, W, algnM, beta, orderC, C); beta = 1; }
    free(W);
  }
  free(batchRows); free(segU);
}

/* src/hyacin_herk.cpp:386-407 */
void ho_herk_batch(char alg, double penalty, int32_t targetK, int32_t batches, int32_t segM, int32_t lastM, int32_t N, int Atype, const void* A, int64_t lda, int32_t u, const int32_t* vexp, int32_t beta, int32_t orderC, uint64_t* C) {
  if (N <= 0 || orderC <= 0 || Atype > HO_F16_COMPLEX) { return; }
  plan_cfg_t cfg = { alg, penalty, targetK };
  if (batches <= 1) { herk_dispatcher(&cfg, lastM, N, Atype, A, lda, u, vexp, beta, orderC, C); } else { herk_batch_dispatcher(&cfg, batches, segM, lastM, N, Atype, A, lda, u, vexp, beta, orderC, C); }
}

/* ------------------------------------------------------------------ */
/* Dequantize (src/fp_i63tp_dequantize.cu)                             */
/* ------------------------------------------------------------------ */
static int clz64(uint64_t x) { return x ? __builtin_clzll(x) : 64; }
static int32_t iexp(int orderA, const uint64_t* A, int64_t strideA) { /* :6-11 */
  int32_t e = 64 - clz64(A[0]);
  if (1 < orderA) { int32_t n = 127 - clz64(A[strideA]); e = 63 < n ? n : e; }
  if (2 < orderA) { int32_t n = 190 - clz64(A[2 * strideA]); e = 126 < n ? n : e; }
  return e;
}

/* :17-54; returns the bit length the type choice is based on */
int32_t ho_dequantize_init(int32_t corr, int32_t f64_capable, int32_t N, int32_t orderC, const uint64_t* C, const int32_t* vexp, int Atype, int* Gtype, int32_t* gElemBytes) {
  static const int32_t type_bytes[12] = { 8, 16, 4, 8, 2, 4, 16, 32, 12, 24, 16, 32 };
  int64_t strideC = ((int64_t)N * N + N) / 2; int32_t bx = INT_MIN, by = 0;
  for (int32_t i = 0; i < N; ++i) { int32_t expA = vexp[i]; if (expA < INT_MAX) {
    int32_t eA = iexp(orderC, &C[((uint64_t)i * ((uint64_t)i + 3)) >> 1], strideC), kx = eA - (expA + expA);
    if (kx == bx) { by = eA > by ? eA : by; } else if (bx < kx) { bx = kx; by = eA; } } }
  int32_t bits = by - (corr + corr); int g;
  if (bits <= 23) { g = HO_F32_COMPLEX; } else if (bits <= 52) { g = HO_F64_COMPLEX; } else if (bits <= 71 && !f64_capable) { g = 9; } else if (bits <= 95 && !f64_capable) { g = 11; } else { g = HO_DD_COMPLEX; }
  if (!type_is_complex(Atype)) { g &= ~1; }
  if (Gtype) { *Gtype = g; } if (gElemBytes) { *gElemBytes = type_bytes[g]; } return by;
}

typedef struct { double x, y; } dd_t;
static void two_sum(double a, double b, double* s, double* e) { *s = a + b; double d = a - *s, sd = *s + d; *e = (b + d) + (a - sd); } /* internal.hpp:181-182 */
static dd_t dd_renorm(dd_t a) { double s = a.x + a.y, d = a.x - s; dd_t r = { s, a.y + d }; return r; } /* :199-200 */
static dd_t dd_add(dd_t a, dd_t b) { double s, e; two_sum(a.x, b.x, &s, &e); dd_t r = { s, (a.y + b.y) + e }; return dd_renorm(r); } /* :213-214 */
static dd_t conv_i64_dd(uint64_t i) { dd_t r = { scalbn((double)(int32_t)(i >> 32), 32), (double)(uint32_t)i }; return r; } /* dequantize.cu:56 */
static double conv_a63_f64(int orderA, const uint64_t* a, int32_t e) { /* :57-62 */
  double res = (double)(int64_t)a[orderA - 1];
  if (2 < orderA) { dd_t i = conv_i64_dd(a[1]); res = (scalbn(res, 63) + i.x) + i.y; }
  if (1 < orderA) { dd_t i = conv_i64_dd(a[0]); res = (scalbn(res, 63) + i.x) + i.y; }
  return scalbn(res, e);
}
static dd_t conv_a63_dd(int orderA, const uint64_t* a, int32_t e) { /* :64-69 */
  dd_t res = dd_renorm(conv_i64_dd(a[orderA - 1]));
  if (2 < orderA) { dd_t s = { scalbn(res.x, 63), scalbn(res.y, 63) }; res = dd_add(s, dd_renorm(conv_i64_dd(a[1]))); }
  if (1 < orderA) { dd_t s = { scalbn(res.x, 63), scalbn(res.y, 63) }; res = dd_add(s, dd_renorm(conv_i64_dd(a[0]))); }
  dd_t r = { scalbn(res.x, e), scalbn(res.y, e) }; return r;
}

/* :121-129.  G layouts: F32/F64 scalar; DD {hi, lo}; complex = {re, im} of those. */
void ho_dequantize(int32_t N, int32_t orderC, const uint64_t* C, const int32_t* vexp, int Gtype, void* G, int64_t ldg) {
  int64_t strideC = ((int64_t)N * N + N) / 2; int Complex = type_is_complex(Gtype);
  #pragma omp parallel for schedule(dynamic, 8)
  for (int32_t x = 0; x < N; ++x) for (int32_t y = 0; y <= x; ++y) {
    int32_t ex = vexp[x], ey = vexp[y]; int zero = (ex == INT_MAX || ey == INT_MAX); int32_t e = zero ? 0 : -(ex + ey);
    uint64_t r[3] = { 0, 0, 0 }, im[3] = { 0, 0, 0 }; const uint64_t* Cp = &C[tri_index(y, x)];
    for (int l = 0; l < orderC; ++l) { r[l] = Cp[l * strideC]; if (Complex) { im[l] = Cp[(orderC + l) * strideC]; } }
    int64_t up = y + (int64_t)x * ldg, lo = x + (int64_t)y * ldg;
    switch (Gtype & ~1) {
      case HO_F64: { double vr = zero ? 0. : conv_a63_f64(orderC, r, e), vi = (zero || !Complex) ? 0. : conv_a63_f64(orderC, im, e); double* g = (double*)G;
        if (Complex) { g[2 * up] = vr; g[2 * up + 1] = vi; g[2 * lo] = vr; g[2 * lo + 1] = -vi; } else { g[up] = vr; g[lo] = vr; } } break;
      case HO_F32: { float vr = zero ? 0.f : (float)conv_a63_f64(orderC, r, e), vi = (zero || !Complex) ? 0.f : (float)conv_a63_f64(orderC, im, e); float* g = (float*)G;
        if (Complex) { g[2 * up] = vr; g[2 * up + 1] = vi; g[2 * lo] = vr; g[2 * lo + 1] = -vi; } else { g[up] = vr; g[lo] = vr; } } break;
      case HO_DD: { dd_t z = { 0., 0. }, vr = zero ? z : conv_a63_dd(orderC, r, e), vi = (zero || !Complex) ? z : conv_a63_dd(orderC, im, e); double* g = (double*)G;
        if (Complex) { g[4 * up] = vr.x; g[4 * up + 1] = vr.y; g[4 * up + 2] = vi.x; g[4 * up + 3] = vi.y; g[4 * lo] = vr.x; g[4 * lo + 1] = vr.y; g[4 * lo + 2] = -vi.x; g[4 * lo + 3] = -vi.y; }
        else { g[2 * up] = vr.x; g[2 * up + 1] = vr.y; g[2 * lo] = vr.x; g[2 * lo + 1] = vr.y; } } break;
      default: break;
    }
  }
}

/* ------------------------------------------------------------------ */
/* Pivoted Cholesky (src/hyacin_potrfp.cu:119-318), FP64 and           */
/* double-double, real and complex.  Sequential restatement of the     */
/* left-looking step: same pivot rule (first maximum of the updated    */
/* diagonal), same stop rule (remaining trace <= eps^2 trace(G) or K   */
/* columns), same in-place layout (row k of R in row k of the          */
/* column-permuted G), 1-based pivots.                                 */
/* ------------------------------------------------------------------ */
static dd_t dd_neg(dd_t a) { dd_t r = { -a.x, -a.y }; return r; }
static dd_t dd_sub(dd_t a, dd_t b) { double s, e; two_sum(a.x, -b.x, &s, &e); dd_t r = { s, (a.y - b.y) + e }; return dd_renorm(r); } /* potrfp.cu:6 */
static dd_t dd_mul(dd_t a, dd_t b) { double p = a.x * b.x; dd_t r = { p, fma(a.x, b.y, a.y * b.x) + fma(a.x, b.x, -p) }; return dd_renorm(r); } /* :21 */
static dd_t dd_sqr(dd_t a) { double p = a.x * a.x; dd_t r = { p, fma(a.x + a.x, a.y, fma(a.x, a.x, -p)) }; return dd_renorm(r); } /* :41 */
static dd_t dd_increment(dd_t x) { dd_t t = { 1.5, x.x }; dd_t y = dd_renorm(t); y.y += x.y; return y; } /* :57 */
/* :58-63: returns sqrt(r) and replaces r by 1/sqrt(r) */
static dd_t dd_sqrt_fl(dd_t* r) {
  int e; dd_t rx = { frexp(1.0 / sqrt(r->x), &e), 0. }; int e2 = e + e - 1; dd_t x = { scalbn(-r->x, e2), scalbn(-r->y, e2) };
  rx = dd_mul(rx, dd_increment(dd_mul(x, dd_sqr(rx)))); rx = dd_mul(rx, dd_increment(dd_mul(x, dd_sqr(rx))));
  x = *r; r->x = scalbn(rx.x, e); r->y = scalbn(rx.y, e); return dd_mul(x, *r);
}
static int dd_less(dd_t a, dd_t b) { return a.x < b.x || (a.x == b.x && a.y < b.y); } /* :104 */

/* G: N x N column-major in the Gtype layout (F64 / F64_COMPLEX / DD / DD_COMPLEX); overwritten.
 * Returns the rank; jpiv gets the 1-based pivots.  Loop structure of potrf_iter_kernel (:214-272):
 * step with the pivot chosen at the end of the previous step, then re-evaluate (max, trace) of the
 * updated diagonal; continue iff trace > eps^2 trace(G), a positive diagonal is left and fewer than
 * K columns are done (K == N: until one column is left, which is then counted). */
int32_t ho_potrfp(double eps, int32_t K, int32_t N, int Gtype, void* G, int64_t ldg, int32_t* jpiv) {
  int Complex = type_is_complex(Gtype), dd = ((Gtype & ~1) == HO_DD); int w = (dd ? 2 : 1) * (Complex ? 2 : 1);
  double* g = (double*)G; double eps2 = eps * eps;
  #define GE(r, c) (&g[((int64_t)(r) + (int64_t)(c) * ldg) * w])
  if (N <= 0) { return 0; } if (K > N || K <= 0) { K = N; }
  dd_t* D = (dd_t*)malloc(sizeof(dd_t) * N), *row_re = (dd_t*)malloc(sizeof(dd_t) * N), *row_im = (dd_t*)malloc(sizeof(dd_t) * N);
  double trace = 0.; dd_t best = { 0., 0. }; int32_t j = -1;
  for (int32_t i = 0; i < N; ++i) {
    double* e = GE(i, i); D[i].x = e[0]; D[i].y = dd ? e[1] : 0.; jpiv[i] = i + 1; trace += D[i].x;
    if (dd ? dd_less(best, D[i]) : (best.x < D[i].x)) { best = D[i]; j = i; }
  }
  double thresh = eps2 * trace; int32_t iterN = (K == N) ? 1 : (N - K), M = 0, Nrem = N;
  dd_t rinv = best, sq = { 0., 0. };
  if (0 <= j) { if (dd) { sq = dd_sqrt_fl(&rinv); } else { sq.x = sqrt(best.x); rinv.x = 1. / sq.x; rinv.y = 0.; } }
  if (j < 0 || !(iterN < N)) { int32_t r = (j < 0) ? 0 : (int32_t)(N == 1); free(D); free(row_re); free(row_im); return r; }
  for (;;) {
    int32_t k = M;
    /* (1) S[l] = G[l, j] - sum_{t<k} conj(R[t, l]) R[t, j] over the trailing rows l */
    for (int32_t l = k; l < N; ++l) {
      double* e = GE(l, j); dd_t sr = { 0., 0. }, si = { 0., 0. };
      if (dd) { sr.x = e[0]; sr.y = e[1]; if (Complex) { si.x = e[2]; si.y = e[3]; } } else { sr.x = e[0]; if (Complex) { si.x = e[1]; } }
      for (int32_t t = 0; t < k; ++t) {
        double* a = GE(t, l), *b = GE(t, j);
        if (dd) {
          dd_t ar = { a[0], a[1] }, br = { b[0], b[1] };
          if (Complex) { dd_t ai = { a[2], a[3] }, bi = { b[2], b[3] };
            sr = dd_sub(sr, dd_add(dd_mul(ar, br), dd_mul(ai, bi))); si = dd_sub(si, dd_sub(dd_mul(ar, bi), dd_mul(ai, br)));
          } else { sr = dd_sub(sr, dd_mul(ar, br)); }
        } else if (Complex) { sr.x = fma(-a[0], b[0], fma(-a[1], b[1], sr.x)); si.x = fma(-a[0], b[1], fma(a[1], b[0], si.x)); }
        else { sr.x = fma(-a[0], b[0], sr.x); }
      }
      row_re[l] = sr; row_im[l] = si;
    }
    ++M; --Nrem;
    /* (2) symmetric swap j <-> k of pivots, diagonal, the finished R rows and the trailing block */
    if (j != k) {
      int32_t tp = jpiv[j]; jpiv[j] = jpiv[k]; jpiv[k] = tp; dd_t td = D[j]; D[j] = D[k]; D[k] = td;
      for (int32_t r = 0; r < N; ++r) for (int c = 0; c < w; ++c) { double t0 = GE(r, j)[c]; GE(r, j)[c] = GE(r, k)[c]; GE(r, k)[c] = t0; }
      for (int32_t c2 = k; c2 < N; ++c2) for (int c = 0; c < w; ++c) { double t0 = GE(j, c2)[c]; GE(j, c2)[c] = GE(k, c2)[c]; GE(k, c2)[c] = t0; }
      dd_t tr = row_re[j]; row_re[j] = row_re[k]; row_re[k] = tr; tr = row_im[j]; row_im[j] = row_im[k]; row_im[k] = tr;
    }
    /* R[k, k] = sqrt(d); R[k, l] = conj(S[l]) / sqrt(d); d_l -= |R[k, l]|^2 */
    { double* e = GE(k, k); if (dd) { e[0] = sq.x; e[1] = sq.y; if (Complex) { e[2] = 0.; e[3] = 0.; } } else { e[0] = sq.x; if (Complex) { e[1] = 0.; } } }
    for (int32_t l = k + 1; l < N; ++l) {
      double* e = GE(k, l);
      if (dd) {
        dd_t rr = dd_mul(rinv, row_re[l]);
        if (Complex) { dd_t ri = dd_mul(rinv, dd_neg(row_im[l])); e[0] = rr.x; e[1] = rr.y; e[2] = ri.x; e[3] = ri.y; D[l] = dd_sub(D[l], dd_add(dd_sqr(rr), dd_sqr(ri))); }
        else { e[0] = rr.x; e[1] = rr.y; D[l] = dd_sub(D[l], dd_sqr(rr)); }
      } else {
        double rr = rinv.x * row_re[l].x;
        if (Complex) { double ri = -rinv.x * row_im[l].x; e[0] = rr; e[1] = ri; D[l].x = fma(-rr, rr, fma(-ri, ri, D[l].x)); } else { e[0] = rr; D[l].x = fma(-rr, rr, D[l].x); }
      }
    }
    /* (3) next pivot, remaining trace, eager next diagonal */
    double rem = 0.; best.x = 0.; best.y = 0.; j = -1;
    for (int32_t i = M; i < N; ++i) { rem += D[i].x; if (dd ? dd_less(best, D[i]) : (best.x < D[i].x)) { best = D[i]; j = i; } }
    if (!(thresh < rem)) { j = -1; }
    rinv = best;
    if (dd) { sq = dd_sqrt_fl(&rinv); } else { sq.x = sqrt(best.x); sq.y = 0.; rinv.x = 1. / sq.x; rinv.y = 0.; }
    if (M < N) { double* e = GE(M, M); if (Nrem == 1) { if (dd) { e[0] = sq.x; e[1] = sq.y; if (Complex) { e[2] = 0.; e[3] = 0.; } } else { e[0] = sq.x; if (Complex) { e[1] = 0.; } } } }
    if (j < 0 || Nrem <= iterN) { break; }
  }
  free(D); free(row_re); free(row_im);
  #undef GE
  return M + (int32_t)(Nrem == 1);
}
