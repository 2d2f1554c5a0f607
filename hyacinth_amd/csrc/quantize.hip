/*
 * quantize.hip -- floating point -> int8 limb / CRT-residue panels (HBM-bound).
 *
 * Replaces the reference's src/quantize_limbs.cu, src/quantize_crt_real.cu and
 * src/quantize_crt_complex.cu.  Every element x of column j becomes the integer
 * q = RNE(x * 2^vexp[j]) (96-bit two's complement) and is written as
 *   limbs:        balanced base-256 digits d_l in [-128, 127], q = sum d_l 256^l;
 *                 complex writes three digit groups, of re + im, re and im;
 *   CRT real:     q mod m_x, stored in int8 (values above 127 wrap by -m_x);
 *   CRT complex:  moduli x < 20: (re - i_x im) mod m_x and (re + i_x im) mod m_x with i_x^2 = -1;
 *                 moduli x >= 20: (re + im) mod m_x, re mod m_x, im mod m_x.
 * A column with vexp[j] == INT_MAX is all zero.
 *
 * Output layout (same as the reference): panel p, column j, row k at
 * B[p * N * ldb + j * ldb + k]; rows are the contraction dimension of the Gram
 * kernel, so every MFMA operand fetch is a contiguous run of K.
 *
 * One thread quantizes four consecutive rows of one column and stores one
 * packed dword per panel (byte stores when B + row is not 4-byte aligned).
 */
#include <type_traits>
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include "hyk_common.h"
#include "crt_tables.h"
#include "hyacin_kernels.h"

namespace {

constexpr int Q_THREADS = 256;
constexpr int Q_ROWS = 4;

__device__ __forceinline__ float half_bits(uint16_t b) { __half_raw r; r.x = b; return __half2float(__half(r)); }

/* loaders: element -> decomposed real / imaginary parts (integer path) or doubles (FP64 residue path) */
struct ElemF64 { static constexpr int cplx = 0; using T = uint64_t; static __device__ __forceinline__ void load(const T* p, hyk::Dec& re, hyk::Dec& im) { re = hyk::decompose_f64(*p); im = hyk::Dec{ 0, 0, 0 }; }
  static __device__ __forceinline__ void load_f64(const T* p, double& re, double& im) { re = __longlong_as_double((long long)*p); im = 0.; } };
struct ElemF32 { static constexpr int cplx = 0; using T = uint32_t; static __device__ __forceinline__ void load(const T* p, hyk::Dec& re, hyk::Dec& im) { re = hyk::decompose_f32(*p); im = hyk::Dec{ 0, 0, 0 }; }
  static __device__ __forceinline__ void load_f64(const T* p, double& re, double& im) { re = (double)__uint_as_float(*p); im = 0.; } };
struct ElemF16 { static constexpr int cplx = 0; using T = uint16_t; static __device__ __forceinline__ void load(const T* p, hyk::Dec& re, hyk::Dec& im) { re = hyk::decompose_f16(*p); im = hyk::Dec{ 0, 0, 0 }; }
  static __device__ __forceinline__ void load_f64(const T* p, double& re, double& im) { re = (double)half_bits(*p); im = 0.; } };
struct ElemF64C { static constexpr int cplx = 1; using T = ulonglong2; static __device__ __forceinline__ void load(const T* p, hyk::Dec& re, hyk::Dec& im) { T v = *p; re = hyk::decompose_f64(v.x); im = hyk::decompose_f64(v.y); }
  static __device__ __forceinline__ void load_f64(const T* p, double& re, double& im) { T v = *p; re = __longlong_as_double((long long)v.x); im = __longlong_as_double((long long)v.y); } };
struct ElemF32C { static constexpr int cplx = 1; using T = uint2; static __device__ __forceinline__ void load(const T* p, hyk::Dec& re, hyk::Dec& im) { T v = *p; re = hyk::decompose_f32(v.x); im = hyk::decompose_f32(v.y); }
  static __device__ __forceinline__ void load_f64(const T* p, double& re, double& im) { T v = *p; re = (double)__uint_as_float(v.x); im = (double)__uint_as_float(v.y); } };
struct ElemF16C { static constexpr int cplx = 1; using T = uint32_t; static __device__ __forceinline__ void load(const T* p, hyk::Dec& re, hyk::Dec& im) { T v = *p; re = hyk::decompose_f16(v & 0xffffu); im = hyk::decompose_f16(v >> 16); }
  static __device__ __forceinline__ void load_f64(const T* p, double& re, double& im) { T v = *p; re = (double)half_bits((uint16_t)(v & 0xffffu)); im = (double)half_bits((uint16_t)(v >> 16)); } };

/* The Q_ROWS consecutive elements of a thread: full, 16-byte aligned groups come in as 16-byte non-temporal vector loads
 * issued back to back (A is read exactly once); ragged or unaligned groups element by element; missing rows read as zero. */
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
template <typename T>
__device__ __forceinline__ void fetch_rows(const T* __restrict__ src, int valid, T (&tmp)[Q_ROWS]) {
  constexpr int BYTES = (int)sizeof(T) * Q_ROWS;
  if (valid == Q_ROWS && ((uintptr_t)src & (BYTES >= 16 ? 15u : 7u)) == 0) {
    if constexpr (BYTES >= 16) {
      #pragma unroll
      for (int i = 0; i < BYTES / 16; ++i) { reinterpret_cast<u32x4*>(tmp)[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src) + i); }
    } else { *reinterpret_cast<u32x2*>(tmp) = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(src)); }
  } else {
    #pragma unroll
    for (int r = 0; r < Q_ROWS; ++r) { tmp[r] = T{}; if (r < valid) { tmp[r] = src[r]; } }
  }
}

__device__ __forceinline__ void store_panel(int8_t* dst, uint32_t packed, int valid, bool aligned) {
  if (aligned && valid == Q_ROWS) { __builtin_nontemporal_store(packed, reinterpret_cast<uint32_t*>(dst)); }   /* written once, read by another kernel: past the caches */
  else { for (int r = 0; r < valid; ++r) { dst[r] = (int8_t)(packed >> (8 * r)); } }
}

/* ------------------------------------------------------------------ limbs */
/* The work of one thread: Q_ROWS consecutive rows i0 .. of column j, given as raw elements (missing rows zero). */
template <typename E>
__device__ __forceinline__ void limbs_rows(int32_t order, int32_t expon, const typename E::T (&raw)[Q_ROWS], int valid, int8_t* out, bool aligned, int64_t strideB) {
  constexpr int GROUPS = E::cplx ? 3 : 1;
  if (expon == HYK_INT_MAX) { for (int p = 0; p < order * GROUPS; ++p) { store_panel(out + p * strideB, 0u, valid, aligned); } return; }
  /* Small values first: q = rint(x 2^expon) is exact in a double while |q| < 2^50 (every plan for FP16 / FP32 storage, and
   * FP64 up to six digits), and its two's complement bytes then come from a 32-bit integer (|q| < 2^29: FP16 storage, three
   * digits) or a 64-bit one instead of the 96-bit path. */
  { double re[Q_ROWS], im[Q_ROWS]; double big = 0.;
    #pragma unroll
    for (int r = 0; r < Q_ROWS; ++r) {
      double a = 0., b = 0.; E::load_f64(&raw[r], a, b);
      re[r] = __builtin_rint(__builtin_ldexp(a, expon)); im[r] = __builtin_rint(__builtin_ldexp(b, expon));
      big = __builtin_fmax(big, __builtin_fmax(__builtin_fabs(re[r]), __builtin_fabs(im[r])));
      if (!(re[r] == re[r]) || !(im[r] == im[r])) { big = __builtin_inf(); }   /* a NaN goes the long way like anything else out of range */
    }
    /* one group at a time (a rolled loop: unrolled, the 3 x order panel addresses and digit words of a complex element cost
     * more registers, and with them resident wavefronts, than the loop costs instructions); the digits of a group unrolled */
    auto digits = [&](auto zero, auto signShift, auto bytes) {
      using Q = decltype(zero);
      #pragma unroll 1
      for (int g = 0; g < GROUPS; ++g) {
        Q q[Q_ROWS];
        #pragma unroll
        for (int r = 0; r < Q_ROWS; ++r) { const Q a = (Q)re[r]; if constexpr (E::cplx) { const Q b = (Q)im[r]; q[r] = g == 0 ? a + b : (g == 1 ? a : b); } else { q[r] = a; } }
        uint32_t carry[Q_ROWS] = { 0, 0, 0, 0 }; int8_t* dst = out + (int64_t)(g * order) * strideB;
        #pragma unroll
        for (int l = 0; l < 12; ++l) {
          if (l < order) {
            uint32_t packed = 0;
            #pragma unroll
            for (int r = 0; r < Q_ROWS; ++r) {
              const uint32_t t = (uint32_t)((q[r] >> (l < bytes() ? 8 * l : signShift())) & 0xff) + carry[r];
              packed |= (t & 0xffu) << (8 * r); carry[r] = (t >> 8) + ((t >> 7) & 1u);
            }
            store_panel(dst, packed, valid, aligned); dst += strideB;
          }
        }
      }
    };
    if (big < 0x1p29) { digits((int32_t)0, std::integral_constant<int, 31>{}, std::integral_constant<int, 4>{}); return; }
    if (big < 0x1p50) { digits((long long)0, std::integral_constant<int, 63>{}, std::integral_constant<int, 8>{}); return; }
  }
  /* the long way: 96-bit integers, one group at a time (the values are worked out again per group: this path is rare, and
   * holding all three groups would set the register count of the whole kernel) */
  #pragma unroll 1
  for (int g = 0; g < GROUPS; ++g) {
    hyk::I96 q[Q_ROWS];
    #pragma unroll
    for (int r = 0; r < Q_ROWS; ++r) {
      hyk::Dec re{ 0, 0, 0 }, im{ 0, 0, 0 }; E::load(&raw[r], re, im);
      if constexpr (E::cplx) { q[r] = g == 0 ? hyk::i96_add(hyk::round_scaled(re, expon), hyk::round_scaled(im, expon)) : hyk::round_scaled(g == 1 ? re : im, expon); }
      else { q[r] = hyk::round_scaled(re, expon); }
    }
    uint32_t carry[Q_ROWS] = { 0, 0, 0, 0 };
    #pragma unroll 1
    for (int l = 0; l < order; ++l) {
      uint32_t packed = 0;
      #pragma unroll
      for (int r = 0; r < Q_ROWS; ++r) { uint32_t t = hyk::i96_byte(q[r], l) + carry[r]; packed |= (t & 0xffu) << (8 * r); carry[r] = (t >> 8) + ((t >> 7) & 1u); }
      store_panel(out + (int64_t)(g * order + l) * strideB, packed, valid, aligned);
    }
  }
}
struct LimbsRows { template <typename E> static __device__ __forceinline__ void run(int32_t order, int32_t expon, const typename E::T (&raw)[Q_ROWS], int valid, int8_t* out, bool aligned, int64_t strideB) { limbs_rows<E>(order, expon, raw, valid, out, aligned, strideB); } };

/* ------------------------------------------------------------------ CRT */
/* DOTS = dwords of the biased two's complement of q that the byte dot products cover: |q| < 2^(32 DOTS - 1) */
template <int X> struct RealMod { static constexpr hyk::DotMod k = hyk::make_dotmod(hyk_crt_real_mo[X]); };
template <int X> struct CplxMod { static constexpr hyk::DotMod k = hyk::make_dotmod(hyk_crt_cplx_mo[X]); static constexpr uint32_t im = hyk_crt_cplx_im[X]; };

template <typename E, int DOTS, int X>
__device__ __forceinline__ void crt_real_step(int32_t order, const hyk::I96 (&q)[Q_ROWS], int8_t* out, int64_t strideB, int valid, bool aligned) {
  if constexpr (X < HYK_CRT_REAL_COUNT) {
    if (X < order) {
      constexpr hyk::DotMod k = RealMod<X>::k; uint32_t packed = 0;
      #pragma unroll
      for (int r = 0; r < Q_ROWS; ++r) { packed |= ((uint32_t)(uint8_t)hyk::stored_residue_dot<DOTS>(q[r], k)) << (8 * r); }
      store_panel(out + (int64_t)X * strideB, packed, valid, aligned);
      crt_real_step<E, DOTS, X + 1>(order, q, out, strideB, valid, aligned);
    }
  }
}

template <int DOTS> struct CrtRealRows {
  template <typename E> static __device__ __forceinline__ void run(int32_t order, int32_t expon, const typename E::T (&raw)[Q_ROWS], int valid, int8_t* out, bool aligned, int64_t strideB) {
    if (expon == HYK_INT_MAX) { for (int p = 0; p < order; ++p) { store_panel(out + p * strideB, 0u, valid, aligned); } return; }
    hyk::I96 q[Q_ROWS];
    #pragma unroll
    for (int r = 0; r < Q_ROWS; ++r) { hyk::Dec re{ 0, 0, 0 }, im{ 0, 0, 0 }; E::load(&raw[r], re, im); q[r] = hyk::round_scaled(re, expon); }
    crt_real_step<E, DOTS, 0>(order, q, out, strideB, valid, aligned);
  }
};

template <typename E, int DOTS, int X>
__device__ __forceinline__ void crt_cplx_step(int32_t order, const hyk::I96 (&qr)[Q_ROWS], const hyk::I96 (&qi)[Q_ROWS], int8_t* out, int64_t strideB, int valid, bool aligned) {
  if constexpr (X < HYK_CRT_CPLX_COUNT) {
    if (X < order) {
      constexpr hyk::DotMod k = CplxMod<X>::k; constexpr uint32_t im = CplxMod<X>::im, centre = hyk::stored_centre(k.m); uint32_t p0 = 0, p1 = 0, p2 = 0;
      #pragma unroll
      for (int r = 0; r < Q_ROWS; ++r) {
        const uint32_t a = hyk::residue_dot<DOTS>(qr[r], k, 0u), b = hyk::residue_dot<DOTS>(qi[r], k, 0u);   /* canonical */
        if constexpr (X < HYK_CRT_CPLX_SPLIT) {
          /* (re -+ iota im) mod m, stored as the reference does: ((t + c) mod m) - c, c = max(m - 128, 0) */
          const int32_t p = (int32_t)hyk::reduce_small(a + (k.m - im) * b + centre, k) - (int32_t)centre, q = (int32_t)hyk::reduce_small(a + im * b + centre, k) - (int32_t)centre;
          p0 |= ((uint32_t)(uint8_t)p) << (8 * r); p1 |= ((uint32_t)(uint8_t)q) << (8 * r);
        } else {
          uint32_t s = a + b; s = s >= k.m ? s - k.m : s;
          p0 |= ((uint32_t)(uint8_t)hyk::residue_to_i8(s, k.m)) << (8 * r); p1 |= ((uint32_t)(uint8_t)hyk::residue_to_i8(a, k.m)) << (8 * r); p2 |= ((uint32_t)(uint8_t)hyk::residue_to_i8(b, k.m)) << (8 * r);
        }
      }
      if constexpr (X < HYK_CRT_CPLX_SPLIT) {
        store_panel(out + (int64_t)(2 * X) * strideB, p0, valid, aligned); store_panel(out + (int64_t)(2 * X + 1) * strideB, p1, valid, aligned);
      } else {
        constexpr int base = 2 * HYK_CRT_CPLX_SPLIT + 3 * (X - HYK_CRT_CPLX_SPLIT);
        store_panel(out + (int64_t)base * strideB, p0, valid, aligned); store_panel(out + (int64_t)(base + 1) * strideB, p1, valid, aligned); store_panel(out + (int64_t)(base + 2) * strideB, p2, valid, aligned);
      }
      crt_cplx_step<E, DOTS, X + 1>(order, qr, qi, out, strideB, valid, aligned);
    }
  }
}

__device__ __forceinline__ int crt_cplx_panels(int32_t order) { return 2 * (order < HYK_CRT_CPLX_SPLIT ? order : HYK_CRT_CPLX_SPLIT) + 3 * (order > HYK_CRT_CPLX_SPLIT ? order - HYK_CRT_CPLX_SPLIT : 0); }
template <int DOTS> struct CrtCplxRows {
  template <typename E> static __device__ __forceinline__ void run(int32_t order, int32_t expon, const typename E::T (&raw)[Q_ROWS], int valid, int8_t* out, bool aligned, int64_t strideB) {
    if (expon == HYK_INT_MAX) { const int panels = crt_cplx_panels(order); for (int p = 0; p < panels; ++p) { store_panel(out + p * strideB, 0u, valid, aligned); } return; }
    hyk::I96 qr[Q_ROWS], qi[Q_ROWS];
    #pragma unroll
    for (int r = 0; r < Q_ROWS; ++r) { hyk::Dec re{ 0, 0, 0 }, im{ 0, 0, 0 }; E::load(&raw[r], re, im); qr[r] = hyk::round_scaled(re, expon); qi[r] = hyk::round_scaled(im, expon); }
    crt_cplx_step<E, DOTS, 0>(order, qr, qi, out, strideB, valid, aligned);
  }
};

/* ------------------------------------------------------------------ CRT, quantized values below 2^51
 * q = rint(x * 2^vexp) is then exact in a double (ldexp and rint are exact operations), and every residue costs three
 * FP64 instructions (hyk::residue_f64) instead of byte dot products and an integer reduction. */
template <int X> struct RealF64 { static constexpr hyk::F64Mod k = hyk::make_f64mod(hyk_crt_real_mo[X], hyk::stored_delta(hyk_crt_real_mo[X])); };
template <int X> struct CplxF64 {
  static constexpr hyk::F64Mod stored = hyk::make_f64mod(hyk_crt_cplx_mo[X], hyk::stored_delta(hyk_crt_cplx_mo[X]));
  static constexpr hyk::F64Mod sym = hyk::make_f64mod(hyk_crt_cplx_mo[X], 0.0);   /* any small representative */
  static constexpr double im = (double)hyk_crt_cplx_im[X];
};
/* Integer -> byte without a conversion instruction: adding 1.5 * 2^52 to an integer-valued double |r| < 2^51 leaves r, in
 * two's complement, in the low bits of the sum's mantissa.  For the real path the constant is folded into the residue's
 * second multiply-add (a + 1.5 * 2^52 is still exact for |a| < 2^51), so a residue byte costs three FP64 instructions. */
constexpr double LOW_BITS = 6755399441055744.0;   /* 1.5 * 2^52 */
__device__ __forceinline__ uint32_t low_word(double r) { return (uint32_t)__double2loint(r + LOW_BITS); }
__device__ __forceinline__ uint32_t low_word_of_biased(double rPlusBias) { return (uint32_t)__double2loint(rPlusBias); }
__device__ __forceinline__ double residue_f64_biased(double a, double aBiased, const hyk::F64Mod& k) {
  return __builtin_fma(k.negM, __builtin_rint(__builtin_fma(a, k.inv, k.tieShift)), aBiased);
}
/* low bytes of four words -> one dword (row 0 in the lowest byte) */
__device__ __forceinline__ uint32_t pack4(uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3) {
  const uint32_t lo = __builtin_amdgcn_perm(w1, w0, 0x0c0c0400u), hi = __builtin_amdgcn_perm(w3, w2, 0x0c0c0400u);
  return __builtin_amdgcn_perm(hi, lo, 0x05040100u);
}
static_assert(Q_ROWS == 4, "pack4 packs the four rows of a thread");

template <int X>
__device__ __forceinline__ void crt_real_f64_step(int32_t order, const double (&a)[Q_ROWS], const double (&ab)[Q_ROWS], int8_t* out, int64_t strideB, int valid, bool aligned) {
  if constexpr (X < HYK_CRT_REAL_COUNT) {
    if (X < order) {
      constexpr hyk::F64Mod k = RealF64<X>::k; uint32_t w[Q_ROWS];
      #pragma unroll
      for (int r = 0; r < Q_ROWS; ++r) { w[r] = low_word_of_biased(residue_f64_biased(a[r], ab[r], k)); }
      store_panel(out + (int64_t)X * strideB, pack4(w[0], w[1], w[2], w[3]), valid, aligned);
      crt_real_f64_step<X + 1>(order, a, ab, out, strideB, valid, aligned);
    }
  }
}

struct CrtRealF64Rows {
  template <typename E> static __device__ __forceinline__ void run(int32_t order, int32_t expon, const typename E::T (&raw)[Q_ROWS], int valid, int8_t* out, bool aligned, int64_t strideB) {
    if (expon == HYK_INT_MAX) { for (int p = 0; p < order; ++p) { store_panel(out + p * strideB, 0u, valid, aligned); } return; }
    double a[Q_ROWS], ab[Q_ROWS];
    #pragma unroll
    for (int r = 0; r < Q_ROWS; ++r) { double re = 0., im = 0.; E::load_f64(&raw[r], re, im); a[r] = __builtin_rint(__builtin_ldexp(re, expon)); ab[r] = a[r] + LOW_BITS; }
    crt_real_f64_step<0>(order, a, ab, out, strideB, valid, aligned);
  }
};

template <int X>
__device__ __forceinline__ void crt_cplx_f64_step(int32_t order, const double (&ar)[Q_ROWS], const double (&ai)[Q_ROWS], int8_t* out, int64_t strideB, int valid, bool aligned) {
  if constexpr (X < HYK_CRT_CPLX_COUNT) {
    if (X < order) {
      using K = CplxF64<X>; uint32_t w0[Q_ROWS], w1[Q_ROWS], w2[Q_ROWS];
      #pragma unroll
      for (int r = 0; r < Q_ROWS; ++r) {
        if constexpr (X < HYK_CRT_CPLX_SPLIT) {
          /* only the imaginary part is reduced first: |rb| <= m / 2, so re -+ iota rb is exact and stays below 2^51 */
          const double rb = hyk::residue_f64(ai[r], K::sym);
          w0[r] = low_word(hyk::residue_f64(__builtin_fma(-K::im, rb, ar[r]), K::stored));
          w1[r] = low_word(hyk::residue_f64(__builtin_fma(K::im, rb, ar[r]), K::stored)); w2[r] = 0u;
        } else {
          w0[r] = low_word(hyk::residue_f64(ar[r] + ai[r], K::stored)); w1[r] = low_word(hyk::residue_f64(ar[r], K::stored)); w2[r] = low_word(hyk::residue_f64(ai[r], K::stored));
        }
      }
      const uint32_t p0 = pack4(w0[0], w0[1], w0[2], w0[3]), p1 = pack4(w1[0], w1[1], w1[2], w1[3]), p2 = pack4(w2[0], w2[1], w2[2], w2[3]); (void)p2;
      if constexpr (X < HYK_CRT_CPLX_SPLIT) {
        store_panel(out + (int64_t)(2 * X) * strideB, p0, valid, aligned); store_panel(out + (int64_t)(2 * X + 1) * strideB, p1, valid, aligned);
      } else {
        constexpr int base = 2 * HYK_CRT_CPLX_SPLIT + 3 * (X - HYK_CRT_CPLX_SPLIT);
        store_panel(out + (int64_t)base * strideB, p0, valid, aligned); store_panel(out + (int64_t)(base + 1) * strideB, p1, valid, aligned); store_panel(out + (int64_t)(base + 2) * strideB, p2, valid, aligned);
      }
      crt_cplx_f64_step<X + 1>(order, ar, ai, out, strideB, valid, aligned);
    }
  }
}

struct CrtCplxF64Rows {
  template <typename E> static __device__ __forceinline__ void run(int32_t order, int32_t expon, const typename E::T (&raw)[Q_ROWS], int valid, int8_t* out, bool aligned, int64_t strideB) {
    if (expon == HYK_INT_MAX) { const int panels = crt_cplx_panels(order); for (int p = 0; p < panels; ++p) { store_panel(out + p * strideB, 0u, valid, aligned); } return; }
    double ar[Q_ROWS], ai[Q_ROWS];
    #pragma unroll
    for (int r = 0; r < Q_ROWS; ++r) {
      double re = 0., im = 0.; E::load_f64(&raw[r], re, im);
      ar[r] = __builtin_rint(__builtin_ldexp(re, expon)); ai[r] = __builtin_rint(__builtin_ldexp(im, expon));
    }
    crt_cplx_f64_step<0>(order, ar, ai, out, strideB, valid, aligned);
  }
};

/* A column-major (M x N, leading dimension lda): one thread takes Q_ROWS consecutive rows of one column straight from memory. */
template <typename E, typename ROWS>
__global__ __launch_bounds__(Q_THREADS) void quantize_kernel(int32_t M, int32_t order, const typename E::T* __restrict__ A, int64_t lda, const int32_t* __restrict__ vexp, int8_t* __restrict__ B, int64_t ldb, int64_t strideB) {
  const int32_t j = blockIdx.y; const int64_t i0 = ((int64_t)blockIdx.x * Q_THREADS + threadIdx.x) * Q_ROWS;
  if (i0 >= M) { return; }
  const int valid = (M - i0) < Q_ROWS ? (int)(M - i0) : Q_ROWS; const int32_t expon = vexp[j];
  int8_t* out = B + (int64_t)j * ldb + i0; const bool aligned = ((uintptr_t)out & 3u) == 0;
  typename E::T raw[Q_ROWS];
  if (expon != HYK_INT_MAX) { fetch_rows(&A[(int64_t)j * lda + i0], valid, raw); } else { for (int r = 0; r < Q_ROWS; ++r) { raw[r] = typename E::T{}; } }
  ROWS::template run<E>(order, expon, raw, valid, out, aligned, strideB);
}

/* A stored as its (conjugate) transpose: the N x M matrix S with op(A)[k, j] = S[j + k lda] (conjugated when CONJ), i.e.
 * the rows of op(A) are contiguous in memory.  A workgroup moves a tile of TJ columns x T_ROWS rows through LDS (reads
 * run along j, whole rows of the stored matrix; the quantized bytes leave along k, 128 per panel and column), then every
 * thread quantizes groups of Q_ROWS rows exactly as in the column-major kernel.  Replaces the transposing copy of the
 * reference (src/lra.cpp:63-69, src/matcopy.cu:36-43) together with the kernel that followed it. */
/* tile shape by element size: the stored rows of a tile are TJ elements long (at least 128 bytes), a column of it leaves as
 * T_ROWS panel bytes per panel; 256 rows (one wavefront per column, 256-byte runs as in the column-major kernel) where 33 KB
 * of LDS hold them */
template <typename T> struct TileCols { static constexpr int value = sizeof(T) >= 4 ? 32 : 64; };
template <typename T> struct TileRows { static constexpr int value = sizeof(T) == 4 ? 256 : 128; };
template <typename E> __device__ __forceinline__ typename E::T conj_elem(typename E::T v) {
  if constexpr (!E::cplx) { return v; }
  else if constexpr (sizeof(typename E::T) == 16) { v.y ^= 0x8000000000000000ull; return v; }
  else if constexpr (sizeof(typename E::T) == 8) { v.y ^= 0x80000000u; return v; }
  else { return v ^ 0x80000000u; }   /* two halves in one word: the imaginary part is the upper one */
}
template <typename E, typename ROWS, bool CONJ>
__global__ __launch_bounds__(Q_THREADS) void quantize_transposed_kernel(int32_t M, int32_t N, int32_t order, const typename E::T* __restrict__ S, int64_t lda, const int32_t* __restrict__ vexp, int8_t* __restrict__ B, int64_t ldb, int64_t strideB) {
  using T = typename E::T; constexpr int TJ = TileCols<T>::value, T_ROWS = TileRows<T>::value, PITCH = T_ROWS + 1;
  extern __shared__ __attribute__((aligned(16))) unsigned char tileBytes[];
  T* tile = reinterpret_cast<T*>(tileBytes);
  const int32_t j0 = blockIdx.y * TJ;
  /* Whole tiles of an aligned matrix come in as 16-byte pieces along the stored rows, all requested before the first is
   * used; ragged or unaligned tiles element by element. */
  constexpr int VE = sizeof(T) >= 16 ? 1 : 16 / (int)sizeof(T), PIECES = TJ / VE, ITER = PIECES * T_ROWS / Q_THREADS;
  static_assert(PIECES * T_ROWS % Q_THREADS == 0, "the pieces of a tile divide evenly among the threads");
  const int64_t k0 = (int64_t)blockIdx.x * T_ROWS;
  if ((((uintptr_t)S) & 15u) == 0 && ((lda * (int64_t)sizeof(T)) & 15) == 0 && j0 + TJ <= N) {
    u32x4 piece[ITER];
    #pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int e = threadIdx.x + it * Q_THREADS, g = e % PIECES, kk = e / PIECES;
      piece[it] = u32x4{ 0u, 0u, 0u, 0u };
      if (k0 + kk < M) { piece[it] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(&S[(int64_t)(j0 + g * VE) + (k0 + kk) * lda])); }
    }
    #pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int e = threadIdx.x + it * Q_THREADS, g = e % PIECES, kk = e / PIECES;
      #pragma unroll
      for (int c = 0; c < VE; ++c) {
        T v; __builtin_memcpy(&v, reinterpret_cast<const char*>(&piece[it]) + c * sizeof(T), sizeof(T));
        if constexpr (CONJ) { v = conj_elem<E>(v); }
        tile[(g * VE + c) * PITCH + kk] = v;
      }
    }
  } else {
    for (int e = threadIdx.x; e < TJ * T_ROWS; e += Q_THREADS) {
      const int jj = e % TJ, kk = e / TJ; T v = T{};
      if (j0 + jj < N && k0 + kk < M) { v = S[(int64_t)(j0 + jj) + (k0 + kk) * lda]; if constexpr (CONJ) { v = conj_elem<E>(v); } }
      tile[jj * PITCH + kk] = v;
    }
  }
  __syncthreads();
  constexpr int GROUPS = T_ROWS / Q_ROWS;   /* row groups per column */
  for (int e = threadIdx.x; e < TJ * GROUPS; e += Q_THREADS) {
    const int kg = e % GROUPS, jj = e / GROUPS; const int32_t j = j0 + jj; const int64_t i0 = k0 + (int64_t)kg * Q_ROWS;
    if (j >= N || i0 >= M) { continue; }
    const int valid = (M - i0) < Q_ROWS ? (int)(M - i0) : Q_ROWS; const int32_t expon = vexp[j];
    int8_t* out = B + (int64_t)j * ldb + i0; const bool aligned = ((uintptr_t)out & 3u) == 0;
    T raw[Q_ROWS];
    #pragma unroll
    for (int r = 0; r < Q_ROWS; ++r) { raw[r] = tile[jj * PITCH + kg * Q_ROWS + r]; }
    ROWS::template run<E>(order, expon, raw, valid, out, aligned, strideB);
  }
}

/* rows [row0, row1) of `panels` panels set to zero: the Gram kernel contracts over whole 128-row blocks */
__global__ void zero_rows_kernel(int8_t* __restrict__ B, int64_t ldb, int64_t cols, int32_t row0, int32_t row1) {
  const int64_t c = blockIdx.x; const int32_t len = row1 - row0; int8_t* p = B + c * ldb + row0;
  for (int32_t i = threadIdx.x; i < len; i += blockDim.x) { p[i] = 0; }
  (void)cols;
}

template <typename E, typename ROWS>
int launch_quantize(hipStream_t stream, char op, int32_t M, int32_t N, int32_t order, const void* A, int64_t lda, const int32_t* vexp, int8_t* B, int64_t ldb) {
  using T = typename E::T; const int64_t strideB = (int64_t)N * ldb;
  if (op == 'N') {
    dim3 grid((uint32_t)((M + Q_THREADS * Q_ROWS - 1) / (Q_THREADS * Q_ROWS)), (uint32_t)N);
    quantize_kernel<E, ROWS><<<grid, Q_THREADS, 0, stream>>>(M, order, (const T*)A, lda, vexp, B, ldb, strideB);
  } else {
    constexpr int TJ = TileCols<T>::value, T_ROWS = TileRows<T>::value; const size_t lds = (size_t)TJ * (T_ROWS + 1) * sizeof(T);
    dim3 grid((uint32_t)((M + T_ROWS - 1) / T_ROWS), (uint32_t)((N + TJ - 1) / TJ));
    if (op == 'C' && E::cplx) {
      if (lds > 65536 && hipFuncSetAttribute(reinterpret_cast<const void*>(&quantize_transposed_kernel<E, ROWS, true>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) { return -3; }
      quantize_transposed_kernel<E, ROWS, true><<<grid, Q_THREADS, lds, stream>>>(M, N, order, (const T*)A, lda, vexp, B, ldb, strideB);
    } else {
      if (lds > 65536 && hipFuncSetAttribute(reinterpret_cast<const void*>(&quantize_transposed_kernel<E, ROWS, false>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) { return -3; }
      quantize_transposed_kernel<E, ROWS, false><<<grid, Q_THREADS, lds, stream>>>(M, N, order, (const T*)A, lda, vexp, B, ldb, strideB);
    }
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

template <typename ROWS>
int launch_quantize_type(hipStream_t stream, char op, int32_t M, int32_t N, int32_t order, int32_t Atype, const void* A, int64_t lda, const int32_t* vexp, int8_t* B, int64_t ldb) {
  switch (Atype) {
    case HYK_F64: return launch_quantize<ElemF64, ROWS>(stream, op, M, N, order, A, lda, vexp, B, ldb);
    case HYK_F32: return launch_quantize<ElemF32, ROWS>(stream, op, M, N, order, A, lda, vexp, B, ldb);
    case HYK_F16: return launch_quantize<ElemF16, ROWS>(stream, op, M, N, order, A, lda, vexp, B, ldb);
    case HYK_F64C: return launch_quantize<ElemF64C, ROWS>(stream, op, M, N, order, A, lda, vexp, B, ldb);
    case HYK_F32C: return launch_quantize<ElemF32C, ROWS>(stream, op, M, N, order, A, lda, vexp, B, ldb);
    case HYK_F16C: return launch_quantize<ElemF16C, ROWS>(stream, op, M, N, order, A, lda, vexp, B, ldb);
    default: return -1;
  }
}

char norm_op(char op) { return (op == 'T' || op == 't') ? 'T' : ((op == 'C' || op == 'c') ? 'C' : 'N'); }

}  // namespace

extern "C" int hykQuantizeLimbsOp(hipStream_t stream, char opA, int32_t M, int32_t N, int32_t orderA, int32_t Atype, const void* A, int64_t lda, const int32_t* vexp, int8_t* B, int64_t ldb) {
  if (M <= 0 || N <= 0) { return 0; }
  const char op = norm_op(opA);
  if (orderA < 1 || orderA > 12 || N > 65535 || ldb < M || lda < (op == 'N' ? M : N)) { return -1; }
  return launch_quantize_type<LimbsRows>(stream, op, M, N, orderA, Atype, A, lda, vexp, B, ldb);
}

extern "C" int hykQuantizeLimbs(hipStream_t stream, int32_t M, int32_t N, int32_t orderA, int32_t Atype, const void* A, int64_t lda, const int32_t* vexp, int8_t* B, int64_t ldb) {
  return hykQuantizeLimbsOp(stream, 'N', M, N, orderA, Atype, A, lda, vexp, B, ldb);
}

/* maxBits: an upper bound on the bit length of |q| (u + 1 covers re + im as well); <= 0 means unknown */
extern "C" int hykQuantizeCrtOp(hipStream_t stream, char opA, int32_t M, int32_t N, int32_t orderA, int32_t Atype, const void* A, int64_t lda, const int32_t* vexp, int8_t* B, int64_t ldb, int32_t maxBits) {
  if (M <= 0 || N <= 0) { return 0; }
  const int cplx = Atype & 1; const char op = norm_op(opA);
  if (orderA < 1 || orderA > (cplx ? HYK_CRT_CPLX_COUNT : HYK_CRT_REAL_COUNT) || N > 65535 || ldb < M || lda < (op == 'N' ? M : N)) { return -1; }
  const int dots = (0 < maxBits && maxBits <= 31) ? 1 : (0 < maxBits && maxBits <= 63) ? 2 : 3;
  const bool viaF64 = (0 < maxBits && maxBits <= 51);   /* |q|, and |re + im| for complex input, below 2^51: exact in a double */
  if (!cplx) {
    if (viaF64) { return launch_quantize_type<CrtRealF64Rows>(stream, op, M, N, orderA, Atype, A, lda, vexp, B, ldb); }
    if (dots == 1) { return launch_quantize_type<CrtRealRows<1>>(stream, op, M, N, orderA, Atype, A, lda, vexp, B, ldb); }
    if (dots == 2) { return launch_quantize_type<CrtRealRows<2>>(stream, op, M, N, orderA, Atype, A, lda, vexp, B, ldb); }
    return launch_quantize_type<CrtRealRows<3>>(stream, op, M, N, orderA, Atype, A, lda, vexp, B, ldb);
  }
  if (viaF64) { return launch_quantize_type<CrtCplxF64Rows>(stream, op, M, N, orderA, Atype, A, lda, vexp, B, ldb); }
  if (dots == 1) { return launch_quantize_type<CrtCplxRows<1>>(stream, op, M, N, orderA, Atype, A, lda, vexp, B, ldb); }
  if (dots == 2) { return launch_quantize_type<CrtCplxRows<2>>(stream, op, M, N, orderA, Atype, A, lda, vexp, B, ldb); }
  return launch_quantize_type<CrtCplxRows<3>>(stream, op, M, N, orderA, Atype, A, lda, vexp, B, ldb);
}

extern "C" int hykQuantizeCrt(hipStream_t stream, int32_t M, int32_t N, int32_t orderA, int32_t Atype, const void* A, int64_t lda, const int32_t* vexp, int8_t* B, int64_t ldb, int32_t maxBits) {
  return hykQuantizeCrtOp(stream, 'N', M, N, orderA, Atype, A, lda, vexp, B, ldb, maxBits);
}

extern "C" int hykZeroRows(hipStream_t stream, int8_t* B, int64_t ldb, int64_t cols, int32_t row0, int32_t row1) {
  if (cols <= 0 || row1 <= row0) { return 0; }
  if (cols > 2147483647ll) { return -1; }
  zero_rows_kernel<<<(uint32_t)cols, 128, 0, stream>>>(B, ldb, cols, row0, row1); return 0;
}
