/*
 * jacobi_rounds.h -- the one-sided Jacobi rounds on the N x r factor B (kernels and the per-sweep launch logic), as templates
 * over XT, the type of the elements of B in memory and of the rows a thread keeps in registers: double for FP64 storage,
 * float for FP32 / FP16 storage (the reference runs its SVD in the precision of the output storage type,
 * src/gram_evd.cu:96-98).  The small Gram matrix of a round, the rotation parameters and everything that decides a
 * rotation stay in FP64 for both: with float rows a thread sums its few products in float and hands the partial sums on
 * as doubles.  Included by tail.hip (double) and tail_f32.hip (float), one set of instantiations each.
 */
#pragma once
#include <type_traits>
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include "hyk_common.h"
#include "hyacin_kernels.h"

/* the float instantiations live in tail_f32.hip; same arguments as hykJacobiSweepTop plus the per-thread settings of tail.hip */
int hyk_jacobi_sweep_f32(hipStream_t stream, int32_t Complex, int32_t N, int32_t r, int32_t head, int32_t top, float* B, double tol, int32_t* rotations, double* carry, int variant, int splitTest);

namespace {

constexpr int T_THREADS = 256;

/* value of lane `j` (the same j in every lane, known at compile time after unrolling) in every lane: two scalar
 * register reads instead of a trip through the LDS crossbar */
__device__ __forceinline__ double lane_value(double v, int j) {
  const long long b = __double_as_longlong(v);
  const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)b, j), hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(b >> 32), j);
  return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}
__device__ __forceinline__ int lane_value(int v, int j) { return __builtin_amdgcn_readlane(v, j); }

/* Sums NV values (a power of two, at most 64) over the wavefront with NV - 1 + 6 - log2(NV) exchanges instead of 6 NV: in
 * the first log2(NV) steps a lane keeps one half of its values and trades the other half with its partner, so that it
 * ends with one value.  Returns, in every lane, the sum of value index_of(lane): the low log2(NV) bits of the lane,
 * reversed. */
/* lane exchange inside a row of 16 lanes through the data-parallel primitives (no LDS round trip):
 * CTRL 0xB1 / 0x4E: partner lane ^ 1 / lane ^ 2 (quad permutations); 0x124 / 0x128: lane - 4 / lane - 8 modulo 16 */
template <int CTRL>
__device__ __forceinline__ double row_exchange(double v) {
  const long long b = __double_as_longlong(v);
  const unsigned lo = (unsigned)__builtin_amdgcn_update_dpp(0, (int)(unsigned)b, CTRL, 0xf, 0xf, false);
  const unsigned hi = (unsigned)__builtin_amdgcn_update_dpp(0, (int)(unsigned)(b >> 32), CTRL, 0xf, 0xf, false);
  return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}
/* partner at distance OFF (1, 2: exchange with lane ^ OFF; 4, 8: the value of lane - OFF modulo 16, which sums a row just
 * as well and keeps the low bits of the lane; 16, 32: lane ^ OFF through the LDS crossbar) */
template <int OFF>
__device__ __forceinline__ double partner_value(double v) {
  if constexpr (OFF == 1) { return row_exchange<0xB1>(v); }
  else if constexpr (OFF == 2) { return row_exchange<0x4E>(v); }
  else if constexpr (OFF == 4) { return row_exchange<0x124>(v); }
  else if constexpr (OFF == 8) { return row_exchange<0x128>(v); }
  else { return __shfl_xor(v, OFF, 64); }
}

template <int NV>
__device__ __forceinline__ double wave_sum_split(double (&v)[NV]) {
  static_assert(NV >= 1 && NV <= 64 && (NV & (NV - 1)) == 0, "a power of two");
  const int lane = threadIdx.x & 63;
  /* splitting steps exchange with lane ^ off and need a true exchange: distances 1 and 2 by quad permutation, further
   * ones through the crossbar; the summing steps after them take the cheapest form of each distance */
  auto split = [&](auto n_, auto off_) {
    constexpr int n = decltype(n_)::value, off = decltype(off_)::value;
    const bool upper = (lane & off) != 0;
    #pragma unroll
    for (int i = 0; i < n / 2; ++i) {
      const double keep = upper ? v[i + n / 2] : v[i], send = upper ? v[i] : v[i + n / 2];
      if constexpr (off <= 2) { v[i] = keep + partner_value<off>(send); } else { v[i] = keep + __shfl_xor(send, off, 64); }
    }
  };
  if constexpr (NV >= 2) { split(std::integral_constant<int, NV>{}, std::integral_constant<int, 1>{}); }
  if constexpr (NV >= 4) { split(std::integral_constant<int, NV / 2>{}, std::integral_constant<int, 2>{}); }
  if constexpr (NV >= 8) { split(std::integral_constant<int, NV / 4>{}, std::integral_constant<int, 4>{}); }
  if constexpr (NV >= 16) { split(std::integral_constant<int, NV / 8>{}, std::integral_constant<int, 8>{}); }
  if constexpr (NV >= 32) { split(std::integral_constant<int, NV / 16>{}, std::integral_constant<int, 16>{}); }
  if constexpr (NV >= 64) { split(std::integral_constant<int, NV / 32>{}, std::integral_constant<int, 32>{}); }
  double s = v[0];
  if constexpr (NV < 2) { s += partner_value<1>(s); }
  if constexpr (NV < 4) { s += partner_value<2>(s); }
  if constexpr (NV < 8) { s += partner_value<4>(s); }
  if constexpr (NV < 16) { s += partner_value<8>(s); }
  if constexpr (NV < 32) { s += partner_value<16>(s); }
  if constexpr (NV < 64) { s += partner_value<32>(s); }
  return s;
}
/* The same sums taken from the top: the halving steps at distances 32 and 16 are register swaps between lane halves
 * (v_permlane32_swap / v_permlane16_swap: after swapping a and b, a + b holds the sum of a in the lower lanes and of b in
 * the upper ones; three instructions per double instead of the seven of a select-and-exchange), and only NV / 4 values
 * are left for the distances below.  NV a power of two, 4 .. 32.  Returns, in every lane, the sum of value
 * lane >> (6 - log2 NV). */
typedef unsigned v2u_t __attribute__((ext_vector_type(2)));
template <int OFF>
__device__ __forceinline__ double swap_add(double a, double b) {
  const long long ab = __double_as_longlong(a), bb = __double_as_longlong(b);
  v2u_t lo, hi;
  if constexpr (OFF == 32) { lo = __builtin_amdgcn_permlane32_swap((unsigned)ab, (unsigned)bb, false, false); hi = __builtin_amdgcn_permlane32_swap((unsigned)(ab >> 32), (unsigned)(bb >> 32), false, false); }
  else { lo = __builtin_amdgcn_permlane16_swap((unsigned)ab, (unsigned)bb, false, false); hi = __builtin_amdgcn_permlane16_swap((unsigned)(ab >> 32), (unsigned)(bb >> 32), false, false); }
  return __longlong_as_double((long long)(((unsigned long long)hi.x << 32) | lo.x)) + __longlong_as_double((long long)(((unsigned long long)hi.y << 32) | lo.y));
}
template <int OFF>
__device__ __forceinline__ double xor_value(double v) {   /* the value of lane ^ OFF, OFF <= 8 */
  if constexpr (OFF == 4) { return __shfl_xor(v, 4, 64); } else { return partner_value<OFF>(v); }   /* a rotation by 8 inside a row of 16 is lane ^ 8 */
}
template <int NV>
__device__ __forceinline__ double wave_sum_swap(double (&v)[NV]) {
  static_assert(NV >= 4 && NV <= 32 && (NV & (NV - 1)) == 0, "a power of two, 4 .. 32");
  const int lane = threadIdx.x & 63;
  #pragma unroll
  for (int i = 0; i < NV / 2; ++i) { v[i] = swap_add<32>(v[i], v[i + NV / 2]); }
  #pragma unroll
  for (int i = 0; i < NV / 4; ++i) { v[i] = swap_add<16>(v[i], v[i + NV / 4]); }
  auto split = [&](auto n_, auto off_) {
    constexpr int n = decltype(n_)::value, off = decltype(off_)::value;
    const bool upper = (lane & off) != 0;
    #pragma unroll
    for (int i = 0; i < n / 2; ++i) {
      const double keep = upper ? v[i + n / 2] : v[i], send = upper ? v[i] : v[i + n / 2];
      v[i] = keep + xor_value<off>(send);
    }
  };
  if constexpr (NV >= 8) { split(std::integral_constant<int, NV / 4>{}, std::integral_constant<int, 8>{}); }
  if constexpr (NV >= 16) { split(std::integral_constant<int, NV / 8>{}, std::integral_constant<int, 4>{}); }
  if constexpr (NV >= 32) { split(std::integral_constant<int, NV / 16>{}, std::integral_constant<int, 2>{}); }
  double s = v[0];
  if constexpr (NV < 8) { s += xor_value<8>(s); }
  if constexpr (NV < 16) { s += xor_value<4>(s); }
  if constexpr (NV < 32) { s += xor_value<2>(s); }
  s += xor_value<1>(s);
  return s;
}
template <int NV> __device__ __forceinline__ int split_index(int lane) {
  int idx = 0, half = NV >> 1;
  #pragma unroll
  for (int bit = 1; bit < NV; bit <<= 1, half >>= 1) { if (lane & bit) { idx += half; } }
  return idx;
}

__device__ __forceinline__ double block_sum(double v, double* scratch) {
  for (int off = 32; off > 0; off >>= 1) { v += __shfl_xor(v, off, 64); }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) { scratch[threadIdx.x >> 6] = v; }
  __syncthreads();
  double s = 0.; for (int w = 0; w < T_THREADS / 64; ++w) { s += scratch[w]; }
  return s;
}

/* The sweep kernels report the largest squared cosine g^2 / (alpha beta) they met, rotated or not, as the bit pattern of a
 * double at rotations + 2 (non-negative doubles order like their bit patterns, so an integer maximum does it). */
__device__ __forceinline__ void report_cosine(int32_t* rotations, double cos2) {
  if (cos2 > 0.) { atomicMax(reinterpret_cast<unsigned long long*>(rotations + 2), (unsigned long long)__double_as_longlong(cos2)); }
}
__device__ __forceinline__ double squared_cosine(double g2, double alpha, double beta) {
  const double ab = alpha * beta;
  return ab > 0. ? g2 / ab : (g2 > 0. ? 1. : 0.);   /* a column whose carried norm has collapsed counts as not converged */
}

template <bool CPLX, typename XT>
__global__ __launch_bounds__(T_THREADS) void jacobi_round_kernel(int32_t N, int32_t n, int32_t r, int32_t head, int32_t top, int32_t round, XT* __restrict__ B, double tol, int32_t* __restrict__ rotations) {
  __shared__ double scratch[T_THREADS / 64];
  const int i = blockIdx.x; int p, q;
  if (i == 0) { p = n - 1; q = round; } else { p = (round + i) % (n - 1); q = (round - i + (n - 1)) % (n - 1); }
  if (p >= r || q >= r) { return; }
  if (p > q) { int t = p; p = q; q = t; }
  if (p >= top) { return; }                        /* both columns belong to the tail that is left alone */
  constexpr int W = CPLX ? 2 : 1;
  XT* bp = &B[(int64_t)p * N * W]; XT* bq = &B[(int64_t)q * N * W];   /* arithmetic in FP64 whatever the storage */
  double alpha = 0., beta = 0., gre = 0., gim = 0.;
  for (int k = threadIdx.x; k < N; k += T_THREADS) {
    if constexpr (CPLX) {
      const double pr = bp[2 * k], pi = bp[2 * k + 1], qr = bq[2 * k], qi = bq[2 * k + 1];
      alpha += pr * pr + pi * pi; beta += qr * qr + qi * qi; gre += pr * qr + pi * qi; gim += pr * qi - pi * qr;   /* conj(p) q */
    } else { const double pv = bp[k], qv = bq[k]; alpha += pv * pv; beta += qv * qv; gre += pv * qv; }
  }
  alpha = block_sum(alpha, scratch); beta = block_sum(beta, scratch); gre = block_sum(gre, scratch); if constexpr (CPLX) { gim = block_sum(gim, scratch); }
  const double g2 = gre * gre + gim * gim;
  if (threadIdx.x == 0 && p < head) { report_cosine(rotations, squared_cosine(g2, alpha, beta)); }
  if (!(g2 > tol * tol * alpha * beta) || !(g2 > 0.)) { return; }
  const double gabs = sqrt(g2), zeta = (beta - alpha) / (2. * gabs);
  const double t = (zeta >= 0. ? 1. : -1.) / (fabs(zeta) + sqrt(1. + zeta * zeta)), cs = 1. / sqrt(1. + t * t), sn = cs * t;
  const double er = gre / gabs, ei = gim / gabs;   /* e^{i phi}; column q is first multiplied by e^{-i phi} so that the cross term is real */
  for (int k = threadIdx.x; k < N; k += T_THREADS) {
    if constexpr (CPLX) {
      const double pr = bp[2 * k], pi = bp[2 * k + 1], q0 = bq[2 * k], q1 = bq[2 * k + 1];
      const double qr = q0 * er + q1 * ei, qi = q1 * er - q0 * ei;
      bp[2 * k] = (XT)(cs * pr - sn * qr); bp[2 * k + 1] = (XT)(cs * pi - sn * qi); bq[2 * k] = (XT)(sn * pr + cs * qr); bq[2 * k + 1] = (XT)(sn * pi + cs * qi);
    } else { const double pv = bp[k], qv = bq[k] * er; bp[k] = (XT)(cs * pv - sn * qv); bq[k] = (XT)(sn * pv + cs * qv); }
  }
  if (threadIdx.x == 0) { atomicAdd(rotations, 1); }
}

/* ------------------------------------------------------------------ blocked one-sided Jacobi
 * A round of the plain kernel above moves every column through memory once per pair it takes part in.  Here a workgroup
 * takes a pair of column blocks (BC columns each), keeps its rows of all 2 BC columns in registers (thread t owns rows
 * t, t + 256, ...) and rotates every cross pair (BC steps of BC disjoint pairs) before writing them back: BC times fewer
 * passes over B per sweep.  In the first round of a sweep the 2 BC columns go through a full round-robin instead, which
 * also covers the pairs inside each block.  Column norms are summed once per round and carried through the rotations
 * (alpha' = alpha - t gamma, beta' = beta + t gamma); only the BC cross products of a step need a workgroup reduction.
 * Blocks of 8 columns (512 threads, 4 rows each) halve the passes again but take 2.7 times as long per round on this
 * device (half as many workgroups as compute units, twice the reduction work per workgroup): 4-column blocks stay. */
/* Sums NV values over the workgroup; lane i < NV of every wavefront returns the sum of value i.  `red` holds two halves of
 * HALF doubles used alternately (`parity`), so that one barrier per call is enough: a wavefront can only be two calls
 * ahead of the slowest one after that one has left the half. */
template <int NV, int THREADS, int HALF>
__device__ __forceinline__ double block_sum_lanes(double (&v)[NV], double* red, int parity) {
  static_assert((THREADS / 64) * NV <= HALF, "a half holds one value per wavefront and summand");
  static_assert(NV <= 64, "one lane per summand");
  double* mine = red + parity * HALF;
  if constexpr ((NV & (NV - 1)) == 0) {
    const double part = wave_sum_split<NV>(v);
    if ((threadIdx.x & 63) < NV) { mine[(threadIdx.x >> 6) * NV + split_index<NV>(threadIdx.x & 63)] = part; }
  } else {
    #pragma unroll
    for (int i = 0; i < NV; ++i) {
      #pragma unroll
      for (int off = 32; off > 0; off >>= 1) { v[i] += __shfl_xor(v[i], off, 64); }
    }
    if ((threadIdx.x & 63) == 0) {
      #pragma unroll
      for (int i = 0; i < NV; ++i) { mine[(threadIdx.x >> 6) * NV + i] = v[i]; }
    }
  }
  __syncthreads();
  double s = 0.; const int lane = threadIdx.x & 63;
  if (lane < NV) { for (int w = 0; w < THREADS / 64; ++w) { s += mine[w * NV + lane]; } }
  return s;
}
/* the same, every thread gets all NV sums */
template <int NV, int THREADS, int HALF>
__device__ __forceinline__ void block_sum_many(double (&v)[NV], double* red, int parity) {
  const double s = block_sum_lanes<NV, THREADS, HALF>(v, red, parity);
  #pragma unroll
  for (int i = 0; i < NV; ++i) { v[i] = lane_value(s, i); }
}

template <typename XT, bool CPLX, int ROWS, int BC, bool FULL, int THREADS>
__global__ __launch_bounds__(THREADS) void jacobi_block_round_kernel(int32_t N, int32_t nb, int32_t r, int32_t head, int32_t top, int32_t round, XT* __restrict__ B, double tol, int32_t* __restrict__ rotations) {
  constexpr int W = CPLX ? 2 : 1, NC = 2 * BC, GV = BC * W;
  constexpr int HALF = (THREADS / 64) * (NC > GV ? NC : GV);
  __shared__ double red[2 * HALF];
  const int i = blockIdx.x; int P, Q;
  if (i == 0) { P = nb - 1; Q = round; } else { P = (round + i) % (nb - 1); Q = (round - i + (nb - 1)) % (nb - 1); }
  if (P > Q) { const int t = P; P = Q; Q = t; }
  int col[NC]; bool live[NC];
  #pragma unroll
  for (int c = 0; c < NC; ++c) { col[c] = (c < BC ? P : Q) * BC + (c % BC); live[c] = col[c] < r; }
  if (!live[0] || col[0] >= top) { return; }      /* both blocks beyond the last column, or wholly in the tail that is left alone */
  /* rows of this thread */
  double x[NC][ROWS][W];
  #pragma unroll
  for (int c = 0; c < NC; ++c) {
    #pragma unroll
    for (int m = 0; m < ROWS; ++m) {
      const int k = threadIdx.x + m * THREADS;
      #pragma unroll
      for (int w = 0; w < W; ++w) { x[c][m][w] = (live[c] && k < N) ? (double)B[((int64_t)col[c] * N + k) * W + w] : 0.; }   /* rows and arithmetic in FP64 whatever the storage */
    }
  }
  double norm[NC];
  #pragma unroll
  for (int c = 0; c < NC; ++c) {
    double s = 0.;
    #pragma unroll
    for (int m = 0; m < ROWS; ++m) {
      #pragma unroll
      for (int w = 0; w < W; ++w) { s += x[c][m][w] * x[c][m][w]; }
    }
    norm[c] = s;
  }
  block_sum_many<NC, THREADS, HALF>(norm, red, 0);
  int applied = 0; double worst = 0.;
  /* FULL: first round of a sweep, all pairs of the 2 BC columns (round-robin); otherwise the BC x BC cross pairs */
  constexpr int STEPS = FULL ? NC - 1 : BC;
  #pragma unroll
  for (int step = 0; step < STEPS; ++step) {
    double g[GV];
    #pragma unroll
    for (int j = 0; j < BC; ++j) {
      const int fa = (j == 0) ? NC - 1 : (step + j) % (NC - 1), fb = (j == 0) ? step : (step - j + (NC - 1)) % (NC - 1);
      const int c0 = FULL ? (fa < fb ? fa : fb) : j, c1 = FULL ? (fa < fb ? fb : fa) : BC + (j + step) % BC;
      double gr = 0., gi = 0.;
      #pragma unroll
      for (int m = 0; m < ROWS; ++m) {
        if constexpr (CPLX) { gr += x[c0][m][0] * x[c1][m][0] + x[c0][m][1] * x[c1][m][1]; gi += x[c0][m][0] * x[c1][m][1] - x[c0][m][1] * x[c1][m][0]; }
        else { gr += x[c0][m][0] * x[c1][m][0]; }
      }
      g[j * W] = gr; if constexpr (CPLX) { g[j * W + 1] = gi; }
    }
    /* lane j < BC of every wavefront works out the rotation of pair j (square roots and divisions once instead of BC
     * times per thread), then the lanes hand the parameters round */
    const double sum = block_sum_lanes<GV, THREADS, HALF>(g, red, (step + 1) & 1);
    const int lane = threadIdx.x & 63;
    double gre = sum, gim = 0.;
    if constexpr (CPLX) { gre = __shfl(sum, 2 * lane, 64); gim = __shfl(sum, 2 * lane + 1, 64); }
    double alpha = 0., beta = 0.; bool pairLive = false, counted = false;
    #pragma unroll
    for (int j = 0; j < BC; ++j) {
      const int fa = (j == 0) ? NC - 1 : (step + j) % (NC - 1), fb = (j == 0) ? step : (step - j + (NC - 1)) % (NC - 1);
      const int c0 = FULL ? (fa < fb ? fa : fb) : j, c1 = FULL ? (fa < fb ? fb : fa) : BC + (j + step) % BC;
      if (lane == j) { alpha = norm[c0]; beta = norm[c1]; pairLive = live[c0] && live[c1] && (col[c0] < top || col[c1] < top); counted = col[c0] < head || col[c1] < head; }
    }
    const double g2 = gre * gre + gim * gim;
    if (pairLive && counted) {                     /* worst = max(worst, squared_cosine(g2, alpha, beta)), dividing only where the maximum moves */
      const double ab = alpha * beta;
      if (ab > 0.) { if (g2 > worst * ab) { worst = g2 / ab; } } else if (g2 > 0.) { worst = fmax(worst, 1.); }
    }
    const bool rotate = pairLive && g2 > tol * tol * alpha * beta && g2 > 0.;
    double cs = 1., sn = 0., er = 1., ei = 0., shift = 0.;
    if (rotate) {
      /* t = tan of the rotation angle = sign(d) h / (|d| + sqrt(d^2 + h^2)) with d = beta - alpha, h = 2 |g|: the smaller
       * root of t^2 + 2 (d / h) t - 1 = 0 without the division by h; d and h are first scaled by one power of two, so
       * that their squares neither overflow nor vanish.  One square root, one division and one reciprocal square root
       * in sequence (the textbook order takes three of each kind, each waiting for the one before). */
      double gabs;
      if constexpr (CPLX) { gabs = sqrt(g2); const double inv = 1. / gabs; er = gre * inv; ei = gim * inv; }
      else { gabs = fabs(gre); er = gre < 0. ? -1. : 1.; }
      const double d = beta - alpha, h = 2. * gabs;
      const int e = __builtin_amdgcn_frexp_exp(fmax(fabs(d), h));
      const double ds = ldexp(fabs(d), -e), hs = ldexp(h, -e);
      const double t = copysign(hs / (ds + sqrt(ds * ds + hs * hs)), d);
      cs = rsqrt(1. + t * t); sn = cs * t; shift = t * gabs;
    }
    #pragma unroll
    for (int j = 0; j < BC; ++j) {
      const int fa = (j == 0) ? NC - 1 : (step + j) % (NC - 1), fb = (j == 0) ? step : (step - j + (NC - 1)) % (NC - 1);
      const int c0 = FULL ? (fa < fb ? fa : fb) : j, c1 = FULL ? (fa < fb ? fb : fa) : BC + (j + step) % BC;
      if (lane_value((int)rotate, j)) {
        const double csj = lane_value(cs, j), snj = lane_value(sn, j), shj = lane_value(shift, j);
        if constexpr (CPLX) {
          const double erj = lane_value(er, j), eij = lane_value(ei, j);
          #pragma unroll
          for (int m = 0; m < ROWS; ++m) {
            const double pr = x[c0][m][0], pi = x[c0][m][1], q0 = x[c1][m][0], q1 = x[c1][m][1];
            const double qr = q0 * erj + q1 * eij, qi = q1 * erj - q0 * eij;
            x[c0][m][0] = csj * pr - snj * qr; x[c0][m][1] = csj * pi - snj * qi; x[c1][m][0] = snj * pr + csj * qr; x[c1][m][1] = snj * pi + csj * qi;
          }
        } else {
          /* real: e^{i phi} = +-1, folded into the coefficients of column c1 as a sign bit (same bits as multiplying the column first) */
          const long long flip = (long long)(unsigned long long)(unsigned)lane_value((int)(er < 0.), j) << 63;
          const double aj = __longlong_as_double(__double_as_longlong(snj) ^ flip), bj = __longlong_as_double(__double_as_longlong(csj) ^ flip);
          #pragma unroll
          for (int m = 0; m < ROWS; ++m) {
            const double pv = x[c0][m][0], qv = x[c1][m][0];
            x[c0][m][0] = csj * pv - aj * qv; x[c1][m][0] = snj * pv + bj * qv;
          }
        }
        norm[c0] -= shj; norm[c1] += shj; ++applied;
      }
    }
  }
  #pragma unroll
  for (int off = BC / 2; off > 0; off >>= 1) { worst = fmax(worst, __shfl_xor(worst, off, 64)); }   /* lanes 0 .. BC-1 hold the pairs */
  if (threadIdx.x == 0) { report_cosine(rotations, worst); }
  if (applied == 0) { return; }                  /* nothing rotated (same decision in every thread): the columns in memory are current */
  #pragma unroll
  for (int c = 0; c < NC; ++c) {
    #pragma unroll
    for (int m = 0; m < ROWS; ++m) {
      const int k = threadIdx.x + m * THREADS;
      if (live[c] && k < N) {
        #pragma unroll
        for (int w = 0; w < W; ++w) { B[((int64_t)col[c] * N + k) * W + w] = (XT)x[c][m][w]; }
      }
    }
  }
  if (threadIdx.x == 0) { atomicAdd(rotations, applied); }
}

/* ------------------------------------------------------------------ blocked one-sided Jacobi in Gram space (real)
 * The kernel above pays one workgroup reduction, one barrier and one chain of square roots and divisions per step.  Here a
 * round takes ONE reduction: the Gram matrix of the workgroup's 2 BC columns (all NC (NC + 1) / 2 products, summed over the
 * rows).  The first wavefront then runs the steps on that small matrix alone (G <- J^T G J per step, kept in LDS) and leaves the list of rotations in
 * LDS; after one more barrier every thread replays the list on its rows.  Same pairs, same order, same rotation rule as the
 * step kernel; the cross products of later steps come out of the updated Gram matrix instead of fresh dot products (both
 * carry rounding noise of the size eps |x_i| |x_j|; the next round starts from fresh sums again). */
struct RotRec { double cs, sn, a, b; };   /* x_c0' = cs x_c0 - a x_c1,  x_c1' = sn x_c0 + b x_c1;  sn == 0: no rotation */
/* The same rotation on columns kept as scale x vector (x_c = s_c u_c), as two shears in sequence: u_c0' = u_c0 - t1 u_c1, then
 * u_c1' = u_c1 + t2 u_c0' with t1 = a s_c1 / (cs s_c0), t2 = a cs s_c0 / s_c1, and s_c0' = cs s_c0, s_c1' = b s_c1 / cs^2: two
 * multiply-adds per row, in place, instead of two products and two multiply-adds; the scales (within 2^-8 .. 2^8 over the at
 * most 15 rotations a column meets in a round) are multiplied in once, before the columns are stored.  t1 == t2 == 0: no
 * rotation. */
struct FastRot { double t1, t2; };

/* 1 / z and 1 / sqrt(z) for z of ordinary size (no scaling, no fix-up of special values): hardware approximation, two
 * Newton steps; the result is within an ulp or two of the exact one. */
__device__ __forceinline__ double rcp_newton(double z) {
  double y = __builtin_amdgcn_rcp(z);
  y = fma(y, fma(-z, y, 1.), y); y = fma(y, fma(-z, y, 1.), y);
  return y;
}
__device__ __forceinline__ double rsqrt_newton(double z) {
  double y = __builtin_amdgcn_rsq(z);
  y = fma(0.5 * y, fma(-z * y, y, 1.), y); y = fma(0.5 * y, fma(-z * y, y, 1.), y);
  return y;
}

__device__ __forceinline__ void wave_lds_sync() {   /* LDS operations of one wavefront complete in order: only the compiler must not move them */
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier(); __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

/* Phase timing of the real Gram-space round (measurement builds only, -DHYK_JACOBI_TIMING): workgroup 1's first thread
 * stamps the 100 MHz counter between the phases and adds the differences to the six 64-bit words behind the 16 bytes of
 * `rotations` that the sweep uses. */
#ifdef HYK_JACOBI_TIMING
#define HYK_JDECL() long long hyk_t0 = 0, hyk_t1 = 0, hyk_t2 = 0, hyk_t3 = 0, hyk_t4 = 0, hyk_t5 = 0, hyk_t6 = 0
#define HYK_JSTAMP(i) if (blockIdx.x == 1 && threadIdx.x == 0) { hyk_t##i = (long long)__builtin_readcyclecounter(); }
#define HYK_JWAIT() asm volatile("s_waitcnt vmcnt(0)" ::: "memory")
#define HYK_JREPORT() if (blockIdx.x == 1 && threadIdx.x == 0) { unsigned long long* w = reinterpret_cast<unsigned long long*>(rotations) + 2; \
  atomicAdd(&w[0], (unsigned long long)(hyk_t1 - hyk_t0)); atomicAdd(&w[1], (unsigned long long)(hyk_t2 - hyk_t1)); atomicAdd(&w[2], (unsigned long long)(hyk_t3 - hyk_t2)); \
  atomicAdd(&w[3], (unsigned long long)(hyk_t4 - hyk_t3)); atomicAdd(&w[4], (unsigned long long)(hyk_t5 - hyk_t4)); atomicAdd(&w[5], (unsigned long long)(hyk_t6 - hyk_t5)); }
#else
#define HYK_JDECL()
#define HYK_JSTAMP(i)
#define HYK_JWAIT()
#define HYK_JREPORT()
#endif

/* CARRY: the products inside a block (x_i . x_j, i < j in the same block of BC columns) travel with the block from round
 * to round in `carry` (BC (BC - 1) / 2 doubles per block) instead of being summed again: the first round of a sweep (FULL)
 * sums everything and writes them, the other rounds sum the norms and the BC^2 cross products only (80 of 136 products
 * for BC = 8) and take the rest from the small matrix as the previous round's steps left it.  The norms and the cross
 * products, which decide every rotation of the round, are always fresh; what is carried only feeds the update of cross
 * products inside a round, multiplied by the sine of a rotation. */
template <int BC> __device__ __forceinline__ void carried_pair(int t, int& i, int& j) { i = 0; while (t >= BC - 1 - i) { t -= BC - 1 - i; ++i; } j = i + 1 + t; }

/* PASSES = 2: factors with twice the rows that fit the registers.  The rows are taken in two halves: the sums of the first
 * half, then of the second (which stays in registers), the steps, and the replay on the second half and then on the first,
 * loaded again: three loads and two stores of half the rows instead of one each of all, for blocks twice as wide. */
/* SPLIT: two workgroups per block pair, partners on one XCD.  Both load all rows, form the same sums in the same order and
 * therefore work out the same rotations, bit for bit; each replays them on one half of the rows only (the first or the last
 * two of a thread's four) and stores that half: the second read of the pair's rows comes out of the L2 the partner filled,
 * and the replay of the first wavefront and the stores, which end a round, are half as long.  For the launches that leave
 * half of the compute units idle otherwise.
 * The round works in place, so a partner must never load rows that the other has already rotated and stored, however far
 * apart the device dispatches the two.  One 32-bit word per pair and round (zero before the launch) orders them:
 *   bits 0-1  workgroups that have arrived (fetch-add on arrival);
 *   bit 2, 3  this half's workgroup has all its loads (rows and carried products) in registers;
 *   bit 4     one workgroup has taken the whole pair.
 * Before it stores, a workgroup looks at the word.  The partner has loaded: it stores its half.  The partner has arrived
 * but not finished loading: it waits (the partner is running and sets its bit without waiting for anything; the wait is
 * bounded all the same and, given up, raises rotations[1], which the host reports as a failure).  The partner has not
 * arrived: a compare-and-swap from exactly "one arrival, my loads done" sets bit 4, and this workgroup then rotates and
 * stores both halves (it loads the other half's rows again and replays the round's rotations from LDS); a partner that
 * arrives afterwards finds bit 4 in what its fetch-add returns and leaves without storing anything (whatever it has
 * loaded meanwhile is discarded).  If the swap fails, the partner has arrived in between: wait as above.  So no load
 * whose values are used can observe a store of the same launch.  The cosine, the rotation count and the carried
 * products are written by the workgroup that is sure to finish: the first half's, or the one that took the pair. */
template <typename XT, int ROWS, int BC, bool FULL, int THREADS, bool CARRY, int PASSES, bool SPLIT = false>
__global__ __launch_bounds__(THREADS) void jacobi_gram_round_kernel(int32_t N, int32_t nb, int32_t r, int32_t head, int32_t top, int32_t round, XT* __restrict__ B, double tol, int32_t* __restrict__ rotations, double* __restrict__ carry, uint32_t* __restrict__ pairWords, int32_t splitTest) {
  constexpr int NC = 2 * BC, NG = NC * (NC + 1) / 2, WAVES = THREADS / 64, STEPS = FULL ? NC - 1 : BC, GS = NC + 1;
  constexpr bool SLIM = CARRY && !FULL;                    /* norms and cross products only */
  constexpr uint32_t PW_COUNT = 3u, PW_LOADED = 4u, PW_TAKEN = 16u;   /* the pair's word: arrivals, loaded bits (<< half), pair taken by one workgroup */
  constexpr int PWAVE = WAVES - 1;                          /* the wavefront that handles the word (not the first: nothing may sit on the chain of steps) */
  constexpr int NW = BC * (BC - 1) / 2, NP = SLIM ? NC + BC * BC : NG;
  constexpr int CH = NP >= 32 ? 32 : 16, TAIL = NP % CH;
  static_assert((TAIL & (TAIL - 1)) == 0 && (TAIL == 0 || TAIL >= 4) && BC * BC <= 64 && 2 * NW <= 64, "tail chunk a power of two; one lane of the first wavefront per pair of pairs and per carried product");
  auto pair_of = [](int p, int& c0, int& c1) {
    if (!SLIM) { c0 = p % NC; c1 = (c0 + p / NC) % NC; }
    else if (p < NC) { c0 = p; c1 = p; }
    else { c0 = (p - NC) / BC; c1 = BC + (p - NC) % BC; }
  };
  __shared__ double part[WAVES][NP];
  __shared__ double Gs[NC * GS];
  __shared__ RotRec rot[STEPS][BC];
  __shared__ FastRot fast[STEPS][BC];
  __shared__ double scale[NC];
  __shared__ double iscale[NC];
  __shared__ double fixed[BC][2];
  __shared__ int32_t pairCol[BC][2];
  __shared__ int32_t appliedAll;
  __shared__ int32_t stepsReady;
  __shared__ double worstAll;
  __shared__ int32_t pairTaken;     /* split rounds: the partner has taken the whole pair, nothing to do here */
  __shared__ int32_t storeMode;     /* split rounds: 0 undecided, 1 this half only, 2 both halves, 3 gave up */
  /* Workgroups go to the 8 XCDs in turn.  Pair i of a round takes its blocks over from the pairs i - 1 and i + 1 of the round
   * before: with the pairs numbered so that neighbours run on the same XCD, most of what a workgroup loads was written
   * through the L2 it sits behind. */
  static_assert(!SPLIT || (!FULL && PASSES == 1 && ROWS == 4), "the split round halves the four rows of a thread");
  const int pairs = nb / 2, xcd = blockIdx.x % 8, slot = (int)(blockIdx.x / 8), half = SPLIT ? (slot & 1) : 0;   /* XCD x takes a contiguous range of pairs */
  if (SPLIT && (slot >> 1) >= pairs / 8 + (xcd < pairs % 8 ? 1 : 0)) { return; }   /* the grid is rounded up to whole XCD rows */
  const int i = xcd * (pairs / 8) + (xcd < pairs % 8 ? xcd : pairs % 8) + (SPLIT ? (slot >> 1) : slot); int P, Q;
  constexpr int RROWS = SPLIT ? ROWS / 2 : ROWS;   /* rows of a thread that this workgroup rotates and stores: registers x[c][0 .. RROWS) once the sums are done */
  if (i == 0) { P = nb - 1; Q = round; } else { P = (round + i) % (nb - 1); Q = (round - i + (nb - 1)) % (nb - 1); }
  if (P > Q) { const int t = P; P = Q; Q = t; }
  int col[NC]; bool live[NC];
  #pragma unroll
  for (int c = 0; c < NC; ++c) { col[c] = (c < BC ? P : Q) * BC + (c % BC); live[c] = col[c] < r; }
  if (!live[0]) { return; }
  /* Columns from `top` on are the tail that is left alone: pairs of two tail columns are not rotated.  A block pair wholly
   * in the tail has nothing to do, except in the first round of a sweep, which also refreshes the carried products. */
  if (!FULL && col[0] >= top) { return; }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  HYK_JDECL(); HYK_JSTAMP(0);
  [[maybe_unused]] double carried = 0.;
  if constexpr (SLIM) { if (wave == 0 && lane < 2 * NW) { carried = carry[(int64_t)(lane < NW ? P : Q) * NW + lane % NW]; } }
  [[maybe_unused]] uint32_t* const word = SPLIT ? &pairWords[(int64_t)(round - 1) * pairs + i] : nullptr;
  [[maybe_unused]] uint32_t arrival = 0u;

  static_assert(PASSES == 1 || PASSES == 2, "all rows at once or in two halves");
  XT x[NC][ROWS];
  typedef XT xt2 __attribute__((ext_vector_type(2)));
  /* a thread owns pairs of adjacent rows: one load or store per pair where the columns are aligned to a pair (N even) */
  static_assert(ROWS % 2 == 0, "rows are owned in adjacent pairs");
  const bool vec2 = (N & 1) == 0 && (reinterpret_cast<uintptr_t>(B) & (2 * sizeof(XT) - 1)) == 0;
  auto row_of = [&](int pass, int m) { return 2 * (int)threadIdx.x + (m & 1) + (m >> 1) * 2 * THREADS + pass * ROWS * THREADS; };
  auto load_rows = [&](int pass) {
    if (vec2) {
      #pragma unroll
      for (int c = 0; c < NC; ++c) {
        #pragma unroll
        for (int m = 0; m < ROWS; m += 2) {
          const int k = row_of(pass, m); xt2 v = { (XT)0, (XT)0 };
          if (live[c] && k < N) { v = *reinterpret_cast<const xt2*>(&B[(int64_t)col[c] * N + k]); }
          x[c][m] = v.x; x[c][m + 1] = v.y;
        }
      }
    } else {
      #pragma unroll
      for (int c = 0; c < NC; ++c) {
        #pragma unroll
        for (int m = 0; m < ROWS; ++m) { const int k = row_of(pass, m); x[c][m] = (live[c] && k < N) ? B[(int64_t)col[c] * N + k] : (XT)0; }
      }
    }
  };
  auto store_rows = [&](int pass, int half) {
    if (vec2) {
      #pragma unroll
      for (int c = 0; c < NC; ++c) {
        #pragma unroll
        for (int m = 0; m < RROWS; m += 2) {
          const int k = row_of(pass, m + half * RROWS);
          /* past the caches: the next round's readers find the rows in memory either way, and the end of the launch has less to write back (a sweep at N = r = 2048: 4.70 -> 4.60 ms; the complex kernel loses with the same stores) */
          if (live[c] && k < N) { __builtin_nontemporal_store(xt2{ x[c][m], x[c][m + 1] }, reinterpret_cast<xt2*>(&B[(int64_t)col[c] * N + k])); }
        }
      }
    } else {
      #pragma unroll
      for (int c = 0; c < NC; ++c) {
        #pragma unroll
        for (int m = 0; m < RROWS; ++m) { const int k = row_of(pass, m + half * RROWS); if (live[c] && k < N) { B[(int64_t)col[c] * N + k] = x[c][m]; } }
      }
    }
  };
  #pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
  load_rows(pass);
  /* arrival at the pair's word, asked behind the row loads (memory answers a wavefront in order, and an atomic takes longer than a load: asked first, it would hold this wavefront's rows back); the answer is needed after the sums */
  if constexpr (SPLIT) {
    if (wave == PWAVE && lane == 0) {
      /* tests (hykJacobiSetSplitTest 1 / 2): this half's workgroup arrives only after the partner has taken the pair, as a workgroup does that the device dispatches late */
      if ((splitTest == 1 && half == 1) || (splitTest == 2 && half == 0)) { for (int spin = 0; spin < (1 << 22) && !(__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & PW_TAKEN); ++spin) { __builtin_amdgcn_s_sleep(8); } }
      arrival = __hip_atomic_fetch_add(word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  HYK_JWAIT(); HYK_JSTAMP(1);
  /* products numbered by diagonal: p = d NC + c stands for (c, (c + d) % NC), d = 0 .. NC / 2 (the last diagonal only for
   * c < NC / 2): every unordered pair once, and p splits back into the pair by shifts.  Summed over the wavefront 32 at a time. */
  #pragma unroll
  for (int chunk = 0; chunk < NP / CH; ++chunk) {
    double v[CH];
    #pragma unroll
    for (int q = 0; q < CH; ++q) {
      int c0 = 0, c1 = 0; pair_of(chunk * CH + q, c0, c1);
      XT sum = (XT)0;   /* a thread's few products in the precision of its rows, the sums across threads in FP64 */
      #pragma unroll
      for (int m = 0; m < ROWS; ++m) { sum = fma(x[c0][m], x[c1][m], sum); }
      v[q] = (double)sum;
    }
    const double tot = wave_sum_swap<CH>(v);
    if ((lane & (64 / CH - 1)) == 0) { double* slot = &part[wave][chunk * CH + lane / (64 / CH)]; *slot = pass == 0 ? tot : *slot + tot; }
  }
  if constexpr (TAIL > 0) {
    double v[TAIL];
    #pragma unroll
    for (int q = 0; q < TAIL; ++q) {
      int c0 = 0, c1 = 0; pair_of((NP / CH) * CH + q, c0, c1);
      XT sum = (XT)0;   /* a thread's few products in the precision of its rows, the sums across threads in FP64 */
      #pragma unroll
      for (int m = 0; m < ROWS; ++m) { sum = fma(x[c0][m], x[c1][m], sum); }
      v[q] = (double)sum;
    }
    const double tot = wave_sum_swap<TAIL>(v);
    if ((lane & (64 / TAIL - 1)) == 0) { double* slot = &part[wave][(NP / CH) * CH + lane / (64 / TAIL)]; *slot = pass == 0 ? tot : *slot + tot; }
  }
  }   /* passes */
  HYK_JSTAMP(2);
  if constexpr (SPLIT) {   /* the rows of this workgroup's half into the first registers; the others are done with */
    #pragma unroll
    for (int c = 0; c < NC; ++c) {
      #pragma unroll
      for (int m = 0; m < RROWS; ++m) {
        XT lo = x[c][m], hi = x[c][m + RROWS];
        asm volatile("" : "+v"(lo), "+v"(hi));   /* two values, not one element picked by a run-time index (which would put the rows into scratch memory) */
        x[c][m] = half ? hi : lo;
      }
    }
  }
  if (threadIdx.x == 0) { stepsReady = 0; }
  if constexpr (SPLIT) {
    if (wave == 0) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }   /* the carried products are in registers too (the rows are: the sums have used them) */
    if (wave == PWAVE && lane == 0) { pairTaken = (arrival & PW_TAKEN) ? 1 : 0; storeMode = 0; }
  }
  __syncthreads();
  if constexpr (SPLIT) {
    if (pairTaken) { return; }   /* uniform: the partner rotates and stores both halves; what was loaded here may be half rotated and is dropped */
    if (splitTest == 3 && half == 1) { return; }   /* tests: a partner that arrives and is never heard of again */
    /* Every load of this workgroup has returned: each thread has used its rows in the sums, and the barrier has passed.  Say
     * so.  The atomic is issued after that point in program order and orders nothing else: what the partner stores once it
     * has seen the bit cannot reach loads that have already delivered their values (a release here would also write the
     * XCD's L2 back, which holds the last round's rows: a microsecond per round for nothing). */
    if (wave == PWAVE && lane == 0) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); __hip_atomic_fetch_or(word, PW_LOADED << half, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
  }
  HYK_JSTAMP(3);
  /* From here on the wavefronts meet through `stepsReady` only: the first wavefront publishes the number of steps whose
   * rotations are in `fast` (and STEPS + 1 once the scales and the rotation count are there as well), the others replay
   * a step on their rows as soon as it is out, while the first one works on the next. */
  if (wave == 0) {
    for (int idx = lane; idx < NP; idx += 64) {
      double tot = 0.;
      #pragma unroll
      for (int w = 0; w < WAVES; ++w) { tot += part[w][idx]; }
      int c0 = 0, c1 = 0; pair_of(idx, c0, c1);
      Gs[c0 * GS + c1] = tot; Gs[c1 * GS + c0] = tot;
    }
    if constexpr (SLIM) {
      if (lane < 2 * NW) { int ci, cj; carried_pair<BC>(lane % NW, ci, cj); const int base = lane < NW ? 0 : BC; Gs[(base + ci) * GS + base + cj] = carried; Gs[(base + cj) * GS + base + ci] = carried; }
    }
    if (lane < NC) { scale[lane] = 1.; iscale[lane] = 1.; }
    wave_lds_sync();
    int applied = 0; double worst = 0.;
    /* One rotation from the 2 x 2 Gram block (alpha, gre; gre, beta) of two columns that are kept as scale x vector
     * (x = s u; s and 1 / s travel together).  rr is the plain rotation for the small matrix; fr the same rotation on the
     * vectors as two shears in sequence, u0 <- u0 - t1 u1, then u1 <- u1 + t2 u0 with the new u0: t1 = sigma tan s1 / s0,
     * t2 = sigma sin cos s0 / s1, and the scales become cos s0 and sigma s1 / cos (sigma = sign of gre).  Everything on
     * this chain holds up the whole workgroup: reciprocal square roots from the hardware approximation and two Newton
     * steps (operands within [1/4, 2]), no division (1 / cos and 1 / (1 + |d| / rho) come out of the second root). */
    auto rotation = [&](double alpha, double beta, double gre, bool pairLive, bool counted, double& s0, double& is0, double& s1, double& is1, RotRec& rr, FastRot& fr, double& na, double& nbeta, bool mine) {
      const double g2 = gre * gre, ab = alpha * beta;
      if (mine && pairLive && counted && g2 > 0.) { worst = fmax(worst, fmin(g2 * __builtin_amdgcn_rcp(ab), 1.)); }   /* an indicator: the approximate reciprocal will do */
      const bool rotate = pairLive && g2 > tol * tol * ab && g2 > 0.;
      rr = RotRec{ 1., 0., 0., 1. }; fr = FastRot{ 0., 0. }; na = alpha; nbeta = beta;
      if (rotate) {
        /* d = beta - alpha, h = 2 |g|, both scaled by one power of two so that rho^2 = d^2 + h^2 lies in [1/4, 2):
         * cos^2 = (1 + |d| / rho) / 2 >= 1/2, sin = sign(d) h / (2 rho cos), tan = sin / cos */
        const double gabs = fabs(gre), d = beta - alpha, h = 2. * gabs;
        const int e = __builtin_amdgcn_frexp_exp(fmax(fabs(d), h));
        const double ds = ldexp(fabs(d), -e), hs = ldexp(h, -e);
        const double q = rsqrt_newton(fma(ds, ds, hs * hs)), c2 = fma(0.5 * ds, q, 0.5), w = rsqrt_newton(c2);   /* w = 1 / cos */
        const double cs = c2 * w, sn = copysign(0.5 * hs * q * w, d), tn = sn * w;
        rr.cs = cs; rr.sn = sn; rr.a = gre < 0. ? -sn : sn; rr.b = gre < 0. ? -cs : cs;
        const double shift = tn * gabs; na = alpha - shift; nbeta = beta + shift;
        if (sn != 0.) {
          if (mine) { ++applied; }
          const double sw = gre < 0. ? -w : w;
          fr.t1 = (sw * sn) * (s1 * is0); fr.t2 = (rr.a * cs) * (s0 * is1);
          s0 = cs * s0; is0 = w * is0; s1 = sw * s1; is1 = rr.b * is1;
        }
      }
    };
    if constexpr (FULL) {
      for (int step = 0; step < STEPS; ++step) {
        if (lane < BC) {
          const int j = lane;
          const int fa = (j == 0) ? NC - 1 : (step + j) % (NC - 1), fb = (j == 0) ? step : (step - j + (NC - 1)) % (NC - 1);
          const int c0 = fa < fb ? fa : fb, c1 = fa < fb ? fb : fa;
          const int i0 = (c0 < BC ? P : Q) * BC + (c0 % BC), i1 = (c1 < BC ? P : Q) * BC + (c1 % BC);
          RotRec rr; FastRot fr; double na, nbeta, s0 = scale[c0], s1 = scale[c1], is0 = iscale[c0], is1 = iscale[c1];
          rotation(Gs[c0 * GS + c0], Gs[c1 * GS + c1], Gs[c0 * GS + c1], i0 < r && i1 < r && (i0 < top || i1 < top), i0 < head || i1 < head, s0, is0, s1, is1, rr, fr, na, nbeta, true);
          scale[c0] = s0; scale[c1] = s1; iscale[c0] = is0; iscale[c1] = is1;
          rot[step][j] = rr; fast[step][j] = fr; fixed[j][0] = na; fixed[j][1] = nbeta; pairCol[j][0] = c0; pairCol[j][1] = c1;
        }
        wave_lds_sync();
        /* G <- J^T G J, one lane per pair of pairs: the 2 x 2 block (rows of pair jr, columns of pair jc) takes the column
         * rotation of jc and the row rotation of jr at once; the blocks are disjoint, so one pass does the step.  What a
         * rotation fixes (its own block: alpha - t gamma, beta + t gamma, 0) is written as such. */
        if (lane < BC * BC) {
          const int jr = lane / BC, jc = lane % BC, r0 = pairCol[jr][0], r1 = pairCol[jr][1], k0 = pairCol[jc][0], k1 = pairCol[jc][1];
          const RotRec rw = rot[step][jr], cl = rot[step][jc];
          const double g00 = Gs[r0 * GS + k0], g01 = Gs[r0 * GS + k1], g10 = Gs[r1 * GS + k0], g11 = Gs[r1 * GS + k1];
          const double h00 = cl.cs * g00 - cl.a * g01, h01 = cl.sn * g00 + cl.b * g01, h10 = cl.cs * g10 - cl.a * g11, h11 = cl.sn * g10 + cl.b * g11;
          double y00 = rw.cs * h00 - rw.a * h10, y10 = rw.sn * h00 + rw.b * h10, y01 = rw.cs * h01 - rw.a * h11, y11 = rw.sn * h01 + rw.b * h11;
          if (jr == jc && rw.sn != 0.) { y00 = fixed[jr][0]; y11 = fixed[jr][1]; y01 = 0.; y10 = 0.; }
          Gs[r0 * GS + k0] = y00; Gs[r0 * GS + k1] = y01; Gs[r1 * GS + k0] = y10; Gs[r1 * GS + k1] = y11;
        }
        wave_lds_sync();
      }
    } else {
      /* Cross pairs only (step s pairs column j of the first block with column (j + s) % BC of the second): the small
       * matrix lives in registers.  Lane (jr, jc) holds the 2 x 2 block rows {jr, BC + (jr + s) % BC} x columns
       * {jc, BC + (jc + s) % BC}; the diagonal lanes (j, j) hold alpha, gamma, beta of pair j and work out its rotation,
       * which the lanes of row j and of column j fetch by lane index (sigma cos and sin: two values say it all); after the
       * update three of the four entries move one lane on to where the next step's pairing wants them.  No LDS memory on
       * the chain from one step to the next. */
      const int jr = (lane / BC) % BC, jc = lane % BC; const bool diag = jr == jc && lane < BC * BC;
      double y00 = Gs[jr * GS + jc], y01 = Gs[jr * GS + BC + jc], y10 = Gs[(BC + jr) * GS + jc], y11 = Gs[(BC + jr) * GS + BC + jc];
      double s0 = 1., is0 = 1., s1 = 1., is1 = 1.;
      const int rowSrc = jr * (BC + 1), colSrc = jc * (BC + 1);
      const int next01 = jr * BC + (jc + 1) % BC, next10 = ((jr + 1) % BC) * BC + jc, next11 = ((jr + 1) % BC) * BC + (jc + 1) % BC;
      const int i0 = P * BC + jr;
      for (int step = 0; step < STEPS; ++step) {
        const int i1 = Q * BC + (jr + step) % BC;
        RotRec rr; FastRot fr; double na, nbeta;
        rotation(y00, y11, y01, i0 < r && i1 < r && (i0 < top || i1 < top), i0 < head || i1 < head, s0, is0, s1, is1, rr, fr, na, nbeta, diag);
        if (diag) { fast[step][jr] = fr; }
        const double rb = __shfl(rr.b, rowSrc, 64), rs = __shfl(rr.sn, rowSrc, 64), cb = __shfl(rr.b, colSrc, 64), cn = __shfl(rr.sn, colSrc, 64);
        const double rc = fabs(rb), ra = rb < 0. ? -rs : rs, cc = fabs(cb), ca = cb < 0. ? -cn : cn;   /* b = sigma cos, a = sigma sin */
        const double h00 = fma(cc, y00, -(ca * y01)), h01 = fma(cn, y00, cb * y01), h10 = fma(cc, y10, -(ca * y11)), h11 = fma(cn, y10, cb * y11);
        double z00 = fma(rc, h00, -(ra * h10)), z10 = fma(rs, h00, rb * h10), z01 = fma(rc, h01, -(ra * h11)), z11 = fma(rs, h01, rb * h11);
        if (diag && rr.sn != 0.) { z00 = na; z11 = nbeta; z01 = 0.; z10 = 0.; }
        y00 = z00; y01 = __shfl(z01, next01, 64); y10 = __shfl(z10, next10, 64); y11 = __shfl(z11, next11, 64); s1 = __shfl(s1, next11, 64); is1 = __shfl(is1, next11, 64);
        if (lane == 0) { __hip_atomic_store(&stepsReady, step + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP); }
      }
      /* after BC steps every entry is back where it started */
      if (lane < BC * BC) { Gs[jr * GS + jc] = y00; Gs[(BC + jr) * GS + BC + jc] = y11; }
      if (diag) { scale[jr] = s0; scale[BC + jr] = s1; }
    }
    #pragma unroll
    for (int off = 32; off > 0; off >>= 1) { worst = fmax(worst, __shfl_xor(worst, off, 64)); applied += __shfl_xor(applied, off, 64); }
    if (lane == 0) { appliedAll = applied; worstAll = worst; if constexpr (!SPLIT) { report_cosine(rotations, worst); if (applied > 0) { atomicAdd(rotations, applied); } } }
    wave_lds_sync();
    if constexpr (CARRY && !SPLIT) {   /* the products inside the two blocks as the steps have left them */
      if (lane < 2 * NW) { int ci, cj; carried_pair<BC>(lane % NW, ci, cj); const int base = lane < NW ? 0 : BC; carry[(int64_t)(lane < NW ? P : Q) * NW + lane % NW] = Gs[(base + ci) * GS + base + cj]; }
    }
    if (lane == 0) { __hip_atomic_store(&stepsReady, STEPS + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP); }
  }
  HYK_JSTAMP(4);
  auto wait_steps = [&](int want) {
    if (wave != 0) { while (__hip_atomic_load(&stepsReady, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < want) { __builtin_amdgcn_s_sleep(1); } }
  };
  /* replay the rotations on the rows of this thread (records fetched one ahead); the half in registers first */
  #pragma unroll
  for (int pass = PASSES - 1; pass >= 0; --pass) {
  if (pass != PASSES - 1) { load_rows(pass); }
  [[maybe_unused]] uint32_t early = 0u;   /* split rounds: the pair's word as it was at the second step (asked for then, looked at when the stores are due) */
  #pragma unroll
  for (int step = 0; step < STEPS; ++step) {
    if (pass == PASSES - 1) { wait_steps(FULL ? STEPS + 1 : step + 1); }
    if constexpr (SPLIT) {
      if (wave == PWAVE && lane == 0) {
        if (step == 1) { early = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }   /* asked for early: the answer takes longer than a step, and this wavefront must not wait for it */
        /* the usual case: the partner had loaded long before, and the others learn it before they are through with the last step */
        if (step == STEPS - 1 && (early & (PW_LOADED << (half ^ 1)))) { __hip_atomic_store(&storeMode, 1 | 4, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }
      }
    }
    /* Nothing of the compiler's moves across this point: not the records of later steps (fetched ahead they would wait in
     * scratch memory), and not the arithmetic of this thread's rows either (it is needed only when the rows are stored, and
     * would otherwise sink behind the waits for all later steps, which takes the overlap away). */
    #pragma unroll
    for (int c = 0; c < NC; ++c) {
      #pragma unroll
      for (int m = 0; m < RROWS; ++m) { asm volatile("" : "+v"(x[c][m]) : : "memory"); }
    }
    FastRot recs[BC];   /* the records of a step come in together: one LDS latency per step, not one per rotation */
    #pragma unroll
    for (int j = 0; j < BC; ++j) { recs[j] = fast[step][j]; }
    #pragma unroll
    for (int j = 0; j < BC; ++j) {
      const XT t1 = (XT)recs[j].t1, t2 = (XT)recs[j].t2;
      const int fa = (j == 0) ? NC - 1 : (step + j) % (NC - 1), fb = (j == 0) ? step : (step - j + (NC - 1)) % (NC - 1);
      const int c0 = FULL ? (fa < fb ? fa : fb) : j, c1 = FULL ? (fa < fb ? fb : fa) : BC + (j + step) % BC;
      #pragma unroll
      for (int m = 0; m < RROWS; ++m) { x[c0][m] = fma(-t1, x[c1][m], x[c0][m]); x[c1][m] = fma(t2, x[c0][m], x[c1][m]); }   /* t1 = t2 = 0: no rotation */
    }
  }
  if (pass == PASSES - 1) { wait_steps(STEPS + 1); }
  if constexpr (SPLIT) {
    /* Who stores what (see the comment above the kernel).  One lane settles it and says so in storeMode (bit 2: settled). */
    if (wave == PWAVE && lane == 0 && !(early & (PW_LOADED << (half ^ 1)))) {
      const uint32_t mine = PW_LOADED << half, theirs = PW_LOADED << (half ^ 1);
      int decided = 0;
      for (int spin = 0; decided == 0 && spin < (splitTest == 3 ? 256 : (1 << 22)); ++spin) {
        const uint32_t seen = __hip_atomic_load(word, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
        if (seen & theirs) { decided = 1; }
        else if ((seen & PW_COUNT) == 1u) {   /* alone so far */
          uint32_t expected = 1u | mine;
          if (seen == expected && __hip_atomic_compare_exchange_strong(word, &expected, expected | PW_TAKEN, __ATOMIC_ACQ_REL, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) { decided = 2; }
        } else { __builtin_amdgcn_s_sleep(2); }   /* the partner is here and loading */
      }
      if (decided == 0) { decided = 3; atomicExch(&rotations[1], 1); }   /* never seen with a running partner: no stores rather than wrong ones */
      __hip_atomic_store(&storeMode, decided | 4, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    while (!(__hip_atomic_load(&storeMode, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) & 4)) { __builtin_amdgcn_s_sleep(1); }
    /* cosine, rotation count and carried products from the workgroup that is sure to finish; nothing waits for them */
    if (wave == PWAVE) {
      const int m = storeMode & 3;
      if (m == 2 || (m == 1 && half == 0)) {
        if (lane == 0) { report_cosine(rotations, worstAll); if (appliedAll > 0) { atomicAdd(rotations, appliedAll); } }
        if constexpr (CARRY) {   /* the products inside the two blocks as the steps have left them: the partner, if there is one, has read its own already */
          if (lane < 2 * NW) { int ci, cj; carried_pair<BC>(lane % NW, ci, cj); const int base = lane < NW ? 0 : BC; carry[(int64_t)(lane < NW ? P : Q) * NW + lane % NW] = Gs[(base + ci) * GS + base + cj]; }
        }
      }
    }
  }
  [[maybe_unused]] const int mode = SPLIT ? (storeMode & 3) : 1;
  if (SPLIT && mode == 3) { return; }
  if (appliedAll == 0) { return; }   /* uniform over the workgroup: nothing was rotated, the columns stay as they are */
  #pragma unroll
  for (int c = 0; c < NC; ++c) {
    const XT sc = (XT)scale[c];
    #pragma unroll
    for (int m = 0; m < RROWS; ++m) { x[c][m] *= sc; }
  }
  HYK_JSTAMP(5);
  store_rows(pass, half);
  HYK_JWAIT(); HYK_JSTAMP(6);
  if constexpr (SPLIT) {
    if (mode == 2) {   /* the partner was not there: its half as well, from memory (nobody else writes these rows in this launch) */
      const int other = half ^ 1;
      #pragma unroll
      for (int c = 0; c < NC; ++c) {
        #pragma unroll
        for (int m = 0; m < RROWS; ++m) { const int k = row_of(pass, m + other * RROWS); x[c][m] = (live[c] && k < N) ? B[(int64_t)col[c] * N + k] : (XT)0; }
      }
      #pragma unroll
      for (int step = 0; step < STEPS; ++step) {
        #pragma unroll
        for (int j = 0; j < BC; ++j) {
          const XT t1 = (XT)fast[step][j].t1, t2 = (XT)fast[step][j].t2; const int c0 = j, c1 = BC + (j + step) % BC;   /* a split round is never the first of a sweep: cross pairs only */
          #pragma unroll
          for (int m = 0; m < RROWS; ++m) { x[c0][m] = fma(-t1, x[c1][m], x[c0][m]); x[c1][m] = fma(t2, x[c0][m], x[c1][m]); }
        }
      }
      #pragma unroll
      for (int c = 0; c < NC; ++c) {
        const XT sc = (XT)scale[c];
        #pragma unroll
        for (int m = 0; m < RROWS; ++m) { x[c][m] *= sc; }
      }
      store_rows(pass, other);
    }
  }
  }   /* passes */
  HYK_JREPORT();
}

/* The same round for complex factors.  The Gram matrix is Hermitian, G[c0][c1] = x_c0^H x_c1: NC (NC + 1) / 2 real parts
 * and NC (NC - 1) / 2 imaginary parts, NC^2 sums in all.  A rotation is x_c0' = cs x_c0 - a x_c1, x_c1' = sn x_c0 + b x_c1
 * with a = sn conj(e), b = cs conj(e), e = g / |g| (the phase that makes the cross product real): G <- J^H G J, the row
 * side with the conjugate coefficients. */
struct RotRecC { double cs, sn, ar, ai, br, bi; };   /* sn == 0: no rotation */
struct Cx { double re, im; };
__device__ __forceinline__ Cx cmul(double ar, double ai, Cx b) { return Cx{ ar * b.re - ai * b.im, ar * b.im + ai * b.re }; }

template <typename XT, int ROWS, int BC, bool FULL, int THREADS, int PASSES, bool CARRY>
__global__ __launch_bounds__(THREADS) void jacobi_gram_round_cplx_kernel(int32_t N, int32_t nb, int32_t r, int32_t head, int32_t top, int32_t round, XT* __restrict__ B, double tol, int32_t* __restrict__ rotations, double* __restrict__ carry) {
  constexpr int NC = 2 * BC, NG = NC * (NC + 1) / 2, NT = NC * NC, WAVES = THREADS / 64, STEPS = FULL ? NC - 1 : BC, GS = NC + 1;
  /* CARRY as in the real kernel: the products inside a block (real and imaginary part, 2 NW doubles per block) come from
   * the round before; summed are the NC norms and the BC^2 cross products (real parts, then imaginary parts) */
  constexpr bool SLIM = CARRY && !FULL;
  constexpr int NW = BC * (BC - 1) / 2, NP = SLIM ? NC + 2 * BC * BC : NT;
  constexpr int CH = SLIM ? 2 * BC : (NP >= 32 ? 32 : NP), TAIL = NP % CH;   /* 40 sums: five times 8; 12: three times 4 */
  static_assert(TAIL == 0 && CH >= 4 && BC * BC <= 64 && 4 * NW <= 64, "whole chunks and a power-of-two tail; one lane of the first wavefront per pair of pairs and per carried value");
  /* which sum number q is: real or imaginary part of the product of columns (c0, c1) */
  auto sum_of = [](int q, bool& isIm, int& c0, int& c1) {
    if (!SLIM) { isIm = q >= NG; const int p = isIm ? q - NG + NC : q; c0 = p % NC; c1 = (c0 + p / NC) % NC; }
    else if (q < NC) { isIm = false; c0 = q; c1 = q; }
    else { const int e = q - NC; isIm = e >= BC * BC; const int f = e % (BC * BC); c0 = f / BC; c1 = BC + f % BC; }
  };
  __shared__ double part[WAVES][NP];
  __shared__ double Gre[NC * GS], Gim[NC * GS];
  __shared__ RotRecC rot[STEPS][BC];
  __shared__ double fixed[BC][2];
  __shared__ int32_t pairCol[BC][2];
  __shared__ int32_t appliedAll;
  __shared__ int32_t stepsReady;
  const int pairs = gridDim.x, xcd = blockIdx.x % 8, i = xcd * (pairs / 8) + (xcd < pairs % 8 ? xcd : pairs % 8) + (int)(blockIdx.x / 8); int P, Q;   /* neighbouring pairs on one XCD, as in the real kernel */
  if (i == 0) { P = nb - 1; Q = round; } else { P = (round + i) % (nb - 1); Q = (round - i + (nb - 1)) % (nb - 1); }
  if (P > Q) { const int t = P; P = Q; Q = t; }
  int col[NC]; bool live[NC];
  #pragma unroll
  for (int c = 0; c < NC; ++c) { col[c] = (c < BC ? P : Q) * BC + (c % BC); live[c] = col[c] < r; }
  if (!live[0]) { return; }
  /* Columns from `top` on are the tail that is left alone: pairs of two tail columns are not rotated.  A block pair wholly
   * in the tail has nothing to do, except in the first round of a sweep, which also refreshes the carried products. */
  if (!FULL && col[0] >= top) { return; }
  static_assert(PASSES == 1 || PASSES == 2, "all rows at once or in two halves (as in the real kernel)");
  XT x[NC][ROWS][2];
  auto load_rows = [&](int pass) {
    #pragma unroll
    for (int c = 0; c < NC; ++c) {
      #pragma unroll
      for (int m = 0; m < ROWS; ++m) {
        const int k = threadIdx.x + (pass * ROWS + m) * THREADS;
        #pragma unroll
        for (int w = 0; w < 2; ++w) { x[c][m][w] = (live[c] && k < N) ? B[((int64_t)col[c] * N + k) * 2 + w] : (XT)0; }
      }
    }
  };
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  HYK_JDECL(); HYK_JSTAMP(0);
  [[maybe_unused]] double carried = 0.;
  if constexpr (SLIM) { if (wave == 0 && lane < 4 * NW) { carried = carry[(int64_t)(lane < 2 * NW ? P : Q) * 2 * NW + lane % (2 * NW)]; } }
  /* sum q < NG: real part of pair p = q; q >= NG: imaginary part of pair p = q - NG + NC (the diagonal has none); pairs
   * numbered by diagonal as in the real kernel */
  #pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
  if (pass > 0) { asm volatile("" ::: "memory"); }   /* the second half is loaded when the first is done with, not before */
  load_rows(pass);
  HYK_JWAIT(); HYK_JSTAMP(1);
  #pragma unroll
  for (int chunk = 0; chunk < NP / CH + (TAIL > 0 ? 1 : 0); ++chunk) {
    constexpr int dummy = 0; (void)dummy;
    double v[CH];
    #pragma unroll
    for (int e = 0; e < CH; ++e) {
      bool isIm = false; int c0 = 0, c1 = 0; if (chunk * CH + e < NP) { sum_of(chunk * CH + e, isIm, c0, c1); }
      XT sum = (XT)0;   /* as in the real kernel: a thread's products in the precision of its rows, everything after in FP64 */
      #pragma unroll
      for (int m = 0; m < ROWS; ++m) {
        if (isIm) { sum = fma(x[c0][m][0], x[c1][m][1], fma(-x[c0][m][1], x[c1][m][0], sum)); }
        else { sum = fma(x[c0][m][0], x[c1][m][0], fma(x[c0][m][1], x[c1][m][1], sum)); }
      }
      v[e] = (double)sum;
    }
    const double tot = wave_sum_swap<CH>(v);
    if ((lane & (64 / CH - 1)) == 0 && chunk * CH + lane / (64 / CH) < NP) { double* slot = &part[wave][chunk * CH + lane / (64 / CH)]; *slot = pass == 0 ? tot : *slot + tot; }
  }
  }   /* passes */
  HYK_JSTAMP(2);
  if (threadIdx.x == 0) { stepsReady = 0; }
  __syncthreads();
  HYK_JSTAMP(3);
  /* from here on the wavefronts meet through stepsReady only, as in the real kernel: the first wavefront publishes the
   * number of steps whose rotations are in `rot`, the others replay a step while the next is worked out */
  if (wave == 0) {
    for (int idx = lane; idx < NP; idx += 64) {
      double tot = 0.;
      #pragma unroll
      for (int w = 0; w < WAVES; ++w) { tot += part[w][idx]; }
      bool isIm = false; int c0 = 0, c1 = 0; sum_of(idx, isIm, c0, c1);
      if (isIm) { Gim[c0 * GS + c1] = tot; Gim[c1 * GS + c0] = -tot; }
      else { Gre[c0 * GS + c1] = tot; Gre[c1 * GS + c0] = tot; if (c0 == c1) { Gim[c0 * GS + c0] = 0.; } }
    }
    if constexpr (SLIM) {
      if (lane < 4 * NW) {
        int ci, cj; carried_pair<BC>((lane % (2 * NW)) % NW, ci, cj); const int base = lane < 2 * NW ? 0 : BC; const bool im = lane % (2 * NW) >= NW;
        if (im) { Gim[(base + ci) * GS + base + cj] = carried; Gim[(base + cj) * GS + base + ci] = -carried; }
        else { Gre[(base + ci) * GS + base + cj] = carried; Gre[(base + cj) * GS + base + ci] = carried; }
      }
    }
    wave_lds_sync();
    int applied = 0; double worst = 0.;
    for (int step = 0; step < STEPS; ++step) {
      if (lane < BC) {
        const int j = lane;
        int c0, c1;
        if constexpr (FULL) {
          const int fa = (j == 0) ? NC - 1 : (step + j) % (NC - 1), fb = (j == 0) ? step : (step - j + (NC - 1)) % (NC - 1);
          c0 = fa < fb ? fa : fb; c1 = fa < fb ? fb : fa;
        } else { c0 = j; c1 = BC + (j + step) % BC; }
        const double alpha = Gre[c0 * GS + c0], beta = Gre[c1 * GS + c1], gre = Gre[c0 * GS + c1], gim = Gim[c0 * GS + c1];
        const int i0 = (c0 < BC ? P : Q) * BC + (c0 % BC), i1 = (c1 < BC ? P : Q) * BC + (c1 % BC);
        const bool pairLive = i0 < r && i1 < r && (i0 < top || i1 < top), counted = i0 < head || i1 < head;
        const double g2 = gre * gre + gim * gim;
        if (pairLive && counted && g2 > 0.) { worst = fmax(worst, fmin(g2 * __builtin_amdgcn_rcp(alpha * beta), 1.)); }   /* an indicator: the approximate reciprocal will do */
        const bool rotate = pairLive && g2 > tol * tol * alpha * beta && g2 > 0.;
        RotRecC rr = { 1., 0., 0., 0., 1., 0. }; double na = alpha, nbeta = beta;
        if (rotate) {
          /* as in the real kernel: no division and no library square root on the chain every wavefront waits for */
          const double inv = rsqrt_newton(g2), gabs = g2 * inv, er = gre * inv, ei = gim * inv, d = beta - alpha, h = 2. * gabs;
          const int e = __builtin_amdgcn_frexp_exp(fmax(fabs(d), h));
          const double ds = ldexp(fabs(d), -e), hs = ldexp(h, -e);
          const double q = rsqrt_newton(fma(ds, ds, hs * hs)), c2 = fma(0.5 * ds, q, 0.5), w = rsqrt_newton(c2);
          const double cs = c2 * w, sn = copysign(0.5 * hs * q * w, d), shift = sn * w * gabs;
          rr.cs = cs; rr.sn = sn; rr.ar = sn * er; rr.ai = -sn * ei; rr.br = cs * er; rr.bi = -cs * ei;
          na = alpha - shift; nbeta = beta + shift;
          if (sn != 0.) { ++applied; }
        }
        rot[step][j] = rr; fixed[j][0] = na; fixed[j][1] = nbeta; pairCol[j][0] = c0; pairCol[j][1] = c1;
      }
      wave_lds_sync();
      if (lane < BC * BC) {
        const int jr = lane / BC, jc = lane % BC, r0 = pairCol[jr][0], r1 = pairCol[jr][1], k0 = pairCol[jc][0], k1 = pairCol[jc][1];
        const RotRecC rw = rot[step][jr], cl = rot[step][jc];
        const Cx g00 = { Gre[r0 * GS + k0], Gim[r0 * GS + k0] }, g01 = { Gre[r0 * GS + k1], Gim[r0 * GS + k1] };
        const Cx g10 = { Gre[r1 * GS + k0], Gim[r1 * GS + k0] }, g11 = { Gre[r1 * GS + k1], Gim[r1 * GS + k1] };
        /* columns: h_x0 = cs g_x0 - a g_x1, h_x1 = sn g_x0 + b g_x1 */
        const Cx a01 = cmul(cl.ar, cl.ai, g01), a11 = cmul(cl.ar, cl.ai, g11), b01 = cmul(cl.br, cl.bi, g01), b11 = cmul(cl.br, cl.bi, g11);
        const Cx h00 = { cl.cs * g00.re - a01.re, cl.cs * g00.im - a01.im }, h01 = { cl.sn * g00.re + b01.re, cl.sn * g00.im + b01.im };
        const Cx h10 = { cl.cs * g10.re - a11.re, cl.cs * g10.im - a11.im }, h11 = { cl.sn * g10.re + b11.re, cl.sn * g10.im + b11.im };
        /* rows: y_0k = cs h_0k - conj(a) h_1k, y_1k = sn h_0k + conj(b) h_1k */
        const Cx c10 = cmul(rw.ar, -rw.ai, h10), c11 = cmul(rw.ar, -rw.ai, h11), d10 = cmul(rw.br, -rw.bi, h10), d11 = cmul(rw.br, -rw.bi, h11);
        Cx y00 = { rw.cs * h00.re - c10.re, rw.cs * h00.im - c10.im }, y01 = { rw.cs * h01.re - c11.re, rw.cs * h01.im - c11.im };
        Cx y10 = { rw.sn * h00.re + d10.re, rw.sn * h00.im + d10.im }, y11 = { rw.sn * h01.re + d11.re, rw.sn * h01.im + d11.im };
        if (jr == jc && rw.sn != 0.) { y00 = Cx{ fixed[jr][0], 0. }; y11 = Cx{ fixed[jr][1], 0. }; y01 = Cx{ 0., 0. }; y10 = Cx{ 0., 0. }; }
        Gre[r0 * GS + k0] = y00.re; Gim[r0 * GS + k0] = y00.im; Gre[r0 * GS + k1] = y01.re; Gim[r0 * GS + k1] = y01.im;
        Gre[r1 * GS + k0] = y10.re; Gim[r1 * GS + k0] = y10.im; Gre[r1 * GS + k1] = y11.re; Gim[r1 * GS + k1] = y11.im;
      }
      wave_lds_sync();
      if (lane == 0) { __hip_atomic_store(&stepsReady, step + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP); }
    }
    #pragma unroll
    for (int off = BC / 2; off > 0; off >>= 1) { worst = fmax(worst, __shfl_xor(worst, off, 64)); applied += __shfl_xor(applied, off, 64); }
    if (lane == 0) { report_cosine(rotations, worst); appliedAll = applied; if (applied > 0) { atomicAdd(rotations, applied); } }
    if constexpr (CARRY) {
      if (lane < 4 * NW) {
        int ci, cj; carried_pair<BC>((lane % (2 * NW)) % NW, ci, cj); const int base = lane < 2 * NW ? 0 : BC; const bool im = lane % (2 * NW) >= NW;
        carry[(int64_t)(lane < 2 * NW ? P : Q) * 2 * NW + lane % (2 * NW)] = im ? Gim[(base + ci) * GS + base + cj] : Gre[(base + ci) * GS + base + cj];
      }
    }
    wave_lds_sync();
    if (lane == 0) { __hip_atomic_store(&stepsReady, STEPS + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP); }
  }
  HYK_JSTAMP(4);
  auto wait_steps = [&](int want) {
    if (wave != 0) { while (__hip_atomic_load(&stepsReady, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < want) { __builtin_amdgcn_s_sleep(1); } }
  };
  #pragma unroll
  for (int pass = PASSES - 1; pass >= 0; --pass) {   /* the half in registers first */
  if (pass != PASSES - 1) { asm volatile("" ::: "memory"); load_rows(pass); }
  #pragma unroll
  for (int step = 0; step < STEPS; ++step) {
    if (pass == PASSES - 1) { wait_steps(step + 1); }
    /* nothing of the compiler's moves across this point (see the real kernel) */
    #pragma unroll
    for (int c = 0; c < NC; ++c) {
      #pragma unroll
      for (int m = 0; m < ROWS; ++m) { asm volatile("" : "+v"(x[c][m][0]), "+v"(x[c][m][1]) : : "memory"); }
    }
    RotRecC recs[BC];   /* the records of a step come in together */
    #pragma unroll
    for (int j = 0; j < BC; ++j) { recs[j] = rot[step][j]; }
    #pragma unroll
    for (int j = 0; j < BC; ++j) {
      struct { XT cs, sn, ar, ai, br, bi; } rr = { (XT)recs[j].cs, (XT)recs[j].sn, (XT)recs[j].ar, (XT)recs[j].ai, (XT)recs[j].br, (XT)recs[j].bi };
      const int fa = (j == 0) ? NC - 1 : (step + j) % (NC - 1), fb = (j == 0) ? step : (step - j + (NC - 1)) % (NC - 1);
      const int c0 = FULL ? (fa < fb ? fa : fb) : j, c1 = FULL ? (fa < fb ? fb : fa) : BC + (j + step) % BC;
      if (recs[j].sn != 0.) {
        #pragma unroll
        for (int m = 0; m < ROWS; ++m) {
          const XT pr = x[c0][m][0], pi = x[c0][m][1], qr = x[c1][m][0], qi = x[c1][m][1];
          x[c0][m][0] = fma(rr.cs, pr, fma(rr.ai, qi, -(rr.ar * qr))); x[c0][m][1] = fma(rr.cs, pi, fma(-rr.ar, qi, -(rr.ai * qr)));
          x[c1][m][0] = fma(rr.sn, pr, fma(rr.br, qr, -(rr.bi * qi))); x[c1][m][1] = fma(rr.sn, pi, fma(rr.br, qi, rr.bi * qr));
        }
      }
    }
  }
  if (pass == PASSES - 1) { wait_steps(STEPS + 1); }
  if (appliedAll == 0) { return; }   /* uniform over the workgroup: nothing was rotated */
  HYK_JSTAMP(5);
  #pragma unroll
  for (int c = 0; c < NC; ++c) {
    #pragma unroll
    for (int m = 0; m < ROWS; ++m) {
      const int k = threadIdx.x + (pass * ROWS + m) * THREADS;
      if (live[c] && k < N) { B[((int64_t)col[c] * N + k) * 2] = x[c][m][0]; B[((int64_t)col[c] * N + k) * 2 + 1] = x[c][m][1]; }
    }
  }
  HYK_JWAIT(); HYK_JSTAMP(6);
  }   /* passes */
  HYK_JREPORT();
}

static int compute_units() {   /* of the device current on this thread */
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) { return n; }
  return 0;
}

/* bytes of the products that travel with the blocks from round to round (enough for every round kernel: 28 doubles per block of 8 real columns) */
static size_t carried_bytes(int32_t r) { return ((size_t)r / 4 + 2) * 28 * sizeof(double); }
/* and of the words that order the two workgroups of a pair in the split rounds: one per pair and round of 8-column blocks */
static size_t pair_word_bytes(int32_t r) { const size_t nb = (((size_t)r + 7) / 8 + 1) & ~(size_t)1; return (nb * nb / 2 * sizeof(uint32_t) + 255) / 256 * 256; }

template <int ROWS, int BC, int THREADS = T_THREADS, int PASSES = 1, typename XT>
static int gram_sweep(hipStream_t stream, int32_t N, int32_t r, int32_t head, int32_t top, XT* B, double tol, int32_t* rotations, double* carry, int splitTest) {
  const int blocks = (r + BC - 1) / BC, nb = (blocks + 1) & ~1;
  if constexpr (ROWS == 4 && PASSES == 1 && BC == 8) {
    /* two workgroups per pair (one per compute unit: 512 threads with their rows in registers) while all of them still run side by side */
    const int splitGrid = 16 * ((nb / 2 + 7) / 8);
    if (carry && splitGrid <= compute_units()) {
      uint32_t* words = reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(carry) + carried_bytes(r));
      if (hykGramWorkspaceClear(stream, words, pair_word_bytes(r)) != 0) { return -3; }
      jacobi_gram_round_kernel<XT, ROWS, BC, true, THREADS, true, PASSES><<<nb / 2, THREADS, 0, stream>>>(N, nb, r, head, top, 0, B, tol, rotations, carry, nullptr, 0);
      for (int round = 1; round < nb - 1; ++round) { jacobi_gram_round_kernel<XT, ROWS, BC, false, THREADS, true, PASSES, true><<<splitGrid, THREADS, 0, stream>>>(N, nb, r, head, top, round, B, tol, rotations, carry, words, splitTest); }
      return hipGetLastError() == hipSuccess ? 0 : -3;
    }
  }
  if (carry) {
    jacobi_gram_round_kernel<XT, ROWS, BC, true, THREADS, true, PASSES><<<nb / 2, THREADS, 0, stream>>>(N, nb, r, head, top, 0, B, tol, rotations, carry, nullptr, 0);
    for (int round = 1; round < nb - 1; ++round) { jacobi_gram_round_kernel<XT, ROWS, BC, false, THREADS, true, PASSES><<<nb / 2, THREADS, 0, stream>>>(N, nb, r, head, top, round, B, tol, rotations, carry, nullptr, 0); }
  } else {
    jacobi_gram_round_kernel<XT, ROWS, BC, true, THREADS, false, PASSES><<<nb / 2, THREADS, 0, stream>>>(N, nb, r, head, top, 0, B, tol, rotations, nullptr, nullptr, 0);
    for (int round = 1; round < nb - 1; ++round) { jacobi_gram_round_kernel<XT, ROWS, BC, false, THREADS, false, PASSES><<<nb / 2, THREADS, 0, stream>>>(N, nb, r, head, top, round, B, tol, rotations, nullptr, nullptr, 0); }
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

template <int ROWS, int BC, int THREADS = T_THREADS, int PASSES = 1, typename XT>
static int gram_sweep_cplx(hipStream_t stream, int32_t N, int32_t r, int32_t head, int32_t top, XT* B, double tol, int32_t* rotations, double* carry) {
  const int blocks = (r + BC - 1) / BC, nb = (blocks + 1) & ~1;
  if (carry) {
    jacobi_gram_round_cplx_kernel<XT, ROWS, BC, true, THREADS, PASSES, true><<<nb / 2, THREADS, 0, stream>>>(N, nb, r, head, top, 0, B, tol, rotations, carry);
    for (int round = 1; round < nb - 1; ++round) { jacobi_gram_round_cplx_kernel<XT, ROWS, BC, false, THREADS, PASSES, true><<<nb / 2, THREADS, 0, stream>>>(N, nb, r, head, top, round, B, tol, rotations, carry); }
  } else {
    jacobi_gram_round_cplx_kernel<XT, ROWS, BC, true, THREADS, PASSES, false><<<nb / 2, THREADS, 0, stream>>>(N, nb, r, head, top, 0, B, tol, rotations, nullptr);
    for (int round = 1; round < nb - 1; ++round) { jacobi_gram_round_cplx_kernel<XT, ROWS, BC, false, THREADS, PASSES, false><<<nb / 2, THREADS, 0, stream>>>(N, nb, r, head, top, round, B, tol, rotations, nullptr); }
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

template <bool CPLX, int ROWS, int BC, int THREADS = T_THREADS, typename XT>
static int blocked_sweep(hipStream_t stream, int32_t N, int32_t r, int32_t head, int32_t top, XT* B, double tol, int32_t* rotations) {
  const int blocks = (r + BC - 1) / BC, nb = (blocks + 1) & ~1;
  jacobi_block_round_kernel<XT, CPLX, ROWS, BC, true, THREADS><<<nb / 2, THREADS, 0, stream>>>(N, nb, r, head, top, 0, B, tol, rotations);
  for (int round = 1; round < nb - 1; ++round) { jacobi_block_round_kernel<XT, CPLX, ROWS, BC, false, THREADS><<<nb / 2, THREADS, 0, stream>>>(N, nb, r, head, top, round, B, tol, rotations); }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

/* One sweep over the r columns of B: which kernel takes it.  variant: 0 Gram-space rounds, 8-column blocks for real factors
 * where they fit (default); 1 the step kernel everywhere; 2 Gram-space rounds with the narrower blocks.  Rows of type float
 * take half the registers of doubles, so a workgroup holds twice as many of them: where double factors go through their
 * rows in two halves (2048 < N <= 4096), float factors take them at once. */
template <typename XT>
static int sweep_top(hipStream_t stream, int32_t Complex, int32_t N, int32_t r, int32_t head, int32_t top, XT* B, double tol, int32_t* rotations, double* carry, int variant, int splitTest) {
  if (N <= 0 || r <= 1) { return 0; }
  if (top > r) { top = r; } if (top < 0) { top = 0; } if (head > r) { head = r; } if (head < 0) { head = 0; }
  constexpr bool F = std::is_same<XT, float>::value;
  /* real factors: Gram-space rounds; blocks of 8 columns where the rows of 16 columns fit the registers of 512 threads
   * (half as many rounds, each 1.4 times as long at N = 2048), blocks of 4 otherwise */
  if (!Complex && r >= 32 && variant == 0) {
    /* up to 1024 rows: four rows per thread on 256 threads, so that a round can go to two workgroups per pair (gram_sweep), while they all run side by side */
    if (N <= 4 * 256 && carry && 16 * ((((r + 7) / 8 + 1) / 2 + 7) / 8) <= compute_units()) { return gram_sweep<4, 8, 256>(stream, N, r, head, top, B, tol, rotations, carry, splitTest); }
    if (N <= 2 * 512) { return gram_sweep<2, 8, 512>(stream, N, r, head, top, B, tol, rotations, carry, splitTest); }
    if (N <= 4 * 512) { return gram_sweep<4, 8, 512>(stream, N, r, head, top, B, tol, rotations, carry, splitTest); }
    if constexpr (F) { if (N <= 8 * 512) { return gram_sweep<8, 8, 512>(stream, N, r, head, top, B, tol, rotations, carry, splitTest); } }
    else { if (N <= 8 * 512) { return gram_sweep<4, 8, 512, 2>(stream, N, r, head, top, B, tol, rotations, carry, splitTest); } }
  }
  if (!Complex && r >= 16 && variant != 1) {
    if (N <= 4 * T_THREADS) { return gram_sweep<4, 4>(stream, N, r, head, top, B, tol, rotations, carry, splitTest); }
    if (N <= 8 * T_THREADS) { return gram_sweep<8, 4>(stream, N, r, head, top, B, tol, rotations, carry, splitTest); }
    if (N <= 8 * 512) { return gram_sweep<8, 4, 512>(stream, N, r, head, top, B, tol, rotations, carry, splitTest); }
  }
  if (!Complex && r >= 16) {
    if (N <= 4 * T_THREADS) { return blocked_sweep<false, 4, 4>(stream, N, r, head, top, B, tol, rotations); }
    if (N <= 8 * T_THREADS) { return blocked_sweep<false, 8, 4>(stream, N, r, head, top, B, tol, rotations); }
    if (N <= 8 * 512) { return blocked_sweep<false, 8, 4, 512>(stream, N, r, head, top, B, tol, rotations); }
  }
  if (Complex && r >= 16 && variant != 1) {
    if (N <= 4 * T_THREADS) { return gram_sweep_cplx<4, 4>(stream, N, r, head, top, B, tol, rotations, carry); }
    if (N <= 4 * 512) { return gram_sweep_cplx<4, 4, 512>(stream, N, r, head, top, B, tol, rotations, carry); }
    if constexpr (F) { if (N <= 8 * 512) { return gram_sweep_cplx<8, 4, 512>(stream, N, r, head, top, B, tol, rotations, carry); } }
    else { if (N <= 8 * 512) { return variant == 0 ? gram_sweep_cplx<4, 4, 512, 2>(stream, N, r, head, top, B, tol, rotations, carry) : gram_sweep_cplx<8, 2, 512>(stream, N, r, head, top, B, tol, rotations, carry); } }
  }
  if (Complex && r >= 16) {
    if (N <= 4 * T_THREADS) { return blocked_sweep<true, 4, 4>(stream, N, r, head, top, B, tol, rotations); }
    if (N <= 4 * 512) { return blocked_sweep<true, 4, 4, 512>(stream, N, r, head, top, B, tol, rotations); }
    if (N <= 8 * 512) { return blocked_sweep<true, 8, 2, 512>(stream, N, r, head, top, B, tol, rotations); }
  }
  const int n = (r + 1) & ~1;
  for (int round = 0; round < n - 1; ++round) {
    if (Complex) { jacobi_round_kernel<true, XT><<<n / 2, T_THREADS, 0, stream>>>(N, n, r, head, top, round, B, tol, rotations); } else { jacobi_round_kernel<false, XT><<<n / 2, T_THREADS, 0, stream>>>(N, n, r, head, top, round, B, tol, rotations); }
  }
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

}  // namespace
