/*
 * potrfp.hip -- diagonal-pivoted Cholesky of the dequantized Gram matrix,
 * P^T G P ~= R^H R, stopped when the remaining trace drops to eps^2 trace(G) or
 * after K columns.  Arithmetic in FP64 or double-double, real or complex.
 *
 * Replaces the reference's src/hyacin_potrfp.cu (persistent left-looking
 * kernel, three grid barriers per column, columns swapped in place).  The
 * MI355X design keeps the left-looking recurrence
 *     S[l]     = G[l, c] - sum_{t<k} conj(R[t, l]) R[t, c]
 *     R[k, l]  = conj(S[l]) / sqrt(d_c),   d_l -= |R[k, l]|^2
 * but (i) never moves a column: pivots are recorded, finished columns are
 * flagged, and R is kept column-wise (Rt[l * ldr + t] = R[t, l]) so that both
 * operands of every dot product are contiguous; (ii) exchanges one small
 * record per workgroup and column instead of passing grid barriers: every
 * workgroup publishes its (max, trace) partial with write-through stores
 * tagged with the column number, polls the records of all workgroups and
 * reduces them itself.
 * No cache is written back or invalidated on the way: what crosses workgroups
 * (records, the factor entries of the pivot column) is stored write-through
 * and loaded past the caches, everything else is private to its owner;
 * (iii) one wavefront owns a column for the whole run (its diagonal entry and
 * its finished flag never leave the wavefront), lanes split the dot product.
 * Ties between equal diagonal entries are broken towards the smaller column
 * index (the reference breaks them towards the smaller position in its swapped
 * order).  The emitted pivot vector follows the reference's swap sequence
 * (jpiv[k] <-> jpiv[position of the pivot]) and is 1-based.
 *
 * Cooperative launch: at most one workgroup per compute unit, all resident.
 */
#include <hip/hip_runtime.h>
#include <atomic>
#include <cstdio>
#include "hyk_common.h"
#include "hyk_dd.h"
#include "hyacin_kernels.h"

namespace {

using hyk::dd_t;

constexpr int P_THREADS = 1024;   /* 16 wavefronts per compute unit: the dot products are latency-bound loads of the factor */
constexpr int P_WAVES = P_THREADS / 64;

/* What a workgroup publishes per column: seven 32-bit pieces (bx, by, trace as two halves each, the index of its best
 * column or -1), every piece in a 64-bit word of its own under the epoch it belongs to: word = epoch << 32 | piece.  A
 * 64-bit store is indivisible, so a reader that finds the epoch in a word has that word's piece, whatever order the
 * words arrive in; no word has to wait for another. */
struct Record { uint64_t w[8]; };
constexpr int RECORD_WORDS = 7;
constexpr int STAGE_BYTES = 48 * 1024;
constexpr int MAX_WORKGROUPS = 256;
constexpr int SPIN_LIMIT = 1 << 22;   /* polls of one record before the run is given up (seconds; a healthy wait is microseconds) */

struct PotrfArgs {
  int32_t N, K, ldr; double eps2;
  const double* G; int64_t ldg;
  double* Rt; double* D; int32_t* jpiv; int32_t* pos; Record* records; int32_t* rankOut;
};

/* scalar types: value = re (+ i im), each part a dd_t (lo part unused in FP64 mode) */
template <bool DD> struct Real {
  dd_t v;
  __device__ __forceinline__ static Real zero() { return Real{ dd_t{ 0., 0. } }; }
  __device__ __forceinline__ static Real load(const double* p) { if constexpr (DD) { return Real{ dd_t{ p[0], p[1] } }; } else { return Real{ dd_t{ p[0], 0. } }; } }
  __device__ __forceinline__ void store(double* p) const { p[0] = v.x; if constexpr (DD) { p[1] = v.y; } }
  /* for data that another workgroup reads or wrote: loads that bypass the non-coherent cache levels, stores that write through */
  __device__ __forceinline__ static Real load_shared(const double* p) { Real r; r.v.x = __hip_atomic_load(const_cast<double*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); r.v.y = 0.; if constexpr (DD) { r.v.y = __hip_atomic_load(const_cast<double*>(p) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); } return r; }
  __device__ __forceinline__ void store_shared(double* p) const { __hip_atomic_store(p, v.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); if constexpr (DD) { __hip_atomic_store(p + 1, v.y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); } }
  __device__ __forceinline__ Real operator+(Real b) const { if constexpr (DD) { return Real{ hyk::dd_add(v, b.v) }; } else { return Real{ dd_t{ v.x + b.v.x, 0. } }; } }
  __device__ __forceinline__ Real operator-(Real b) const { if constexpr (DD) { return Real{ hyk::dd_sub(v, b.v) }; } else { return Real{ dd_t{ v.x - b.v.x, 0. } }; } }
  __device__ __forceinline__ Real operator*(Real b) const { if constexpr (DD) { return Real{ hyk::dd_mul(v, b.v) }; } else { return Real{ dd_t{ v.x * b.v.x, 0. } }; } }
  __device__ __forceinline__ Real neg() const { return Real{ dd_t{ -v.x, -v.y } }; }
  __device__ __forceinline__ bool less(Real b) const { if constexpr (DD) { return hyk::dd_less(v, b.v); } else { return v.x < b.v.x; } }
  /* acc - a*b */
  __device__ __forceinline__ static Real fnma(Real a, Real b, Real acc) { if constexpr (DD) { return Real{ hyk::dd_sub(acc.v, hyk::dd_mul(a.v, b.v)) }; } else { return Real{ dd_t{ fma(-a.v.x, b.v.x, acc.v.x), 0. } }; } }
  __device__ __forceinline__ Real shfl_xor(int m) const { Real r; r.v.x = __shfl_xor(v.x, m, 64); if constexpr (DD) { r.v.y = __shfl_xor(v.y, m, 64); } else { r.v.y = 0.; } return r; }
};

template <bool DD> __device__ __forceinline__ void sqrt_rsqrt(Real<DD> d, Real<DD>& sq, Real<DD>& rs) {
  if constexpr (DD) { dd_t r = hyk::dd_rsqrt(d.v); rs.v = r; sq.v = hyk::dd_mul(d.v, r); } else { double s = sqrt(d.v.x); sq.v = dd_t{ s, 0. }; rs.v = dd_t{ 1.0 / s, 0. }; }
}

template <bool DD, bool CPLX> struct Width { static constexpr int real = DD ? 2 : 1; static constexpr int elem = real * (CPLX ? 2 : 1); };

/* deterministic block arg-max: larger value wins, ties to the smaller index; idx < 0 means "no positive entry" */
__device__ __forceinline__ void better(bool dd, double& bx, double& by, int32_t& bi, double ox, double oy, int32_t oi) {
  if (oi < 0) { return; }
  bool gt = dd ? (bx < ox || (bx == ox && by < oy)) : (bx < ox);
  bool eq = dd ? (bx == ox && by == oy) : (bx == ox);
  if (bi < 0 || gt || (eq && oi < bi)) { bx = ox; by = oy; bi = oi; }
}

/* arg-max / sum over the lanes of a wavefront by `steps` butterfly exchanges (the low 2^steps lanes of every aligned group end up equal) */
template <bool DD, int STEPS>
__device__ __forceinline__ void wave_reduce(double& bx, double& by, int32_t& bi, double& tr) {
  #pragma unroll
  for (int m = 1 << (STEPS - 1); m > 0; m >>= 1) {
    const double ox = __shfl_xor(bx, m, 64), oy = __shfl_xor(by, m, 64), ot = __shfl_xor(tr, m, 64); const int32_t oi = __shfl_xor(bi, m, 64);
    better(DD, bx, by, bi, ox, oy, oi); tr += ot;
  }
}

/* LDS: partials of the wavefronts (x, y, t, i), partials of the wavefronts that collected records (rx, ry, rt, ri: a later phase of
 * the same step, which must not overwrite what the first wavefront may still be reading), and the give-up flag */
constexpr int POLL_WAVES = MAX_WORKGROUPS / 64;
struct Exchange { double x[P_WAVES], y[P_WAVES], t[P_WAVES], rx[POLL_WAVES], ry[POLL_WAVES], rt[POLL_WAVES]; int32_t i[P_WAVES], ri[POLL_WAVES]; int32_t failed; };

/* Every wavefront holds one partial in its lane 0 (a wavefront works on one column at a time); afterwards the lanes
 * 0..15 of the first wavefront hold the workgroup's result.  One barrier. */
template <bool DD>
__device__ __forceinline__ void reduce_leaders(Exchange& ex, double& bx, double& by, int32_t& bi, double& tr) {
  static_assert(P_WAVES == 16, "four butterfly steps");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { ex.x[wave] = bx; ex.y[wave] = by; ex.i[wave] = bi; ex.t[wave] = tr; }
  __syncthreads();
  if (wave == 0) {
    bx = by = tr = 0.; bi = -1;
    if (lane < P_WAVES) { bx = ex.x[lane]; by = ex.y[lane]; bi = ex.i[lane]; tr = ex.t[lane]; }
    wave_reduce<DD, 4>(bx, by, bi, tr);
  }
}

/* Threads t < workgroups hold the records they collected; afterwards every thread holds the result over all of them
 * (combined in one fixed order, so that all workgroups take the same decisions).  One barrier. */
template <bool DD>
__device__ __forceinline__ void reduce_records(Exchange& ex, int workgroups, double& bx, double& by, int32_t& bi, double& tr) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, pollWaves = (workgroups + 63) >> 6;
  if (wave < pollWaves) { wave_reduce<DD, 6>(bx, by, bi, tr); if (lane == 0) { ex.rx[wave] = bx; ex.ry[wave] = by; ex.ri[wave] = bi; ex.rt[wave] = tr; } }
  __syncthreads();
  bx = ex.rx[0]; by = ex.ry[0]; bi = ex.ri[0]; tr = ex.rt[0];
  for (int w = 1; w < pollWaves; ++w) { better(DD, bx, by, bi, ex.rx[w], ex.ry[w], ex.ri[w]); tr += ex.rt[w]; }
}

/* Publishes this workgroup's partial for `epoch`: lane j < 7 of the first wavefront stores word j (after the workgroup
 * reduction every lane holds the result). */
__device__ __forceinline__ void publish(Record* rec, double bx, double by, double tr, int32_t bi, uint32_t epoch) {
  const int j = threadIdx.x;
  if (j < RECORD_WORDS) {
    const uint64_t src = (uint64_t)__double_as_longlong(j < 2 ? bx : j < 4 ? by : tr);
    const uint32_t piece = j == 6 ? (uint32_t)bi : (uint32_t)(src >> (32 * (j & 1)));
    __hip_atomic_store(&rec->w[j], ((uint64_t)epoch << 32) | piece, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

/* Thread t < workgroups waits for record t of `epoch` and takes it as its reduction input; a wait that gives up raises ex.failed. */
__device__ __forceinline__ void collect(Exchange& ex, Record* recs, int workgroups, uint32_t epoch, double& bx, double& by, int32_t& bi, double& tr) {
  bx = by = tr = 0.; bi = -1; bool ok = true;
  if ((int)threadIdx.x < workgroups) {
    Record* rec = &recs[threadIdx.x]; uint64_t v[RECORD_WORDS]; int spins = 0;
    for (;;) {
      bool complete = true;
      #pragma unroll
      for (int j = 0; j < RECORD_WORDS; ++j) { v[j] = __hip_atomic_load(&rec->w[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
      #pragma unroll
      for (int j = 0; j < RECORD_WORDS; ++j) { complete = complete && (uint32_t)(v[j] >> 32) == epoch; }
      if (complete) { break; }
      if (++spins > SPIN_LIMIT) { ok = false; break; }
      __builtin_amdgcn_s_sleep(1);
    }
    if (ok) {
      bx = __longlong_as_double((long long)((v[0] & 0xffffffffull) | (v[1] << 32))); by = __longlong_as_double((long long)((v[2] & 0xffffffffull) | (v[3] << 32)));
      tr = __longlong_as_double((long long)((v[4] & 0xffffffffull) | (v[5] << 32))); bi = (int32_t)(uint32_t)v[6];
    }
  }
  if (!ok) { ex.failed = 1; }
}

template <bool DD, bool CPLX>
__global__ __launch_bounds__(P_THREADS) void potrfp_kernel(const PotrfArgs a) {
  uint32_t epoch = 0;
  using R = Real<DD>; constexpr int WR = Width<DD, CPLX>::real, WE = Width<DD, CPLX>::elem;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwg = gridDim.x, wg = blockIdx.x;
  const int gwave = wg * P_WAVES + wave, nwaves = nwg * P_WAVES;
  const int N = a.N;
  /* column gwave + i nwaves belongs to this wavefront for the whole run; bit i of finished: it has been a pivot */
  uint64_t finished = 0;
  __shared__ Exchange ex;
  constexpr int STAGE = STAGE_BYTES / (WE * 8);   /* factor entries of the pivot column that fit the LDS stage */
  __shared__ __attribute__((aligned(16))) double stage[STAGE_BYTES / 8];
  if (tid == 0) { ex.failed = 0; }
  __syncthreads();

  /* init: diagonal, pivot bookkeeping (workgroup 0 keeps it), first arg-max and trace */
  double bx = 0., by = 0., tr = 0.; int32_t bi = -1;
  for (int l = gwave; l < N; l += nwaves) {
    if (lane == 0) {
      R d = R::load(&a.G[((int64_t)l + (int64_t)l * a.ldg) * WE]); d.store_shared(&a.D[(int64_t)l * WR]); tr += d.v.x;
      if (d.v.x > 0.) { better(DD, bx, by, bi, d.v.x, d.v.y, l); }
    }
  }
  if (wg == 0) { for (int l = tid; l < N; l += P_THREADS) { a.jpiv[l] = l + 1; a.pos[l] = l; } }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  reduce_leaders<DD>(ex, bx, by, bi, tr);
  ++epoch;
  publish(&a.records[(epoch & 1) * MAX_WORKGROUPS + wg], bx, by, tr, bi, epoch);
  collect(ex, &a.records[(epoch & 1) * MAX_WORKGROUPS], nwg, epoch, bx, by, bi, tr);
  reduce_records<DD>(ex, nwg, bx, by, bi, tr);
  bool alive = ex.failed == 0;
  const double thresh = a.eps2 * tr;
  const int Kstop = a.K >= N ? N - 1 : a.K;   /* with K == N the last column is appended without a test (see below) */
  int k = 0;
  while (alive && bi >= 0 && k < Kstop) {
    const int c = bi; R dc{ dd_t{ bx, by } }, sq, rho; sqrt_rsqrt<DD>(dc, sq, rho);
    if (wg == 0 && tid == 0) {
      /* R[k, c] = sqrt(d_c); pivot bookkeeping in the reference's swap order */
      double* rc = &a.Rt[((int64_t)c * a.ldr + k) * WE]; sq.store(rc); if constexpr (CPLX) { R::zero().store(rc + WR); }
      const int p = a.pos[c], c0 = a.jpiv[k] - 1; a.jpiv[k] = c + 1; a.jpiv[p] = c0 + 1; a.pos[c] = k; a.pos[c0] = p;
    }
    /* column c of R, shared by every dot product of this step: Rt[c][0..k), written by the wavefront that owns c.  The
     * workgroup fetches it once into LDS (what exceeds the stage is read from memory by every wavefront); the barrier
     * of the previous step's reduction has made the stage free. */
    const double* rcol = &a.Rt[(int64_t)c * a.ldr * WE];
    const int staged = k < STAGE ? k : STAGE;
    for (int e = tid; e < staged * WE; e += P_THREADS) { stage[e] = __hip_atomic_load(const_cast<double*>(rcol) + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
    __syncthreads();
    bx = by = tr = 0.; bi = -1;
    int slot = 0;
    for (int l = gwave; l < N; l += nwaves, ++slot) {
      if (l == c) { finished |= 1ull << slot; }
      if ((finished >> slot) & 1ull) { continue; }
      const double* rl = &a.Rt[(int64_t)l * a.ldr * WE];
      /* G[l, c] and d_l are needed only after the dot product: request them first so their latency hides under it */
      const double* g = &a.G[((int64_t)l + (int64_t)c * a.ldg) * WE];
      const R gre0 = R::load(g), d0 = R::load(&a.D[(int64_t)l * WR]); R gim0 = R::zero(); if constexpr (CPLX) { gim0 = R::load(g + WR); }
      R sre = R::zero(), sim = R::zero();
      #pragma unroll 8
      for (int t = lane; t < staged; t += 64) {
        if constexpr (CPLX) {
          R ar = R::load(&rl[(int64_t)t * WE]), ai = R::load(&rl[(int64_t)t * WE + WR]), br = R::load(&stage[t * WE]), bim = R::load(&stage[t * WE + WR]);
          sre = R::fnma(ar, br, sre); sre = R::fnma(ai, bim, sre); sim = R::fnma(ar, bim, sim); sim = R::fnma(ai.neg(), br, sim);
        } else { sre = R::fnma(R::load(&rl[(int64_t)t * WE]), R::load(&stage[t * WE]), sre); }
      }
      #pragma unroll 2
      for (int t = staged + lane; t < k; t += 64) {
        if constexpr (CPLX) {
          R ar = R::load(&rl[(int64_t)t * WE]), ai = R::load(&rl[(int64_t)t * WE + WR]), br = R::load_shared(&rcol[(int64_t)t * WE]), bim = R::load_shared(&rcol[(int64_t)t * WE + WR]);
          /* S -= conj(a) b:  re -= ar br + ai bi;  im -= ar bi - ai br */
          sre = R::fnma(ar, br, sre); sre = R::fnma(ai, bim, sre); sim = R::fnma(ar, bim, sim); sim = R::fnma(ai.neg(), br, sim);
        } else { sre = R::fnma(R::load(&rl[(int64_t)t * WE]), R::load_shared(&rcol[(int64_t)t * WE]), sre); }
      }
      for (int m = 32; m > 0; m >>= 1) { sre = sre + sre.shfl_xor(m); if constexpr (CPLX) { sim = sim + sim.shfl_xor(m); } }
      if (lane == 0) {
        sre = sre + gre0; R rr = rho * sre; double* out = &a.Rt[((int64_t)l * a.ldr + k) * WE]; rr.store_shared(out);
        R d = d0;
        if constexpr (CPLX) { sim = sim + gim0; R ri = (rho * sim).neg(); ri.store_shared(out + WR); d = d - (rr * rr + ri * ri); } else { d = d - rr * rr; }
        d.store_shared(&a.D[(int64_t)l * WR]); tr += d.v.x;
        if (d.v.x > 0.) { better(DD, bx, by, bi, d.v.x, d.v.y, l); }
      }
    }
    /* the factor entries have to be in memory before the record that lets other workgroups go on; a workgroup barrier
     * does not wait for the stores of its wavefronts, so every wavefront waits for its own */
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    reduce_leaders<DD>(ex, bx, by, bi, tr);
    ++k; ++epoch;
    publish(&a.records[(epoch & 1) * MAX_WORKGROUPS + wg], bx, by, tr, bi, epoch);
    collect(ex, &a.records[(epoch & 1) * MAX_WORKGROUPS], nwg, epoch, bx, by, bi, tr);
    reduce_records<DD>(ex, nwg, bx, by, bi, tr);
    alive = ex.failed == 0;
    if (!(thresh < tr)) { bi = -1; }
  }
  /* reference quirk (src/hyacin_potrfp.cu:271): when exactly one column is left it is counted and its diagonal written */
  int rank = k;
  if (alive && N - k == 1) {
    if (wg == 0 && tid == 0) {
      const int c = a.jpiv[k] - 1;   /* positions k.. of the swap order hold the columns that were never a pivot */
      R d = R::load_shared(&a.D[(int64_t)c * WR]); R sq = R::zero(), rho; if (d.v.x > 0.) { sqrt_rsqrt<DD>(d, sq, rho); }
      double* rc = &a.Rt[((int64_t)c * a.ldr + k) * WE]; sq.store(rc); if constexpr (CPLX) { R::zero().store(rc + WR); }
    }
    rank = k + 1;
  }
  if (wg == 0 && tid == 0) { *a.rankOut = alive ? rank : -1; }
}

/* tags of an earlier run must not pass for an epoch of this one */
__global__ void clear_records_kernel(Record* r) { for (int j = 0; j < 8; ++j) { r[threadIdx.x].w[j] = 0ull; } }

/* one-time per kernel: how many workgroups may be co-resident */
template <bool DD, bool CPLX> int launch(hipStream_t stream, PotrfArgs& args, int cus) {
  int perCu = 0; if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCu, potrfp_kernel<DD, CPLX>, P_THREADS, 0) != hipSuccess || perCu < 1) { return -3; }
  int grid = cus < MAX_WORKGROUPS ? cus : MAX_WORKGROUPS; const int want = (args.N + P_WAVES - 1) / P_WAVES; if (grid > want) { grid = want; } if (grid < 1) { grid = 1; }
  if ((int64_t)grid * P_WAVES * 64 < args.N) { return -1; }   /* a wavefront tracks at most 64 columns */
  void* params[] = { &args };
  hipError_t e = hipLaunchCooperativeKernel(reinterpret_cast<const void*>(&potrfp_kernel<DD, CPLX>), dim3(grid), dim3(P_THREADS), params, 0, stream);
  return e == hipSuccess ? 0 : -3;
}

}  // namespace

extern "C" size_t hykPotrfpWorkspaceBytes(int32_t N, int32_t Gtype) {
  if (N <= 0) { return 0; }
  const size_t wr = ((Gtype & ~1) == HYK_DD) ? 2 : 1;
  /* D | pos | records (two epochs x MAX_WORKGROUPS) + alignment slack */
  return (size_t)N * wr * 8 + (size_t)N * 4 + 2 * MAX_WORKGROUPS * sizeof(Record) + 256;
}

extern "C" int hykPotrfp(hipStream_t stream, int32_t computeUnits, double eps, int32_t K, int32_t N, int32_t Gtype, const void* G, int64_t ldg, void* Rt, int32_t ldr, int32_t* jpiv, void* workspace, int32_t* rankOut) {
  if (N <= 0) { return 0; }
  if (!workspace) { return -1; }
  if (K <= 0 || K > N) { K = N; }
  if (ldg < N || ldr < (K < N ? K + 1 : N) || computeUnits < 1) { return -1; }
  const bool dd = (Gtype & ~1) == HYK_DD, cplx = Gtype & 1;
  if (!dd && (Gtype & ~1) != HYK_F64) { return -1; }
  PotrfArgs a; a.N = N; a.K = K; a.ldr = ldr; a.eps2 = eps * eps; a.G = (const double*)G; a.ldg = ldg; a.Rt = (double*)Rt; a.jpiv = jpiv; a.rankOut = rankOut;
  char* w = (char*)workspace; a.D = (double*)w; w += (size_t)N * (dd ? 2 : 1) * 8; a.pos = (int32_t*)w; w += (size_t)N * 4;
  w = (char*)(((uintptr_t)w + 63) & ~(uintptr_t)63); a.records = (Record*)w;
  clear_records_kernel<<<1, 2 * MAX_WORKGROUPS, 0, stream>>>(a.records);
  if (dd) { return cplx ? launch<true, true>(stream, a, computeUnits) : launch<true, false>(stream, a, computeUnits); }
  return cplx ? launch<false, true>(stream, a, computeUnits) : launch<false, false>(stream, a, computeUnits);
}

/* ---- the same factorisation for callers that cannot allocate device memory ----
 * The diagonal, the position table and the exchange records live in a file-scope device array instead of a workspace
 * argument.  Every device holds its own copy of the array at its own address; the address is looked up once per device
 * (with that device current) and only that pointer is ever handed to kernels. */
constexpr int32_t STATIC_MAX_N = 8192;
constexpr size_t STATIC_BYTES = (size_t)STATIC_MAX_N * 16 + (size_t)STATIC_MAX_N * 4 + 2 * MAX_WORKGROUPS * sizeof(Record) + 256;
static __device__ __align__(256) unsigned char scratch[STATIC_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::atomic<void*> g_scratchPtr[MAX_DEVICES];

/* device address of `scratch` on the current device; nullptr (and a message) when the runtime refuses */
void* static_scratch() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) { return nullptr; }
  void* p = g_scratchPtr[dev].load(std::memory_order_acquire);
  if (p) { return p; }
  const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !p) { std::fprintf(stderr, "hyacin: hipGetSymbolAddress(scratch) failed on device %d: %s\n", dev, hipGetErrorString(e)); return nullptr; }
  g_scratchPtr[dev].store(p, std::memory_order_release);   /* two threads racing here store the same address */
  return p;
}
}  // namespace

extern "C" int32_t hykPotrfpStaticMaxN(void) { return STATIC_MAX_N; }

extern "C" int hykPotrfpStatic(hipStream_t stream, int32_t computeUnits, double eps, int32_t K, int32_t N, int32_t Gtype, const void* G, int64_t ldg, void* Rt, int32_t ldr, int32_t* jpiv, int32_t* rankOut) {
  if (N <= 0) { return 0; }
  if (N > STATIC_MAX_N) { std::fprintf(stderr, "hyacin: hykPotrfpStatic: N = %d exceeds the built-in scratch (N <= %d); use hykPotrfp with a workspace\n", N, STATIC_MAX_N); return -2; }
  if (hykPotrfpWorkspaceBytes(N, Gtype) > STATIC_BYTES) { return -2; }
  void* ws = static_scratch();
  if (!ws) { return -3; }
  return hykPotrfp(stream, computeUnits, eps, K, N, Gtype, G, ldg, Rt, ldr, jpiv, ws, rankOut);
}
