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

/* one-time per kernel: how many workgroups may be co-resident */
template <bool DD, bool CPLX> int launch(hipStream_t stream, PotrfArgs& args, int cus) {
  int perCu = 0; if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCu, potrfp_kernel<DD, CPLX>, P_THREADS, 0) != hipSuccess || perCu < 1) { return -3; }
  int grid = cus < MAX_WORKGROUPS ? cus : MAX_WORKGROUPS; const int want = (args.N + P_WAVES - 1) / P_WAVES; if (grid > want) { grid = want; } if (grid < 1) { grid = 1; }
  if ((int64_t)grid * P_WAVES * 64 < args.N) { return -1; }   /* a wavefront tracks at most 64 columns */
  void* params[] = { &args };
  hipError_t e = hipLaunchCooperativeKernel(reinterpret_cast<const void*>(&potrfp_kernel<DD, CPLX>), dim3(grid), dim3(P_THREADS), params, 0, stream);
  return e == hipSuccess ? 0 : -3;
}


/* ====================================================================================================================
 * Blocked, right-looking form (N <= 8192): the factorization advances in panels of PB columns.
 *
 *  - Panel.  One wavefront per 64 columns is an *agent* (wavefront 0 of workgroup a < agents); a lane owns one column
 *    for the whole run: its remaining diagonal entry lives in a register, its entries of the current panel's rows in
 *    LDS.  The trailing matrix G' is kept up to date by the update phase, so a step needs, per lane, G'[l, c] and the
 *    dot product of at most PB - 1 factor entries.  Per step an agent publishes ONE 128-byte record (arg-max and trace
 *    of its columns and the candidate's newest factor entry, every 32-bit piece in a 64-bit word tagged with the step
 *    number) and every agent polls all records, one lane per record, and reduces them inside the wavefront: no
 *    workgroup barrier and no LDS on the chain from one pivot to the next.  The factor entries of a step are stored
 *    after its record (the one entry another agent can need before they are visible travels in the record).
 *  - Update.  After a panel every workgroup drops the new pivots from its sorted list of remaining columns and all
 *    workgroups apply the rank-PB update G'[l, m] -= sum_t conj(R[t, l]) R[t, m] to the pairs l < m of remaining
 *    columns, in 64 x 64 tiles (operands in LDS, a 4 x 4 block per lane).  Only the strict upper triangle of G' is kept;
 *    the panel reads G'[l, c] as conj(G'[c, l]) where l > c.  G is overwritten (as in the reference).
 *  - What crosses workgroups (records, factor entries, G', pivots) is stored write-through and loaded past the
 *    non-coherent cache levels; a counter that every workgroup bumps after its update tiles is the one grid-wide
 *    rendezvous per panel.  Every wait is bounded and gives up for the whole grid.
 * ==================================================================================================================== */
namespace blk {

constexpr int THREADS = 256;        /* four wavefronts: the first leads (agent or waiter), all four update */
constexpr int PB = 16;              /* columns per panel */
constexpr int MAX_AGENTS = 128;     /* 64 columns each */
constexpr int MAX_N = MAX_AGENTS * 64;
constexpr int REC_WORDS = 16;       /* 128 bytes per record */
constexpr int TILE = 64;
constexpr int SPIN = 1 << 21;
constexpr int CTL_WORDS = 32;       /* control block: [0], [1] tagged panel summary; [8] update counter */

struct Args {
  int32_t N, K, ldr, agents; double eps2;
  double* G; int64_t ldg; double* Rt; int32_t* jpiv; int32_t* pos; uint64_t* records; uint64_t* ctl; int32_t* rankOut;
};

__device__ __forceinline__ uint64_t ld_shared_u64(const uint64_t* p) { return __hip_atomic_load(const_cast<uint64_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_shared_u64(uint64_t* p, uint64_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ int32_t ld_shared_i32(const int32_t* p) { return __hip_atomic_load(const_cast<int32_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_shared_i32(int32_t* p, int32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

/* what an agent publishes per step, all wavefront-uniform */
struct Msg { double bx, by, tr, n[4]; int32_t bi; };

/* lane j < 15 stores word j = epoch << 32 | piece j; pieces: the halves of bx, by, tr, n[0..3], then the index */
__device__ __forceinline__ void publish(uint64_t* rec, const Msg& m, uint32_t epoch) {
  const int j = threadIdx.x & 63, q = j >> 1;
  double v = m.bx; v = q == 1 ? m.by : v; v = q == 2 ? m.tr : v; v = q == 3 ? m.n[0] : v; v = q == 4 ? m.n[1] : v; v = q == 5 ? m.n[2] : v; v = q == 6 ? m.n[3] : v;
  const uint64_t bits = (uint64_t)__double_as_longlong(v);
  const uint32_t piece = j == 14 ? (uint32_t)m.bi : (uint32_t)(bits >> (32 * (j & 1)));
  if (j < 15) { st_shared_u64(&rec[j], ((uint64_t)epoch << 32) | piece); }
}

/* waits for record `r` of `epoch` (bounded); false when the wait gave up */
__device__ __forceinline__ bool read_record(const uint64_t* rec, uint32_t epoch, Msg& m) {
  uint64_t v[15];
  for (int spins = 0;; ++spins) {
    bool complete = true;
    #pragma unroll
    for (int j = 0; j < 15; ++j) { v[j] = ld_shared_u64(&rec[j]); }
    #pragma unroll
    for (int j = 0; j < 15; ++j) { complete = complete && (uint32_t)(v[j] >> 32) == epoch; }
    if (complete) { break; }
    if (spins > SPIN) { return false; }
    __builtin_amdgcn_s_sleep(1);
  }
  auto dbl = [&](int q) { return __longlong_as_double((long long)((v[2 * q] & 0xffffffffull) | (v[2 * q + 1] << 32))); };
  m.bx = dbl(0); m.by = dbl(1); m.tr = dbl(2); m.n[0] = dbl(3); m.n[1] = dbl(4); m.n[2] = dbl(5); m.n[3] = dbl(6); m.bi = (int32_t)(uint32_t)v[14];
  return true;
}

/* All records of `epoch` -> in every lane: the best column over all agents (its value, its newest factor entry) and the
 * total trace.  Lane i reads records i and i + 64.  Every agent runs the same instructions on the same data, so all
 * agents take the same decisions.  Returns false when a wait gave up. */
template <bool DD>
__device__ __forceinline__ bool collect(const uint64_t* recs, int agents, uint32_t epoch, Msg& out) {
  const int lane = threadIdx.x & 63; bool ok = true;
  Msg m; m.bx = m.by = m.tr = 0.; m.bi = -1; m.n[0] = m.n[1] = m.n[2] = m.n[3] = 0.;
  if (lane < agents) { ok = read_record(&recs[(size_t)lane * REC_WORDS], epoch, m); if (!ok) { m.bi = -1; m.tr = 0.; } }
  if (lane + 64 < agents) {
    Msg o; const bool ok2 = read_record(&recs[(size_t)(lane + 64) * REC_WORDS], epoch, o); ok = ok && ok2;
    if (ok2) {
      const int before = m.bi; better(DD, m.bx, m.by, m.bi, o.bx, o.by, o.bi); m.tr += o.tr;
      if (m.bi != before) { m.n[0] = o.n[0]; m.n[1] = o.n[1]; m.n[2] = o.n[2]; m.n[3] = o.n[3]; }
    }
  }
  out.bx = m.bx; out.by = m.by; out.bi = m.bi; out.tr = m.tr;
  wave_reduce<DD, 6>(out.bx, out.by, out.bi, out.tr);
  /* the winner's newest entry sits in the lane that read its record */
  const int src = out.bi >= 0 ? ((out.bi >> 6) & 63) : 0;
  #pragma unroll
  for (int q = 0; q < 4; ++q) { out.n[q] = __shfl(m.n[q], src, 64); }
  return __all(ok);
}

template <bool DD, bool CPLX>
__global__ __launch_bounds__(THREADS) void potrfp_blocked_kernel(const Args a) {
  using R = Real<DD>; constexpr int WR = Width<DD, CPLX>::real, WE = Width<DD, CPLX>::elem;
  extern __shared__ __attribute__((aligned(16))) double lds[];
  /* LDS: [operands / own rows: 2 * TILE * PB * WE doubles][pivot rows: PB * WE doubles][remaining columns: N uint16] */
  double* const own = lds;                              /* agent: own[(t * 64 + lane) * WE + w]; update: operand A */
  double* const opB = lds + TILE * PB * WE;             /* update: operand B */
  double* const prow = lds + 2 * TILE * PB * WE;        /* agent: factor entries of the pivot column in this panel */
  uint16_t* const list = reinterpret_cast<uint16_t*>(prow + PB * WE);
  __shared__ int32_t info[4];                           /* panel end, finished, failed */
  __shared__ int32_t piv[PB];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wg = blockIdx.x, nwg = gridDim.x;
  const int N = a.N, P = a.agents; const bool agent = wave == 0 && wg < P;
  const int l = wg * 64 + lane; const bool mine = agent && l < N;

  for (int i = tid; i < N; i += THREADS) { list[i] = (uint16_t)i; }
  if (wg == 0) { for (int i = tid; i < N; i += THREADS) { st_shared_i32(&a.jpiv[i], i + 1); st_shared_i32(&a.pos[i], i); } }
  if (tid == 0) { info[0] = 0; info[1] = 0; info[2] = 0; }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  int na = N;

  /* agent state */
  R d = R::zero(); bool dead = !mine; uint32_t epoch = 0; Msg cur; cur.bi = -1; cur.bx = cur.by = cur.tr = 0.; cur.n[0] = cur.n[1] = cur.n[2] = cur.n[3] = 0.;
  double thresh = 0.; int k = 0; bool failed = false, stop = false;
  const int Kstop = a.K >= N ? N - 1 : a.K;
  if (agent) {
    Msg m; m.bx = m.by = m.tr = 0.; m.bi = -1; m.n[0] = m.n[1] = m.n[2] = m.n[3] = 0.;
    if (mine) { d = R::load_shared(&a.G[((int64_t)l + (int64_t)l * a.ldg) * WE]); m.tr = d.v.x; if (d.v.x > 0.) { m.bx = d.v.x; m.by = d.v.y; m.bi = l; } }
    wave_reduce<DD, 6>(m.bx, m.by, m.bi, m.tr);
    ++epoch; publish(&a.records[((size_t)(epoch & 1) * MAX_AGENTS + wg) * REC_WORDS], m, epoch);
    failed = !collect<DD>(&a.records[(size_t)(epoch & 1) * MAX_AGENTS * REC_WORDS], P, epoch, cur);
    thresh = a.eps2 * cur.tr;
    stop = failed || cur.bi < 0 || k >= Kstop;
  }

  for (int kb = 0, panel = 0;; kb += PB, ++panel) {
    if (wave == 0) {
      if (agent && !failed) {
        if (panel > 0) {   /* every workgroup has applied the previous panel to G' */
          const uint32_t want = (uint32_t)nwg * (uint32_t)panel; int spins = 0;
          while (__hip_atomic_load(reinterpret_cast<uint32_t*>(&a.ctl[8]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want) { if (++spins > SPIN) { failed = true; break; } __builtin_amdgcn_s_sleep(1); }
        }
        while (!failed && !stop && k < kb + PB) {
          const int c = cur.bi, j = k - kb; R dc{ dd_t{ cur.bx, cur.by } }, sq, rho; sqrt_rsqrt<DD>(dc, sq, rho);
          /* factor entries R[kb .. k, c] of the pivot column: lane t fetches entry t, the newest one came with the record */
          if (lane < j - 1) {
            const double* src = &a.Rt[((int64_t)c * a.ldr + kb + lane) * WE];
            #pragma unroll
            for (int w = 0; w < WE; ++w) { prow[lane * WE + w] = __hip_atomic_load(const_cast<double*>(src) + w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
          }
          if (lane == 0 && j > 0) {
            #pragma unroll
            for (int w = 0; w < WE; ++w) { prow[(j - 1) * WE + w] = cur.n[w]; }
          }
          R rr = R::zero(), ri = R::zero();
          const bool work = !dead && l != c;
          if (work) {
            R gre, gim = R::zero();
            if (l < c) { const double* g = &a.G[((int64_t)l + (int64_t)c * a.ldg) * WE]; gre = R::load_shared(g); if constexpr (CPLX) { gim = R::load_shared(g + WR); } }
            else { const double* g = &a.G[((int64_t)c + (int64_t)l * a.ldg) * WE]; gre = R::load_shared(g); if constexpr (CPLX) { gim = R::load_shared(g + WR).neg(); } }
            R sre = gre, sim = gim;
            for (int t = 0; t < j; ++t) {
              const double* o = &own[(t * 64 + lane) * WE]; const double* b = &prow[t * WE];
              if constexpr (CPLX) {
                const R ar = R::load(o), ai = R::load(o + WR), br = R::load(b), bim = R::load(b + WR);
                /* S -= conj(a) b:  re -= ar br + ai bi;  im -= ar bi - ai br */
                sre = R::fnma(ar, br, sre); sre = R::fnma(ai, bim, sre); sim = R::fnma(ar, bim, sim); sim = R::fnma(ai.neg(), br, sim);
              } else { sre = R::fnma(R::load(o), R::load(b), sre); }
            }
            rr = rho * sre; if constexpr (CPLX) { ri = (rho * sim).neg(); }
            if constexpr (CPLX) { d = d - (rr * rr + ri * ri); } else { d = d - rr * rr; }
          }
          if (!dead && l == c) { rr = sq; ri = R::zero(); dead = true; }
          const bool wrote = work || (mine && l == c);
          if (wrote) { double* o = &own[(j * 64 + lane) * WE]; rr.store(o); if constexpr (CPLX) { ri.store(o + WR); } }
          /* arg-max and trace of the columns this agent still has, and the candidate's newest entry */
          Msg m; m.bx = m.by = m.tr = 0.; m.bi = -1;
          if (!dead) { m.tr = d.v.x; if (d.v.x > 0.) { m.bx = d.v.x; m.by = d.v.y; m.bi = l; } }
          wave_reduce<DD, 6>(m.bx, m.by, m.bi, m.tr);
          { const int src = m.bi >= 0 ? (m.bi & 63) : 0;
            m.n[0] = __shfl(rr.v.x, src, 64); m.n[1] = m.n[2] = m.n[3] = 0.;
            if constexpr (DD) { m.n[1] = __shfl(rr.v.y, src, 64); }
            if constexpr (CPLX) { m.n[WR] = __shfl(ri.v.x, src, 64); if constexpr (DD) { m.n[WR + 1] = __shfl(ri.v.y, src, 64); } } }
          ++k; ++epoch;
          const bool last = (k == kb + PB) || (k >= Kstop);   /* the update (or the host) reads this panel's factor entries next */
          double* out = &a.Rt[((int64_t)l * a.ldr + (k - 1)) * WE];
          if (last) { if (wrote) { rr.store_shared(out); if constexpr (CPLX) { ri.store_shared(out + WR); } } asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
          publish(&a.records[((size_t)(epoch & 1) * MAX_AGENTS + wg) * REC_WORDS], m, epoch);
          if (!last && wrote) { rr.store_shared(out); if constexpr (CPLX) { ri.store_shared(out + WR); } }
          if (wg == 0 && lane == 0) {   /* pivot bookkeeping in the reference's swap order */
            const int p = ld_shared_i32(&a.pos[c]), c0 = ld_shared_i32(&a.jpiv[k - 1]) - 1;
            st_shared_i32(&a.jpiv[k - 1], c + 1); st_shared_i32(&a.jpiv[p], c0 + 1); st_shared_i32(&a.pos[c], k - 1); st_shared_i32(&a.pos[c0], p);
          }
          failed = !collect<DD>(&a.records[(size_t)(epoch & 1) * MAX_AGENTS * REC_WORDS], P, epoch, cur);
          if (!(thresh < cur.tr)) { cur.bi = -1; }
          stop = failed || cur.bi < 0 || k >= Kstop;
        }
        if (wg == 0) {   /* panel summary for every workgroup: columns done, and whether the factorization ends here */
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          const uint32_t seq = (uint32_t)panel + 1u;
          if (lane == 0) { st_shared_u64(&a.ctl[0], ((uint64_t)seq << 32) | (uint32_t)k); st_shared_u64(&a.ctl[1], ((uint64_t)seq << 32) | (uint32_t)((stop ? 1 : 0) | (failed ? 2 : 0))); }
        }
      }
      /* every leader waits for the summary */
      { const uint32_t seq = (uint32_t)panel + 1u; uint64_t s0 = 0, s1 = 0; int spins = 0; bool got = false;
        while (!failed) {
          s0 = ld_shared_u64(&a.ctl[0]); s1 = ld_shared_u64(&a.ctl[1]);
          if ((uint32_t)(s0 >> 32) == seq && (uint32_t)(s1 >> 32) == seq) { got = true; break; }
          if (++spins > SPIN) { failed = true; break; }
          __builtin_amdgcn_s_sleep(4);
        }
        if (lane == 0) { info[0] = got ? (int32_t)(uint32_t)s0 : 0; info[1] = got ? (int32_t)((uint32_t)s1 & 1u) : 1; info[2] = (failed || (got && ((uint32_t)s1 & 2u))) ? 1 : 0; }
      }
    }
    __syncthreads();
    const int ke = info[0], fin = info[1], bad = info[2];
    __syncthreads();   /* info is rewritten in the next round */
    if (bad) { failed = true; break; }
    if (fin) { break; }
    const int nbk = ke - kb;

    /* ---- update phase ---- */
    if (tid < nbk) { piv[tid] = ld_shared_i32(&a.jpiv[kb + tid]) - 1; }
    __syncthreads();
    { /* drop the new pivots from the sorted list of remaining columns */
      constexpr int PER = MAX_N / THREADS; uint16_t keep[PER]; int16_t to[PER];
      #pragma unroll
      for (int e = 0; e < PER; ++e) {
        const int idx = tid + e * THREADS; to[e] = -1;
        if (idx < na) { const int v = list[idx]; int shift = 0; bool gone = false; for (int i = 0; i < nbk; ++i) { shift += piv[i] < v ? 1 : 0; gone = gone || piv[i] == v; } keep[e] = (uint16_t)v; if (!gone) { to[e] = (int16_t)(idx - shift); } }
      }
      __syncthreads();
      #pragma unroll
      for (int e = 0; e < PER; ++e) { if (to[e] >= 0) { list[to[e]] = keep[e]; } }
      na -= nbk;
      __syncthreads();
    }
    const int nT = (na + TILE - 1) / TILE, tiles = nT * (nT + 1) / 2;
    for (int tile = wg; tile < tiles; tile += nwg) {
      int J = (int)((sqrtf(8.f * (float)tile + 1.f) - 1.f) * 0.5f); while ((J + 1) * (J + 2) / 2 <= tile) { ++J; } while (J * (J + 1) / 2 > tile) { --J; }
      const int I = tile - J * (J + 1) / 2;
      /* operands: the panel's factor entries of 64 remaining columns each, op[(t * 64 + col) * WE + w] */
      for (int e = tid; e < 2 * TILE * PB; e += THREADS) {
        const int which = e / (TILE * PB), r = e % (TILE * PB), col = r / PB, t = r % PB; if (which == 1 && I == J) { break; }
        const int li = (which ? J : I) * TILE + col; double* dst = &(which ? opB : own)[(t * 64 + col) * WE];
        if (li < na && t < nbk) {
          const double* src = &a.Rt[((int64_t)list[li] * a.ldr + kb + t) * WE];
          #pragma unroll
          for (int w = 0; w < WE; ++w) { dst[w] = __hip_atomic_load(const_cast<double*>(src) + w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
        } else {
          #pragma unroll
          for (int w = 0; w < WE; ++w) { dst[w] = 0.; }
        }
      }
      __syncthreads();
      const double* A = own; const double* B = I == J ? own : opB;
      const int ry = (wave >> 1) * 32 + (lane & 7), cx = (wave & 1) * 32 + (lane >> 3);
      R sre[4][4], sim[4][4];
      #pragma unroll
      for (int i = 0; i < 4; ++i) {
        #pragma unroll
        for (int jj = 0; jj < 4; ++jj) { sre[i][jj] = R::zero(); sim[i][jj] = R::zero(); }
      }
      for (int t = 0; t < nbk; ++t) {
        R ar[4], ai[4], br[4], bi[4];
        #pragma unroll
        for (int i = 0; i < 4; ++i) {
          const double* pa = &A[(t * 64 + ry + 8 * i) * WE]; const double* pb = &B[(t * 64 + cx + 8 * i) * WE];
          ar[i] = R::load(pa); br[i] = R::load(pb); if constexpr (CPLX) { ai[i] = R::load(pa + WR); bi[i] = R::load(pb + WR); }
        }
        #pragma unroll
        for (int i = 0; i < 4; ++i) {
          #pragma unroll
          for (int jj = 0; jj < 4; ++jj) {
            /* G'[l, m] -= conj(R[t, l]) R[t, m] */
            sre[i][jj] = R::fnma(ar[i], br[jj], sre[i][jj]);
            if constexpr (CPLX) { sre[i][jj] = R::fnma(ai[i], bi[jj], sre[i][jj]); sim[i][jj] = R::fnma(ar[i], bi[jj], sim[i][jj]); sim[i][jj] = R::fnma(ai[i].neg(), br[jj], sim[i][jj]); }
          }
        }
      }
      #pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int li = I * TILE + ry + 8 * i; if (li >= na) { continue; } const int lcol = list[li];
        #pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int mi = J * TILE + cx + 8 * jj; if (mi >= na || li >= mi) { continue; } const int mcol = list[mi];
          double* g = &a.G[((int64_t)lcol + (int64_t)mcol * a.ldg) * WE];
          (R::load_shared(g) + sre[i][jj]).store_shared(g);
          if constexpr (CPLX) { (R::load_shared(g + WR) + sim[i][jj]).store_shared(g + WR); }
        }
      }
      __syncthreads();
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) { __hip_atomic_fetch_add(reinterpret_cast<uint32_t*>(&a.ctl[8]), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
  }

  /* reference quirk (src/hyacin_potrfp.cu:271): when exactly one column is left it is counted and its diagonal written */
  if (agent && !failed && N - k == 1 && !dead) {
    R sq = R::zero(), rho; if (d.v.x > 0.) { sqrt_rsqrt<DD>(d, sq, rho); }
    double* rc = &a.Rt[((int64_t)l * a.ldr + k) * WE]; sq.store(rc); if constexpr (CPLX) { R::zero().store(rc + WR); }
  }
  if (wg == 0 && tid == 0) { *a.rankOut = failed ? -1 : ((N - k == 1) ? k + 1 : k); }
}

template <bool DD, bool CPLX> int launch(hipStream_t stream, Args& args, int cus) {
  constexpr int WE = Width<DD, CPLX>::elem;
  const size_t ldsBytes = (size_t)(2 * TILE * PB * WE + PB * WE) * 8 + (size_t)args.N * 2 + 16;
  const void* fn = reinterpret_cast<const void*>(&potrfp_blocked_kernel<DD, CPLX>);
  if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes) != hipSuccess) { return -3; }
  int perCu = 0; if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCu, potrfp_blocked_kernel<DD, CPLX>, THREADS, ldsBytes) != hipSuccess || perCu < 1) { return -3; }
  int grid = cus < 256 ? cus : 256; if (grid < args.agents) { return -1; }
  void* params[] = { &args };
  return hipLaunchCooperativeKernel(fn, dim3(grid), dim3(THREADS), params, (unsigned)ldsBytes, stream) == hipSuccess ? 0 : -3;
}

__global__ void clear_kernel(uint64_t* p, int words) { for (int i = threadIdx.x; i < words; i += blockDim.x) { p[i] = 0ull; } }

}  // namespace blk

}  // namespace

namespace {
/* workspace: [pos: N int32][exchange area: records / control words of either kernel][D: N reals (left-looking kernel)] */
constexpr size_t EXCHANGE_BYTES = 2 * blk::MAX_AGENTS * blk::REC_WORDS * 8 + blk::CTL_WORDS * 8;
static_assert(EXCHANGE_BYTES >= 2 * MAX_WORKGROUPS * sizeof(Record), "the exchange area holds the records of either kernel");
size_t align256(size_t v) { return (v + 255) / 256 * 256; }

int run_potrfp(hipStream_t stream, bool blocked, int32_t computeUnits, double eps, int32_t K, int32_t N, int32_t Gtype, void* G, int64_t ldg, void* Rt, int32_t ldr, int32_t* jpiv, void* workspace, int32_t* rankOut) {
  if (N <= 0) { return 0; }
  if (!workspace || !G || !Rt || !jpiv || !rankOut) { return -1; }
  if (K <= 0 || K > N) { K = N; }
  if (ldg < N || ldr < (K < N ? K + 1 : N) || computeUnits < 1) { return -1; }
  const bool dd = (Gtype & ~1) == HYK_DD, cplx = Gtype & 1;
  if (!dd && (Gtype & ~1) != HYK_F64) { return -1; }
  char* w = (char*)workspace; int32_t* pos = (int32_t*)w; w += align256((size_t)N * 4); uint64_t* exchange = (uint64_t*)w; w += EXCHANGE_BYTES; double* D = (double*)w;
  blk::clear_kernel<<<1, 256, 0, stream>>>(exchange, (int)(EXCHANGE_BYTES / 8));
  const int agents = (N + 63) / 64, grid = computeUnits < 256 ? computeUnits : 256;
  if (blocked && N <= blk::MAX_N && agents <= grid) {
    blk::Args b; b.N = N; b.K = K; b.ldr = ldr; b.agents = agents; b.eps2 = eps * eps; b.G = (double*)G; b.ldg = ldg; b.Rt = (double*)Rt; b.jpiv = jpiv; b.pos = pos;
    b.records = exchange; b.ctl = exchange + 2 * blk::MAX_AGENTS * blk::REC_WORDS; b.rankOut = rankOut;
    if (dd) { return cplx ? blk::launch<true, true>(stream, b, computeUnits) : blk::launch<true, false>(stream, b, computeUnits); }
    return cplx ? blk::launch<false, true>(stream, b, computeUnits) : blk::launch<false, false>(stream, b, computeUnits);
  }
  PotrfArgs a; a.N = N; a.K = K; a.ldr = ldr; a.eps2 = eps * eps; a.G = (const double*)G; a.ldg = ldg; a.Rt = (double*)Rt; a.jpiv = jpiv; a.rankOut = rankOut;
  a.D = D; a.pos = pos; a.records = (Record*)exchange;
  if (dd) { return cplx ? launch<true, true>(stream, a, computeUnits) : launch<true, false>(stream, a, computeUnits); }
  return cplx ? launch<false, true>(stream, a, computeUnits) : launch<false, false>(stream, a, computeUnits);
}
}  // namespace

extern "C" size_t hykPotrfpWorkspaceBytes(int32_t N, int32_t Gtype) {
  if (N <= 0) { return 0; }
  const size_t wr = ((Gtype & ~1) == HYK_DD) ? 2 : 1;
  return align256((size_t)N * 4) + EXCHANGE_BYTES + align256((size_t)N * wr * 8);
}

extern "C" int hykPotrfp(hipStream_t stream, int32_t computeUnits, double eps, int32_t K, int32_t N, int32_t Gtype, void* G, int64_t ldg, void* Rt, int32_t ldr, int32_t* jpiv, void* workspace, int32_t* rankOut) {
  return run_potrfp(stream, true, computeUnits, eps, K, N, Gtype, G, ldg, Rt, ldr, jpiv, workspace, rankOut);
}

extern "C" int hykPotrfpLeftLooking(hipStream_t stream, int32_t computeUnits, double eps, int32_t K, int32_t N, int32_t Gtype, void* G, int64_t ldg, void* Rt, int32_t ldr, int32_t* jpiv, void* workspace, int32_t* rankOut) {
  return run_potrfp(stream, false, computeUnits, eps, K, N, Gtype, G, ldg, Rt, ldr, jpiv, workspace, rankOut);
}

/* ---- the same factorisation for callers that cannot allocate device memory ----
 * The diagonal, the position table and the exchange records live in a file-scope device array instead of a workspace
 * argument.  Every device holds its own copy of the array at its own address; the address is looked up once per device
 * (with that device current) and only that pointer is ever handed to kernels. */
constexpr int32_t STATIC_MAX_N = 8192;
constexpr size_t STATIC_BYTES = (size_t)STATIC_MAX_N * 4 + EXCHANGE_BYTES + (size_t)STATIC_MAX_N * 16;   /* hykPotrfpWorkspaceBytes(8192, double-double) */
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

extern "C" int hykPotrfpStatic(hipStream_t stream, int32_t computeUnits, double eps, int32_t K, int32_t N, int32_t Gtype, void* G, int64_t ldg, void* Rt, int32_t ldr, int32_t* jpiv, int32_t* rankOut) {
  if (N <= 0) { return 0; }
  if (N > STATIC_MAX_N) { std::fprintf(stderr, "hyacin: hykPotrfpStatic: N = %d exceeds the built-in scratch (N <= %d); use hykPotrfp with a workspace\n", N, STATIC_MAX_N); return -2; }
  if (hykPotrfpWorkspaceBytes(N, Gtype) > STATIC_BYTES) { return -2; }
  void* ws = static_scratch();
  if (!ws) { return -3; }
  return hykPotrfp(stream, computeUnits, eps, K, N, Gtype, G, ldg, Rt, ldr, jpiv, ws, rankOut);
}
