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
/* hykPotrfpSetPlainLaunch: the kernels here are launched cooperatively (the runtime then guarantees that all workgroups are
 * resident, which their waits for each other rely on).  With this set, a grid that the occupancy query says fits the device
 * is started with a plain launch instead: on an otherwise idle device that comes to the same, and a grid that does not
 * become resident after all fails safe (every wait is bounded and gives the run up with rank -1).  The same plain launch
 * is what a call falls back to when the runtime refuses the cooperative one (seen when a second process on the device has
 * made cooperative launches of its own): the refusal is cleared from the runtime's error state and not reported. */
std::atomic<int> g_plainLaunch{ 0 };

bool fits_device(int grid, int perCu) {
  int dev = 0, units = 0;
  return hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && (int64_t)grid <= (int64_t)units * perCu;
}

constexpr int SPIN_LIMIT = 1 << 22;   /* polls of one record before the run is given up (seconds; a healthy wait is microseconds) */

struct PotrfArgs {
  int32_t N, K, ldr; double eps2;
  const double* G; int64_t ldg;
  double* Rt; double* D; int32_t* jpiv; int32_t* pos; Record* records; int32_t* rankOut; double* traceOut;
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
  if (wg == 0 && tid == 0) { *a.rankOut = alive ? rank : -1; if (a.traceOut) { *a.traceOut = 0.; } }   /* this kernel has no cut (hykPotrfpWanted) */
}

/* one-time per kernel: how many workgroups may be co-resident */
template <bool DD, bool CPLX> int launch(hipStream_t stream, PotrfArgs& args, int cus) {
  int perCu = 0; if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCu, potrfp_kernel<DD, CPLX>, P_THREADS, 0) != hipSuccess || perCu < 1) { return -3; }
  int grid = cus < MAX_WORKGROUPS ? cus : MAX_WORKGROUPS; const int want = (args.N + P_WAVES - 1) / P_WAVES; if (grid > want) { grid = want; } if (grid < 1) { grid = 1; }
  if ((int64_t)grid * P_WAVES * 64 < args.N) { return -1; }   /* a wavefront tracks at most 64 columns */
  const bool fits = fits_device(grid, perCu);
  if (!(g_plainLaunch.load(std::memory_order_relaxed) && fits)) {
    void* params[] = { &args };
    if (hipLaunchCooperativeKernel(reinterpret_cast<const void*>(&potrfp_kernel<DD, CPLX>), dim3(grid), dim3(P_THREADS), params, 0, stream) == hipSuccess) { return 0; }
    (void)hipGetLastError();   /* refused: not to be found by the next call that asks for the last error */
    if (!fits) { return -3; }
  }
  potrfp_kernel<DD, CPLX><<<grid, P_THREADS, 0, stream>>>(args); return hipGetLastError() == hipSuccess ? 0 : -3;
}


/* ====================================================================================================================
 * Blocked, right-looking form (N <= 8192): the factorization advances in panels of PB columns.
 *
 *  - Panel.  One wavefront per 64 columns is an *agent* (wavefront 0 of workgroup a < agents; column l belongs to agent
 *    l % agents); a lane owns one column for the whole run: its remaining diagonal entry lives in a register, its entries of the current panel's rows in
 *    LDS.  The trailing matrix G' is kept up to date by the update phase, so a step needs, per lane, G'[l, c] and a
 *    dot product of at most PB - 1 factor entries.  Per step an agent publishes ONE record (arg-max and trace of its
 *    columns and the candidate's newest factor entry; every 32-bit piece in a 64-bit word tagged with the step number,
 *    word j of all agents side by side so that a poll of all records touches two or three cache lines per word) and
 *    every agent polls all records, one lane per record, and reduces them inside the wavefront with data-parallel
 *    lane exchanges: no workgroup barrier and no LDS on the chain from one pivot to the next.  The factor entries of a
 *    step are stored after its record (the one entry another agent can need before they are visible travels in the
 *    record).  While a step runs, the agents fetch what the next step needs if the runner-up of the last arg-max
 *    becomes the pivot (its column of G' and its factor entries); when it does, the step starts without waiting for
 *    memory.
 *  - Update.  After a panel every workgroup drops the new pivots from its sorted list of remaining columns and all
 *    workgroups apply the rank-PB update G'[l, m] -= sum_t conj(R[t, l]) R[t, m] to the pairs l < m of remaining
 *    columns, in 64 x 64 tiles (operands in LDS, a 4 x 4 block per lane).  Only the strict upper triangle of G' is kept;
 *    the panel reads G'[l, c] as conj(G'[c, l]) where l > c.  G is overwritten (as in the reference).
 *  - What crosses workgroups (records, factor entries, G', the panel summary) is stored write-through and loaded past
 *    the non-coherent cache levels; a counter that every workgroup bumps after its update tiles is the one grid-wide
 *    rendezvous per panel.  Every wait is bounded and gives up for the whole grid.
 * ==================================================================================================================== */
namespace blk {

constexpr int THREADS = 256;        /* four wavefronts: the first leads (agent or waiter), all four update */
constexpr int MAX_PB = 32;          /* columns per panel: 32 for real matrices, 16 for complex ones */
constexpr int MAX_AGENTS = 128;     /* 64 columns each */
constexpr int MAX_N = MAX_AGENTS * 64;
constexpr int REC_WORDS = 16;       /* at most 15 tagged words per record */
constexpr int TILE = 64;
constexpr int SPIN = 1 << 21;
constexpr int CTL_WORDS = 64;       /* control block: [0 .. 2 + PB/2) tagged panel summary; [32] update counter; [40 .. 50) timing sums */
constexpr int CTL_COUNTER = 32, CTL_TIMING = 40;

struct Args {
  int32_t N, K, ldr, agents; double eps2;
  double* G; int64_t ldg; double* Rt; int32_t* jpiv; uint64_t* records; uint64_t* ctl; int32_t* rankOut;
  /* wanted / cut: a caller that uses the `wanted` leading values of the factor only lets the factorization end once what is
   * left of G weighs little against them (hykPotrfpWanted); traceOut: the trace of what is left when the factorization ends */
  int32_t wanted; double cut; double* traceOut;
};

__device__ __forceinline__ uint64_t ld_shared_u64(const uint64_t* p) { return __hip_atomic_load(const_cast<uint64_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_shared_u64(uint64_t* p, uint64_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

/* ---- wavefront-wide arg-max / sum without LDS: six exchange steps, after which every lane holds the result.
 * Steps 0..3 stay inside a row of 16 lanes (quad permutations, then the two mirror patterns: any pairing that joins
 * two groups holding equal values does), steps 4 and 5 swap rows / halves between two registers. */
template <int STEP> __device__ __forceinline__ void pair_u32(uint32_t v, uint32_t& x, uint32_t& y) {
  if constexpr (STEP == 0) { x = v; y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xf, 0xf, false); }
  else if constexpr (STEP == 1) { x = v; y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xf, 0xf, false); }
  else if constexpr (STEP == 2) { x = v; y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xf, 0xf, false); }
  else if constexpr (STEP == 3) { x = v; y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xf, 0xf, false); }
  else if constexpr (STEP == 4) { const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false); x = r[0]; y = r[1]; }
  else { const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false); x = r[0]; y = r[1]; }
}
template <int STEP> __device__ __forceinline__ void pair_f64(double v, double& x, double& y) {
  const uint64_t b = (uint64_t)__double_as_longlong(v); uint32_t xl, yl, xh, yh;
  pair_u32<STEP>((uint32_t)b, xl, yl); pair_u32<STEP>((uint32_t)(b >> 32), xh, yh);
  x = __longlong_as_double((long long)(((uint64_t)xh << 32) | xl)); y = __longlong_as_double((long long)(((uint64_t)yh << 32) | yl));
}
template <bool DD, int STEP> __device__ __forceinline__ void reduce_step(double& bx, double& by, int32_t& bi, double& tr) {
  double x0, x1, y0 = 0., y1 = 0., t0, t1; uint32_t i0, i1;
  pair_f64<STEP>(bx, x0, x1); if constexpr (DD) { pair_f64<STEP>(by, y0, y1); } pair_u32<STEP>((uint32_t)bi, i0, i1); pair_f64<STEP>(tr, t0, t1);
  bx = x0; by = y0; bi = (int32_t)i0; better(DD, bx, by, bi, x1, y1, (int32_t)i1); tr = t0 + t1;
}
template <bool DD> __device__ __forceinline__ void reduce_wave_full(double& bx, double& by, int32_t& bi, double& tr) {
  reduce_step<DD, 0>(bx, by, bi, tr); reduce_step<DD, 1>(bx, by, bi, tr); reduce_step<DD, 2>(bx, by, bi, tr);
  reduce_step<DD, 3>(bx, by, bi, tr); reduce_step<DD, 4>(bx, by, bi, tr); reduce_step<DD, 5>(bx, by, bi, tr);
}
template <int STEP> __device__ __forceinline__ void max_sum_step(double& bx, double& tr) {
  double x0, x1, t0, t1; pair_f64<STEP>(bx, x0, x1); pair_f64<STEP>(tr, t0, t1); bx = x0 < x1 ? x1 : x0; tr = t0 + t1;
}
/* The usual case has one largest high word: then only that maximum and the trace go through the six exchange steps, and
 * the low word and the index are read from the one lane that holds the maximum.  Candidates have bx > 0, lanes without
 * one bx = 0 and bi = -1.  Equal high words (or no candidate) take the full reduction; both give the same result. */
template <bool DD> __device__ __forceinline__ void reduce_wave(double& bx, double& by, int32_t& bi, double& tr) {
  double mx = bx, t = tr;
  max_sum_step<0>(mx, t); max_sum_step<1>(mx, t); max_sum_step<2>(mx, t); max_sum_step<3>(mx, t); max_sum_step<4>(mx, t); max_sum_step<5>(mx, t);
  const uint64_t holders = __ballot(bi >= 0 && bx == mx);
  if (__popcll(holders) == 1) {
    const int src = __builtin_amdgcn_readfirstlane((int)__ffsll((long long)holders) - 1);
    bx = mx; tr = t; bi = __builtin_amdgcn_readlane(bi, src);
    if constexpr (DD) {
      const uint64_t b = (uint64_t)__double_as_longlong(by);
      const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)b, src), hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(b >> 32), src);
      by = __longlong_as_double((long long)(((uint64_t)hi << 32) | lo));
    } else { by = 0.; }
  } else { reduce_wave_full<DD>(bx, by, bi, tr); }
}

/* acc -= a b without renormalising acc (its low word collects the error terms; renorm() once at the end) */
template <bool DD> __device__ __forceinline__ void fnma_acc(const Real<DD>& a, const Real<DD>& b, Real<DD>& acc) {
  if constexpr (DD) {
    const double p = a.v.x * b.v.x; double e = fma(a.v.x, b.v.x, -p); e = fma(a.v.x, b.v.y, e); e = fma(a.v.y, b.v.x, e);
    const double s = acc.v.x - p, bb = s - acc.v.x, err = (acc.v.x - (s - bb)) + (-p - bb);
    acc.v.x = s; acc.v.y = (acc.v.y + err) - e;
  } else { acc.v.x = fma(-a.v.x, b.v.x, acc.v.x); }
}
template <bool DD> __device__ __forceinline__ Real<DD> renorm(Real<DD> a) {
  if constexpr (DD) { double s, e; hyk::two_sum(a.v.x, a.v.y, s, e); return Real<DD>{ dd_t{ s, e } }; } else { return a; }
}

/* what an agent publishes per step (wavefront-uniform): doubles bx, tr, n[0 .. WE), by (double-double only), then the index */
template <bool DD, bool CPLX> struct Rec {
  static constexpr int WE = Width<DD, CPLX>::elem, ND = 2 + WE + (DD ? 1 : 0), NW = 2 * ND + 1;
  double bx, by, tr, n[4]; int32_t bi;
  __device__ __forceinline__ void clear() { bx = by = tr = 0.; bi = -1; n[0] = n[1] = n[2] = n[3] = 0.; }
};

/* word j of agent i for the step parity: recs[(parity * REC_WORDS + j) * MAX_AGENTS + i] */
template <bool DD, bool CPLX>
__device__ __forceinline__ void publish(uint64_t* recs, int agent, const Rec<DD, CPLX>& m, uint32_t epoch) {
  using RC = Rec<DD, CPLX>; const int j = threadIdx.x & 63, q = j >> 1;
  double v = m.bx; v = q == 1 ? m.tr : v;
  #pragma unroll
  for (int w = 0; w < RC::WE; ++w) { v = q == 2 + w ? m.n[w] : v; }
  if constexpr (DD) { v = q == 2 + RC::WE ? m.by : v; }
  const uint64_t bits = (uint64_t)__double_as_longlong(v);
  const uint32_t piece = j == RC::NW - 1 ? (uint32_t)m.bi : (uint32_t)(bits >> (32 * (j & 1)));
  if (j < RC::NW) { st_shared_u64(&recs[((size_t)(epoch & 1) * REC_WORDS + j) * MAX_AGENTS + agent], ((uint64_t)epoch << 32) | piece); }
}

/* waits for the record of agent i (bounded); false when the wait gave up.  Two polls are kept in flight, so that a record
 * is seen at most half a memory latency after it has become visible. */
template <bool DD, bool CPLX>
__device__ __forceinline__ bool read_record(const uint64_t* recs, int i, uint32_t epoch, Rec<DD, CPLX>& m) {
  using RC = Rec<DD, CPLX>; uint64_t va[RC::NW], vb[RC::NW], v[RC::NW]; const uint64_t* base = &recs[(size_t)(epoch & 1) * REC_WORDS * MAX_AGENTS + i];
  auto poll = [&](uint64_t (&w)[RC::NW]) {
    #pragma unroll
    for (int j = 0; j < RC::NW; ++j) { w[j] = ld_shared_u64(base + (size_t)j * MAX_AGENTS); }
  };
  auto complete = [&](const uint64_t (&w)[RC::NW]) {
    bool all = true;
    #pragma unroll
    for (int j = 0; j < RC::NW; ++j) { all = all && (uint32_t)(w[j] >> 32) == epoch; }
    return all;
  };
  poll(va);
  for (int spins = 0;; ++spins) {
    poll(vb);
    if (complete(va)) {
      #pragma unroll
      for (int j = 0; j < RC::NW; ++j) { v[j] = va[j]; }
      break;
    }
    poll(va);
    if (complete(vb)) {
      #pragma unroll
      for (int j = 0; j < RC::NW; ++j) { v[j] = vb[j]; }
      break;
    }
    if (spins > SPIN) { return false; }
  }
  auto dbl = [&](int q) { return __longlong_as_double((long long)((v[2 * q] & 0xffffffffull) | (v[2 * q + 1] << 32))); };
  m.bx = dbl(0); m.tr = dbl(1); m.by = 0.; m.n[0] = m.n[1] = m.n[2] = m.n[3] = 0.;
  #pragma unroll
  for (int w = 0; w < RC::WE; ++w) { m.n[w] = dbl(2 + w); }
  if constexpr (DD) { m.by = dbl(2 + RC::WE); }
  m.bi = (int32_t)(uint32_t)v[RC::NW - 1];
  return true;
}

/* value of a wavefront-uniform lane's register in every lane */
__device__ __forceinline__ double lane_f64(double v, int src) {
  const int s = __builtin_amdgcn_readfirstlane(src); const uint64_t b = (uint64_t)__double_as_longlong(v);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)b, s), hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(b >> 32), s);
  return __longlong_as_double((long long)(((uint64_t)hi << 32) | lo));
}

/* All records of `epoch` -> in every lane: the best column over all agents (value, newest factor entry) and the total
 * trace; m / m2 keep what this lane read (records i and i + 64: the better one, the other one) for runner_up().  Column l
 * belongs to agent l % agents.  Every agent runs the same instructions on the same data, so all agents take the same
 * decisions. */
template <bool DD, bool CPLX>
__device__ __forceinline__ bool collect(const uint64_t* recs, int agents, uint32_t epoch, Rec<DD, CPLX>& out, Rec<DD, CPLX>& m, Rec<DD, CPLX>& m2) {
  using RC = Rec<DD, CPLX>; const int lane = threadIdx.x & 63; bool ok = true;
  m.clear(); m2.clear();
  if (lane < agents) { ok = read_record<DD, CPLX>(recs, lane, epoch, m); if (!ok) { m.clear(); } }
  if (lane + 64 < agents) {
    RC o; const bool ok2 = read_record<DD, CPLX>(recs, lane + 64, epoch, o); ok = ok && ok2;
    if (ok2) {
      const double t = m.tr + o.tr; double bx = m.bx, by = m.by; int32_t bi = m.bi; better(DD, bx, by, bi, o.bx, o.by, o.bi);
      if (bi != m.bi) { m2 = m; m = o; } else { m2 = o; }
      m.tr = t;
    }
  }
  out.bx = m.bx; out.by = m.by; out.bi = m.bi; out.tr = m.tr;
  reduce_wave<DD>(out.bx, out.by, out.bi, out.tr);
  const int src = out.bi >= 0 ? ((out.bi % agents) & 63) : 0;   /* the winner's newest entry sits in the lane that read its record */
  #pragma unroll
  for (int q = 0; q < 4; ++q) { out.n[q] = q < RC::WE ? lane_f64(m.n[q], src) : 0.; }
  return __all(ok);
}
/* the best column of the agents other than the winner's, with its newest entry: the same reduction with the winner's record left out */
template <bool DD, bool CPLX>
__device__ __forceinline__ void runner_up(int agents, int winner, const Rec<DD, CPLX>& m, const Rec<DD, CPLX>& m2, Rec<DD, CPLX>& second) {
  using RC = Rec<DD, CPLX>; const RC& r = (winner >= 0 && m.bi == winner) ? m2 : m; double dummy = 0.;
  second.bx = r.bx; second.by = r.by; second.bi = r.bi; second.tr = 0.;
  reduce_wave<DD>(second.bx, second.by, second.bi, dummy);
  const int src = second.bi >= 0 ? ((second.bi % agents) & 63) : 0;
  #pragma unroll
  for (int q = 0; q < 4; ++q) { second.n[q] = q < RC::WE ? lane_f64(r.n[q], src) : 0.; }
}

/* -DHYK_POTRFP_TIMING: the first agent adds up, in wall-clock ticks of 10 ns, where its steps spend their time, and leaves
 * the sums in the control words CTL_TIMING .. of the workspace (a measuring build; the stamps themselves cost time) */
#ifdef HYK_POTRFP_TIMING
#define HYK_STAMP(slot) do { const long long now_ = wall_clock64(); tsum[slot] += now_ - tlast; tlast = now_; } while (0)
#define HYK_COUNT(slot) do { tsum[slot] += 1; } while (0)
#else
#define HYK_STAMP(slot) do { } while (0)
#define HYK_COUNT(slot) do { } while (0)
#endif

template <bool DD, bool CPLX>
__global__ __launch_bounds__(THREADS) void potrfp_blocked_kernel(const Args a) {
#ifdef HYK_POTRFP_TIMING
  long long tsum[10] = { 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 }, tlast = wall_clock64();
#endif
  using R = Real<DD>; using RC = Rec<DD, CPLX>; constexpr int WR = Width<DD, CPLX>::real, WE = Width<DD, CPLX>::elem, PB = CPLX ? 16 : 32;
  extern __shared__ __attribute__((aligned(16))) double lds[];
  /* LDS: [operands / own rows: 2 * TILE * PB * WE doubles][pivot rows: PB * WE doubles][remaining columns, pivot order, positions: N uint16 each] */
  double* const own = lds;                              /* agent: own[(t * 64 + lane) * WE + w]; update: operand A */
  double* const opB = lds + TILE * PB * WE;             /* update: operand B */
  double* const prow = lds + 2 * TILE * PB * WE;        /* agent: factor entries of the pivot column in this panel */
  uint16_t* const list = reinterpret_cast<uint16_t*>(prow + PB * WE);
  uint16_t* const order = list + a.N;                   /* first workgroup: column at each position of the reference's swap order */
  uint16_t* const where = order + a.N;                  /* ... and the position of each column */
  __shared__ int32_t info[4];                           /* panel end, finished, failed */
  __shared__ int32_t piv[MAX_PB];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wg = blockIdx.x, nwg = gridDim.x;
  const int N = a.N, P = a.agents; const bool agent = wave == 0 && wg < P;
  const int l = lane * P + wg; const bool mine = agent && l < N;   /* columns dealt round-robin to the agents: neighbouring columns (often neighbours in size) sit with different agents */

  for (int i = tid; i < N; i += THREADS) { list[i] = (uint16_t)i; order[i] = (uint16_t)i; where[i] = (uint16_t)i; }
  if (tid == 0) { info[0] = 0; info[1] = 0; info[2] = 0; }
  __syncthreads();
  int na = N;

  /* agent state */
  R d = R::zero(); bool dead = !mine; uint32_t epoch = 0; RC cur, nxt, seen, seen2; cur.clear(); nxt.clear(); seen.clear(); seen2.clear();
  double thresh = 0., traceFirst = 0., normFirst2 = 0., traceWanted = 0.; int k = 0; bool failed = false, stop = false, cutInForce = false; int mypiv = 0;
  /* what was fetched for the runner-up: its column of G' and (lane t) its factor entry t of this panel */
  int specCol = -1; R specGre = R::zero(), specGim = R::zero(); double specRow[WE], specNew[WE];
  #pragma unroll
  for (int w = 0; w < WE; ++w) { specRow[w] = 0.; specNew[w] = 0.; }
  const int Kstop = a.K >= N ? N - 1 : a.K;
  if (agent) {
    RC m; m.clear();
    if (mine) { d = R::load_shared(&a.G[((int64_t)l + (int64_t)l * a.ldg) * WE]); m.tr = d.v.x; if (d.v.x > 0.) { m.bx = d.v.x; m.by = d.v.y; m.bi = l; } }
    reduce_wave<DD>(m.bx, m.by, m.bi, m.tr);
    ++epoch; publish<DD, CPLX>(a.records, wg, m, epoch);
    failed = !collect<DD, CPLX>(a.records, P, epoch, cur, seen, seen2);
    thresh = a.eps2 * cur.tr;
    stop = failed || cur.bi < 0 || k >= Kstop;
  }

  for (int kb = 0, panel = 0;; kb += PB, ++panel) {
    if (wave == 0) {
      if (agent && !failed) {
        HYK_STAMP(7);
        if (panel > 0) {   /* every workgroup has applied the previous panel to G' */
          const uint32_t want = (uint32_t)nwg * (uint32_t)panel; int spins = 0;
          while (__hip_atomic_load(reinterpret_cast<uint32_t*>(&a.ctl[CTL_COUNTER]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want) { if (++spins > SPIN) { failed = true; break; } }
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");   /* pairs with the release of the bump below: what the other workgroups wrote to G' and Rt before they bumped the counter is what the loads from here on see */
        }
        specCol = -1;
        HYK_STAMP(0);
        while (!failed && !stop && k < kb + PB) {
          HYK_COUNT(9);
          /* the second way to end (hykPotrfpWanted): a step takes the squared norm of its row of the factor off the trace of
           * what is left, so the traces around steps 1 and `wanted` give the norms nu_1 and nu_w of those rows, and
           * b = cut nu_1 nu_w; after `wanted` steps it becomes the threshold if what is left of G is within 32 b already (a floor
           * right under the wanted values).  Every agent holds the same record, so all decide alike. */
          if (k == 0) { traceFirst = cur.tr; }
          if (k == 1) { normFirst2 = traceFirst - cur.tr; }
          if (k + 1 == a.wanted) { traceWanted = cur.tr; }
          if (a.cut > 0. && k == a.wanted) {
            const double normWanted2 = traceWanted - cur.tr, b = (normFirst2 > 0. && normWanted2 > 0.) ? a.cut * sqrt(normFirst2 * normWanted2) : 0.;
            if (cur.tr <= 32. * b && thresh < b) { thresh = b; cutInForce = true; }
          }
          const int c = cur.bi, j = k - kb; R dc{ dd_t{ cur.bx, cur.by } }, sq, rho; sqrt_rsqrt<DD>(dc, sq, rho);
          const bool hit = specCol == c; const bool work = !dead && l != c;
          if (lane == j) { mypiv = c; }
          /* factor entries R[kb .. k, c] of the pivot column: entry t from lane t (fetched ahead on a hit: entries 0 .. j-3;
           * else 0 .. j-2 now), the newer ones came with the records */
          R gre = specGre, gim = specGim;
          if (hit) {
            HYK_COUNT(8);
            if (lane < j - 2) {
              #pragma unroll
              for (int w = 0; w < WE; ++w) { prow[lane * WE + w] = specRow[w]; }
            }
            if (lane == 0 && j > 1) {
              #pragma unroll
              for (int w = 0; w < WE; ++w) { prow[(j - 2) * WE + w] = specNew[w]; }
            }
          } else {
            if (lane < j - 1) {
              const double* src = &a.Rt[((int64_t)c * a.ldr + kb + lane) * WE];
              #pragma unroll
              for (int w = 0; w < WE; ++w) { prow[lane * WE + w] = __hip_atomic_load(const_cast<double*>(src) + w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
            }
            if (work) {
              if (l < c) { const double* g = &a.G[((int64_t)l + (int64_t)c * a.ldg) * WE]; gre = R::load_shared(g); if constexpr (CPLX) { gim = R::load_shared(g + WR); } }
              else { const double* g = &a.G[((int64_t)c + (int64_t)l * a.ldg) * WE]; gre = R::load_shared(g); if constexpr (CPLX) { gim = R::load_shared(g + WR).neg(); } }
            }
          }
          if (lane == 0 && j > 0) {
            #pragma unroll
            for (int w = 0; w < WE; ++w) { prow[(j - 1) * WE + w] = cur.n[w]; }
          }
          R rr = R::zero(), ri = R::zero();
          if (work) {
            R sre = gre, sim = gim;
            #pragma unroll 4
            for (int t = 0; t < j; ++t) {   /* unrolled so that the LDS reads of several entries are in flight together */
              const double* o = &own[(t * 64 + lane) * WE]; const double* b = &prow[t * WE];
              if constexpr (CPLX) {
                const R ar = R::load(o), ai = R::load(o + WR), br = R::load(b), bim = R::load(b + WR);
                /* S -= conj(a) b:  re -= ar br + ai bi;  im -= ar bi - ai br */
                fnma_acc<DD>(ar, br, sre); fnma_acc<DD>(ai, bim, sre); fnma_acc<DD>(ar, bim, sim); fnma_acc<DD>(ai.neg(), br, sim);
              } else { fnma_acc<DD>(R::load(o), R::load(b), sre); }
            }
            sre = renorm<DD>(sre); rr = rho * sre; if constexpr (CPLX) { sim = renorm<DD>(sim); ri = (rho * sim).neg(); }
            if constexpr (CPLX) { d = d - (rr * rr + ri * ri); } else { d = d - rr * rr; }
          }
          if (!dead && l == c) { rr = sq; ri = R::zero(); dead = true; }
          const bool wrote = work || (mine && l == c);
          if (wrote) { double* o = &own[(j * 64 + lane) * WE]; rr.store(o); if constexpr (CPLX) { ri.store(o + WR); } }
          HYK_STAMP(1);
          /* arg-max and trace of the columns this agent still has, and the candidate's newest entry */
          RC m; m.clear();
          if (!dead) { m.tr = d.v.x; if (d.v.x > 0.) { m.bx = d.v.x; m.by = d.v.y; m.bi = l; } }
          reduce_wave<DD>(m.bx, m.by, m.bi, m.tr);
          { const int src = m.bi >= 0 ? m.bi / P : 0;
            m.n[0] = lane_f64(rr.v.x, src);
            if constexpr (DD) { m.n[1] = lane_f64(rr.v.y, src); }
            if constexpr (CPLX) { m.n[WR] = lane_f64(ri.v.x, src); if constexpr (DD) { m.n[WR + 1] = lane_f64(ri.v.y, src); } } }
          HYK_STAMP(2);
          ++k; ++epoch;
          const bool last = (k == kb + PB) || (k >= Kstop);   /* the update (or the host) reads this panel's factor entries next */
          double* out = &a.Rt[((int64_t)l * a.ldr + (k - 1)) * WE];
          if (last) { if (wrote) { rr.store_shared(out); if constexpr (CPLX) { ri.store_shared(out + WR); } } asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
          publish<DD, CPLX>(a.records, wg, m, epoch);
          if (!last && wrote) { rr.store_shared(out); if constexpr (CPLX) { ri.store_shared(out + WR); } }
          /* fetch ahead for the runner-up c2 of the arg-max that chose this step's pivot: G'[l, c2] and its factor entries
           * 0 .. j-2 (what is certainly in memory by now); not across a panel end, where G' changes.  Issued after the
           * record, so that nothing on the way to the record waits for these loads. */
          runner_up<DD, CPLX>(P, c, seen, seen2, nxt);
          const int c2 = nxt.bi; const bool ahead = c2 >= 0 && j + 1 < PB && k < Kstop;
          if (ahead) {
            if (lane < j - 1) {
              const double* src = &a.Rt[((int64_t)c2 * a.ldr + kb + lane) * WE];
              #pragma unroll
              for (int w = 0; w < WE; ++w) { specRow[w] = __hip_atomic_load(const_cast<double*>(src) + w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
            }
            if (!dead && l != c2) {
              if (l < c2) { const double* g = &a.G[((int64_t)l + (int64_t)c2 * a.ldg) * WE]; specGre = R::load_shared(g); if constexpr (CPLX) { specGim = R::load_shared(g + WR); } }
              else { const double* g = &a.G[((int64_t)c2 + (int64_t)l * a.ldg) * WE]; specGre = R::load_shared(g); if constexpr (CPLX) { specGim = R::load_shared(g + WR).neg(); } }
            }
            #pragma unroll
            for (int w = 0; w < WE; ++w) { specNew[w] = nxt.n[w]; }
          }
          specCol = ahead ? c2 : -1;
          if (wg == 0 && lane == 0) {   /* pivot bookkeeping in the reference's swap order */
            const int p = where[c], c0 = order[k - 1]; order[k - 1] = (uint16_t)c; order[p] = (uint16_t)c0; where[c] = (uint16_t)(k - 1); where[c0] = (uint16_t)p;
          }
          HYK_STAMP(3);
          failed = !collect<DD, CPLX>(a.records, P, epoch, cur, seen, seen2);
          HYK_STAMP(4);
          if (!(thresh < cur.tr)) { cur.bi = -1; }
          stop = failed || cur.bi < 0 || k >= Kstop;
        }
        if (wg == 0) {   /* panel summary for every workgroup: columns done, whether the factorization ends here, the new pivots */
          const uint32_t seq = (uint32_t)panel + 1u; const int pl = lane >= 2 ? lane - 2 : 0;
          const int q0 = __shfl(mypiv, (2 * pl) & 63, 64), q1 = __shfl(mypiv, (2 * pl + 1) & 63, 64);   /* lane t holds the pivot of step t of this panel */
          uint32_t payload = (uint32_t)q0 | ((uint32_t)q1 << 16); payload = lane == 0 ? (uint32_t)k : payload; payload = lane == 1 ? (uint32_t)((stop ? 1 : 0) | (failed ? 2 : 0)) : payload;
          if (lane < 2 + PB / 2) { st_shared_u64(&a.ctl[lane], ((uint64_t)seq << 32) | payload); }
        }
      }
      /* every leader waits for the summary */
      { const uint32_t seq = (uint32_t)panel + 1u; uint64_t s = 0; int spins = 0; bool got = false;
        while (!failed) {
          if (lane < 2 + PB / 2) { s = ld_shared_u64(&a.ctl[lane]); }
          if (__all(lane >= 2 + PB / 2 || (uint32_t)(s >> 32) == seq)) { got = true; break; }
          if (++spins > SPIN) { failed = true; break; }
          __builtin_amdgcn_s_sleep(2);
        }
        const uint32_t w0 = (uint32_t)__shfl((int)(uint32_t)s, 0, 64), w1 = (uint32_t)__shfl((int)(uint32_t)s, 1, 64);
        if (lane == 0) { info[0] = got ? (int32_t)w0 : 0; info[1] = got ? (int32_t)(w1 & 1u) : 1; info[2] = (failed || (got && (w1 & 2u))) ? 1 : 0; }
        if (got && lane >= 2 && lane < 2 + PB / 2) { piv[2 * (lane - 2)] = (int32_t)((uint32_t)s & 0xffffu); piv[2 * (lane - 2) + 1] = (int32_t)(((uint32_t)s >> 16) & 0xffffu); }
      }
    }
    __syncthreads();
    HYK_STAMP(5);
    const int ke = info[0], fin = info[1], bad = info[2];
    if (bad) { failed = true; break; }
    if (fin) { break; }
    const int nbk = ke - kb;

    /* ---- update phase ---- */
    /* drop the new pivots from the sorted list of remaining columns: an entry moves down by the number of pivots below it */
    for (int base = 0; base < na; base += THREADS) {
      const int idx = base + tid; int v = 0, to = -1;
      if (idx < na) { v = list[idx]; int shift = 0; bool gone = false; for (int i = 0; i < nbk; ++i) { shift += piv[i] < v ? 1 : 0; gone = gone || piv[i] == v; } if (!gone) { to = idx - shift; } }
      __syncthreads();
      if (to >= 0) { list[to] = (uint16_t)v; }
      __syncthreads();
    }
    na -= nbk;
    const int nT = (na + TILE - 1) / TILE, tiles = nT * (nT + 1) / 2;
    for (int tile = wg; tile < tiles; tile += nwg) {
      int J = (int)((sqrtf(8.f * (float)tile + 1.f) - 1.f) * 0.5f); while ((J + 1) * (J + 2) / 2 <= tile) { ++J; } while (J * (J + 1) / 2 > tile) { --J; }
      const int I = tile - J * (J + 1) / 2;
      /* operands: the panel's factor entries of 64 remaining columns each, op[(t * 64 + col) * WE + w]; all loads of a
       * thread are issued before the first is stored, so that their latencies overlap */
      { constexpr int PER = TILE * PB / THREADS;
        #pragma unroll
        for (int which = 0; which < 2; ++which) {
          if (which == 1 && I == J) { break; }
          double v[PER][WE];
          #pragma unroll
          for (int e = 0; e < PER; ++e) {
            const int r = tid + e * THREADS, col = r / PB, t = r % PB, li = (which ? J : I) * TILE + col;
            #pragma unroll
            for (int w = 0; w < WE; ++w) { v[e][w] = 0.; }
            if (li < na && t < nbk) {
              const double* src = &a.Rt[((int64_t)list[li] * a.ldr + kb + t) * WE];
              #pragma unroll
              for (int w = 0; w < WE; ++w) { v[e][w] = __hip_atomic_load(const_cast<double*>(src) + w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
            }
          }
          #pragma unroll
          for (int e = 0; e < PER; ++e) {
            const int r = tid + e * THREADS, col = r / PB, t = r % PB; double* dst = &(which ? opB : own)[(t * 64 + col) * WE];
            #pragma unroll
            for (int w = 0; w < WE; ++w) { dst[w] = v[e][w]; }
          }
        }
      }
      __syncthreads();
      const double* A = own; const double* B = I == J ? own : opB;
      const int ry = (wave >> 1) * 32 + (lane & 7), cx = (wave & 1) * 32 + (lane >> 3);
      /* G'[l, m] for the 16 pairs of this lane: requested now, needed after the products */
      R gre[4][4], gim[4][4]; double* gp[4][4];
      #pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int li = I * TILE + ry + 8 * i; const int lcol = li < na ? list[li] : 0;
        #pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int mi = J * TILE + cx + 8 * jj; gp[i][jj] = nullptr; gre[i][jj] = R::zero(); gim[i][jj] = R::zero();
          if (li < na && mi < na && li < mi) {
            double* g = &a.G[((int64_t)lcol + (int64_t)list[mi] * a.ldg) * WE]; gp[i][jj] = g;
            gre[i][jj] = R::load_shared(g); if constexpr (CPLX) { gim[i][jj] = R::load_shared(g + WR); }
          }
        }
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
            fnma_acc<DD>(ar[i], br[jj], gre[i][jj]);
            if constexpr (CPLX) { fnma_acc<DD>(ai[i], bi[jj], gre[i][jj]); fnma_acc<DD>(ar[i], bi[jj], gim[i][jj]); fnma_acc<DD>(ai[i].neg(), br[jj], gim[i][jj]); }
          }
        }
      }
      #pragma unroll
      for (int i = 0; i < 4; ++i) {
        #pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          if (gp[i][jj]) { renorm<DD>(gre[i][jj]).store_shared(gp[i][jj]); if constexpr (CPLX) { renorm<DD>(gim[i][jj]).store_shared(gp[i][jj] + WR); } }
        }
      }
      __syncthreads();
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   /* every thread's stores of this panel's update have left (the release below names the order; this wait is what makes it cheap for the one thread that bumps) */
    __syncthreads();
    if (tid == 0) { __hip_atomic_fetch_add(reinterpret_cast<uint32_t*>(&a.ctl[CTL_COUNTER]), 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT); }
    HYK_STAMP(6);
  }
#ifdef HYK_POTRFP_TIMING
  if (wg == 0 && tid == 0) { for (int i = 0; i < 10; ++i) { a.ctl[CTL_TIMING + i] = (uint64_t)tsum[i]; } }
#endif

  /* reference quirk (src/hyacin_potrfp.cu:271): when exactly one column is left it is counted and its diagonal written */
  if (agent && !failed && N - k == 1 && !dead) {
    R sq = R::zero(), rho; if (d.v.x > 0.) { sqrt_rsqrt<DD>(d, sq, rho); }
    double* rc = &a.Rt[((int64_t)l * a.ldr + k) * WE]; sq.store(rc); if constexpr (CPLX) { R::zero().store(rc + WR); }
  }
  __syncthreads();
  if (wg == 0) {
    if (tid == 0) { info[3] = k; }   /* the agent's count of columns done */
    __syncthreads();
    for (int i = tid; i < N; i += THREADS) { a.jpiv[i] = (int32_t)order[i] + 1; }
    if (tid == 0) {
      *a.rankOut = failed ? -1 : ((N - info[3] == 1) ? info[3] + 1 : info[3]);
      if (a.traceOut) { *a.traceOut = (!cutInForce || failed || N - info[3] <= 1 || !(cur.tr > 0.)) ? 0. : cur.tr; }   /* the trace of what is left of G (the first agent's copy of the last record) */
    }
  }
}

template <bool DD, bool CPLX> int launch(hipStream_t stream, Args& args, int cus) {
  constexpr int WE = Width<DD, CPLX>::elem, PB = CPLX ? 16 : 32;
  const size_t ldsBytes = (size_t)(2 * TILE * PB * WE + PB * WE) * 8 + (size_t)args.N * 6 + 16;
  const void* fn = reinterpret_cast<const void*>(&potrfp_blocked_kernel<DD, CPLX>);
  if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes) != hipSuccess) { return -3; }
  int perCu = 0; if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCu, potrfp_blocked_kernel<DD, CPLX>, THREADS, ldsBytes) != hipSuccess || perCu < 1) { return -3; }
  int grid = cus < 256 ? cus : 256; if (grid < args.agents) { return -1; }
  const bool fits = fits_device(grid, perCu);
  if (!(g_plainLaunch.load(std::memory_order_relaxed) && fits)) {   /* hykPotrfpSetPlainLaunch: see there */
    void* params[] = { &args };
    if (hipLaunchCooperativeKernel(fn, dim3(grid), dim3(THREADS), params, (unsigned)ldsBytes, stream) == hipSuccess) { return 0; }
    (void)hipGetLastError();
    if (!fits) { return -3; }
  }
  potrfp_blocked_kernel<DD, CPLX><<<grid, THREADS, ldsBytes, stream>>>(args); return hipGetLastError() == hipSuccess ? 0 : -3;
}

__global__ void clear_kernel(uint64_t* p, int words) { for (int i = threadIdx.x; i < words; i += blockDim.x) { p[i] = 0ull; } }

}  // namespace blk

}  // namespace

namespace {
/* workspace: [pos: N int32][exchange area: records / control words of either kernel][D: N reals (left-looking kernel)] */
constexpr size_t EXCHANGE_BYTES = 2 * blk::MAX_AGENTS * blk::REC_WORDS * 8 + blk::CTL_WORDS * 8;   /* 33 280 bytes */
static_assert(EXCHANGE_BYTES >= 2 * MAX_WORKGROUPS * sizeof(Record), "the exchange area holds the records of either kernel");
size_t align256(size_t v) { return (v + 255) / 256 * 256; }

int run_potrfp(hipStream_t stream, bool blocked, int32_t computeUnits, double eps, int32_t K, int32_t N, int32_t Gtype, void* G, int64_t ldg, void* Rt, int32_t ldr, int32_t* jpiv, void* workspace, int32_t* rankOut, int32_t wanted = 0, double cut = 0., double* traceOut = nullptr) {
  if (N <= 0) { return 0; }
  if (!workspace || !G || !Rt || !jpiv || !rankOut) { return -1; }
  if (K <= 0 || K > N) { K = N; }
  if (ldg < N || ldr < (K < N ? K + 1 : N) || computeUnits < 1 || !(cut >= 0.)) { return -1; }
  const bool dd = (Gtype & ~1) == HYK_DD, cplx = Gtype & 1;
  if (!dd && (Gtype & ~1) != HYK_F64) { return -1; }
  char* w = (char*)workspace; int32_t* pos = (int32_t*)w; w += align256((size_t)N * 4); uint64_t* exchange = (uint64_t*)w; w += EXCHANGE_BYTES; double* D = (double*)w;
  blk::clear_kernel<<<1, 256, 0, stream>>>(exchange, (int)(EXCHANGE_BYTES / 8));
  const int agents = (N + 63) / 64, grid = computeUnits < 256 ? computeUnits : 256;
  if (blocked && N <= blk::MAX_N && agents <= grid) {
    blk::Args b; b.N = N; b.K = K; b.ldr = ldr; b.agents = agents; b.eps2 = eps * eps; b.G = (double*)G; b.ldg = ldg; b.Rt = (double*)Rt; b.jpiv = jpiv;
    b.records = exchange; b.ctl = exchange + 2 * blk::MAX_AGENTS * blk::REC_WORDS; b.rankOut = rankOut;
    b.wanted = (wanted > 0 && wanted < N) ? wanted : 0; b.cut = b.wanted ? cut : 0.; b.traceOut = traceOut;
    if (dd) { return cplx ? blk::launch<true, true>(stream, b, computeUnits) : blk::launch<true, false>(stream, b, computeUnits); }
    return cplx ? blk::launch<false, true>(stream, b, computeUnits) : blk::launch<false, false>(stream, b, computeUnits);
  }
  PotrfArgs a; a.N = N; a.K = K; a.ldr = ldr; a.eps2 = eps * eps; a.G = (const double*)G; a.ldg = ldg; a.Rt = (double*)Rt; a.jpiv = jpiv; a.rankOut = rankOut; a.traceOut = traceOut;
  a.D = D; a.pos = pos; a.records = (Record*)exchange;
  if (dd) { return cplx ? launch<true, true>(stream, a, computeUnits) : launch<true, false>(stream, a, computeUnits); }
  return cplx ? launch<false, true>(stream, a, computeUnits) : launch<false, false>(stream, a, computeUnits);
}
}  // namespace

extern "C" int hykPotrfpSetPlainLaunch(int32_t enable) { g_plainLaunch.store(enable ? 1 : 0, std::memory_order_relaxed); return 0; }

extern "C" size_t hykPotrfpWorkspaceBytes(int32_t N, int32_t Gtype) {
  if (N <= 0) { return 0; }
  const size_t wr = ((Gtype & ~1) == HYK_DD) ? 2 : 1;
  return align256((size_t)N * 4) + EXCHANGE_BYTES + align256((size_t)N * wr * 8);
}

extern "C" int hykPotrfp(hipStream_t stream, int32_t computeUnits, double eps, int32_t K, int32_t N, int32_t Gtype, void* G, int64_t ldg, void* Rt, int32_t ldr, int32_t* jpiv, void* workspace, int32_t* rankOut) {
  return run_potrfp(stream, true, computeUnits, eps, K, N, Gtype, G, ldg, Rt, ldr, jpiv, workspace, rankOut);
}

extern "C" int hykPotrfpWanted(hipStream_t stream, int32_t computeUnits, double eps, int32_t K, int32_t wanted, double cut, int32_t N, int32_t Gtype, void* G, int64_t ldg, void* Rt, int32_t ldr, int32_t* jpiv, void* workspace, int32_t* rankOut, double* traceOut) {
  return run_potrfp(stream, true, computeUnits, eps, K, N, Gtype, G, ldg, Rt, ldr, jpiv, workspace, rankOut, wanted, cut, traceOut);
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
