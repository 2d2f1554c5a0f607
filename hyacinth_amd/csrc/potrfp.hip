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
 * operands of every dot product are contiguous; (ii) needs one grid barrier per
 * column: every workgroup reduces the per-workgroup (max, trace) partials
 * itself after the barrier, so no second barrier distributes the winner;
 * (iii) one wavefront owns a column, lanes split the dot product.
 * Ties between equal diagonal entries are broken towards the smaller column
 * index (the reference breaks them towards the smaller position in its swapped
 * order).  The emitted pivot vector follows the reference's swap sequence
 * (jpiv[k] <-> jpiv[position of the pivot]) and is 1-based.
 *
 * Cooperative launch: at most one workgroup per compute unit, all resident.
 */
#include <hip/hip_runtime.h>
#include "hyk_common.h"
#include "hyk_dd.h"
#include "hyacin_kernels.h"

namespace {

using hyk::dd_t;

constexpr int P_THREADS = 1024;   /* 16 wavefronts per compute unit: the dot products are latency-bound loads of the factor */
constexpr int P_WAVES = P_THREADS / 64;

struct Partial { double bx, by, trace; int32_t idx, pad; };

struct PotrfArgs {
  int32_t N, K, ldr; double eps2;
  const double* G; int64_t ldg;
  double* Rt; double* D; int32_t* done; int32_t* jpiv; int32_t* pos; Partial* partials; int32_t* rankOut; uint32_t* arrivals;
};

/* scalar types: value = re (+ i im), each part a dd_t (lo part unused in FP64 mode) */
template <bool DD> struct Real {
  dd_t v;
  __device__ __forceinline__ static Real zero() { return Real{ dd_t{ 0., 0. } }; }
  __device__ __forceinline__ static Real load(const double* p) { if constexpr (DD) { return Real{ dd_t{ p[0], p[1] } }; } else { return Real{ dd_t{ p[0], 0. } }; } }
  __device__ __forceinline__ void store(double* p) const { p[0] = v.x; if constexpr (DD) { p[1] = v.y; } }
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

/* workgroup arg-max / sum: shuffles inside each wavefront, one exchange through LDS between them (two barriers) */
template <bool DD>
__device__ __forceinline__ void wave_reduce(double& bx, double& by, int32_t& bi, double& tr) {
  #pragma unroll
  for (int m = 32; m > 0; m >>= 1) {
    const double ox = __shfl_xor(bx, m, 64), oy = __shfl_xor(by, m, 64), ot = __shfl_xor(tr, m, 64); const int32_t oi = __shfl_xor(bi, m, 64);
    better(DD, bx, by, bi, ox, oy, oi); tr += ot;
  }
}
template <bool DD>
__device__ __forceinline__ void block_reduce(double& bx, double& by, int32_t& bi, double& tr) {
  __shared__ double sx[P_WAVES], sy[P_WAVES], st[P_WAVES]; __shared__ int32_t si[P_WAVES];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  wave_reduce<DD>(bx, by, bi, tr);
  if (lane == 0) { sx[wave] = bx; sy[wave] = by; si[wave] = bi; st[wave] = tr; }
  __syncthreads();
  bx = by = tr = 0.; bi = -1;
  if (lane < P_WAVES) { bx = sx[lane]; by = sy[lane]; bi = si[lane]; tr = st[lane]; }
  wave_reduce<DD>(bx, by, bi, tr);     /* every wavefront reduces the same P_WAVES entries: no broadcast needed */
  __syncthreads();
}

/* Grid barrier for the co-resident workgroups of the cooperative launch: one arrival counter that only grows, so no
 * reset phase; barrier number `epoch` (1, 2, ...) is passed once the counter has reached epoch * workgroups.  The fences
 * publish this workgroup's global writes before the arrival and drop stale cache lines after the release. */
__device__ __forceinline__ void grid_barrier(uint32_t* arrivals, uint32_t workgroups, uint32_t epoch) {
  __syncthreads();
  if (threadIdx.x == 0) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    __hip_atomic_fetch_add(arrivals, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t target = epoch * workgroups;
    while (__hip_atomic_load(arrivals, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) { __builtin_amdgcn_s_sleep(1); }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  }
  __syncthreads();
}

template <bool DD, bool CPLX>
__global__ __launch_bounds__(P_THREADS) void potrfp_kernel(const PotrfArgs a) {
  uint32_t epoch = 0;
  using R = Real<DD>; constexpr int WR = Width<DD, CPLX>::real, WE = Width<DD, CPLX>::elem;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwg = gridDim.x, wg = blockIdx.x;
  const int gthread = wg * P_THREADS + tid, nthreads = nwg * P_THREADS, gwave = wg * P_WAVES + wave, nwaves = nwg * P_WAVES;
  const int N = a.N;

  /* init: diagonal, pivot bookkeeping, first arg-max and trace */
  double bx = 0., by = 0., tr = 0.; int32_t bi = -1;
  for (int l = gthread; l < N; l += nthreads) {
    R d = R::load(&a.G[((int64_t)l + (int64_t)l * a.ldg) * WE]); d.store(&a.D[(int64_t)l * WR]);
    a.done[l] = 0; a.jpiv[l] = l + 1; a.pos[l] = l; tr += d.v.x;
    if (d.v.x > 0.) { better(DD, bx, by, bi, d.v.x, d.v.y, l); }
  }
  block_reduce<DD>(bx, by, bi, tr);
  if (tid == 0) { a.partials[wg] = Partial{ bx, by, tr, bi, 0 }; }
  grid_barrier(a.arrivals, (uint32_t)nwg, ++epoch);
  bx = by = tr = 0.; bi = -1;
  if (tid < nwg) { Partial p = a.partials[tid]; bx = p.bx; by = p.by; bi = p.idx; tr = p.trace; }
  block_reduce<DD>(bx, by, bi, tr);
  const double thresh = a.eps2 * tr;
  const int Kstop = a.K >= N ? N - 1 : a.K;   /* with K == N the last column is appended without a test (see below) */
  int k = 0;
  while (bi >= 0 && k < Kstop) {
    const int c = bi; R dc{ dd_t{ bx, by } }, sq, rho; sqrt_rsqrt<DD>(dc, sq, rho);
    if (wg == 0 && tid == 0) {
      /* R[k, c] = sqrt(d_c); pivot bookkeeping in the reference's swap order */
      double* rc = &a.Rt[((int64_t)c * a.ldr + k) * WE]; sq.store(rc); if constexpr (CPLX) { R::zero().store(rc + WR); }
      const int p = a.pos[c], c0 = a.jpiv[k] - 1; a.jpiv[k] = c + 1; a.jpiv[p] = c0 + 1; a.pos[c] = k; a.pos[c0] = p; a.done[c] = 1;
    }
    /* column c of R, shared by every dot product of this step: Rt[c][0..k) */
    const double* rcol = &a.Rt[(int64_t)c * a.ldr * WE];
    bx = by = tr = 0.; bi = -1;
    for (int l = gwave; l < N; l += nwaves) {
      if (l == c || a.done[l]) { continue; }
      const double* rl = &a.Rt[(int64_t)l * a.ldr * WE];
      /* G[l, c] and d_l are needed only after the dot product: request them first so their latency hides under it */
      const double* g = &a.G[((int64_t)l + (int64_t)c * a.ldg) * WE];
      const R gre0 = R::load(g), d0 = R::load(&a.D[(int64_t)l * WR]); R gim0 = R::zero(); if constexpr (CPLX) { gim0 = R::load(g + WR); }
      R sre = R::zero(), sim = R::zero();
      #pragma unroll 8
      for (int t = lane; t < k; t += 64) {
        if constexpr (CPLX) {
          R ar = R::load(&rl[(int64_t)t * WE]), ai = R::load(&rl[(int64_t)t * WE + WR]), br = R::load(&rcol[(int64_t)t * WE]), bim = R::load(&rcol[(int64_t)t * WE + WR]);
          /* S -= conj(a) b:  re -= ar br + ai bi;  im -= ar bi - ai br */
          sre = R::fnma(ar, br, sre); sre = R::fnma(ai, bim, sre); sim = R::fnma(ar, bim, sim); sim = R::fnma(ai.neg(), br, sim);
        } else { sre = R::fnma(R::load(&rl[(int64_t)t * WE]), R::load(&rcol[(int64_t)t * WE]), sre); }
      }
      for (int m = 32; m > 0; m >>= 1) { sre = sre + sre.shfl_xor(m); if constexpr (CPLX) { sim = sim + sim.shfl_xor(m); } }
      if (lane == 0) {
        sre = sre + gre0; R rr = rho * sre; double* out = &a.Rt[((int64_t)l * a.ldr + k) * WE]; rr.store(out);
        R d = d0;
        if constexpr (CPLX) { sim = sim + gim0; R ri = (rho * sim).neg(); ri.store(out + WR); d = d - (rr * rr + ri * ri); } else { d = d - rr * rr; }
        d.store(&a.D[(int64_t)l * WR]); tr += d.v.x;
        if (d.v.x > 0.) { better(DD, bx, by, bi, d.v.x, d.v.y, l); }
      }
    }
    block_reduce<DD>(bx, by, bi, tr);
    ++k;
    Partial* part = &a.partials[(k & 1) * nwg];
    if (tid == 0) { part[wg] = Partial{ bx, by, tr, bi, 0 }; }
    grid_barrier(a.arrivals, (uint32_t)nwg, ++epoch);
    bx = by = tr = 0.; bi = -1;
    if (tid < nwg) { Partial p = part[tid]; bx = p.bx; by = p.by; bi = p.idx; tr = p.trace; }
    block_reduce<DD>(bx, by, bi, tr);
    if (!(thresh < tr)) { bi = -1; }
  }
  /* reference quirk (src/hyacin_potrfp.cu:271): when exactly one column is left it is counted and its diagonal written */
  int rank = k;
  if (N - k == 1) {
    if (wg == 0 && tid == 0) {
      int c = -1; for (int l = 0; l < N; ++l) { if (!a.done[l]) { c = l; } }
      if (c >= 0) { R d = R::load(&a.D[(int64_t)c * WR]); R sq = R::zero(), rho; if (d.v.x > 0.) { sqrt_rsqrt<DD>(d, sq, rho); } double* rc = &a.Rt[((int64_t)c * a.ldr + k) * WE]; sq.store(rc); if constexpr (CPLX) { R::zero().store(rc + WR); } }
    }
    rank = k + 1;
  }
  if (wg == 0 && tid == 0) { *a.rankOut = rank; }
}

__global__ void clear_word_kernel(uint32_t* p) { *p = 0u; }

/* one-time per kernel: how many workgroups may be co-resident */
template <bool DD, bool CPLX> int launch(hipStream_t stream, PotrfArgs& args, int cus) {
  int perCu = 0; if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&perCu, potrfp_kernel<DD, CPLX>, P_THREADS, 0) != hipSuccess || perCu < 1) { return -3; }
  int grid = cus < 256 ? cus : 256; const int want = (args.N + P_WAVES - 1) / P_WAVES; if (grid > want) { grid = want; } if (grid < 1) { grid = 1; }
  void* params[] = { &args };
  hipError_t e = hipLaunchCooperativeKernel(reinterpret_cast<const void*>(&potrfp_kernel<DD, CPLX>), dim3(grid), dim3(P_THREADS), params, 0, stream);
  return e == hipSuccess ? 0 : -3;
}

}  // namespace

extern "C" size_t hykPotrfpWorkspaceBytes(int32_t N, int32_t Gtype) {
  if (N <= 0) { return 0; }
  const size_t wr = ((Gtype & ~1) == HYK_DD) ? 2 : 1;
  /* D | done | pos | partials(2 x 256) */
  return (size_t)N * wr * 8 + (size_t)N * 4 * 2 + 2 * 256 * sizeof(Partial) + 256 + 256;
}

extern "C" int hykPotrfp(hipStream_t stream, int32_t computeUnits, double eps, int32_t K, int32_t N, int32_t Gtype, const void* G, int64_t ldg, void* Rt, int32_t ldr, int32_t* jpiv, void* workspace, int32_t* rankOut) {
  if (N <= 0) { return 0; }
  if (K <= 0 || K > N) { K = N; }
  if (ldg < N || ldr < (K < N ? K + 1 : N) || computeUnits < 1) { return -1; }
  const bool dd = (Gtype & ~1) == HYK_DD, cplx = Gtype & 1;
  if (!dd && (Gtype & ~1) != HYK_F64) { return -1; }
  PotrfArgs a; a.N = N; a.K = K; a.ldr = ldr; a.eps2 = eps * eps; a.G = (const double*)G; a.ldg = ldg; a.Rt = (double*)Rt; a.jpiv = jpiv; a.rankOut = rankOut;
  char* w = (char*)workspace; a.D = (double*)w; w += (size_t)N * (dd ? 2 : 1) * 8; a.done = (int32_t*)w; w += (size_t)N * 4; a.pos = (int32_t*)w; w += (size_t)N * 4;
  w = (char*)(((uintptr_t)w + 15) & ~(uintptr_t)15); a.partials = (Partial*)w; w += 2 * 256 * sizeof(Partial);
  w = (char*)(((uintptr_t)w + 63) & ~(uintptr_t)63); a.arrivals = (uint32_t*)w;
  clear_word_kernel<<<1, 1, 0, stream>>>(a.arrivals);
  if (dd) { return cplx ? launch<true, true>(stream, a, computeUnits) : launch<true, false>(stream, a, computeUnits); }
  return cplx ? launch<false, true>(stream, a, computeUnits) : launch<false, false>(stream, a, computeUnits);
}
