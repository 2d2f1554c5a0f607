/*
 * gram_mfma.hip -- the int8 Gram contraction on the CDNA4 matrix cores, and the
 * kernels that turn its accumulators into the 63-bit-limb integer Gram.
 *
 * Replaces, in the reference, the cuBLAS int8 GEMMs of src/hyacin_herk.cpp:61-251
 * together with the int32 -> accumulator kernels src/limbs_diag.cu,
 * src/limbs_cross_real.cu, src/limbs_cross_imag.cu, src/crt_diag_real.cu,
 * src/crt_rotate.cu, src/crt_extra_real.cu, src/crt_extra_imag.cu (all fused into
 * the contraction's epilogue: the int32 products never reach HBM), and
 * src/crt_reconstruct_real.cu / src/crt_reconstruct_complex.cu.
 *
 * Data layout.  int8 panels, K-contiguous: panel p, column j, row k at
 * panels[p * panelStride + j * ldb + k]; K (rows) is a multiple of 128 with the
 * padding rows zero.  Accumulators: plane q, packed-triangle entry
 * y + x(x+1)/2 (y <= x) at acc[q * planeStride + entry]; uint32 sums of
 * canonical residues for the CRT path, int64 sums for the limb path.
 *
 * Work decomposition.  A work item is (group, 256x256 tile (ta <= tb) of the
 * upper block triangle, K split).  A group is a list of panel pairs
 * (lanePanel, aPanel) whose products  W[y, x] = sum_k lanePanel[k, y] *
 * aPanel[k, x]  (y in block ta, x in block tb) are summed in int32 on the
 * MFMA accumulators, plus an epilogue rule that says which accumulator planes
 * receive  +-W  or  (c * W) mod m.  Exact integer addition commutes, so items
 * combine through atomics in any order and the result is bit-identical to any
 * serial schedule.  Lower-triangle products (needed by the complex paths) are
 * expressed as groups with the two panels swapped, so that the lane dimension of
 * the MFMA output always runs along the contiguous index of the packed triangle.
 *
 * Mapping to the chip.  One 256-thread workgroup (4 wavefronts, 2x2, each
 * 128x128 = 4x4 v_mfma_i32_32x32x32_i8 tiles, 256 accumulator registers per
 * lane) per item and per compute unit.  Three generations of the main loop
 * live here, selectable for measurement (hykGramSetSlab): operand slabs staged
 * global -> registers -> LDS (gram_kernel), direct global -> LDS loads into a
 * ring of four 64-K-byte stages (gram_dma_kernel), and the default, direct
 * loads of whole 128-byte lines into a ring of ten half-tile units that fills
 * the 160 KB of LDS (gram_ring_kernel).  In all of them the 16-byte LDS slots
 * are XOR-swizzled per row so that fragment reads are bank-conflict free.
 * Workgroups are dispatched round-robin over the 8 XCDs, so item =
 * (blockIdx % 8) * itemsPerXcd + blockIdx / 8 keeps the items that run
 * together on one XCD (one L2) on the same panels and K range.
 */
#include <vector>
#include <type_traits>
#include <atomic>
#include <hip/hip_runtime.h>
#include "hyk_common.h"
#include "crt_tables.h"
#include "hyacin_kernels.h"

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int TILE = 256;        /* output tile edge per workgroup */
constexpr int WAVE_TILE = 128;   /* output tile edge per wavefront */
constexpr int G_THREADS = 256;
constexpr int MAX_GROUPS = 48;
constexpr int MAX_PAIRS = 192;
constexpr int XCDS = 8;

enum { EPI_MOD = 0, EPI_I64 = 1 };

struct GramGroup {
  uint16_t pairBegin, pairCount;
  uint16_t planeRe, planeIm;
  uint32_t m, d, c32;       /* EPI_MOD: modulus, floor(2^32/m), 2^32 mod m */
  uint32_t mulRe, mulIm;    /* EPI_MOD: multipliers in [0, m), 0 = no contribution; EPI_I64: 0 none, 1 add, 2 subtract */
};

struct GramArgs {
  const int8_t* panels; int64_t ldb, panelStride;
  void* acc; int64_t planeStride;
  int32_t N, nT, tileCount, kLen, kSplits, K, groupCount, totalItems, itemsPerXcd;
  int32_t exclusive;                /* 1: this launch's items are the only writers of their accumulator entries */
  uint32_t tileMagic, splitMagic;   /* floor(2^32 / d) + 1: x / d == mulhi(x, magic) while x * d < 2^32 (checked on the host); 0 for d == 1 */
  /* set-aligned schedule (ring kernel): a set = the tileCount tiles of one (group, K split); slots = compute units per XCD */
  int32_t slotShift, roundsPerXcd, setCount, mainRounds, leftover, perRound; uint32_t mainMagic, leftMagic;
  int32_t pairShift;                /* 1: groups 2 s and 2 s + 1 read the same panels and take turns inside one set (complex residues) */
  GramGroup groups[MAX_GROUPS];
  uint32_t pairs[MAX_PAIRS];  /* lanePanel | aPanel << 16 */
};

/* element (i, j) of a 32x32 MFMA result held in accumulator register r of a lane */
__device__ __forceinline__ int acc_row(int r, int lane) { return ((r >> 2) << 3) + ((lane >> 5) << 2) + (r & 3); }

/* Epilogue shared by the contraction kernels (expanded in place: the accumulators must stay in registers): lane
 * dimension j <-> y (contiguous in the packed triangle), register dimension i <-> x.  Items that are the only writers of
 * their accumulator entries (one K split, planes not shared between groups: EXCL) store; all others add atomically. */
#define HYK_GRAM_PUT(TYPE, PLANE, VALUE) { TYPE* p_ = &dst[(int64_t)(PLANE) * args.planeStride + e]; if constexpr (EXCL_) { *p_ = (VALUE); } else { atomicAdd(p_, (VALUE)); } }
#define HYK_GRAM_EPILOGUE(EXCL) { \
  constexpr bool EXCL_ = (EXCL); const bool diagTile = (ta == tb); \
  _Pragma("unroll") for (int a = 0; a < 4; ++a) { \
    _Pragma("unroll") for (int b = 0; b < 4; ++b) { \
      __builtin_amdgcn_sched_barrier(0);   /* one 32x32 block at a time: keeps the accumulator copies out of scratch */ \
      const int y = y0 + wy * WAVE_TILE + b * 32 + (lane & 31); \
      _Pragma("unroll") for (int r = 0; r < 16; ++r) { \
        const int x = x0 + wx * WAVE_TILE + a * 32 + acc_row(r, lane); \
        if (x < args.N && y < args.N && (!diagTile || y <= x)) { \
          const int64_t e = hyk::tri_index(y, x); const int32_t w = acc[a][b][r]; \
          if constexpr (EPI == EPI_MOD) { \
            uint32_t* dst = reinterpret_cast<uint32_t*>(args.acc); \
            const uint32_t v = hyk::reduce_i32(w, grp.m, grp.d, grp.c32); \
            if (grp.mulRe) HYK_GRAM_PUT(uint32_t, grp.planeRe, grp.mulRe == 1u ? v : hyk::reduce_u32(v * grp.mulRe, grp.m, grp.d)) \
            if (grp.mulIm) HYK_GRAM_PUT(uint32_t, grp.planeIm, grp.mulIm == 1u ? v : hyk::reduce_u32(v * grp.mulIm, grp.m, grp.d)) \
          } else { \
            unsigned long long* dst = reinterpret_cast<unsigned long long*>(args.acc); \
            const unsigned long long pos = (unsigned long long)(long long)w, negv = (unsigned long long)(-(long long)w); \
            if (grp.mulRe) HYK_GRAM_PUT(unsigned long long, grp.planeRe, grp.mulRe == 1u ? pos : negv) \
            if (grp.mulIm) HYK_GRAM_PUT(unsigned long long, grp.planeIm, grp.mulIm == 1u ? pos : negv) \
          } \
        } \
      } \
    } \
  } \
}

template <int BK> struct Slab {
  static constexpr int PITCH = BK;                      /* bytes per tile row in LDS, unpadded; 16-byte slots are XOR-swizzled per row */
  static constexpr int TILE_BYTES = TILE * PITCH;
  static constexpr int PIECES = TILE * BK / 16;         /* 16-byte pieces per operand tile */
  static constexpr int PER_THREAD = PIECES / G_THREADS; /* pieces each thread moves per operand tile */
  static constexpr int PER_ROW = BK / 16;
  /* Slot swizzle: piece kq of row r sits in slot kq ^ swz(r).  Fragment reads touch the same kq of 8 (or 16) consecutive
   * rows: the swizzle spreads them over all 32 (or 64) banks; a parked row still occupies its own contiguous BK bytes, so
   * the writes are conflict-free as well. */
  __device__ static __forceinline__ int swz(int row) {
    if constexpr (BK == 64) { return (((row >> 1) ^ (row >> 3)) & 1) | (((row >> 2) & 1) << 1); }
    else { return ((row ^ (row >> 3)) & 1) | (row & 6); }
  }
};

template <int BK, int EPI>
__global__ __launch_bounds__(G_THREADS, 1) void gram_kernel(const GramArgs args) {
  using S = Slab<BK>;
  extern __shared__ __align__(16) int8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wy = wave & 1, wx = wave >> 1;

  /* XCD-aware item mapping.  Everything derived from the item is wave-uniform and stays in scalar registers: divisions go
   * through host-made reciprocals (the hardware divides on the vector ALU), the triangular root is a short scalar search. */
  const int item = (int)(blockIdx.x % XCDS) * args.itemsPerXcd + (int)(blockIdx.x / XCDS);
  if ((int)(blockIdx.x / XCDS) >= args.itemsPerXcd || item >= args.totalItems) { return; }
  const int gk = args.tileMagic ? (int)(((uint64_t)(uint32_t)item * args.tileMagic) >> 32) : item, t = item - gk * args.tileCount;
  const int g = args.splitMagic ? (int)(((uint64_t)(uint32_t)gk * args.splitMagic) >> 32) : gk, ks = gk - g * args.kSplits;
  int tb = 0; while ((tb + 1) * (tb + 2) / 2 <= t) { ++tb; }
  const int ta = t - tb * (tb + 1) / 2;
  const GramGroup grp = args.groups[g];
  const int k0 = ks * args.kLen, kEnd = (k0 + args.kLen) < args.K ? (k0 + args.kLen) : args.K, slabs = (kEnd - k0) / BK;
  const int y0 = ta * TILE, x0 = tb * TILE;

  /* per-thread global source offsets (column clamped to N-1: out-of-range columns only feed masked outputs) */
  int64_t srcLane[S::PER_THREAD], srcA[S::PER_THREAD]; int dstOff[S::PER_THREAD];
  #pragma unroll
  for (int r = 0; r < S::PER_THREAD; ++r) {
    const int p = tid + r * G_THREADS, row = p / S::PER_ROW, kq = p % S::PER_ROW;
    int cy = y0 + row; cy = cy < args.N ? cy : args.N - 1; int cx = x0 + row; cx = cx < args.N ? cx : args.N - 1;
    srcLane[r] = (int64_t)cy * args.ldb + kq * 16; srcA[r] = (int64_t)cx * args.ldb + kq * 16; dstOff[r] = row * S::PITCH + ((kq ^ S::swz(row)) << 4);
  }

  v16i acc[4][4];
  #pragma unroll
  for (int a = 0; a < 4; ++a) {
    #pragma unroll
    for (int b = 0; b < 4; ++b) {
      #pragma unroll
      for (int r = 0; r < 16; ++r) { acc[a][b][r] = 0; }
    }
  }

  const int iters = slabs * grp.pairCount;
  /* Global -> register -> LDS pipeline.  HBM / L2 latency is longer than one slab of MFMA work, so the loads of a slab are
   * issued three slabs ahead into one of two register sets, parked in LDS one slab ahead, and contracted from LDS. */
  v4i stg[2][2 * S::PER_THREAD];
  /* Position of the slab requested last (pair within the group, slab within the K range) and its panel addresses; all
   * wave-uniform and kept in scalar registers.  The loop body has no control flow: past the last slab the position stays
   * put and the loads re-read the last slab (never parked), so the outstanding-load counter can be waited on exactly.
   * peek() loads the descriptor of the following pair early; advance() consumes it right after a barrier, where the
   * LDS / scalar-load counter is drained anyway. */
  int curPair = 0, curSlab = 0, issued = 1; uint32_t ppNext = args.pairs[grp.pairBegin];
  const int8_t* baseLane = args.panels + (int64_t)(ppNext & 0xffffu) * args.panelStride + k0;
  const int8_t* baseA = args.panels + (int64_t)(ppNext >> 16) * args.panelStride + k0;
  auto peek = [&]() { const int q = curPair + 1 < (int)grp.pairCount ? curPair + 1 : (int)grp.pairCount - 1; ppNext = args.pairs[grp.pairBegin + q]; };
  auto advance = [&]() {
    const bool more = issued < iters, wrap = more && (curSlab + 1 == slabs);
    const int8_t* candLane = args.panels + (int64_t)(ppNext & 0xffffu) * args.panelStride + k0;
    const int8_t* candA = args.panels + (int64_t)(ppNext >> 16) * args.panelStride + k0;
    baseLane = wrap ? candLane : baseLane + (more ? BK : 0); baseA = wrap ? candA : baseA + (more ? BK : 0);
    curSlab = wrap ? 0 : curSlab + (more ? 1 : 0); curPair += wrap ? 1 : 0; issued += more ? 1 : 0;
  };
  auto issue = [&](v4i (&reg)[2 * S::PER_THREAD]) {
    #pragma unroll
    for (int r = 0; r < S::PER_THREAD; ++r) { reg[r] = *reinterpret_cast<const v4i*>(baseLane + srcLane[r]); }
    #pragma unroll
    for (int r = 0; r < S::PER_THREAD; ++r) { reg[S::PER_THREAD + r] = *reinterpret_cast<const v4i*>(baseA + srcA[r]); }
  };
  auto stash = [&](const v4i (&reg)[2 * S::PER_THREAD], int stage) {
    int8_t* tileLane = lds + stage * 2 * S::TILE_BYTES; int8_t* tileA = tileLane + S::TILE_BYTES;
    #pragma unroll
    for (int r = 0; r < S::PER_THREAD; ++r) { *reinterpret_cast<v4i*>(tileLane + dstOff[r]) = reg[r]; }
    #pragma unroll
    for (int r = 0; r < S::PER_THREAD; ++r) { *reinterpret_cast<v4i*>(tileA + dstOff[r]) = reg[S::PER_THREAD + r]; }
  };

  /* fragment addressing: lanes 0-31 take K bytes [0,16), lanes 32-63 bytes [16,32) of each 32-deep MFMA step; the row of a
   * lane is lane & 31 plus a multiple of 32, so its swizzle is a per-lane constant */
  constexpr int KSTEPS = BK / 32;
  const int rowLane = (wy * WAVE_TILE + (lane & 31)) * S::PITCH, rowA = (wx * WAVE_TILE + (lane & 31)) * S::PITCH, sw = S::swz(lane & 31), hi = lane >> 5;
  int kOff[KSTEPS];
  #pragma unroll
  for (int kk = 0; kk < KSTEPS; ++kk) { kOff[kk] = ((2 * kk + hi) ^ sw) << 4; }
  v4i fl[2][4], fa[2][4];
  auto frags = [&](int stage, int kk, int set) {
    const int8_t* tileLane = lds + stage * 2 * S::TILE_BYTES; const int8_t* tileA = tileLane + S::TILE_BYTES;
    #pragma unroll
    for (int b = 0; b < 4; ++b) { fl[set][b] = *reinterpret_cast<const v4i*>(tileLane + rowLane + b * 32 * S::PITCH + kOff[kk]); }
    #pragma unroll
    for (int a = 0; a < 4; ++a) { fa[set][a] = *reinterpret_cast<const v4i*>(tileA + rowA + a * 32 * S::PITCH + kOff[kk]); }
  };
  auto mfmas = [&](int set) {
    #pragma unroll
    for (int a = 0; a < 4; ++a) {
      #pragma unroll
      for (int b = 0; b < 4; ++b) { acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[set][a], fl[set][b], acc[a][b], 0, 0, 0); }
    }
  };
  /* One slab, software-pipelined.  On entry the fragments of its first K step are already on their way (set 0).
   * While the matrix cores work through a K step, the LDS pipe fetches the fragments of the next step and parks the next
   * slab in the other buffer; one barrier before the last K step publishes that slab, whose first fragments are then
   * requested under the last step's MFMAs together with the global loads of the slab three ahead.
   * sched_group_barrier pins the interleaving: masks 0x8 MFMA, 0x100 LDS read, 0x200 LDS write, 0x20 global read. */
  auto slab = [&](auto parity) {
    constexpr int cur = decltype(parity)::value, nxt = cur ^ 1;
    peek();
    #pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) {
      const bool last = (kk == KSTEPS - 1);
      if (!last) { frags(cur, kk + 1, (kk + 1) & 1); } else { frags(nxt, 0, 0); issue(stg[nxt]); }
      mfmas(kk & 1);
      if (kk == 0) { stash(stg[nxt], nxt); }
      #pragma unroll
      for (int i = 0; i < 8; ++i) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); }
      if (kk == 0) {
        #pragma unroll
        for (int i = 0; i < 8; ++i) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x200, (2 * S::PER_THREAD) / 8, 0); }
      } else if (last) {
        #pragma unroll
        for (int i = 0; i < 8; ++i) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x020, (2 * S::PER_THREAD) / 8, 0); }
      }
      if (kk == KSTEPS - 2) { __syncthreads(); advance(); }
    }
  };

  /* prologue: slabs 0 and 1 requested, slab 0 parked, slab 2 requested, first fragments on their way */
  issue(stg[0]); peek(); advance(); issue(stg[1]);
  stash(stg[0], 0);
  peek(); advance(); issue(stg[0]);
  __syncthreads();
  frags(0, 0, 0);
  int it = 0;
  for (; it + 1 < iters; it += 2) { slab(std::integral_constant<int, 0>{}); slab(std::integral_constant<int, 1>{}); }
  if (it < iters) { slab(std::integral_constant<int, 0>{}); }

  HYK_GRAM_EPILOGUE(false)
}

/* ------------------------------------------------------------------ contraction with direct global -> LDS loads
 * Same work items, same epilogue.  The operand slabs (64 K bytes deep) travel from HBM / L2 straight into a ring of four
 * LDS stages with global_load_lds_dwordx4: no staging registers, no LDS store instructions (at one wavefront per SIMD the
 * 16-byte LDS stores cost more issue time than the fragment reads).  The hardware writes the 64 lanes of such a load to
 * 64 consecutive 16-byte slots, so the slot swizzle is applied on the global side: the lane that owns slot s of row r
 * fetches K piece s ^ swz(r).  The loads are issued from inline assembly: the compiler would otherwise make every LDS
 * read wait for all direct loads in flight.  Their completion is tracked by hand with the vector-memory counter: every
 * slab step issues exactly 8 loads per lane (past the end of the K range it re-requests the last slab into a stage
 * nobody reads again), so "slab j + 1 has landed" is always "at most 16 loads outstanding". */
template <int V> using IC = std::integral_constant<int, V>;
constexpr int DMA_BK = 64, DMA_STAGES = 4, DMA_TILE_BYTES = TILE * DMA_BK, DMA_STAGE_BYTES = 2 * DMA_TILE_BYTES;

__device__ __forceinline__ void dma16(uint32_t ldsAddr, const int8_t* src) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" :: "s"(ldsAddr), "v"(src) : "memory");
}
/* the same with the address as a wave-uniform base plus an unsigned 32-bit offset per lane: no vector arithmetic per load */
__device__ __forceinline__ void dma16(uint32_t ldsAddr, const int8_t* base, uint32_t laneOffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" :: "s"(ldsAddr), "v"(laneOffset), "s"(base) : "memory");
}

template <int EPI, bool EXCL>
__global__ __launch_bounds__(G_THREADS, 1) void gram_dma_kernel(const GramArgs args) {
  using S = Slab<DMA_BK>;
  constexpr int BK = DMA_BK;
  extern __shared__ __align__(16) int8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wy = wave & 1, wx = wave >> 1;

  const int item = (int)(blockIdx.x % XCDS) * args.itemsPerXcd + (int)(blockIdx.x / XCDS);
  if ((int)(blockIdx.x / XCDS) >= args.itemsPerXcd || item >= args.totalItems) { return; }
  const int gk = args.tileMagic ? (int)(((uint64_t)(uint32_t)item * args.tileMagic) >> 32) : item, t = item - gk * args.tileCount;
  const int g = args.splitMagic ? (int)(((uint64_t)(uint32_t)gk * args.splitMagic) >> 32) : gk, ks = gk - g * args.kSplits;
  int tb = 0; while ((tb + 1) * (tb + 2) / 2 <= t) { ++tb; }
  const int ta = t - tb * (tb + 1) / 2;
  const GramGroup grp = args.groups[g];
  const int k0 = ks * args.kLen, kEnd = (k0 + args.kLen) < args.K ? (k0 + args.kLen) : args.K, slabs = (kEnd - k0) / BK;
  const int y0 = ta * TILE, x0 = tb * TILE;

  /* lane tid of load r fills LDS slot p = tid + 256 r of a tile (row p / 4, slot p % 4) */
  int64_t srcLane[S::PER_THREAD], srcA[S::PER_THREAD];
  #pragma unroll
  for (int r = 0; r < S::PER_THREAD; ++r) {
    const int p = tid + r * G_THREADS, row = p / S::PER_ROW, kq = (p % S::PER_ROW) ^ S::swz(row);
    int cy = y0 + row; cy = cy < args.N ? cy : args.N - 1; int cx = x0 + row; cx = cx < args.N ? cx : args.N - 1;
    srcLane[r] = (int64_t)cy * args.ldb + kq * 16; srcA[r] = (int64_t)cx * args.ldb + kq * 16;
  }
  const uint32_t ldsBase = (uint32_t)(size_t)(__attribute__((address_space(3))) int8_t*)lds;
  const uint32_t dmaBase = __builtin_amdgcn_readfirstlane(ldsBase + (uint32_t)wave * 1024u);

  v16i acc[4][4];
  #pragma unroll
  for (int a = 0; a < 4; ++a) {
    #pragma unroll
    for (int b = 0; b < 4; ++b) {
      #pragma unroll
      for (int r = 0; r < 16; ++r) { acc[a][b][r] = 0; }
    }
  }

  const int iters = slabs * grp.pairCount;
  int curPair = 0, curSlab = 0, issued = 1; uint32_t ppNext = args.pairs[grp.pairBegin];
  const int8_t* baseLane = args.panels + (int64_t)(ppNext & 0xffffu) * args.panelStride + k0;
  const int8_t* baseA = args.panels + (int64_t)(ppNext >> 16) * args.panelStride + k0;
  auto peek = [&]() { const int q = curPair + 1 < (int)grp.pairCount ? curPair + 1 : (int)grp.pairCount - 1; ppNext = args.pairs[grp.pairBegin + q]; };
  auto advance = [&]() {
    const bool more = issued < iters, wrap = more && (curSlab + 1 == slabs);
    const int8_t* candLane = args.panels + (int64_t)(ppNext & 0xffffu) * args.panelStride + k0;
    const int8_t* candA = args.panels + (int64_t)(ppNext >> 16) * args.panelStride + k0;
    baseLane = wrap ? candLane : baseLane + (more ? BK : 0); baseA = wrap ? candA : baseA + (more ? BK : 0);
    curSlab = wrap ? 0 : curSlab + (more ? 1 : 0); curPair += wrap ? 1 : 0; issued += more ? 1 : 0;
  };
  /* load i (0..7) of the current slab position into the stage at byte offset stageOff */
  auto dma = [&](int i, uint32_t stageOff) {
    const int r = i & 3; const bool second = i >= 4;
    dma16(dmaBase + stageOff + (second ? (uint32_t)DMA_TILE_BYTES : 0u) + (uint32_t)r * 4096u, (second ? baseA + srcA[r] : baseLane + srcLane[r]));
  };

  constexpr int KSTEPS = BK / 32;
  static_assert(KSTEPS == 2, "the slab step below is written for two MFMA K steps");
  const int rowLane = (wy * WAVE_TILE + (lane & 31)) * S::PITCH, rowA = DMA_TILE_BYTES + (wx * WAVE_TILE + (lane & 31)) * S::PITCH, sw = S::swz(lane & 31), hi = lane >> 5;
  const int k0Off = ((0 + hi) ^ sw) << 4, k1Off = ((2 + hi) ^ sw) << 4;
  v4i fl[2][4], fa[2][4];
  /* fragment read i (0..3 lane operand, 4..7 A operand) of K step kk from the stage at stageOff into register set `set` */
  auto rd = [&](int i, int set, int kk, uint32_t stageOff) {
    const int8_t* base = lds + stageOff + (kk ? k1Off : k0Off);
    if (i < 4) { fl[set][i] = *reinterpret_cast<const v4i*>(base + rowLane + i * 32 * S::PITCH); }
    else { fa[set][i - 4] = *reinterpret_cast<const v4i*>(base + rowA + (i - 4) * 32 * S::PITCH); }
  };
  auto mm = [&](int n, int set) { const int a = n >> 2, b = n & 3; acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[set][a], fl[set][b], acc[a][b], 0, 0, 0); };

  /* A run of MFMAs with fragment reads paired to the first of them, closed for the scheduler so that the direct loads
   * issued between runs stay where they are written. */
  auto run = [&](auto mmFirst_, auto mmCount_, auto mmSet_, auto rdFirst_, auto rdCount_, auto rdSet_, auto rdKk_, uint32_t rdOff) {
    constexpr int mmFirst = decltype(mmFirst_)::value, mmCount = decltype(mmCount_)::value, mmSet = decltype(mmSet_)::value;
    constexpr int rdFirst = decltype(rdFirst_)::value, rdCount = decltype(rdCount_)::value, rdSet = decltype(rdSet_)::value, rdKk = decltype(rdKk_)::value;
    #pragma unroll
    for (int i = 0; i < rdCount; ++i) { rd(rdFirst + i, rdSet, rdKk, rdOff); }
    #pragma unroll
    for (int n = 0; n < mmCount; ++n) { mm(mmFirst + n, mmSet); }
    #pragma unroll
    for (int i = 0; i < rdCount; ++i) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); }
    if constexpr (mmCount > rdCount) { __builtin_amdgcn_sched_group_barrier(0x008, mmCount - rdCount, 0); }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto load = [&](int i, uint32_t stageOff) { dma(i, stageOff); __builtin_amdgcn_sched_barrier(0); };

  /* prologue: slabs 0..2 and the lane-operand half of slab 3 on their way, slab 0 landed and published, its first fragments requested */
  #pragma unroll
  for (int st = 0; st < DMA_STAGES; ++st) {
    if (st) { peek(); advance(); }
    #pragma unroll
    for (int i = 0; i < (st == DMA_STAGES - 1 ? 4 : 8); ++i) { dma(i, (uint32_t)st * DMA_STAGE_BYTES); }
  }
  asm volatile("s_waitcnt vmcnt(20)" ::: "memory");
  __syncthreads();
  #pragma unroll
  for (int i = 0; i < 8; ++i) { rd(i, 0, 0, 0u); }
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_sched_barrier(0);

  /* Steady state, slab `it` in stage it % 4.  The eight loads of a slab are spread over a whole slab time (a burst of them
   * stalls instruction issue behind the address unit): the A-operand half of slab it + 3 goes out under the first K step
   * into the stage freed one slab ago, the lane-operand half of slab it + 4 under the second K step into stage `cur`. */
  for (int it = 0; it < iters; ++it) {
    const uint32_t curOff = (uint32_t)(it & (DMA_STAGES - 1)) * DMA_STAGE_BYTES, nxtOff = (uint32_t)((it + 1) & (DMA_STAGES - 1)) * DMA_STAGE_BYTES,
                   prvOff = (uint32_t)((it + DMA_STAGES - 1) & (DMA_STAGES - 1)) * DMA_STAGE_BYTES;
    /* first K step: MFMAs on set 0, fragments of the second K step into set 1 */
    peek();
    run(IC<0>{}, IC<3>{}, IC<0>{}, IC<0>{}, IC<3>{}, IC<1>{}, IC<1>{}, curOff); load(4, prvOff);
    run(IC<3>{}, IC<3>{}, IC<0>{}, IC<3>{}, IC<3>{}, IC<1>{}, IC<1>{}, curOff); load(5, prvOff);
    run(IC<6>{}, IC<3>{}, IC<0>{}, IC<6>{}, IC<2>{}, IC<1>{}, IC<1>{}, curOff); load(6, prvOff);
    run(IC<9>{}, IC<2>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<1>{}, IC<1>{}, curOff); load(7, prvOff);
    run(IC<11>{}, IC<1>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<1>{}, IC<1>{}, curOff);
    /* slab it + 1 has landed (own loads) and every wave is done reading stage `cur`: publish */
    asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    run(IC<12>{}, IC<4>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<1>{}, IC<1>{}, curOff);
    advance();
    __builtin_amdgcn_sched_barrier(0);
    /* second K step: MFMAs on set 1, first fragments of the next slab into set 0 */
    run(IC<0>{}, IC<4>{}, IC<1>{}, IC<0>{}, IC<4>{}, IC<0>{}, IC<0>{}, nxtOff); load(0, curOff);
    run(IC<4>{}, IC<4>{}, IC<1>{}, IC<4>{}, IC<4>{}, IC<0>{}, IC<0>{}, nxtOff); load(1, curOff);
    run(IC<8>{}, IC<4>{}, IC<1>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<0>{}, nxtOff); load(2, curOff);
    run(IC<12>{}, IC<3>{}, IC<1>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<0>{}, nxtOff); load(3, curOff);
    run(IC<15>{}, IC<1>{}, IC<1>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<0>{}, nxtOff);
    __builtin_amdgcn_s_waitcnt(0xC07F);   /* lgkmcnt(0): set 0 was requested eight MFMAs ago; stating it here keeps waits out of the first K step */
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   /* no direct load may still be writing LDS when the workgroup ends */

  HYK_GRAM_EPILOGUE(EXCL)
}

/* ------------------------------------------------------------------ contraction with full-line direct loads
 * Same work items and epilogue again; what changes is the shape of the global -> LDS traffic.  A direct load that fetches
 * 64 K-bytes of a row touches half a 128-byte cache line, and the L2 / address path is bound by requests, not bytes:
 * with every load instruction covering 8 rows x 128 bytes (whole lines) the same bytes cost about half as much.  K
 * therefore advances in slabs of 128 bytes, and all of LDS (160 KB) is a ring of ten 16 KB units, a unit being half an
 * operand tile (128 rows x 128 K-bytes, 16-byte slots XOR-swizzled per row on the global side).  A slab is four
 * consecutive units: lane rows 0-127, lane rows 128-255, A rows 0-127, A rows 128-255.
 *
 * Schedule of slab j (four MFMA K steps, fragments one step ahead in two register sets):
 *   step 0, 1   fill the two lane units of slab j + 2 (freed by slab j - 1), one load per four MFMAs;
 *   step 2      no loads; at its end slab j + 1 has landed (at most the 8 loads just issued are outstanding) and every
 *               wave has read the last fragments of slab j: barrier;
 *   step 3      first fragments of slab j + 1, and the two A units of slab j + 2 go into units slab j just released.
 * The loads that gate a barrier are always at least three K steps (1536 MFMA cycles) old. */
constexpr int RING_K = 128, RING_UNIT_BYTES = 128 * RING_K, RING_UNITS = 10, RING_BYTES = RING_UNITS * RING_UNIT_BYTES;

template <int EPI, bool EXCL>
__global__ __launch_bounds__(G_THREADS, 1) void gram_ring_kernel(const GramArgs args) {
  using S = Slab<RING_K>;
  extern __shared__ __align__(16) int8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), wy = wave & 1, wx = wave >> 1;

  /* Set-aligned schedule.  The workgroups of an XCD start in the order of their index and, one per compute unit, run in
   * rounds of `slots`.  All tiles of a set (one group, one K split) read the same panels, so a round should hold tiles
   * of one set: a set takes mainRounds whole rounds, and the tileCount % slots tiles left over are packed perRound sets
   * to a round behind all the whole ones.  Round rr of the launch is round rr / 8 of XCD rr % 8, which spreads the
   * left-over rounds (they read the most panel bytes per tile) over the XCDs. */
  const int xcd = (int)(blockIdx.x % XCDS), q = (int)(blockIdx.x / XCDS), slots = 1 << args.slotShift;
  const int round = q >> args.slotShift, slot = q & (slots - 1), rr = round * XCDS + xcd;
  auto divide = [](int v, uint32_t magic) { return magic ? (int)(((uint64_t)(uint32_t)v * magic) >> 32) : v; };
  int set, t;
  if (rr < args.setCount * args.mainRounds) { set = divide(rr, args.mainMagic); t = ((rr - set * args.mainRounds) << args.slotShift) + slot; }
  else {
    if (args.leftover == 0) { return; }
    const int inRound = divide(slot, args.leftMagic); set = (rr - args.setCount * args.mainRounds) * args.perRound + inRound;
    if (inRound >= args.perRound || set >= args.setCount) { return; }
    t = (args.mainRounds << args.slotShift) + (slot - inRound * args.leftover);
  }
  const int sg = divide(set, args.splitMagic), ks = set - sg * args.kSplits, g = (sg << args.pairShift) + (t & ((1 << args.pairShift) - 1)); t >>= args.pairShift;
  /* tiles row by row, (ta, ta), (ta, ta + 1), ..., (ta, nT - 1): the tiles at the end of this order, which the schedule
   * packs into the left-over rounds, form the smallest triangle in the corner and share the fewest row blocks */
  int ta = 0, rowStart = 0; while (rowStart + (args.nT - ta) <= t) { rowStart += args.nT - ta; ++ta; }
  const int tb = ta + (t - rowStart);
  const GramGroup grp = args.groups[g];
  const int k0 = ks * args.kLen, kEnd = (k0 + args.kLen) < args.K ? (k0 + args.kLen) : args.K, slabs = (kEnd - k0) / RING_K;
  const int y0 = ta * TILE, x0 = tb * TILE;

  /* load r (0..3) of a unit: lane tid fills slot tid % 8 of row tid / 8 + 32 r (tile row + 128 for the second half) */
  /* byte offsets from the first row of the tile (the host has checked that 256 rows fit 32 bits) */
  uint32_t srcLane[2][4], srcA[2][4];
  {
    const int rowBase = tid >> 3, kq = (tid & 7) ^ S::swz(rowBase);   /* the swizzle depends on the row modulo 32 only */
    #pragma unroll
    for (int h = 0; h < 2; ++h) {
      #pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = h * 128 + rowBase + 32 * r;
        int cy = y0 + row; cy = cy < args.N ? cy : args.N - 1; int cx = x0 + row; cx = cx < args.N ? cx : args.N - 1;
        srcLane[h][r] = (uint32_t)(cy - y0) * (uint32_t)args.ldb + (uint32_t)kq * 16u; srcA[h][r] = (uint32_t)(cx - x0) * (uint32_t)args.ldb + (uint32_t)kq * 16u;
      }
    }
  }
  const uint32_t ldsBase = (uint32_t)(size_t)(__attribute__((address_space(3))) int8_t*)lds;
  const uint32_t dmaBase = __builtin_amdgcn_readfirstlane(ldsBase + (uint32_t)wave * 1024u);

  v16i acc[4][4];
  #pragma unroll
  for (int a = 0; a < 4; ++a) {
    #pragma unroll
    for (int b = 0; b < 4; ++b) {
      #pragma unroll
      for (int r = 0; r < 16; ++r) { acc[a][b][r] = 0; }
    }
  }

  /* Two request streams run through the same sequence of (pair, slab) positions: the lane units and, half a slab behind,
   * the A units.  Each keeps the position it requested last as wave-uniform scalar state: slabs still to request in the
   * whole item and in the current pair, the pair, the address of the slab.  Past the last slab a stream stays where it
   * is (the ring is filled two slabs ahead, so the last iterations request the last slab again).  The common step is
   * branch-free scalar arithmetic; only the change of pair, once in `slabs` steps, takes a branch and a load. */
  const int iters = __builtin_amdgcn_readfirstlane(slabs * (int)grp.pairCount);
  const int lastPair = __builtin_amdgcn_readfirstlane((int)grp.pairCount - 1), pairBegin = __builtin_amdgcn_readfirstlane((int)grp.pairBegin);
  const int perPair = __builtin_amdgcn_readfirstlane(slabs);
  const uint32_t pp0 = args.pairs[pairBegin];
  const int64_t rowsLane = (int64_t)y0 * args.ldb + k0, rowsA = (int64_t)x0 * args.ldb + k0;
  const int8_t* baseLane = args.panels + (int64_t)(pp0 & 0xffffu) * args.panelStride + rowsLane;
  const int8_t* baseA = args.panels + (int64_t)(pp0 >> 16) * args.panelStride + rowsA;
  int leftL = iters - 1, inPairL = perPair - 1, pairL = 0, leftA = iters - 1, inPairA = perPair - 1, pairA = 0;
  /* (the step is written without booleans that outlive a basic block: such a condition is held as a lane mask and
   * drags the counters into vector registers and vector compares) */
  auto advanceL = [&]() {
    const int go = leftL < 1 ? leftL : 1;                      /* 0 once every slab has been requested */
    baseLane += go * RING_K; leftL -= go; inPairL -= go;
    if (__builtin_expect(inPairL < 0, 0)) {
      pairL = pairL + 1 < lastPair ? pairL + 1 : lastPair; inPairL = perPair - 1;
      baseLane = args.panels + (int64_t)(args.pairs[pairBegin + pairL] & 0xffffu) * args.panelStride + rowsLane;
    }
  };
  auto advanceA = [&]() {
    const int go = leftA < 1 ? leftA : 1;
    baseA += go * RING_K; leftA -= go; inPairA -= go;
    if (__builtin_expect(inPairA < 0, 0)) {
      pairA = pairA + 1 < lastPair ? pairA + 1 : lastPair; inPairA = perPair - 1;
      baseA = args.panels + (int64_t)(args.pairs[pairBegin + pairA] >> 16) * args.panelStride + rowsA;
    }
  };
  /* ring position of the next unit to fill (byte offset, wraps at RING_BYTES) */
  uint32_t fillOff = 0;
  auto next_unit = [&]() { const uint32_t u = fillOff; fillOff += RING_UNIT_BYTES; fillOff = fillOff == (uint32_t)RING_BYTES ? 0u : fillOff; return u; };
  auto fill_lane = [&](int h, int r, uint32_t unitOff) { dma16(dmaBase + unitOff + (uint32_t)r * 4096u, baseLane, srcLane[h][r]); };
  auto fill_a = [&](int h, int r, uint32_t unitOff) { dma16(dmaBase + unitOff + (uint32_t)r * 4096u, baseA, srcA[h][r]); };

  const int rowOff = (lane & 31) * RING_K, sw = S::swz(lane & 31), hi = lane >> 5;
  int kOff[4];
  #pragma unroll
  for (int kk = 0; kk < 4; ++kk) { kOff[kk] = ((2 * kk + hi) ^ sw) << 4; }
  v4i fl[2][4], fa[2][4];
  /* fragment read i (0..3 lane operand, 4..7 A operand) of K step kk; laneUnit / aUnit: byte offsets of this wave's units */
  auto rd = [&](int i, int set, int kk, uint32_t laneUnit, uint32_t aUnit) {
    if (i < 4) { fl[set][i] = *reinterpret_cast<const v4i*>(lds + laneUnit + rowOff + i * 32 * RING_K + kOff[kk]); }
    else { fa[set][i - 4] = *reinterpret_cast<const v4i*>(lds + aUnit + rowOff + (i - 4) * 32 * RING_K + kOff[kk]); }
  };
  auto unit_offset = [&](uint32_t slabOff, int unit) { uint32_t o = slabOff + (uint32_t)unit * RING_UNIT_BYTES; return o >= (uint32_t)RING_BYTES ? o - (uint32_t)RING_BYTES : o; };

  /* prologue: slabs 0 and 1 requested in full (eight units); slab 0 landed and published; its first fragments requested */
  #pragma unroll
  for (int s0 = 0; s0 < 2; ++s0) {
    if (s0) { advanceL(); advanceA(); }
    #pragma unroll
    for (int h = 0; h < 2; ++h) {
      const uint32_t u = next_unit();
      #pragma unroll
      for (int r = 0; r < 4; ++r) { fill_lane(h, r, u); }
    }
    #pragma unroll
    for (int h = 0; h < 2; ++h) {
      const uint32_t u = next_unit();
      #pragma unroll
      for (int r = 0; r < 4; ++r) { fill_a(h, r, u); }
    }
  }
  advanceL();                              /* lane stream: next to request is slab 2; A stream stays on slab 1 until the first barrier */
  asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  __syncthreads();
  uint32_t slabOff = 0;                    /* ring offset of the first unit of the slab being contracted */
  {
    const uint32_t lu = unit_offset(slabOff, wy), au = unit_offset(slabOff, 2 + wx);
    #pragma unroll
    for (int i = 0; i < 8; ++i) { rd(i, 0, 0, lu, au); }
  }
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_sched_barrier(0);

  /* The loop in three versions, chosen once per wavefront.  In a diagonal tile only y <= x is kept: of the 32x32 blocks
   * (a, b) of wavefront (wy, wx), those with 4 wy + b > 4 wx + a lie wholly below the diagonal.  Version 1 (wy == wx)
   * leaves out its six such blocks, version 2 (wy > wx) all sixteen: that wavefront only requests its share of the ring
   * and keeps the barriers.  The device runs this kernel at its power limit, so MFMAs not issued turn into clock. */
  auto contract = [&](auto mode_) {
    constexpr int MODE = decltype(mode_)::value;
    /* MFMA n of a K step works on block (a, b) = (n / 4, n % 4 run back and forth): between consecutive MFMAs only one
     * of the two operands changes */
    auto b_of = [](int n) constexpr { return ((n >> 2) & 1) ? 3 - (n & 3) : (n & 3); };
    auto kept = [b_of](int n) constexpr { return MODE == 0 || (MODE == 1 && b_of(n) <= (n >> 2)); };
    auto mm = [&](int n, int set) { const int a = n >> 2, b = b_of(n); acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[set][a], fl[set][b], acc[a][b], 0, 0, 0); };
    /* a run of MFMAs with fragment reads paired to the first of them, closed for the scheduler */
    auto run = [&](auto mmFirst_, auto mmCount_, auto mmSet_, auto rdFirst_, auto rdCount_, auto rdSet_, auto rdKk_, uint32_t laneUnit, uint32_t aUnit) {
      constexpr int mmFirst = decltype(mmFirst_)::value, mmCount = decltype(mmCount_)::value, mmSet = decltype(mmSet_)::value;
      constexpr int rdFirst = decltype(rdFirst_)::value, rdCount = MODE == 2 ? 0 : decltype(rdCount_)::value, rdSet = decltype(rdSet_)::value, rdKk = decltype(rdKk_)::value;
      int keptCount = 0;
      #pragma unroll
      for (int i = 0; i < rdCount; ++i) { rd(rdFirst + i, rdSet, rdKk, laneUnit, aUnit); }
      #pragma unroll
      for (int n = 0; n < mmCount; ++n) { if (kept(mmFirst + n)) { mm(mmFirst + n, mmSet); ++keptCount; } }
      #pragma unroll
      for (int i = 0; i < rdCount; ++i) { if (i < keptCount) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); } __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); }
      #pragma unroll
      for (int n = rdCount; n < mmCount; ++n) { if (n < keptCount) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); } }
      __builtin_amdgcn_sched_barrier(0);
    };
    for (int it = 0; it < iters; ++it) {
      const uint32_t lu = unit_offset(slabOff, wy), au = unit_offset(slabOff, 2 + wx);
      uint32_t nextOff = slabOff + 4u * RING_UNIT_BYTES; nextOff = nextOff >= (uint32_t)RING_BYTES ? nextOff - (uint32_t)RING_BYTES : nextOff;
      const uint32_t nlu = unit_offset(nextOff, wy), nau = unit_offset(nextOff, 2 + wx);
      /* K step 0: MFMAs on set 0, fragments of step 1 into set 1, lane unit 0 of slab it + 2 */
      { const uint32_t u = next_unit();
        run(IC<0>{}, IC<4>{}, IC<0>{}, IC<0>{}, IC<4>{}, IC<1>{}, IC<1>{}, lu, au); fill_lane(0, 0, u); __builtin_amdgcn_sched_barrier(0);
        run(IC<4>{}, IC<4>{}, IC<0>{}, IC<4>{}, IC<4>{}, IC<1>{}, IC<1>{}, lu, au); fill_lane(0, 1, u); __builtin_amdgcn_sched_barrier(0);
        run(IC<8>{}, IC<4>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<1>{}, IC<1>{}, lu, au); fill_lane(0, 2, u); __builtin_amdgcn_sched_barrier(0);
        run(IC<12>{}, IC<4>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<1>{}, IC<1>{}, lu, au); fill_lane(0, 3, u); __builtin_amdgcn_sched_barrier(0); }
      /* K step 1: MFMAs on set 1, fragments of step 2 into set 0, lane unit 1 of slab it + 2 */
      { const uint32_t u = next_unit();
        run(IC<0>{}, IC<4>{}, IC<1>{}, IC<0>{}, IC<4>{}, IC<0>{}, IC<2>{}, lu, au); fill_lane(1, 0, u); __builtin_amdgcn_sched_barrier(0);
        run(IC<4>{}, IC<4>{}, IC<1>{}, IC<4>{}, IC<4>{}, IC<0>{}, IC<2>{}, lu, au); fill_lane(1, 1, u); __builtin_amdgcn_sched_barrier(0);
        run(IC<8>{}, IC<4>{}, IC<1>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<2>{}, lu, au); fill_lane(1, 2, u); __builtin_amdgcn_sched_barrier(0);
        run(IC<12>{}, IC<4>{}, IC<1>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<2>{}, lu, au); fill_lane(1, 3, u); __builtin_amdgcn_sched_barrier(0); }
      /* K step 2: MFMAs on set 0, fragments of step 3 into set 1, no loads */
      run(IC<0>{}, IC<4>{}, IC<0>{}, IC<0>{}, IC<4>{}, IC<1>{}, IC<3>{}, lu, au);
      run(IC<4>{}, IC<8>{}, IC<0>{}, IC<4>{}, IC<4>{}, IC<1>{}, IC<3>{}, lu, au);
      /* slab it + 1 has landed (own loads: only the eight lane loads above may be outstanding) and every wave has read
       * its last fragments of slab it: publish, release */
      asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
      run(IC<12>{}, IC<4>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<1>{}, IC<3>{}, lu, au);
      advanceL(); advanceA();
      __builtin_amdgcn_sched_barrier(0);
      /* K step 3: MFMAs on set 1, first fragments of slab it + 1 into set 0, both A units of slab it + 2 */
      { const uint32_t u0 = next_unit(), u1 = next_unit();
        run(IC<0>{}, IC<2>{}, IC<1>{}, IC<0>{}, IC<2>{}, IC<0>{}, IC<0>{}, nlu, nau); fill_a(0, 0, u0); __builtin_amdgcn_sched_barrier(0);
        run(IC<2>{}, IC<2>{}, IC<1>{}, IC<2>{}, IC<2>{}, IC<0>{}, IC<0>{}, nlu, nau); fill_a(0, 1, u0); __builtin_amdgcn_sched_barrier(0);
        run(IC<4>{}, IC<2>{}, IC<1>{}, IC<4>{}, IC<2>{}, IC<0>{}, IC<0>{}, nlu, nau); fill_a(0, 2, u0); __builtin_amdgcn_sched_barrier(0);
        run(IC<6>{}, IC<2>{}, IC<1>{}, IC<6>{}, IC<2>{}, IC<0>{}, IC<0>{}, nlu, nau); fill_a(0, 3, u0); __builtin_amdgcn_sched_barrier(0);
        run(IC<8>{}, IC<2>{}, IC<1>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<0>{}, nlu, nau); fill_a(1, 0, u1); __builtin_amdgcn_sched_barrier(0);
        run(IC<10>{}, IC<2>{}, IC<1>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<0>{}, nlu, nau); fill_a(1, 1, u1); __builtin_amdgcn_sched_barrier(0);
        run(IC<12>{}, IC<2>{}, IC<1>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<0>{}, nlu, nau); fill_a(1, 2, u1); __builtin_amdgcn_sched_barrier(0);
        run(IC<14>{}, IC<2>{}, IC<1>{}, IC<0>{}, IC<0>{}, IC<0>{}, IC<0>{}, nlu, nau); fill_a(1, 3, u1); __builtin_amdgcn_sched_barrier(0); }
      __builtin_amdgcn_s_waitcnt(0xC07F);   /* lgkmcnt(0): the fragments of the next slab were requested eight MFMAs ago */
      slabOff = nextOff;
    }
  };
  const int mode = (ta == tb) ? (wy > wx ? 2 : (wy == wx ? 1 : 0)) : 0;
  if (mode == 0) { contract(IC<0>{}); } else if (mode == 1) { contract(IC<1>{}); } else { contract(IC<2>{}); }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   /* no direct load may still be writing LDS when the workgroup ends */

  /* Epilogue: the same entries, values and order of operations per entry as HYK_GRAM_EPILOGUE, with everything that is
   * uniform over the workgroup decided once.  Lane dimension j <-> y (contiguous in the packed triangle), register
   * dimension i <-> x; register r of a block is row xb + 8 (r / 4) + r % 4, so the packed index runs along with
   * tri(x + s) - tri(x) = s x + s (s + 1) / 2.  A signed sum w is reduced as (w + bias) mod m with bias the smallest
   * multiple of m that is >= 2^31: w + bias is non-negative and below 2^32 for every sum the K cap allows (for m = 256
   * a wrap is harmless), so one unsigned reduction gives the canonical residue.  Blocks of a diagonal tile wholly below
   * the diagonal are skipped, those wholly above need no test.  CHECKED: the tile touches the matrix edge or the diagonal.
   * SIMPLE: the group adds its sums unchanged to its real plane only (every real launch, the paired complex residues). */
  const bool inner = (ta != tb) && (x0 + TILE <= args.N) && (y0 + TILE <= args.N);
  const bool simple = grp.mulRe == 1u && grp.mulIm == 0u;
  uint32_t bias = 0u;
  if constexpr (EPI == EPI_MOD) { const uint32_t over = 0x80000000u % grp.m; bias = 0x80000000u + (over ? grp.m - over : 0u); }
  /* 64-bit sums: the two planes of the group and the signs, as wave-uniform values in scalar registers */
  [[maybe_unused]] unsigned long long* wideRe = nullptr; [[maybe_unused]] unsigned long long* wideIm = nullptr;
  [[maybe_unused]] bool hasRe = false, hasIm = false; [[maybe_unused]] int32_t maskRe = 0, maskIm = 0;
  if constexpr (EPI == EPI_I64) {
    auto uniform64 = [](uint64_t v) { return ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32)) << 32) | (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v); };
    wideRe = reinterpret_cast<unsigned long long*>(uniform64((uint64_t)(reinterpret_cast<unsigned long long*>(args.acc) + (int64_t)grp.planeRe * args.planeStride)));
    wideIm = reinterpret_cast<unsigned long long*>(uniform64((uint64_t)(reinterpret_cast<unsigned long long*>(args.acc) + (int64_t)grp.planeIm * args.planeStride)));
    hasRe = __builtin_amdgcn_readfirstlane((int)grp.mulRe) != 0; hasIm = __builtin_amdgcn_readfirstlane((int)grp.mulIm) != 0;
    maskRe = __builtin_amdgcn_readfirstlane(grp.mulRe == 2u ? -1 : 0); maskIm = __builtin_amdgcn_readfirstlane(grp.mulIm == 2u ? -1 : 0);
  }
  /* what the epilogue needs of the arguments, as locals: its sixteen blocks in four versions name them hundreds of times,
   * and past some number of uses the optimiser stops reading a by-value argument structure in place and copies it to
   * scratch memory instead (whose loads count as divergent: the load addresses of the loop above then sit in vector registers) */
  const int32_t nCols = args.N; const int64_t planeStride = args.planeStride; uint32_t* const accBase = reinterpret_cast<uint32_t*>(args.acc);
  auto emit = [&](auto checked_, auto simple_) {
    constexpr bool CHECKED = decltype(checked_)::value != 0, SIMPLE = decltype(simple_)::value != 0;
    /* one 32x32 block; a and b are compile-time values, so the accumulators are named registers whatever the optimiser
     * makes of the loops (a loop over blocks that it declines to unroll indexes them at run time: all 256 go to scratch) */
    auto block = [&](auto a_, auto b_) __attribute__((always_inline)) {   /* (a call that is not inlined would take the address of the kernel arguments, which then live in scratch memory) */
        constexpr int a = decltype(a_)::value, b = decltype(b_)::value;
        __builtin_amdgcn_sched_barrier(0);   /* one 32x32 block at a time: keeps the accumulator copies out of scratch */
        bool diagBlock = false;
        if constexpr (CHECKED) { if (ta == tb) { const int by = 4 * wy + b, bx = 4 * wx + a; if (by > bx) { return; } diagBlock = by == bx; } }
        const int y = y0 + wy * WAVE_TILE + b * 32 + (lane & 31);
        int x = x0 + wx * WAVE_TILE + a * 32 + ((lane >> 5) << 2);
        int64_t e = hyk::tri_index(y, x);
        #pragma unroll
        for (int r = 0; r < 16; ++r) {
          if (r) { if (r & 3) { e += x + 1; x += 1; } else { e += 5 * (int64_t)x + 15; x += 5; } }
          bool ok = true;
          if constexpr (CHECKED) { ok = x < nCols && y < nCols && (!diagBlock || y <= x); }
          if (ok) {
            const int32_t w = acc[a][b][r];
            if constexpr (EPI == EPI_MOD) {
              uint32_t* dst = accBase;
              const uint32_t v = hyk::reduce_u32((uint32_t)w + bias, grp.m, grp.d);
              if constexpr (SIMPLE) {
                uint32_t* at = &dst[(int64_t)grp.planeRe * planeStride + e];
                if constexpr (EXCL) { *at = v; } else { atomicAdd(at, v); }
              } else {
                if (grp.mulRe) { uint32_t* at = &dst[(int64_t)grp.planeRe * planeStride + e]; const uint32_t t = grp.mulRe == 1u ? v : hyk::reduce_u32(v * grp.mulRe, grp.m, grp.d); if constexpr (EXCL) { *at = t; } else { atomicAdd(at, t); } }
                if (grp.mulIm) { uint32_t* at = &dst[(int64_t)grp.planeIm * planeStride + e]; const uint32_t t = grp.mulIm == 1u ? v : hyk::reduce_u32(v * grp.mulIm, grp.m, grp.d); if constexpr (EXCL) { *at = t; } else { atomicAdd(at, t); } }
              }
            } else {   /* 64-bit sums of the limb levels: + W or - W to the real and / or the imaginary plane of the level */
              if constexpr (SIMPLE) {
                unsigned long long* at = wideRe + e; const unsigned long long pos = (unsigned long long)(long long)w;
                if constexpr (EXCL) { *at = pos; } else { atomicAdd(at, pos); }
              } else {   /* (w ^ mask) - mask = -w for mask = -1 (a K range that the cap allows never sums to INT_MIN) */
                if (hasRe) { const unsigned long long t = (unsigned long long)(long long)((w ^ maskRe) - maskRe); if constexpr (EXCL) { wideRe[e] = t; } else { atomicAdd(wideRe + e, t); } }
                if (hasIm) { const unsigned long long t = (unsigned long long)(long long)((w ^ maskIm) - maskIm); if constexpr (EXCL) { wideIm[e] = t; } else { atomicAdd(wideIm + e, t); } }
              }
            }
          }
        }
    };
    block(IC<0>{}, IC<0>{}); block(IC<0>{}, IC<1>{}); block(IC<0>{}, IC<2>{}); block(IC<0>{}, IC<3>{});
    block(IC<1>{}, IC<0>{}); block(IC<1>{}, IC<1>{}); block(IC<1>{}, IC<2>{}); block(IC<1>{}, IC<3>{});
    block(IC<2>{}, IC<0>{}); block(IC<2>{}, IC<1>{}); block(IC<2>{}, IC<2>{}); block(IC<2>{}, IC<3>{});
    block(IC<3>{}, IC<0>{}); block(IC<3>{}, IC<1>{}); block(IC<3>{}, IC<2>{}); block(IC<3>{}, IC<3>{});
  };
  if (mode == 2) { /* every block of this wavefront lies below the diagonal */ }
  else if (inner) { if (simple) { emit(IC<0>{}, IC<1>{}); } else { emit(IC<0>{}, IC<0>{}); } }
  else { if (simple) { emit(IC<1>{}, IC<1>{}); } else { emit(IC<1>{}, IC<0>{}); } }
}

/* ------------------------------------------------------------------ CRT reconstruction */
struct ReconTable {
  int32_t order, rot;   /* rot: the first `rot` moduli of a complex launch hold p and q = Re +- i Im instead of Re and Im */
  uint32_t m[HYK_CRT_CPLX_COUNT], d[HYK_CRT_CPLX_COUNT], minv[HYK_CRT_CPLX_COUNT], iminv[HYK_CRT_CPLX_COUNT];
  uint64_t Pd[HYK_CRT_CPLX_COUNT][3], P[3];
};

/* one modulus of the centred lift: a += s (P/m) with s = (r minv mod m) - (a >= 0 ? m : 0), which keeps |a| < P */
__device__ __forceinline__ void recon_step(hyk::I192& a, uint32_t r, const ReconTable& tab, int x) {
  const uint32_t tt = hyk::reduce_u32(r * tab.minv[x], tab.m[x], tab.d[x]);
  hyk::I192 pd; pd.w[0] = tab.Pd[x][0]; pd.w[1] = tab.Pd[x][1]; pd.w[2] = tab.Pd[x][2];
  if (hyk::i192_is_neg(a)) { hyk::i192_add(a, hyk::i192_mul_small(pd, tt)); }
  else { hyk::i192_add(a, hyk::i192_neg(hyk::i192_mul_small(pd, tab.m[x] - tt))); }
}
/* into [-P/2, P/2), then C (+)= a */
__device__ __forceinline__ void recon_finish(hyk::I192 a, const ReconTable& tab, int32_t beta, int32_t orderC, uint64_t* out, int64_t count) {
  hyk::I192 P; P.w[0] = tab.P[0]; P.w[1] = tab.P[1]; P.w[2] = tab.P[2];
  if (hyk::i192_is_neg(a)) { hyk::i192_add(a, P); }
  hyk::I192 twice = a; hyk::i192_add(twice, a); hyk::I192 diff = twice; hyk::i192_add(diff, hyk::i192_neg(P));
  if (!hyk::i192_is_neg(diff)) { hyk::i192_add(a, hyk::i192_neg(P)); }   /* 2a >= P  ->  a - P */
  if (beta) { hyk::I192 old = hyk::limbs_to_i192(orderC, out, count); hyk::i192_add(a, old); }
  hyk::i192_to_limbs(a, orderC, out, count);
}

/* Entry e: residues from the uint32 sums of its planes (real: plane x; complex: planes x and order + x), centred CRT
 * lift, C (+)= value; the sums are zeroed afterwards.  The rotating moduli of a complex launch arrive as p = W[y, x] and
 * q = W[x, y] of W = P^T Q (one plane each, each written by one group of the contraction): Re = (p + q) / 2,
 * Im = (p - q) / (2 i) mod m are formed here (the reference's accumulate_crt_rotate, src/crt_rotate.cu:5-46, does it
 * in the epilogue of its GEMM). */
__global__ __launch_bounds__(256) void crt_reconstruct_kernel(const ReconTable tab, int64_t count, uint32_t* __restrict__ acc, int64_t planeStride, int32_t beta, int32_t orderC, uint64_t* __restrict__ C, int32_t cplx) {
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= count) { return; }
  hyk::I192 re, im; re.w[0] = re.w[1] = re.w[2] = 0; im = re;
  for (int x = 0; x < tab.order; ++x) {
    uint32_t* s0 = &acc[(int64_t)x * planeStride + e];
    uint32_t r0 = hyk::reduce_u32(*s0, tab.m[x], tab.d[x]); *s0 = 0u;
    if (cplx) {
      uint32_t* s1 = &acc[(int64_t)(tab.order + x) * planeStride + e];
      uint32_t r1 = hyk::reduce_u32(*s1, tab.m[x], tab.d[x]); *s1 = 0u;
      if (x < tab.rot) {
        const uint32_t m = tab.m[x], sum = r0 + r1, dif = r0 + m - r1;
        r0 = hyk::reduce_u32(hyk::reduce_u32(sum, m, tab.d[x]) * ((m + 1u) >> 1), m, tab.d[x]);
        r1 = hyk::reduce_u32(hyk::reduce_u32(dif, m, tab.d[x]) * tab.iminv[x], m, tab.d[x]);
      }
      recon_step(im, r1, tab, x);
    }
    recon_step(re, r0, tab, x);
  }
  recon_finish(re, tab, beta, orderC, &C[e], count);
  if (cplx) { recon_finish(im, tab, beta, orderC, &C[(int64_t)orderC * count + e], count); }
}

/* limb path: C (+)= sum_s T_s 2^(8 s) */
__global__ __launch_bounds__(256) void limb_combine_kernel(int64_t count, int32_t levels, unsigned long long* __restrict__ acc, int64_t planeStride, int32_t beta, int32_t orderC, uint64_t* __restrict__ C, int32_t clear) {
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; const int z = blockIdx.y;
  if (e >= count) { return; }
  hyk::I192 a; a.w[0] = a.w[1] = a.w[2] = 0;
  for (int s = 0; s < levels; ++s) {
    unsigned long long* src = &acc[(int64_t)(z * levels + s) * planeStride + e];
    const int64_t v = (int64_t)*src; if (clear) { *src = 0ull; }
    hyk::i192_add_shifted_i64(a, v, 8u * (uint32_t)s);
  }
  uint64_t* out = &C[(int64_t)z * orderC * count + e];
  if (beta) { hyk::I192 old = hyk::limbs_to_i192(orderC, out, count); hyk::i192_add(a, old); }
  hyk::i192_to_limbs(a, orderC, out, count);
}

__global__ void fill_zero_kernel(uint4* __restrict__ p, int64_t n16) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; if (i < n16) { p[i] = make_uint4(0, 0, 0, 0); }
}

/* ------------------------------------------------------------------ host-side planning */
struct Launch { GramArgs args; int epi; };

/* Tuning and measuring state is per host thread: a setting made on one thread never changes what another thread's calls
 * launch, and nothing here is shared between threads. */
thread_local int g_bk = 0;   /* 0: direct-to-LDS ring of 128-byte rows (default); 2: direct-to-LDS ring of 64-byte rows; 64 / 128: register-staged kernel with that K slab (hykGramSetSlab) */

/* optional per-launch timing of the contraction kernel with HIP events on its own stream */
struct Timed { hipEvent_t start, stop; };
thread_local bool g_profile = false; thread_local std::vector<Timed> g_timed;

template <int BK, int EPI> hipError_t launch_one(hipStream_t stream, const GramArgs& a) {
  const int ldsBytes = 2 * 2 * Slab<BK>::TILE_BYTES;
  static std::atomic<bool> attr{ false };   /* two threads arriving together both set the attribute: harmless */
  if (!attr.load(std::memory_order_acquire)) { hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gram_kernel<BK, EPI>), hipFuncAttributeMaxDynamicSharedMemorySize, ldsBytes); if (e != hipSuccess) { return e; } attr.store(true, std::memory_order_release); }
  const int blocks = a.itemsPerXcd * XCDS;
  Timed t{ nullptr, nullptr };
  if (g_profile) { if (hipEventCreate(&t.start) != hipSuccess || hipEventCreate(&t.stop) != hipSuccess) { return hipErrorUnknown; } (void)hipEventRecord(t.start, stream); }
  gram_kernel<BK, EPI><<<blocks, G_THREADS, ldsBytes, stream>>>(a);
  if (g_profile) { (void)hipEventRecord(t.stop, stream); g_timed.push_back(t); }
  return hipGetLastError();
}

template <int EPI, bool EXCL> hipError_t launch_dma(hipStream_t stream, const GramArgs& a) {
  const int ldsBytes = DMA_STAGES * DMA_STAGE_BYTES;
  static std::atomic<bool> attr{ false };   /* two threads arriving together both set the attribute: harmless */
  if (!attr.load(std::memory_order_acquire)) { hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gram_dma_kernel<EPI, EXCL>), hipFuncAttributeMaxDynamicSharedMemorySize, ldsBytes); if (e != hipSuccess) { return e; } attr.store(true, std::memory_order_release); }
  const int blocks = a.itemsPerXcd * XCDS;
  Timed t{ nullptr, nullptr };
  if (g_profile) { if (hipEventCreate(&t.start) != hipSuccess || hipEventCreate(&t.stop) != hipSuccess) { return hipErrorUnknown; } (void)hipEventRecord(t.start, stream); }
  gram_dma_kernel<EPI, EXCL><<<blocks, G_THREADS, ldsBytes, stream>>>(a);
  if (g_profile) { (void)hipEventRecord(t.stop, stream); g_timed.push_back(t); }
  return hipGetLastError();
}

template <int EPI, bool EXCL> hipError_t launch_ring(hipStream_t stream, const GramArgs& a) {
  static std::atomic<bool> attr{ false };   /* two threads arriving together both set the attribute: harmless */
  if (!attr.load(std::memory_order_acquire)) { hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gram_ring_kernel<EPI, EXCL>), hipFuncAttributeMaxDynamicSharedMemorySize, RING_BYTES); if (e != hipSuccess) { return e; } attr.store(true, std::memory_order_release); }
  const int blocks = XCDS * a.roundsPerXcd * (1 << a.slotShift);
  Timed t{ nullptr, nullptr };
  if (g_profile) { if (hipEventCreate(&t.start) != hipSuccess || hipEventCreate(&t.stop) != hipSuccess) { return hipErrorUnknown; } (void)hipEventRecord(t.start, stream); }
  gram_ring_kernel<EPI, EXCL><<<blocks, G_THREADS, RING_BYTES, stream>>>(a);
  if (g_profile) { (void)hipEventRecord(t.stop, stream); g_timed.push_back(t); }
  return hipGetLastError();
}

int compute_units() {   /* of the device current on this thread */
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0) { return n; }
  return 256;
}

hipError_t launch_gram(hipStream_t stream, GramArgs& a, int epi, int maxProducts, bool unshared, bool paired) {
  /* the ring kernel addresses the 256 rows of a tile with 32-bit byte offsets: longer rows go to the register-staged kernel */
  const int mode = (g_bk == 0 && 255ll * a.ldb + RING_K > 0xffffffffll) ? 128 : g_bk;
  int maxPairs = 1; for (int g = 0; g < a.groupCount; ++g) { maxPairs = a.groups[g].pairCount > maxPairs ? a.groups[g].pairCount : maxPairs; }
  const int bk = mode == 0 ? RING_K : (mode == 2 ? DMA_BK : mode); int kCap = (maxProducts / maxPairs) / bk * bk; if (kCap < bk) { return hipErrorInvalidValue; }
  /* K split.  One workgroup runs per compute unit, so a launch takes rounds = ceil(items / units) item times; an item costs
   * its K range plus a fixed prologue / epilogue (65536 reductions and atomics) worth about 48 x 64 K-bytes of it.  Take
   * the split count that minimises rounds x (K range + epilogue); the cap keeps the int32 sums exact. */
  const int64_t base = (int64_t)a.groupCount * a.tileCount; const int units = compute_units();
  const int minSplits = (a.K + kCap - 1) / kCap; int splits = minSplits; double best = -1.;
  for (int cand = minSplits; cand <= minSplits + 15; ++cand) {
    const int len = ((a.K + cand - 1) / cand + bk - 1) / bk * bk; if (len < 16 * bk && cand > minSplits) { break; }
    const int count = (a.K + len - 1) / len; int64_t rounds = (base * count + units - 1) / units;
    if (mode == 0) {   /* the ring kernel's schedule hands out whole rounds of an XCD (set-aligned rounds, below) */
      const int slots = units / XCDS >= 32 ? 32 : (units / XCDS >= 16 ? 16 : (units / XCDS >= 8 ? 8 : 1)), shift = (paired && (a.groupCount & 1) == 0) ? 1 : 0;
      const int setTiles = a.tileCount << shift; const int64_t sets = (int64_t)(a.groupCount >> shift) * count; const int left = setTiles % slots, per = left ? slots / left : 0;
      rounds = (sets * (setTiles / slots) + (left ? (sets + per - 1) / per : 0) + XCDS - 1) / XCDS;
    }
    const double cost = (double)rounds * ((double)len / 64. + 48.);   /* in units of 64 K-bytes of contraction */
    if (best < 0. || cost < best * 0.98) { best = cost; splits = cand; }   /* a further split has to win by 2 % */
  }
  int kLen = ((a.K + splits - 1) / splits + bk - 1) / bk * bk; if (kLen > kCap) { kLen = kCap; }
  if (kLen > a.K) { kLen = a.K; }
  a.kLen = kLen; a.kSplits = (a.K + kLen - 1) / kLen; a.exclusive = (unshared && a.kSplits == 1 && (mode == 0 || mode == 2)) ? 1 : 0;
  const int64_t total = base * a.kSplits; if (total > 0x7fffffff / 2) { return hipErrorInvalidValue; }
  a.totalItems = (int)total; a.itemsPerXcd = (int)((total + XCDS - 1) / XCDS);
  if (total * a.tileCount >= (1ll << 32) || total * a.kSplits >= (1ll << 32)) { return hipErrorInvalidValue; }
  a.tileMagic = a.tileCount > 1 ? (uint32_t)((1ull << 32) / (uint32_t)a.tileCount) + 1u : 0u; a.splitMagic = a.kSplits > 1 ? (uint32_t)((1ull << 32) / (uint32_t)a.kSplits) + 1u : 0u;
  if (mode == 0) {
    /* set-aligned schedule; compute units per XCD rounded down to a power of two (32 on this device) */
    int slots = units / XCDS; a.slotShift = 0; while ((2 << a.slotShift) <= slots) { ++a.slotShift; } slots = 1 << a.slotShift;
    a.pairShift = (paired && (a.groupCount & 1) == 0) ? 1 : 0; const int setTiles = a.tileCount << a.pairShift;
    a.setCount = (a.groupCount >> a.pairShift) * a.kSplits; a.mainRounds = setTiles / slots; a.leftover = setTiles % slots; a.perRound = a.leftover ? slots / a.leftover : 0;
    const int rounds = a.setCount * a.mainRounds + (a.leftover ? (a.setCount + a.perRound - 1) / a.perRound : 0);
    a.roundsPerXcd = (rounds + XCDS - 1) / XCDS;
    a.mainMagic = a.mainRounds > 1 ? (uint32_t)((1ull << 32) / (uint32_t)a.mainRounds) + 1u : 0u; a.leftMagic = a.leftover > 1 ? (uint32_t)((1ull << 32) / (uint32_t)a.leftover) + 1u : 0u;
    if ((int64_t)rounds * a.mainRounds >= (1ll << 31) || (int64_t)a.setCount * a.kSplits >= (1ll << 31)) { return hipErrorInvalidValue; }
    if (a.exclusive) { return epi == EPI_MOD ? launch_ring<EPI_MOD, true>(stream, a) : launch_ring<EPI_I64, true>(stream, a); }
    return epi == EPI_MOD ? launch_ring<EPI_MOD, false>(stream, a) : launch_ring<EPI_I64, false>(stream, a);
  }
  if (mode == 2) {
    if (a.exclusive) { return epi == EPI_MOD ? launch_dma<EPI_MOD, true>(stream, a) : launch_dma<EPI_I64, true>(stream, a); }
    return epi == EPI_MOD ? launch_dma<EPI_MOD, false>(stream, a) : launch_dma<EPI_I64, false>(stream, a);
  }
  if (bk == 128) { return epi == EPI_MOD ? launch_one<128, EPI_MOD>(stream, a) : launch_one<128, EPI_I64>(stream, a); }
  return epi == EPI_MOD ? launch_one<64, EPI_MOD>(stream, a) : launch_one<64, EPI_I64>(stream, a);
}

void base_args(GramArgs& a, const int8_t* panels, int64_t ldb, int32_t N, int32_t K, void* acc) {
  a.panels = panels; a.ldb = ldb; a.panelStride = (int64_t)N * ldb; a.acc = acc; a.planeStride = ((int64_t)N * N + N) / 2;
  a.N = N; a.nT = (N + TILE - 1) / TILE; a.tileCount = a.nT * (a.nT + 1) / 2; a.K = K; a.groupCount = 0;
}

struct GroupBuilder {
  GramArgs a; int pairs = 0; int epi; int maxProducts; bool unshared; bool paired = false; hipStream_t stream; hipError_t err = hipSuccess;
  /* paired: groups come in adjacent pairs that read the same two panels (set by the caller before the first group) */
  /* unshared: no two groups write the same accumulator plane (true for the real paths) */
  GroupBuilder(hipStream_t s, int epi_, int maxProducts_, bool unshared_, const int8_t* panels, int64_t ldb, int32_t N, int32_t K, void* acc) : epi(epi_), maxProducts(maxProducts_), unshared(unshared_), stream(s) { base_args(a, panels, ldb, N, K, acc); }
  void flush() { if (a.groupCount > 0 && err == hipSuccess) { err = launch_gram(stream, a, epi, maxProducts, unshared, paired); } a.groupCount = 0; pairs = 0; }
  /* begins a group; flushes first when the tables are full */
  GramGroup& begin(int npairs) {
    if (a.groupCount == MAX_GROUPS || pairs + npairs > MAX_PAIRS) { flush(); }
    GramGroup& g = a.groups[a.groupCount++]; g.pairBegin = (uint16_t)pairs; g.pairCount = 0; g.planeRe = g.planeIm = 0; g.m = 1; g.d = 0; g.c32 = 0; g.mulRe = g.mulIm = 0; return g;
  }
  void pair(GramGroup& g, int lanePanel, int aPanel) { a.pairs[pairs] = (uint32_t)lanePanel | ((uint32_t)aPanel << 16); ++pairs; ++g.pairCount; }
};

void set_mod(GramGroup& g, uint32_t m) { g.m = m; g.d = (uint32_t)(0x100000000ull / m); g.c32 = (uint32_t)(0x100000000ull % m); }

hipError_t zero_fill(hipStream_t stream, void* p, size_t bytes) {
  const int64_t n16 = (int64_t)((bytes + 15) / 16); if (n16 == 0) { return hipSuccess; }
  fill_zero_kernel<<<(uint32_t)((n16 + 255) / 256), 256, 0, stream>>>(reinterpret_cast<uint4*>(p), n16); return hipGetLastError();
}

}  // namespace

extern "C" int hykGramProfile(int32_t enable) {
  for (Timed& t : g_timed) { (void)hipEventDestroy(t.start); (void)hipEventDestroy(t.stop); } g_timed.clear(); g_profile = enable != 0; return 0;
}

/* total milliseconds and number of contraction-kernel launches since hykGramProfile(1); waits for them to finish */
extern "C" int hykGramProfileRead(double* totalMs, int32_t* launches) {
  double sum = 0.; for (Timed& t : g_timed) { if (hipEventSynchronize(t.stop) != hipSuccess) { return -3; } float ms = 0.f; if (hipEventElapsedTime(&ms, t.start, t.stop) != hipSuccess) { return -3; } sum += ms; }
  if (totalMs) { *totalMs = sum; } if (launches) { *launches = (int32_t)g_timed.size(); } return 0;
}

/* Register-only MFMA loop: what the matrix cores sustain on this device when nothing else competes for power.  Every lane
 * holds eight int8 operand fragments (hashed lane / block indices when `random`, zeros otherwise) and issues the same
 * 4x4 pattern of v_mfma_i32_32x32x32_i8 as the contraction kernel; block 0 reports its shader-clock and wall-clock spans. */
__global__ __launch_bounds__(G_THREADS, 1) void mfma_ceiling_kernel(int iters, int random, int* sink, long long* clocks) {
  v4i a[4], b[4];
  #pragma unroll
  for (int i = 0; i < 4; ++i) {
    #pragma unroll
    for (int c = 0; c < 4; ++c) {
      uint32_t h = (uint32_t)(threadIdx.x * 8 + i) * 2654435761u + (uint32_t)(blockIdx.x * 4 + c) * 40503u; h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
      a[i][c] = random ? (int)h : 0; b[i][c] = random ? (int)(h * 3266489917u + 0x9e3779b9u) : 0;
    }
  }
  v16i acc[4][4];
  #pragma unroll
  for (int i = 0; i < 4; ++i) {
    #pragma unroll
    for (int j = 0; j < 4; ++j) {
      #pragma unroll
      for (int r = 0; r < 16; ++r) { acc[i][j][r] = 0; }
    }
  }
  const long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
    #pragma unroll
    for (int i = 0; i < 4; ++i) {
      #pragma unroll
      for (int j = 0; j < 4; ++j) { acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i][j], 0, 0, 0); }
    }
  }
  const long long c1 = clock64(), w1 = wall_clock64();
  int sum = 0;
  #pragma unroll
  for (int i = 0; i < 4; ++i) {
    #pragma unroll
    for (int j = 0; j < 4; ++j) {
      #pragma unroll
      for (int r = 0; r < 16; ++r) { sum += acc[i][j][r]; }
    }
  }
  sink[blockIdx.x * G_THREADS + threadIdx.x] = sum;
  if (threadIdx.x == 0 && blockIdx.x == 0) { clocks[0] = c1 - c0; clocks[1] = w1 - w0; }
}

/* Measurement hook (no counterpart in the reference).  Runs the register-only MFMA loop on `blocks` workgroups (one per
 * compute unit is the natural choice) and reports int8 tera-ops per second and the shader clock it ran at.  Allocates and
 * frees its own small buffers and synchronises the stream. */
extern "C" int hykMfmaCeiling(hipStream_t stream, int32_t blocks, int32_t iters, int32_t random, double* teraOps, double* clockGHz) {
  if (blocks <= 0 || iters <= 0) { return -1; }
  int* sink = nullptr; long long* clocks = nullptr; hipEvent_t e0 = nullptr, e1 = nullptr; int rc = -3;
  if (hipMalloc(&sink, (size_t)blocks * G_THREADS * sizeof(int)) == hipSuccess && hipMalloc(&clocks, 2 * sizeof(long long)) == hipSuccess &&
      hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess) {
    mfma_ceiling_kernel<<<blocks, G_THREADS, 0, stream>>>(iters / 8 + 1, random, sink, clocks);   /* warm-up, lets the clock settle */
    (void)hipEventRecord(e0, stream);
    mfma_ceiling_kernel<<<blocks, G_THREADS, 0, stream>>>(iters, random, sink, clocks);
    (void)hipEventRecord(e1, stream);
    long long h[2] = { 0, 1 }; float ms = 0.f;
    if (hipEventSynchronize(e1) == hipSuccess && hipEventElapsedTime(&ms, e0, e1) == hipSuccess && hipMemcpy(h, clocks, sizeof(h), hipMemcpyDeviceToHost) == hipSuccess && ms > 0.f) {
      if (teraOps) { *teraOps = (double)blocks * 4. * (double)iters * 16. * 65536. / ((double)ms * 1e-3) / 1e12; }
      if (clockGHz) { *clockGHz = h[1] > 0 ? (double)h[0] / (double)h[1] * 0.1 : 0.; }   /* wall clock counts at 100 MHz */
      rc = 0;
    }
  }
  if (e0) { (void)hipEventDestroy(e0); } if (e1) { (void)hipEventDestroy(e1); } if (sink) { (void)hipFree(sink); } if (clocks) { (void)hipFree(clocks); }
  return rc;
}

extern "C" int hykGramSetSlab(int32_t bk) { if (bk != 0 && bk != 2 && bk != 64 && bk != 128) { return -1; } g_bk = bk; return 0; }

extern "C" size_t hykGramWorkspaceBytes(int32_t kind, int32_t Complex, int32_t N, int32_t orderA) {
  if (N <= 0 || orderA <= 0) { return 0; }
  const size_t T = ((size_t)N * (size_t)N + (size_t)N) / 2, planes = (size_t)(Complex ? 2 : 1);
  size_t bytes = (kind == HYK_GRAM_LIMBS) ? planes * (size_t)(2 * orderA - 1) * T * 8 : planes * (size_t)orderA * T * 4;
  return (bytes + 255) / 256 * 256;
}

/* Workspace must be zero on entry (hykGramWorkspaceClear) and is zero again on return. */
extern "C" int hykGramWorkspaceClear(hipStream_t stream, void* workspace, size_t bytes) { return zero_fill(stream, workspace, bytes) == hipSuccess ? 0 : -3; }

extern "C" int hykGramCrt(hipStream_t stream, int32_t Complex, int32_t N, int32_t orderA, const int8_t* panels, int64_t ldb, int32_t K, int32_t beta, int32_t orderC, uint64_t* C, void* workspace) {
  if (N <= 0) { return 0; }
  if (orderA < 1 || orderA > (Complex ? HYK_CRT_CPLX_COUNT : HYK_CRT_REAL_COUNT) || orderC < 1 || orderC > 3 || K <= 0 || (K & 127) || ldb < K || (ldb & 15) || ((uintptr_t)panels & 15)) { return -1; }
  /* 131072 products per int32: residues of every modulus but 256 are at most 125 in magnitude, and mod 256 a wrap is harmless */
  /* planes are shared between groups only by the three-product moduli of a complex launch */
  GroupBuilder gb(stream, EPI_MOD, 131072, Complex == 0 || orderA <= HYK_CRT_CPLX_SPLIT, panels, ldb, N, K, workspace);
  ReconTable tab; tab.order = orderA; tab.rot = 0;
  gb.paired = Complex != 0 && orderA <= HYK_CRT_CPLX_SPLIT;
  if (!Complex) {
    for (int x = 0; x < orderA; ++x) { GramGroup& g = gb.begin(1); set_mod(g, hyk_crt_real_mo[x]); g.mulRe = 1; g.planeRe = (uint16_t)x; gb.pair(g, x, x); }
    for (int x = 0; x < orderA; ++x) { tab.m[x] = hyk_crt_real_mo[x]; tab.d[x] = (uint32_t)(0x100000000ull / tab.m[x]); tab.minv[x] = hyk_crt_real_minv[orderA - 1][x]; for (int k = 0; k < 3; ++k) { tab.Pd[x][k] = hyk_crt_real_Pd[orderA - 1][x][k]; } }
    for (int k = 0; k < 3; ++k) { tab.P[k] = hyk_crt_real_P[orderA - 1][k]; }
  } else {
    const int rot = orderA < HYK_CRT_CPLX_SPLIT ? orderA : HYK_CRT_CPLX_SPLIT;
    for (int x = 0; x < rot; ++x) {
      /* W = P^T Q: elements on or above the diagonal are p = Re + i Im, the transposed ones q = Re - i Im (mod m).  Each
       * goes to a plane of its own (p: plane x, q: plane orderA + x), so every accumulator entry has one writer and the
       * contraction can store instead of adding atomically; the reconstruction forms Re = (p + q)/2, Im = (p - q)/(2 i). */
      const uint32_t m = hyk_crt_cplx_mo[x];
      GramGroup& g0 = gb.begin(1); set_mod(g0, m); g0.mulRe = 1; g0.planeRe = (uint16_t)x; gb.pair(g0, 2 * x, 2 * x + 1);
      GramGroup& g1 = gb.begin(1); set_mod(g1, m); g1.mulRe = 1; g1.planeRe = (uint16_t)(orderA + x); gb.pair(g1, 2 * x + 1, 2 * x);
    }
    for (int x = HYK_CRT_CPLX_SPLIT; x < orderA; ++x) {
      /* 3M scheme mod m: Re = S^T S - (R^T I + I^T R), Im = R^T I - I^T R with S = R + I */
      const uint32_t m = hyk_crt_cplx_mo[x]; const int base = 2 * HYK_CRT_CPLX_SPLIT + 3 * (x - HYK_CRT_CPLX_SPLIT);
      GramGroup& gs = gb.begin(1); set_mod(gs, m); gs.mulRe = 1; gs.planeRe = (uint16_t)x; gb.pair(gs, base, base);
      GramGroup& g0 = gb.begin(1); set_mod(g0, m); g0.mulRe = m - 1; g0.mulIm = 1; g0.planeRe = (uint16_t)x; g0.planeIm = (uint16_t)(orderA + x); gb.pair(g0, base + 1, base + 2);
      GramGroup& g1 = gb.begin(1); set_mod(g1, m); g1.mulRe = m - 1; g1.mulIm = m - 1; g1.planeRe = (uint16_t)x; g1.planeIm = (uint16_t)(orderA + x); gb.pair(g1, base + 2, base + 1);
    }
    tab.rot = rot;
    for (int x = 0; x < orderA; ++x) { tab.m[x] = hyk_crt_cplx_mo[x]; tab.d[x] = (uint32_t)(0x100000000ull / tab.m[x]); tab.minv[x] = hyk_crt_cplx_minv[orderA - 1][x]; tab.iminv[x] = x < HYK_CRT_CPLX_SPLIT ? hyk_crt_cplx_iminv[x] : 0u; for (int k = 0; k < 3; ++k) { tab.Pd[x][k] = hyk_crt_cplx_Pd[orderA - 1][x][k]; } }
    for (int k = 0; k < 3; ++k) { tab.P[k] = hyk_crt_cplx_P[orderA - 1][k]; }
  }
  gb.flush(); if (gb.err != hipSuccess) { return -3; }
  const int64_t T = ((int64_t)N * N + N) / 2;
  crt_reconstruct_kernel<<<(uint32_t)((T + 255) / 256), 256, 0, stream>>>(tab, T, reinterpret_cast<uint32_t*>(workspace), T, beta, orderC, C, Complex ? 1 : 0);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}

extern "C" int hykGramLimbs(hipStream_t stream, int32_t Complex, int32_t N, int32_t orderA, const int8_t* panels, int64_t ldb, int32_t K, int32_t beta, int32_t orderC, uint64_t* C, void* workspace) {
  if (N <= 0) { return 0; }
  if (orderA < 1 || orderA > 12 || orderC < 1 || orderC > 3 || K <= 0 || (K & 127) || ldb < K || (ldb & 15) || ((uintptr_t)panels & 15)) { return -1; }
  const int levels = 2 * orderA - 1;
  /* 131071 products of magnitude <= 2^14 fit an int32 */
  GroupBuilder gb(stream, EPI_I64, 131071, Complex == 0, panels, ldb, N, K, workspace);
  /* heaviest levels first so the tail of the launch is made of short items */
  for (int cnt = orderA; cnt >= 1; --cnt) for (int s = 0; s < levels; ++s) {
    const int lo = s < orderA ? 0 : s - orderA + 1, hi = s < orderA ? s : orderA - 1; if (hi - lo + 1 != cnt) { continue; }
    /* digits group 0 (real input: the only one; complex input: re + im): T_s = sum_{i+j=s} A_i^T A_j, upper triangle */
    GramGroup& g = gb.begin(cnt); g.mulRe = 1; g.planeRe = (uint16_t)s; for (int i = lo; i <= hi; ++i) { gb.pair(g, i, s - i); }
    if (Complex) {
      /* X_s = sum_{i+j=s} R_i^T I_j: Re -= X[y,x] + X[x,y], Im += X[y,x] - X[x,y] (3M scheme) */
      GramGroup& g0 = gb.begin(cnt); g0.mulRe = 2; g0.mulIm = 1; g0.planeRe = (uint16_t)s; g0.planeIm = (uint16_t)(levels + s); for (int i = lo; i <= hi; ++i) { gb.pair(g0, orderA + i, 2 * orderA + (s - i)); }
      GramGroup& g1 = gb.begin(cnt); g1.mulRe = 2; g1.mulIm = 2; g1.planeRe = (uint16_t)s; g1.planeIm = (uint16_t)(levels + s); for (int i = lo; i <= hi; ++i) { gb.pair(g1, 2 * orderA + (s - i), orderA + i); }
    }
  }
  gb.flush(); if (gb.err != hipSuccess) { return -3; }
  const int64_t T = ((int64_t)N * N + N) / 2; dim3 grid((uint32_t)((T + 255) / 256), Complex ? 2u : 1u);
  limb_combine_kernel<<<grid, 256, 0, stream>>>(T, levels, reinterpret_cast<unsigned long long*>(workspace), T, beta, orderC, C, 1);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
