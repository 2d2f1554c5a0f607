/* Host-side helpers shared by the C++ drivers of the hyacin.h API. */
#pragma once
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <algorithm>
#include <utility>
#include <vector>
#include <hip/hip_runtime_api.h>
#include "hyacin.h"
#include "hyacin_kernels.h"

namespace hyh {

/* A failed runtime call or kernel launch is reported on stderr once per call site and the call chain carries on,
 * like the reference's release build; silent wrong answers are worse than noise. */
#define HYH_CHECK(call) do { hipError_t hyh_e_ = (call); if (hyh_e_ != hipSuccess) { std::fprintf(stderr, "hyacin: %s failed: %s (%s:%d)\n", #call, hipGetErrorString(hyh_e_), __FILE__, __LINE__); } } while (0)
#define HYH_KERNEL(call) do { int hyh_r_ = (call); if (hyh_r_ != 0) { std::fprintf(stderr, "hyacin: %s returned %d (%s:%d)\n", #call, hyh_r_, __FILE__, __LINE__); } } while (0)

inline bool is_complex(int t) { return (t & 1) != 0; }
inline int elem_bytes(int t) { static const int b[12] = { 8, 16, 4, 8, 2, 4, 16, 32, 12, 24, 16, 32 }; return (t >= 0 && t < 12) ? b[t] : 0; }

/* Stream-ordered scratch from the handle's pool (reference: cudaMallocFromPoolAsync / cudaFreeAsync throughout).
 * When the handle owns its pool, blocks are kept and reused instead of being returned after every call: the runtime's
 * pool calls cost up to a millisecond each for multi-gigabyte blocks, more than the kernels between them.  All work of a
 * handle is ordered on its one stream, so a reused block is never touched by two calls at once.  hyacinDestroy frees them. */
void* scratch_acquire(const hyacinHandle_t* h, size_t bytes, bool* kept);
void scratch_release(const hyacinHandle_t* h, void* p, bool kept);
void scratch_drop_all(const hyacinHandle_t* h);
struct Scratch {
  const hyacinHandle_t* h; void* p = nullptr; bool kept = false;
  Scratch(const hyacinHandle_t* h_, size_t bytes) : h(h_) { if (bytes) { p = scratch_acquire(h, bytes, &kept); } }
  ~Scratch() { if (p) { scratch_release(h, p, kept); } }
  Scratch(const Scratch&) = delete; Scratch& operator=(const Scratch&) = delete;
  template <typename T> T* as() const { return reinterpret_cast<T*>(p); }
};

/* segment timer (reference: src/utils.cpp:39-43,103-114) */
enum class Segment : unsigned char { untimed, dist_kernel, rep_kernel, comm };
void timer_mark(const hyacinHandle_t* h, Segment s);

/* planner (reference: src/hyacin_herk.cpp:11-43) */
struct GramPlan { char alg; int32_t order; int32_t second; };  /* second: limb capacity in bits ('L') or rows per CRT chunk ('C') */
GramPlan gram_algorithm(char alg, int32_t K, int32_t u, int32_t Complex, int32_t segmentK, double batchPenalty);

inline int32_t round_up(int32_t v, int32_t a) { return (v + a - 1) / a * a; }

}  // namespace hyh
