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

/* Failure handling.  A failed runtime call, allocation or kernel-layer call is reported on stderr and recorded as the
 * status of the hyacin.h call that is running on this thread; from then on that call launches nothing more (HYH_KERNEL
 * skips its argument), frees what it holds and returns 0 / leaves its outputs as they are.  The status of the last
 * outermost call stays readable through hykLastStatus() until the thread's next hyacin.h call. */
struct CallStatus { int code = 0; int depth = 0; };
CallStatus& call_status();
inline bool ok() { return call_status().code == 0; }
void fail(int code, const char* what, const char* detail, const char* file, int line);
struct ApiScope {   /* first statement of every hyacin.h function: the outermost one starts with a clean status */
  ApiScope() { CallStatus& s = call_status(); if (s.depth++ == 0) { s.code = 0; } }
  ~ApiScope() { --call_status().depth; }
  ApiScope(const ApiScope&) = delete; ApiScope& operator=(const ApiScope&) = delete;
};
#define HYH_CHECK(call) do { hipError_t hyh_e_ = (call); if (hyh_e_ != hipSuccess) { hyh::fail((int)hyh_e_, #call, hipGetErrorString(hyh_e_), __FILE__, __LINE__); } } while (0)
#define HYH_KERNEL(call) do { if (hyh::ok()) { int hyh_r_ = (call); if (hyh_r_ != 0) { hyh::fail(hyh_r_, #call, "kernel layer refused or failed to launch", __FILE__, __LINE__); } } } while (0)

inline bool is_complex(int t) { return (t & 1) != 0; }
inline int elem_bytes(int t) { static const int b[12] = { 8, 16, 4, 8, 2, 4, 16, 32, 12, 24, 16, 32 }; return (t >= 0 && t < 12) ? b[t] : 0; }

/* Stream-ordered scratch from the handle's pool (reference: cudaMallocFromPoolAsync / cudaFreeAsync throughout).
 * When the handle owns its pool, blocks are kept and reused instead of being returned after every call: the runtime's
 * pool calls cost up to a millisecond each for multi-gigabyte blocks, more than the kernels between them.  The work of a
 * handle is ordered on its stream, so a reused block is never touched by two calls at once; a block that was last used on
 * another stream (the caller has changed handle->hipStream) is handed out after a device-wide wait.  hyacinDestroy frees them. */
void* scratch_acquire(const hyacinHandle_t* h, size_t bytes, bool* kept);
void scratch_release(const hyacinHandle_t* h, void* p, bool kept);
void scratch_drop_all(const hyacinHandle_t* h);
struct Scratch {
  const hyacinHandle_t* h; void* p = nullptr; bool kept = false;
  Scratch(const hyacinHandle_t* h_, size_t bytes) : h(h_) {
    if (bytes && ok()) { p = scratch_acquire(h, bytes, &kept); if (!p) { fail(-4, "scratch allocation", "the memory pool returned no block", __FILE__, __LINE__); } }
  }
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

/* the Gram stages with the storage order of A as an argument ('N' column-major M x N; 'T' / 'C' the stored N x M transpose) */
void quantize_scale_batch(const hyacinHandle_t* h, char op, int32_t batches, int32_t segM, int32_t lastM, int32_t N, int Atype, const void* A, int64_t lda, int32_t uA, int32_t* vexp);
void herk_batch(const hyacinHandle_t* h, char op, int32_t batches, int32_t segM, int32_t lastM, int32_t N, int Atype, const void* A, int64_t lda, int32_t u, const int32_t* vexp, int32_t beta, int32_t orderC, uint64_t* C);

inline int32_t round_up(int32_t v, int32_t a) { return (v + a - 1) / a * a; }

}  // namespace hyh
