/*
 * handle.cpp -- handle lifecycle, environment configuration and the segment timer.
 * Mirrors the reference's src/utils.cpp: hyacinCreate (:56-90), hyacinDestroy (:92-101),
 * register_event (:103-114), hyacinSync_TimerSegments (:116-141).
 *
 * The library needs no vendor BLAS / solver: the rocblasHandle and solverHandle slots are
 * never created here and never used; a caller may leave them null or park its own there.
 */
#include <cstring>
#include <string>
#include <map>
#include <mutex>
#include <atomic>
#include "common.hpp"

namespace {

constexpr uint32_t OWNS_MEMPOOL = 0x4, OWNS_PINNED = 0x8, OWNS_TIMER = 0x10;   /* bit values of src/utils.cpp:45-49 */

struct EventTimer { std::vector<std::pair<hyh::Segment, hipEvent_t>> events; hyh::Segment last = hyh::Segment::untimed; };

/* blocks kept per handle-owned pool; `stream`: the stream whose work used the block last */
struct Block { void* p; size_t bytes; bool busy; hipStream_t stream; };
std::mutex g_keptMutex; std::map<hipMemPool_t, std::vector<Block>> g_kept;

thread_local int g_failAllocation = 0;   /* test hook: the n-th scratch acquisition of this host thread from now on fails */

bool env_get(const char* key, std::string& out) { const char* v = std::getenv(key); if (!v) { return false; } out = v; return true; }
bool env_true(const std::string& s) { return s == "1" || s == "true" || s == "True"; }

}  // namespace

extern "C" void hyacinCreate(hyacinHandle_t* handle) {
  hyh::ApiScope scope;
  if (!handle) { return; }
  HYH_CHECK(hipGetDevice(&handle->DeviceID));
  HYH_CHECK(hipDeviceGetAttribute(&handle->DeviceSMs, hipDeviceAttributeMultiprocessorCount, handle->DeviceID));
  handle->DeviceIsF64Capable = 1;   /* CDNA: full-rate FP64 vector and matrix units */

  std::string s;
  handle->GramMatrixAlgorithm = env_get("HYACIN_GRAM_ALGORITHM", s) && !s.empty() ? s[0] : 'A';
  handle->StrideBatchPerfPenalty = env_get("HYACIN_STRIDE_BATCH_PERF_PENALTY", s) ? std::atof(s.c_str()) : 1.3;
  handle->GramSegmentK = env_get("HYACIN_GRAM_SEGMENT_K", s) ? std::atoi(s.c_str()) : 8192;
  handle->TCGemmTargetK = env_get("HYACIN_TCGEMM_TARGET_K", s) ? std::atoi(s.c_str()) : 8192;
  handle->QuantizeBitCorrection = env_get("HYACIN_QUANTIZE_BITS_CORR", s) ? std::atoi(s.c_str()) : 7;
  handle->QRCPTruncateRank = env_get("HYACIN_QRCP_TRUNCATE_RANK", s) ? std::atoi(s.c_str()) : 1;
  handle->JacobiSVDSweeps = env_get("HYACIN_JACOBI_SVD_SWEEPS", s) ? std::atoi(s.c_str()) : 3;

  if (handle->mempool == nullptr) {
    hipMemPoolProps props; std::memset(&props, 0, sizeof(props));
    props.allocType = hipMemAllocationTypePinned; props.location.type = hipMemLocationTypeDevice; props.location.id = handle->DeviceID;
    hipMemPool_t pool = nullptr;
    if (hipMemPoolCreate(&pool, &props) == hipSuccess && pool) {
      uint64_t threshold = UINT64_MAX; HYH_CHECK(hipMemPoolSetAttribute(pool, hipMemPoolAttrReleaseThreshold, &threshold));
      handle->mempool = pool; handle->HandleOwnedResource |= OWNS_MEMPOOL;
    } else { (void)hipGetLastError(); HYH_CHECK(hipDeviceGetDefaultMemPool(&handle->mempool, handle->DeviceID)); }
  }
  if (handle->pinnedWorkspace == nullptr) { HYH_CHECK(hipHostMalloc(&handle->pinnedWorkspace, 64, hipHostMallocDefault)); handle->HandleOwnedResource |= OWNS_PINNED; }

  if (env_get("HYACIN_PLAIN_LAUNCH", s)) { (void)hykPotrfpSetPlainLaunch(env_true(s) ? 1 : 0); }   /* for runs under a kernel-tracing profiler */
  const bool timer = env_get("HYACIN_CREATE_TIMER", s) ? env_true(s) : false;
  if (timer && handle->timer == nullptr) { handle->timer = new EventTimer(); handle->HandleOwnedResource |= OWNS_TIMER; }
  const bool verbose = env_get("HYACIN_VERBOSE", s) ? env_true(s) : false;
  if (verbose && handle->logger == nullptr) { handle->logger = stdout; }
}

hyh::CallStatus& hyh::call_status() { static thread_local CallStatus s; return s; }

void hyh::fail(int code, const char* what, const char* detail, const char* file, int line) {
  std::fprintf(stderr, "hyacin: %s failed (%d: %s) at %s:%d\n", what, code, detail, file, line);
  CallStatus& s = call_status(); if (s.code == 0) { s.code = code ? code : -1; }
}

extern "C" int hykLastStatus(void) { return hyh::call_status().code; }
extern "C" int hykTestFailAllocation(int32_t nth) { g_failAllocation = nth > 0 ? nth : 0; return 0; }

void* hyh::scratch_acquire(const hyacinHandle_t* h, size_t bytes, bool* kept) {
  void* p = nullptr; *kept = false;
  if (g_failAllocation > 0 && g_failAllocation-- == 1) { return nullptr; }
  if ((h->HandleOwnedResource & OWNS_MEMPOOL) && h->mempool) {
    std::lock_guard<std::mutex> lock(g_keptMutex);
    std::vector<Block>& blocks = g_kept[h->mempool]; Block* best = nullptr;
    for (Block& b : blocks) { if (!b.busy && b.bytes >= bytes && b.bytes / 4 <= bytes && (!best || b.bytes < best->bytes)) { best = &b; } }
    if (best) {
      /* The caller may have put another stream into the handle since the block was last used (the fields may be edited
       * between calls).  Work queued on the old stream may still touch the block, and that stream may no longer exist, so
       * it cannot be waited on by name: the device is. */
      if (best->stream != h->hipStream) { HYH_CHECK(hipDeviceSynchronize()); best->stream = h->hipStream; }
      best->busy = true; *kept = true; return best->p;
    }
    if (blocks.size() >= 64) {   /* many different sizes have come by: return the idle ones to the pool */
      bool foreign = false; for (Block& b : blocks) { foreign = foreign || (!b.busy && b.stream != h->hipStream); }
      if (foreign) { HYH_CHECK(hipDeviceSynchronize()); }   /* a block last used on another stream is freed on this one */
      std::vector<Block> live; for (Block& b : blocks) { if (b.busy) { live.push_back(b); } else { HYH_CHECK(hipFreeAsync(b.p, h->hipStream)); } } blocks.swap(live);
    }
    const size_t rounded = (bytes + 255) / 256 * 256;
    HYH_CHECK(hipMallocFromPoolAsync(&p, rounded, h->mempool, h->hipStream));
    if (p) { blocks.push_back(Block{ p, rounded, true, h->hipStream }); *kept = true; }
    return p;
  }
  HYH_CHECK(hipMallocFromPoolAsync(&p, bytes, h->mempool, h->hipStream));
  return p;
}

void hyh::scratch_release(const hyacinHandle_t* h, void* p, bool kept) {
  if (!kept) { HYH_CHECK(hipFreeAsync(p, h->hipStream)); return; }
  std::lock_guard<std::mutex> lock(g_keptMutex);
  auto it = g_kept.find(h->mempool); if (it == g_kept.end()) { return; }
  for (Block& b : it->second) { if (b.p == p) { b.busy = false; b.stream = h->hipStream; return; } }
}

void hyh::scratch_drop_all(const hyacinHandle_t* h) {
  std::lock_guard<std::mutex> lock(g_keptMutex);
  auto it = g_kept.find(h->mempool); if (it == g_kept.end()) { return; }
  bool foreign = false; for (Block& b : it->second) { foreign = foreign || b.stream != h->hipStream; }
  if (foreign) { HYH_CHECK(hipDeviceSynchronize()); }
  for (Block& b : it->second) { HYH_CHECK(hipFreeAsync(b.p, h->hipStream)); }
  g_kept.erase(it);
}

extern "C" void hyacinDestroy(hyacinHandle_t* handle) {
  hyh::ApiScope scope;
  if (!handle) { return; }
  if ((handle->HandleOwnedResource & OWNS_MEMPOOL) && handle->mempool) { hyh::scratch_drop_all(handle); }
  HYH_CHECK(hipDeviceSynchronize());
  if ((handle->HandleOwnedResource & OWNS_MEMPOOL) && handle->mempool) { HYH_CHECK(hipMemPoolDestroy(handle->mempool)); }
  if ((handle->HandleOwnedResource & OWNS_PINNED) && handle->pinnedWorkspace) { HYH_CHECK(hipHostFree(handle->pinnedWorkspace)); }
  if ((handle->HandleOwnedResource & OWNS_TIMER) && handle->timer) {
    EventTimer* t = (EventTimer*)handle->timer; for (auto& ev : t->events) { HYH_CHECK(hipEventDestroy(ev.second)); } delete t;
  }
  std::memset(handle, 0, sizeof(hyacinHandle_t));
}

void hyh::timer_mark(const hyacinHandle_t* h, hyh::Segment seg) {
  EventTimer* t = (EventTimer*)h->timer;
  if (t && t->last != seg) { hipEvent_t e; HYH_CHECK(hipEventCreate(&e)); HYH_CHECK(hipEventRecord(e, h->hipStream)); t->events.emplace_back(t->last, e); t->last = seg; }
}

extern "C" void hyacinSync_TimerSegments(const hyacinHandle_t* handle, double* eventMs, int32_t lenMs) {
  hyh::ApiScope scope;
  if (handle->timer == nullptr) { HYH_CHECK(hipStreamSynchronize(handle->hipStream)); return; }
  EventTimer* t = (EventTimer*)handle->timer; const int len = (int)t->events.size();
  hipEvent_t e; HYH_CHECK(hipEventCreate(&e)); HYH_CHECK(hipEventRecord(e, handle->hipStream)); HYH_CHECK(hipEventSynchronize(e));
  t->events.emplace_back(t->last, e);
  if (eventMs != nullptr && 0 < lenMs) {
    /* event i closes the segment whose class is events[i].first; the first event only opens the first segment */
    double d = 0., r = 0., c = 0.;
    if (len) { hipEvent_t prev = t->events[0].second;
      for (size_t i = 1; i < t->events.size(); ++i) {
        float ms = 0.f; const hyh::Segment seg = t->events[i].first;
        if (seg != hyh::Segment::untimed) { HYH_CHECK(hipEventElapsedTime(&ms, prev, t->events[i].second)); }
        if (seg == hyh::Segment::dist_kernel) { d += ms; } else if (seg == hyh::Segment::rep_kernel) { r += ms; } else if (seg == hyh::Segment::comm) { c += ms; }
        prev = t->events[i].second;
      } }
    for (int32_t i = 0; i < lenMs; ++i) {
      const char req = static_cast<char>(eventMs[i]);
      eventMs[i] = (req == 'D' || req == 'd') ? d : ((req == 'R' || req == 'r') ? r : ((req == 'C' || req == 'c') ? c : 0.));
    }
  }
  for (auto& ev : t->events) { HYH_CHECK(hipEventDestroy(ev.second)); } t->events.clear(); t->last = hyh::Segment::untimed;
}

/* reference: src/allreduce_1drow.cu:3-5 -- one GPU holds every row, nothing to reduce */
extern "C" void hyacinAllReduce1Drow(const hyacinHandle_t*, int32_t, int32_t, uint64_t, uint64_t*) {}
extern "C" void hyacinAllReduceVExp(const hyacinHandle_t*, uint64_t, int32_t*) {}
