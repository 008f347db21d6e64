// Device memory of the library's own: the records through which workgroups of one launch hand partial tiles to each
// other (the split division of the attention kernel, the K-split shares of the persistent GEMM) and the arrival
// counters that go with them.  One set per (device, stream): launches on one stream run one after the other and can
// share it, launches on different streams get different sets.  A set is created at the first launch that needs one,
// grown when a later launch needs more, and kept until ll_release_stream_memory or the end of the process.  The
// counters are zero whenever no launch is running: every kernel that uses them leaves them at zero.
#include <map>
#include <mutex>
#include <vector>

#include "ll_common.h"

namespace ll {

// A set that a capturing stream has used is part of a recorded graph, which will use the same addresses at every
// replay: such a set is never freed when a later launch needs a larger one (it is kept aside until the release call).
struct ScratchEntry {
  StreamScratch current{};
  bool recorded = false;
  std::vector<StreamScratch> retired;
};
static std::mutex g_scratch_mutex;
static std::map<std::pair<int, hipStream_t>, ScratchEntry> g_scratch;

static void free_scratch(StreamScratch& w) {
  if (w.records) (void)hipFree(w.records);  // waits for the launches that still use it
  if (w.counters) (void)hipFree(w.counters);
  w = StreamScratch{};
}

int stream_scratch(int dev, hipStream_t stream, size_t record_bytes, size_t counters, bool may_allocate, StreamScratch& out,
                   bool* missing, const char* what) {
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (missing) *missing = false;
  if (!may_allocate) {  // the stream is being captured
    const auto it = g_scratch.find({dev, stream});
    if (it == g_scratch.end() || it->second.current.record_bytes < record_bytes ||
        it->second.current.n_counters < counters) {
      if (missing) *missing = true;
      return LL_OK;
    }
    it->second.recorded = true;
    out = it->second.current;
    return LL_OK;
  }
  ScratchEntry& entry = g_scratch[{dev, stream}];
  StreamScratch& w = entry.current;
  if (w.record_bytes < record_bytes || w.n_counters < counters) {
    const size_t want_bytes = record_bytes > w.record_bytes ? record_bytes : w.record_bytes;
    size_t want_counters = counters > w.n_counters ? counters : w.n_counters;
    if (want_counters < 4096) want_counters = 4096;
    if (entry.recorded && w.records) {
      entry.retired.push_back(w);
      w = StreamScratch{};
      entry.recorded = false;
    } else {
      free_scratch(w);
    }
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&w.records), want_bytes);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&w.counters), want_counters * sizeof(int));
    if (e == hipSuccess) e = hipMemsetAsync(w.counters, 0, want_counters * sizeof(int), stream);
    if (e != hipSuccess) {
      set_error("%s: cannot set up %zu bytes for partial results: %s", what, want_bytes, hipGetErrorString(e));
      free_scratch(w);
      if (entry.retired.empty()) g_scratch.erase({dev, stream});
      return LL_ELAUNCH;
    }
    w.record_bytes = want_bytes;
    w.n_counters = want_counters;
  }
  out = w;
  return LL_OK;
}

int release_stream_scratch(int dev, hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  const auto it = g_scratch.find({dev, stream});
  if (it == g_scratch.end()) return LL_OK;
  free_scratch(it->second.current);
  for (StreamScratch& old : it->second.retired) free_scratch(old);
  g_scratch.erase(it);
  return LL_OK;
}

bool stream_is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return true;
  }
  return status != hipStreamCaptureStatusNone;
}

int compute_units_of(int dev, int& cus, const char* what) {
  static std::atomic<int> cached[64];
  if (dev >= 0 && dev < 64 && (cus = cached[dev].load(std::memory_order_relaxed)) > 0) return LL_OK;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
    set_error("%s: cannot read the number of compute units of device %d", what, dev);
    return LL_ELAUNCH;
  }
  if (dev >= 0 && dev < 64) cached[dev].store(cus, std::memory_order_relaxed);
  return LL_OK;
}

}  // namespace ll

extern "C" int ll_release_stream_memory(void* stream) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    ll::set_error("ll_release_stream_memory: hipGetDevice failed");
    return LL_ELAUNCH;
  }
  return ll::release_stream_scratch(dev, static_cast<hipStream_t>(stream));
}
