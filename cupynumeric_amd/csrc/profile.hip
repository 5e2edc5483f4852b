// Event-based launch timing (see profile.h) and its extern "C" controls.
#include "profile.h"

#include <stdint.h>
#include <string.h>

#include <atomic>
#include <mutex>
#include <vector>

#include "../../include/cpn_sort.h"

namespace cpn {

namespace {
struct Record {
  const char* label;
  hipEvent_t start;
  hipEvent_t stop;
  bool closed;
};
std::atomic<bool> g_enabled{false};
std::mutex g_mutex;
std::vector<Record> g_records;
constexpr size_t MAX_RECORDS = 1 << 16;
}  // namespace

bool profiling_enabled() { return g_enabled.load(std::memory_order_relaxed); }

int profile_begin(const char* label, hipStream_t stream)
{
  std::lock_guard<std::mutex> lock(g_mutex);
  if (g_records.size() >= MAX_RECORDS) {
    return -1;
  }
  Record r{label, nullptr, nullptr, false};
  if (hipEventCreate(&r.start) != hipSuccess) {
    return -1;
  }
  if (hipEventCreate(&r.stop) != hipSuccess) {
    (void)hipEventDestroy(r.start);
    return -1;
  }
  (void)hipEventRecord(r.start, stream);
  g_records.push_back(r);
  return static_cast<int>(g_records.size() - 1);
}

void profile_end(int slot, hipStream_t stream)
{
  std::lock_guard<std::mutex> lock(g_mutex);
  if (slot >= 0 && static_cast<size_t>(slot) < g_records.size()) {
    (void)hipEventRecord(g_records[slot].stop, stream);
    g_records[slot].closed = true;
  }
}

}  // namespace cpn

extern "C" {

int cpn_profile_enable(int on)
{
  const bool prev = cpn::g_enabled.exchange(on != 0);
  return prev ? 1 : 0;
}

int cpn_profile_collect(char* labels, uint64_t label_stride, float* milliseconds, int max_records)
{
  std::lock_guard<std::mutex> lock(cpn::g_mutex);
  int n = 0;
  for (auto& r : cpn::g_records) {
    if (r.closed && n < max_records && labels != nullptr && milliseconds != nullptr && label_stride > 0) {
      float ms = -1.0f;
      if (hipEventSynchronize(r.stop) == hipSuccess && hipEventElapsedTime(&ms, r.start, r.stop) == hipSuccess) {
        strncpy(labels + static_cast<size_t>(n) * label_stride, r.label, label_stride - 1);
        labels[static_cast<size_t>(n) * label_stride + label_stride - 1] = 0;
        milliseconds[n]                                                 = ms;
        ++n;
      }
    }
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
  }
  cpn::g_records.clear();
  return n;
}

}  // extern "C"
