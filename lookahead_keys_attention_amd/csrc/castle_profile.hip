// Optional per-kernel timing with HIP events, recorded on the stream each kernel is launched
// on.  Off by default (then ProfScope costs one relaxed load).  Used by bench.py for the
// roofline figures; see castle_profile_enable / castle_profile_read in include/castle_hip.h.
#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>
#include <vector>

#include "castle_profile.h"

namespace castle {
namespace {
struct Record { int slot; hipEvent_t start, stop; };
std::atomic<int> g_enabled{0};
std::mutex g_mu;
std::vector<Record> g_records;        // records of the current window
std::vector<hipEvent_t> g_free;       // recycled events
constexpr size_t kMaxRecords = 1 << 16;

hipEvent_t get_event() {
  if (!g_free.empty()) { hipEvent_t e = g_free.back(); g_free.pop_back(); return e; }
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) return nullptr;
  return e;
}
}  // namespace

ProfScope::ProfScope(int slot, hipStream_t stream) : stream_(stream), index_(-1) {
  if (g_enabled.load(std::memory_order_relaxed) == 0) return;
  std::lock_guard<std::mutex> lock(g_mu);
  if (g_records.size() >= kMaxRecords) return;
  Record r{slot, get_event(), get_event()};
  if (r.start == nullptr || r.stop == nullptr) return;
  hipEventRecord(r.start, stream);
  g_records.push_back(r);
  index_ = (int)g_records.size() - 1;
}

ProfScope::~ProfScope() {
  if (index_ < 0) return;
  std::lock_guard<std::mutex> lock(g_mu);
  if (index_ < (int)g_records.size()) hipEventRecord(g_records[index_].stop, stream_);
}

int profile_enable(int on) {
  std::lock_guard<std::mutex> lock(g_mu);
  for (Record& r : g_records) { g_free.push_back(r.start); g_free.push_back(r.stop); }
  g_records.clear();
  g_enabled.store(on ? 1 : 0, std::memory_order_relaxed);
  return 0;
}

int profile_read(int* slots, float* ms, int max_records) {
  std::lock_guard<std::mutex> lock(g_mu);
  int n = 0;
  for (Record& r : g_records) {
    if (hipEventSynchronize(r.stop) != hipSuccess) return -3;
    float t = 0.f;
    if (hipEventElapsedTime(&t, r.start, r.stop) != hipSuccess) return -3;
    if (n < max_records) { slots[n] = r.slot; ms[n] = t; ++n; }
    g_free.push_back(r.start);
    g_free.push_back(r.stop);
  }
  g_records.clear();
  return n;
}

}  // namespace castle
