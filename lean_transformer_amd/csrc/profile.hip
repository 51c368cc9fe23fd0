// Per-kernel timing behind lt_profile_*: event pairs recorded on the launch stream, aggregated per tag on read.
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "lt_common.h"

namespace {

struct Record {
  std::string tag;
  double flops, bytes;
  hipEvent_t start, stop;
};

std::mutex g_mutex;
bool g_enabled = false;
std::vector<Record> g_records;
std::vector<hipEvent_t> g_free_events;
constexpr size_t MAX_RECORDS = 1 << 16;

hipEvent_t take_event() {
  if (!g_free_events.empty()) {
    hipEvent_t e = g_free_events.back();
    g_free_events.pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) return nullptr;
  return e;
}

void recycle_locked() {
  for (Record& r : g_records) {
    if (r.start) g_free_events.push_back(r.start);
    if (r.stop) g_free_events.push_back(r.stop);
  }
  g_records.clear();
}

}  // namespace

bool lt_profile_active() { return g_enabled; }

void lt_profile_begin(const char* tag, double flops, double bytes, hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_enabled || g_records.size() >= MAX_RECORDS) return;
  Record r{tag, flops, bytes, take_event(), take_event()};
  if (!r.start || !r.stop) return;
  (void)hipEventRecord(r.start, stream);
  g_records.push_back(r);
}

void lt_profile_end(hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (g_records.empty()) return;
  (void)hipEventRecord(g_records.back().stop, stream);
}

extern "C" int lt_profile_enable(int32_t enable) {
  std::lock_guard<std::mutex> lock(g_mutex);
  g_enabled = enable != 0;
  return LT_OK;
}

extern "C" int lt_profile_reset(void) {
  std::lock_guard<std::mutex> lock(g_mutex);
  recycle_locked();
  return LT_OK;
}

extern "C" int lt_profile_read(lt_profile_entry* entries, int32_t max_entries) {
  std::lock_guard<std::mutex> lock(g_mutex);
  std::map<std::string, lt_profile_entry> agg;
  std::vector<std::string> order;
  for (Record& r : g_records) {
    if (hipEventSynchronize(r.stop) != hipSuccess) {
      lt_set_error("lt_profile_read: waiting for an event failed");
      return -LT_ERR_HIP;
    }
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, r.start, r.stop) != hipSuccess) {
      lt_set_error("lt_profile_read: hipEventElapsedTime failed");
      return -LT_ERR_HIP;
    }
    auto it = agg.find(r.tag);
    if (it == agg.end()) {
      lt_profile_entry e;
      memset(&e, 0, sizeof(e));
      snprintf(e.name, sizeof(e.name), "%s", r.tag.c_str());
      it = agg.emplace(r.tag, e).first;
      order.push_back(r.tag);
    }
    it->second.launches += 1;
    it->second.ms += ms;
    it->second.flops += r.flops;
    it->second.bytes += r.bytes;
  }
  int n = 0;
  for (const std::string& tag : order) {
    if (entries && n < max_entries) entries[n] = agg[tag];
    n++;
  }
  return n;
}
