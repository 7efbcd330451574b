// Event-based kernel timing behind nmtg_trace_begin / nmtg_trace_end.
#include "common.hip.h"
#include "trace.hip.h"
#include <cstring>
#include <algorithm>
#include <atomic>
#include <map>
#include <mutex>
#include <vector>

namespace nmtg {
namespace {

struct Record {
  const char* name;
  hipEvent_t start, stop;
};

std::mutex g_mu;
std::atomic<bool> g_on{false};   // read without the lock on every launch
std::vector<Record> g_records;        // records in use since trace_begin
std::vector<Record> g_pool;           // events kept for reuse
constexpr size_t MAX_RECORDS = 1 << 16;

}  // namespace

bool trace_on() { return g_on.load(std::memory_order_relaxed); }

void trace_open(const char* name, hipStream_t st, int* slot) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (!g_on || g_records.size() >= MAX_RECORDS) return;
  Record r{name, nullptr, nullptr};
  if (!g_pool.empty()) {
    r = g_pool.back();
    g_pool.pop_back();
    r.name = name;
  } else {
    if (hipEventCreate(&r.start) != hipSuccess || hipEventCreate(&r.stop) != hipSuccess) {
      (void)hipGetLastError();
      return;
    }
  }
  if (hipEventRecord(r.start, st) != hipSuccess) { (void)hipGetLastError(); g_pool.push_back(r); return; }
  g_records.push_back(r);
  *slot = static_cast<int>(g_records.size()) - 1;
}

void trace_close(hipStream_t st, int slot) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (slot < 0 || slot >= static_cast<int>(g_records.size())) return;
  if (hipEventRecord(g_records[slot].stop, st) != hipSuccess) (void)hipGetLastError();
}

}  // namespace nmtg

using namespace nmtg;

extern "C" int nmtg_trace_begin(void) {
  std::lock_guard<std::mutex> lk(g_mu);
  for (auto& r : g_records) g_pool.push_back(r);
  g_records.clear();
  g_on = true;
  return 0;
}

extern "C" int64_t nmtg_trace_end(char* out, int64_t capacity) {
  std::lock_guard<std::mutex> lk(g_mu);
  g_on = false;
  std::map<std::string, std::pair<int64_t, double>> agg;
  for (auto& r : g_records) {
    float ms = 0.f;
    if (hipEventSynchronize(r.stop) == hipSuccess && hipEventElapsedTime(&ms, r.start, r.stop) == hipSuccess) {
      auto& a = agg[r.name];
      a.first += 1;
      a.second += ms;
    } else {
      (void)hipGetLastError();
    }
    g_pool.push_back(r);
  }
  g_records.clear();
  std::string text;
  for (auto& kv : agg) {
    char line[256];
    snprintf(line, sizeof(line), "%s %lld %.6f\n", kv.first.c_str(), (long long)kv.second.first, kv.second.second);
    text += line;
  }
  if (out != nullptr && capacity > 0) {
    const size_t n = std::min<size_t>(text.size(), static_cast<size_t>(capacity) - 1);
    std::memcpy(out, text.data(), n);
    out[n] = 0;
  }
  return static_cast<int64_t>(text.size());
}
