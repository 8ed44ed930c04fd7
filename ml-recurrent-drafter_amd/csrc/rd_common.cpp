// Error buffer and version of the C ABI.
#include "rd_common.h"

#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

namespace rd {

char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

// ---- kernel timing -----------------------------------------------------------------------------
namespace {
constexpr int kTimingSlots = 16384;
struct TimingState {
  std::mutex mu;
  bool enabled = false;
  std::string only;  // when not empty: the one kernel that is timed
  int used = 0;
  int every = 1;  // of the launches that qualify, every n-th is timed ...
  long seen = 0;  // ... counted from the last rd_timing_enable
  std::vector<hipEvent_t> start, stop;
  std::vector<const char*> name;
};
TimingState& timing() {
  static TimingState t;
  return t;
}
}  // namespace

ScopedTiming::ScopedTiming(const char* name, hipStream_t stream) : stream_(stream), slot_(-1) {
  TimingState& t = timing();
  if (!t.enabled) return;
  std::lock_guard<std::mutex> lock(t.mu);
  if (!t.only.empty() && t.only != name) return;
  if ((t.seen++ % t.every) != 0) return;
  if (t.used >= (int)t.start.size()) return;  // pool exhausted: later launches go untimed
  slot_ = t.used++;
  t.name[slot_] = name;
  (void)hipEventRecord(t.start[slot_], stream_);
}

void timing_events(const char* name, hipEvent_t* start, hipEvent_t* stop) {
  *start = *stop = nullptr;
  TimingState& t = timing();
  if (!t.enabled) return;
  std::lock_guard<std::mutex> lock(t.mu);
  if (!t.only.empty() && t.only != name) return;
  if ((t.seen++ % t.every) != 0) return;
  if (t.used >= (int)t.start.size()) return;
  const int slot = t.used++;
  t.name[slot] = name;
  *start = t.start[slot];
  *stop = t.stop[slot];
}

ScopedTiming::~ScopedTiming() {
  if (slot_ < 0) return;
  (void)hipEventRecord(timing().stop[slot_], stream_);
}

}  // namespace rd

extern "C" int rd_timing_enable(int on) {
  auto& t = rd::timing();
  std::lock_guard<std::mutex> lock(t.mu);
  if (on && t.start.empty()) {
    t.start.resize(rd::kTimingSlots);
    t.stop.resize(rd::kTimingSlots);
    t.name.assign(rd::kTimingSlots, nullptr);
    for (int i = 0; i < rd::kTimingSlots; ++i) {
      if (hipEventCreate(&t.start[i]) != hipSuccess || hipEventCreate(&t.stop[i]) != hipSuccess) {
        t.start.clear(); t.stop.clear(); t.name.clear();
        return rd::fail(RD_ELAUNCH, "rd_timing_enable: hipEventCreate failed");
      }
    }
  }
  t.enabled = on != 0;
  t.used = 0;
  t.seen = 0;
  return RD_OK;
}

extern "C" int rd_timing_sample(int every) {
  RD_REQUIRE(every >= 1, RD_EINVAL, "rd_timing_sample: every %d < 1", every);
  auto& t = rd::timing();
  std::lock_guard<std::mutex> lock(t.mu);
  t.every = every;
  t.seen = 0;
  return RD_OK;
}

extern "C" int rd_timing_select(const char* kernel) {
  auto& t = rd::timing();
  std::lock_guard<std::mutex> lock(t.mu);
  t.only = kernel ? kernel : "";
  return RD_OK;
}

extern "C" int rd_timing_collect(char* out, size_t out_bytes) {
  auto& t = rd::timing();
  std::lock_guard<std::mutex> lock(t.mu);
  std::map<std::string, std::pair<long, double>> acc;
  for (int i = 0; i < t.used; ++i) {
    if (hipEventSynchronize(t.stop[i]) != hipSuccess) continue;
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, t.start[i], t.stop[i]) != hipSuccess) continue;
    auto& e = acc[t.name[i]];
    e.first += 1;
    e.second += ms;
  }
  t.used = 0;
  std::string text;
  char line[160];
  for (auto& kv : acc) {
    snprintf(line, sizeof line, "%s %ld %.6f\n", kv.first.c_str(), kv.second.first, kv.second.second);
    text += line;
  }
  RD_REQUIRE(out && out_bytes > text.size(), RD_EINVAL, "rd_timing_collect: buffer of %zu bytes too small (%zu)",
             out_bytes, text.size() + 1);
  memcpy(out, text.c_str(), text.size() + 1);
  return RD_OK;
}

extern "C" int rd_version(void) { return RD_ABI_VERSION; }
extern "C" const char* rd_last_error(void) { return rd::error_buffer(); }
