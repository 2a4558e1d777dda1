// Version, error-string and profiling entry points of libdcp_hip.so.
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "common.h"

namespace dcp {

char* last_error_buffer() {
  static thread_local char buffer[512] = {0};
  return buffer;
}

namespace {
struct Span {
  std::string name;
  hipEvent_t start, stop;
};
std::mutex g_mu;
bool g_profiling = false;
std::vector<Span> g_spans;
unsigned g_generation = 0;  // bumped whenever a report clears the list: span ids carry it
constexpr int kSpanBits = 24;
}  // namespace

bool profiling_enabled() { return g_profiling; }

int profile_begin(const char* name, hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_mu);
  Span s;
  s.name = name;
  if (hipEventCreate(&s.start) != hipSuccess) return -1;
  if (hipEventCreate(&s.stop) != hipSuccess) {
    (void)hipEventDestroy(s.start);
    return -1;
  }
  (void)hipEventRecord(s.start, stream);
  if (g_spans.size() >= (size_t)1 << kSpanBits) {  // ids are 24 bits of index under 7 bits of generation
    (void)hipEventDestroy(s.start);
    (void)hipEventDestroy(s.stop);
    return -1;
  }
  g_spans.push_back(s);
  return (int)(((g_generation & 0x7f) << kSpanBits) | (unsigned)(g_spans.size() - 1));
}

void profile_end(int span, hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_mu);
  // The span this timer opened: none if its events could not be created, and none if a report
  // has cleared the list in between (the id's generation then differs, and the index may by now
  // name another kernel's span, whose stop event must not be recorded here).
  if (span < 0 || (unsigned)(span >> kSpanBits) != (g_generation & 0x7f)) return;
  const int index = span & ((1 << kSpanBits) - 1);
  if (index < (int)g_spans.size()) (void)hipEventRecord(g_spans[index].stop, stream);
}

}  // namespace dcp

extern "C" int dcp_version(void) { return 100; }

extern "C" const char* dcp_last_error(void) { return dcp::last_error_buffer(); }

extern "C" void dcp_profile_enable(int on) {
  std::lock_guard<std::mutex> lock(dcp::g_mu);
  dcp::g_profiling = on != 0;
}

extern "C" int dcp_profile_report(char* buffer, size_t capacity) {
  std::lock_guard<std::mutex> lock(dcp::g_mu);
  std::map<std::string, std::pair<double, long>> totals;
  for (auto& s : dcp::g_spans) {
    float ms = 0.0f;
    if (hipEventSynchronize(s.stop) == hipSuccess && hipEventElapsedTime(&ms, s.start, s.stop) == hipSuccess) {
      auto& t = totals[s.name];
      t.first += ms;
      t.second += 1;
    }
    (void)hipEventDestroy(s.start);
    (void)hipEventDestroy(s.stop);
  }
  dcp::g_spans.clear();
  ++dcp::g_generation;
  std::string text;
  char line[256];
  for (auto& kv : totals) {
    snprintf(line, sizeof line, "%s %ld %.6f\n", kv.first.c_str(), kv.second.second, kv.second.first);
    text += line;
  }
  if (buffer && capacity > 0) {
    snprintf(buffer, capacity, "%s", text.c_str());
  }
  return (int)text.size() < (int)capacity ? DCP_OK : DCP_ERR_ARG;
}
