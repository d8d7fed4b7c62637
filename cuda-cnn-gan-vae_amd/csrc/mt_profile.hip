// Per-kernel timing with HIP events on the work stream: the counterpart of the reference's event stopwatch and
// scope timer (cuda/ccudatimespent.cu:38-52, cuda/ctimestamp.cu:17-32), but accumulated per label instead of
// printed.  When disabled (the default) a scope costs one branch.
#include <map>
#include <string>
#include <vector>

#include "mt_common.h"

namespace {

struct Pending {
  const char *label;
  hipEvent_t start, stop;
};
struct Total {
  std::string label;
  uint64_t launches = 0;
  double ms = 0.0;
};

bool g_on = false;
int g_muted = 0;   // ProfileMute objects alive
int g_open = 0;    // ProfileScope objects alive that hold a slot of g_pending
std::vector<Pending> g_pending;
std::vector<hipEvent_t> g_free_events;
std::vector<Total> g_totals;
std::map<std::string, size_t> g_index;

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

int flush() {
  if (g_pending.empty()) return MT_OK;
  MT_HIP(hipStreamSynchronize(mt::stream()));
  for (const Pending &p : g_pending) {
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, p.start, p.stop) == hipSuccess) {
      auto it = g_index.find(p.label);
      if (it == g_index.end()) {
        it = g_index.emplace(p.label, g_totals.size()).first;
        g_totals.push_back(Total{p.label});
      }
      g_totals[it->second].launches++;
      g_totals[it->second].ms += ms;
    }
    g_free_events.push_back(p.start);
    g_free_events.push_back(p.stop);
  }
  g_pending.clear();
  return MT_OK;
}

}  // namespace

namespace mt {

bool profiling() { return g_on && g_muted == 0; }

ProfileMute::ProfileMute(bool on_) : on(on_) { if (on) g_muted++; }
ProfileMute::~ProfileMute() { if (on) g_muted--; }

const char *intern_label(const char *name, const char *suffix) {
  static std::map<std::string, std::string> labels;
  std::string key = std::string(name) + "[" + suffix + "]";
  return labels.emplace(key, key).first->second.c_str();
}

ProfileScope::ProfileScope(const char *label) : slot(-1) {
  if (!g_on || g_muted) return;
  if (g_pending.size() >= 16384) {
    // the pending list is emptied only while no scope holds a slot of it; otherwise this sample is dropped
    if (g_open > 0 || flush() != MT_OK) return;
  }
  Pending p{label, take_event(), nullptr};
  if (!p.start) return;
  p.stop = take_event();
  if (!p.stop || hipEventRecord(p.start, stream()) != hipSuccess) {
    g_free_events.push_back(p.start);
    if (p.stop) g_free_events.push_back(p.stop);
    return;
  }
  slot = (int)g_pending.size();
  g_pending.push_back(p);
  g_open++;
}

ProfileScope::~ProfileScope() {
  if (slot < 0) return;
  g_open--;
  (void)hipEventRecord(g_pending[slot].stop, stream());
}

}  // namespace mt

extern "C" {

int mt_profile_enable(int on) {
  if (on) {
    int rc = flush();
    if (rc) return rc;
    g_totals.clear();
    g_index.clear();
    g_on = true;
  } else {
    g_on = false;
    return flush();
  }
  return MT_OK;
}

int mt_profile_entries(void) {
  if (flush() != MT_OK) return -1;
  return (int)g_totals.size();
}

int mt_profile_entry(int index, const char **label, uint64_t *launches, double *total_ms) {
  if (index < 0 || (size_t)index >= g_totals.size()) return mt::fail(MT_E_ARGUMENT, "mt_profile_entry: index %d out of range", index);
  if (label) *label = g_totals[index].label.c_str();
  if (launches) *launches = g_totals[index].launches;
  if (total_ms) *total_ms = g_totals[index].ms;
  return MT_OK;
}

}  // extern "C"
