// Integer tuning knobs (launch shapes, tile variants) that can be changed at run
// time through sarek_hip_set_tunable() without rebuilding; used for sweeps.
#pragma once
#include <atomic>
#include <cstdint>

namespace sarek_hip {
// Value of knob `name`, or `fallback` when it was never set.  An environment
// variable SAREK_HIP_TUNE_<name with '.' replaced by '_'> seeds the knob on first use.
// Takes a lock and walks the table: launch code goes through tunable() below instead.
int64_t tunable_lookup(const char *name, int64_t fallback);
void set_tunable(const char *name, int64_t value);

// One per place that reads a knob: the value it saw last and the table generation it saw it at.
struct TunableSite {
  std::atomic<uint64_t> generation{0};
  std::atomic<int64_t> value{0};
};
extern std::atomic<uint64_t> g_tunable_generation;   // bumped by every set_tunable

inline int64_t tunable_at(TunableSite &site, const char *name, int64_t fallback) {
  const uint64_t now = g_tunable_generation.load(std::memory_order_acquire);
  if (site.generation.load(std::memory_order_acquire) == now) return site.value.load(std::memory_order_relaxed);
  const int64_t v = tunable_lookup(name, fallback);
  site.value.store(v, std::memory_order_relaxed);
  site.generation.store(now, std::memory_order_release);
  return v;
}

// Clock-probe buffer for a launch of `workgroups` workgroups, or nullptr.
unsigned long long *clock_probe(int64_t workgroups);
}  // namespace sarek_hip

// tunable("name", fallback) on a launch path: two atomic loads while no knob has changed since the
// last call from this very place; the table is consulted again after any sarek_hip_set_tunable.
#define tunable(name, fallback)                                        \
  ([&]() -> int64_t {                                                  \
    static ::sarek_hip::TunableSite sarek_tunable_site;                \
    return ::sarek_hip::tunable_at(sarek_tunable_site, name, fallback); \
  }())
