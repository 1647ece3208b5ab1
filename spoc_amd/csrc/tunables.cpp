#include "tunables.hpp"

#include <cstdlib>
#include <map>
#include <mutex>
#include <string>
#include <string_view>

#include <hip/hip_runtime.h>

#include "common.hpp"
#include "sarek_hip.h"

namespace sarek_hip {
namespace {
std::mutex g_mu;
// looked up by the kernels' launch code at every call: no allocation for the key
std::map<std::string, int64_t, std::less<>> &table() {
  static std::map<std::string, int64_t, std::less<>> t;
  return t;
}
unsigned long long *g_probe = nullptr;
int64_t g_probe_pairs = 0;
}  // namespace

unsigned long long *clock_probe(int64_t workgroups) {
  std::lock_guard<std::mutex> lock(g_mu);
  return (g_probe && workgroups <= g_probe_pairs) ? g_probe : nullptr;
}

#undef tunable
std::atomic<uint64_t> g_tunable_generation{1};

int64_t tunable_lookup(const char *name, int64_t fallback) {
  std::lock_guard<std::mutex> lock(g_mu);
  auto &t = table();
  auto it = t.find(std::string_view(name));
  if (it != t.end()) return it->second;
  std::string env = "SAREK_HIP_TUNE_";
  for (const char *p = name; *p; ++p) env.push_back(*p == '.' ? '_' : *p);
  int64_t v = fallback;
  if (const char *e = std::getenv(env.c_str())) v = std::strtoll(e, nullptr, 10);
  t[name] = v;
  return v;
}

void set_tunable(const char *name, int64_t value) {
  std::lock_guard<std::mutex> lock(g_mu);
  table()[name] = value;
  g_tunable_generation.fetch_add(1, std::memory_order_release);
}
}  // namespace sarek_hip

extern "C" int sarek_hip_set_tunable(const char *name, int64_t value) {
  if (!name) return SAREK_HIP_E_INVALID_ARG;
  // knobs of kernels that only the measurement build holds (some of them compute wrong results on purpose)
  if (!sarek_hip::kMeasureBuild)
    for (const char *measure_only : {"gemm16.ablate", "gemm16.ring", "gemm16.tj", "gemm16.mfma", "gemm16.waves", "gemm16.barriers"})
      if (std::string_view(name) == measure_only)
        return sarek_hip::fail(SAREK_HIP_E_UNSUPPORTED, "tunable %s exists in the measurement build only (libsarek_hip_measure.so)",
                               name);
  sarek_hip::set_tunable(name, value);
  return SAREK_HIP_OK;
}

extern "C" int sarek_hip_is_measurement_build(void) { return sarek_hip::kMeasureBuild ? 1 : 0; }

extern "C" int sarek_hip_set_clock_probe(uint64_t *device_pairs, int64_t capacity_pairs,
                                         int64_t *ticks_per_second) {
  using namespace sarek_hip;
  if (!kMeasureBuild)
    return fail(SAREK_HIP_E_UNSUPPORTED, "the in-kernel clock probe exists in the measurement build only (libsarek_hip_measure.so)");
  if (device_pairs && capacity_pairs <= 0)
    return fail(SAREK_HIP_E_INVALID_ARG, "clock probe: capacity must be positive");
  if (ticks_per_second) {
    int dev = 0, khz = 0;
    SAREK_HIP_TRY(hipGetDevice(&dev));
    SAREK_HIP_TRY(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev));
    *ticks_per_second = static_cast<int64_t>(khz) * 1000;
  }
  std::lock_guard<std::mutex> lock(g_mu);
  g_probe = reinterpret_cast<unsigned long long *>(device_pairs);
  g_probe_pairs = device_pairs ? capacity_pairs : 0;
  return SAREK_HIP_OK;
}
