#include "tunables.hpp"

#include <cstdlib>
#include <map>
#include <mutex>
#include <string>

#include "sarek_hip.h"

namespace sarek_hip {
namespace {
std::mutex g_mu;
std::map<std::string, int64_t> &table() {
  static std::map<std::string, int64_t> t;
  return t;
}
}  // namespace

int64_t tunable(const char *name, int64_t fallback) {
  std::lock_guard<std::mutex> lock(g_mu);
  auto &t = table();
  auto it = t.find(name);
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
}
}  // namespace sarek_hip

extern "C" int sarek_hip_set_tunable(const char *name, int64_t value) {
  if (!name) return SAREK_HIP_E_INVALID_ARG;
  sarek_hip::set_tunable(name, value);
  return SAREK_HIP_OK;
}
