// What a BACKEND module says about itself besides its functions (spoc/framework/Framework_sig.ml:137-143,
// 285, 314-319): name, version, execution model, and the registry of backend intrinsics
// (INTRINSIC_REGISTRY, :107-119).  The registry holds name -> (device code, convergence); it starts with
// the entries the CUDA plugin registers (sarek-cuda/Cuda_plugin.ml:47-143) in their HIP spellings and
// takes more at run time.  The code generator has its own table: the registry is for callers that ask
// what a backend offers (sarek/framework/test/test_framework_integration.ml:190-207).
#include <cstring>
#include <map>
#include <mutex>
#include <string>

#include "common.hpp"

namespace sarek_hip {
namespace {

struct Intrinsic {
  std::string codegen;
  int convergence;
};

std::mutex g_mu;

std::map<std::string, Intrinsic> &table() {
  static std::map<std::string, Intrinsic> *t = [] {
    auto *m = new std::map<std::string, Intrinsic>;
    const int U = SAREK_HIP_CONVERGENCE_UNIFORM, D = SAREK_HIP_CONVERGENCE_DIVERGENT, S = SAREK_HIP_CONVERGENCE_SYNC;
    (*m)["thread_id_x"] = {"threadIdx.x", D};
    (*m)["thread_id_y"] = {"threadIdx.y", D};
    (*m)["thread_id_z"] = {"threadIdx.z", D};
    (*m)["block_id_x"] = {"blockIdx.x", U};
    (*m)["block_id_y"] = {"blockIdx.y", U};
    (*m)["block_id_z"] = {"blockIdx.z", U};
    (*m)["block_dim_x"] = {"blockDim.x", U};
    (*m)["block_dim_y"] = {"blockDim.y", U};
    (*m)["block_dim_z"] = {"blockDim.z", U};
    (*m)["global_thread_id"] = {"(threadIdx.x + blockIdx.x * blockDim.x)", D};
    (*m)["block_barrier"] = {"__syncthreads()", S};
    (*m)["warp_barrier"] = {"__builtin_amdgcn_wave_barrier()", S};   // a 64-lane wave, not a 32-lane warp
    (*m)["memory_fence"] = {"__threadfence()", U};
    return m;
  }();
  return *t;
}

// tools/device_info.ml:8-14
std::string format_memory(uint64_t bytes) {
  char buf[64];
  const double gb = static_cast<double>(bytes) / (1024.0 * 1024.0 * 1024.0);
  if (gb >= 1.0) std::snprintf(buf, sizeof(buf), "%.2f GB", gb);
  else std::snprintf(buf, sizeof(buf), "%.0f MB", static_cast<double>(bytes) / (1024.0 * 1024.0));
  return buf;
}

// tools/device_info.ml:16-43 for a device of this backend (never a CPU device; FP64 and atomics always:
// the capabilities record of sarek-cuda/Cuda_plugin_base.ml:177-195 with this device's figures)
std::string device_block(int id, const sarek_hip_device_info &d) {
  char buf[512];
  std::string o;
  std::snprintf(buf, sizeof(buf), "[%d] %s\n    Backend: HIP\n    Memory: %s\n", id, d.name,
                format_memory(d.total_global_mem).c_str());
  o += buf;
  if (d.compute_major > 0) {
    std::snprintf(buf, sizeof(buf), "    Compute Capability: %d.%d\n", d.compute_major, d.compute_minor);
    o += buf;
  }
  std::snprintf(buf, sizeof(buf),
                "    Max Threads/Block: %d\n    Compute Units: %d\n    Warp/Wavefront Size: %d\n"
                "    Features: Atomics, FP64\n",
                d.max_threads_per_block, d.multiprocessor_count, d.warp_size);
  o += buf;
  return o;
}

}  // namespace
}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" {

const char *sarek_hip_backend_name(void) { return "HIP"; }

int sarek_hip_backend_version(int *major, int *minor, int *patch) {
  if (!major || !minor || !patch) return fail(SAREK_HIP_E_INVALID_ARG, "backend_version: NULL argument");
  *major = 1;
  *minor = 0;
  *patch = 0;
  return SAREK_HIP_OK;
}

int sarek_hip_execution_model(void) { return SAREK_HIP_EXECUTION_JIT; }

int sarek_hip_device_report(char *out, size_t cap, size_t *needed, int *device_count) {
  const std::string rule(70, '=');
  std::string o = rule + "\nSAREK Device Information Utility\nMulti-Backend GPU/CPU Device Diagnostic Tool\n" + rule + "\n";
  int count = 0;
  if (sarek_hip_is_available()) {
    if (sarek_hip_device_count(&count) != SAREK_HIP_OK) count = 0;
  }
  if (device_count) *device_count = count;
  if (count == 0) {
    o += "\n\xE2\x9A\xA0 No devices found\nEnsure you have:\n"
         "  - HIP backend: AMD GPU driver + ROCm runtime (libamdhip64, libhiprtc)\n" + rule + "\n";
  } else {
    o += "\nFound " + std::to_string(count) + " device" + (count > 1 ? "s" : "") + ":\n\n";
    for (int i = 0; i < count; ++i) {
      sarek_hip_device_info d;
      if (sarek_hip_device_get_info(i, &d) != SAREK_HIP_OK) continue;     // Device.get i = None: skipped
      o += device_block(i, d) + "\n";
    }
    o += rule + "\nUsage:\n  \xE2\x80\xA2 Device.get N returns device N (0-" + std::to_string(count - 1) + ")\n"
         "  \xE2\x80\xA2 Device.by_framework \"HIP\" filters by backend\n" + rule + "\n";
  }
  if (needed) *needed = o.size() + 1;
  if (!out || cap < o.size() + 1)
    return fail(SAREK_HIP_E_BUFFER_TOO_SMALL, "device_report: %zu bytes needed", o.size() + 1);
  std::memcpy(out, o.c_str(), o.size() + 1);
  return SAREK_HIP_OK;
}

int sarek_hip_intrinsic_register(const char *name, const char *codegen, int convergence) {
  if (!name || !codegen || !*name) return fail(SAREK_HIP_E_INVALID_ARG, "intrinsic_register: NULL or empty argument");
  if (convergence < SAREK_HIP_CONVERGENCE_UNIFORM || convergence > SAREK_HIP_CONVERGENCE_SYNC)
    return fail(SAREK_HIP_E_INVALID_ARG, "intrinsic_register: unknown convergence %d", convergence);
  std::lock_guard<std::mutex> lock(g_mu);
  table()[name] = {codegen, convergence};                     // Hashtbl.replace
  return SAREK_HIP_OK;
}

int sarek_hip_intrinsic_find(const char *name, char *codegen, size_t cap, int *convergence, int *found) {
  if (!name || !found) return fail(SAREK_HIP_E_INVALID_ARG, "intrinsic_find: NULL argument");
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = table().find(name);
  *found = it != table().end();
  if (!*found) return SAREK_HIP_OK;
  if (convergence) *convergence = it->second.convergence;
  if (codegen) {
    if (cap < it->second.codegen.size() + 1)
      return fail(SAREK_HIP_E_BUFFER_TOO_SMALL, "intrinsic_find: %zu bytes needed", it->second.codegen.size() + 1);
    std::snprintf(codegen, cap, "%s", it->second.codegen.c_str());
  }
  return SAREK_HIP_OK;
}

int sarek_hip_intrinsic_list(char *out, size_t cap, size_t *needed) {
  std::string all;                                             // sorted, newline-separated
  {
    std::lock_guard<std::mutex> lock(g_mu);
    for (auto &kv : table()) all += kv.first + "\n";
  }
  if (needed) *needed = all.size() + 1;
  if (!out || cap < all.size() + 1) return fail(SAREK_HIP_E_BUFFER_TOO_SMALL, "intrinsic_list: %zu bytes needed", all.size() + 1);
  std::snprintf(out, cap, "%s", all.c_str());
  return SAREK_HIP_OK;
}

}  // extern "C"
