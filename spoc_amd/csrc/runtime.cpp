// Device / Memory / Stream / Event / Kernel layer of libsarek_hip: the HIP and hiprtc
// calls the plugin's Hip_api module needs, behind the library's status convention.
// Mirrors the responsibilities of sarek-cuda/Cuda_api.ml:35-512 and
// sarek-cuda/Cuda_nvrtc.ml:263-389 (compile with log capture, cached kernels,
// parameter-pointer launch).
#include <hip/hiprtc.h>

#include "code_cache.hpp"

#include <atomic>
#include <cctype>
#include <cstring>
#include <map>
#include <unordered_map>
#include <mutex>
#include <set>
#include <string>
#include <vector>

#include "common.hpp"

struct sarek_hip_kernel_s {
  hipModule_t module = nullptr;
  hipFunction_t function = nullptr;
  std::string name;
  int device = -1;
  bool cached = false;
  std::atomic<unsigned> dynamic_lds_allowed{48u << 10};   // raised on demand, see sarek_hip_kernel_launch
};

namespace sarek_hip {
namespace {

std::mutex g_mu;
bool g_inited = false;
std::set<void *> g_live_allocs;  // device pointers handed out and not yet freed
// Compiled kernels by (device, kernel name, source text): buckets by hash, the text compared on a hit.
struct CachedKernel {
  int dev;
  std::string name, source;
  sarek_hip_kernel kernel;
};
std::unordered_map<uint64_t, std::vector<CachedKernel>> g_kernel_cache;

int rtc_fail(hiprtcResult r, const char *what) {
  return fail(1000 + static_cast<int>(r), "%s: %s", what, hiprtcGetErrorString(r));
}

// 64-bit hash of the source text, eight bytes a step, for the kernel cache (looked up at every
// launch: a byte-at-a-time hash of a 2 KB source costs as much as the launch call itself).
uint64_t hash_text(const char *p, size_t n) {
  uint64_t h = 0x9E3779B97F4A7C15ull ^ n;
  while (n >= 8) {
    uint64_t w;
    std::memcpy(&w, p, 8);
    h = (h ^ w) * 0xFF51AFD7ED558CCDull;
    h ^= h >> 32;
    p += 8;
    n -= 8;
  }
  uint64_t w = 0;
  std::memcpy(&w, p, n);
  h = (h ^ w) * 0xC4CEB9FE1A85EC53ull;
  return h ^ (h >> 29);
}

void copy_log(const std::string &text, char *log, size_t log_len) {
  if (!log || log_len == 0) return;
  size_t n = text.size() < log_len - 1 ? text.size() : log_len - 1;
  std::memcpy(log, text.data(), n);
  log[n] = '\0';
}

// Whether `text` uses the module-qualified name MODULE.something without declaring MODULE itself.
bool uses_module(const std::string &text, const char *module) {
  const std::string name = module;
  bool used = false;
  for (size_t at = text.find(name); at != std::string::npos; at = text.find(name, at + 1)) {
    const bool starts = at == 0 || !(std::isalnum(static_cast<unsigned char>(text[at - 1])) || text[at - 1] == '_');
    if (!starts) continue;
    const char after = at + name.size() < text.size() ? text[at + name.size()] : '\0';
    if (after == '.') used = true;
    else if (!(std::isalnum(static_cast<unsigned char>(after)) || after == '_')) return false;   // the text's own Float
  }
  return used;
}

// OCaml's constants that a kernel may name.  A reference to a value outside the kernel lowers to a variable of that
// name (sarek/ppx/Sarek_lower_ir.ml:378-380), so the text says `sdata[tid] = Float.neg_infinity;` -- as the reference's
// own generated reduction does (benchmarks/generate_backend_code.ml:164) -- which is no C without an object called
// Float.  The Native backend evaluates the OCaml value, a double; these are the same values.
std::string ocaml_constants_for(const std::string &text) {
  std::string o;
  if (uses_module(text, "Float"))
    o += "struct sarek_hip_ocaml_float { double infinity, neg_infinity, nan, pi, epsilon, max_float, min_float, zero, one, "
         "minus_one; };\nstatic constexpr sarek_hip_ocaml_float Float = {__builtin_inf(), -__builtin_inf(), "
         "__builtin_nan(\"\"), 3.141592653589793116, 2.220446049250313081e-16, 1.797693134862315708e+308, "
         "2.225073858507201383e-308, 0.0, 1.0, -1.0};\n";
  if (uses_module(text, "Int32"))
    o += "struct sarek_hip_ocaml_int32 { int max_int, min_int, zero, one, minus_one; };\n"
         "static constexpr sarek_hip_ocaml_int32 Int32 = {2147483647, -2147483647 - 1, 0, 1, -1};\n";
  if (uses_module(text, "Int64"))
    o += "struct sarek_hip_ocaml_int64 { long long max_int, min_int, zero, one, minus_one; };\n"
         "static constexpr sarek_hip_ocaml_int64 Int64 = {9223372036854775807LL, -9223372036854775807LL - 1, 0, 1, -1};\n";
  // Gpu.spoc_powint's device text is a call of that name (sarek/Sarek_stdlib/Gpu.ml:235-247), which nothing in the
  // reference's device headers defines; its OCaml side multiplies `exp` times.
  if (text.find("spoc_powint(") != std::string::npos && text.find("int spoc_powint(") == std::string::npos)
    o += "__device__ __forceinline__ int spoc_powint(int base, int exp) {\n  int acc = 1;\n"
         "  for (; exp > 0; --exp) acc *= base;\n  return acc;\n}\n";
  return o;
}

int compile_impl(const char *source_given, const char *kernel_name, sarek_hip_kernel *out, char *log,
                 size_t log_len) {
  if (!source_given || !kernel_name || !out)
    return fail(SAREK_HIP_E_INVALID_ARG, "kernel_compile: NULL argument");
  if (log && log_len) log[0] = '\0';
  std::string with_constants;
  const char *source = source_given;
  {
    const std::string text = source_given;
    const std::string constants = ocaml_constants_for(text);
    if (!constants.empty()) {
      with_constants = constants + text;
      source = with_constants.c_str();
    }
  }
  int dev = 0;
  SAREK_HIP_TRY(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  SAREK_HIP_TRY(hipGetDeviceProperties(&prop, dev));
  std::string arch = std::string("--offload-arch=") + prop.gcnArchName;

  // Persistent cache: the code object depends on the source, the target and the compiler.
  std::string cache_key;
  if (cache_enabled()) {
    int rtc_major = 0, rtc_minor = 0, runtime_version = 0;
    (void)hiprtcVersion(&rtc_major, &rtc_minor);
    (void)hipRuntimeGetVersion(&runtime_version);
    cache_key = cache_compute_key(std::string(prop.name) + "|" + prop.gcnArchName,
                                  "hiprtc " + std::to_string(rtc_major) + "." + std::to_string(rtc_minor) +
                                      " hip " + std::to_string(runtime_version) + " -O3 -packed-fp32-ops -fwrapv",
                                  source);
    std::vector<char> cached;
    if (cache_get(cache_key, &cached) && !cached.empty()) {
      auto *k = new sarek_hip_kernel_s();
      k->name = kernel_name;
      k->device = dev;
      if (hipModuleLoadData(&k->module, cached.data()) == hipSuccess) {
        if (hipModuleGetFunction(&k->function, k->module, kernel_name) == hipSuccess) {
          *out = k;
          return SAREK_HIP_OK;
        }
        (void)hipModuleUnload(k->module);
      }
      delete k;
      (void)hipGetLastError();
      cache_note_error();   // unusable entry: compile afresh and overwrite it
    }
  }

  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, source, "sarek_kernel.hip", 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) return rtc_fail(r, "hiprtcCreateProgram");
  // Packed FP32 instructions are switched off for generated code as for the library's own kernels
  // (some of their forms have given wrong results on this hardware without any error).
  // -fwrapv: int32 / int64 arithmetic of a kernel wraps modulo 2^32 / 2^64 on the Native backend (OCaml's Int32 and
  // Int64 are defined that way), so an overflow in the device text -- a hash, a linear congruential generator -- must
  // not be something the optimiser may assume away.
  const char *opts[] = {arch.c_str(), "-O3",    "-std=c++17",       "-fwrapv",
                        "-Xclang",    "-target-feature", "-Xclang", "-packed-fp32-ops"};
  r = hiprtcCompileProgram(prog, static_cast<int>(sizeof(opts) / sizeof(opts[0])), opts);
  std::string build_log;
  size_t log_size = 0;
  if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
    build_log.resize(log_size);
    hiprtcGetProgramLog(prog, &build_log[0]);
  }
  copy_log(build_log, log, log_len);
  if (r != HIPRTC_SUCCESS) {
    hiprtcDestroyProgram(&prog);
    return fail(SAREK_HIP_E_COMPILE, "hiprtc compilation of kernel '%s' failed: %s\n%s", kernel_name,
                hiprtcGetErrorString(r), build_log.c_str());
  }
  size_t code_size = 0;
  r = hiprtcGetCodeSize(prog, &code_size);
  if (r != HIPRTC_SUCCESS) {
    hiprtcDestroyProgram(&prog);
    return rtc_fail(r, "hiprtcGetCodeSize");
  }
  std::vector<char> code(code_size);
  r = hiprtcGetCode(prog, code.data());
  hiprtcDestroyProgram(&prog);
  if (r != HIPRTC_SUCCESS) return rtc_fail(r, "hiprtcGetCode");
  if (!cache_key.empty()) cache_put(cache_key, code.data(), code.size());

  auto *k = new sarek_hip_kernel_s();
  k->name = kernel_name;
  k->device = dev;
  hipError_t e = hipModuleLoadData(&k->module, code.data());
  if (e != hipSuccess) {
    delete k;
    return check_hip(e, "hipModuleLoadData");
  }
  e = hipModuleGetFunction(&k->function, k->module, kernel_name);
  if (e != hipSuccess) {
    (void)hipModuleUnload(k->module);
    delete k;
    return check_hip(e, "hipModuleGetFunction");
  }
  *out = k;
  return SAREK_HIP_OK;
}

}  // namespace

// Bumped whenever the compile cache is emptied: handles of cached kernels kept elsewhere are stale from then on.
std::atomic<uint64_t> g_kernel_cache_generation{1};
uint64_t kernel_cache_generation() { return g_kernel_cache_generation.load(std::memory_order_acquire); }
}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" {

int sarek_hip_init(void) {
  std::lock_guard<std::mutex> lock(g_mu);
  if (g_inited) return SAREK_HIP_OK;
  SAREK_HIP_TRY(hipInit(0));
  g_inited = true;
  return SAREK_HIP_OK;
}

int sarek_hip_is_available(void) {
  int n = 0;
  if (hipInit(0) != hipSuccess) return 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n > 0 ? 1 : 0;
}

int sarek_hip_device_count(int *count) {
  if (!count) return fail(SAREK_HIP_E_INVALID_ARG, "device_count: NULL out pointer");
  SAREK_HIP_TRY(hipGetDeviceCount(count));
  return SAREK_HIP_OK;
}

int sarek_hip_device_get_info(int device, sarek_hip_device_info *out) {
  if (!out) return fail(SAREK_HIP_E_INVALID_ARG, "device_get_info: NULL out pointer");
  hipDeviceProp_t p;
  SAREK_HIP_TRY(hipGetDeviceProperties(&p, device));
  std::memset(out, 0, sizeof(*out));
  std::strncpy(out->name, p.name, sizeof(out->name) - 1);
  std::strncpy(out->gcn_arch, p.gcnArchName, sizeof(out->gcn_arch) - 1);
  out->total_global_mem = p.totalGlobalMem;
  out->max_threads_per_block = p.maxThreadsPerBlock;
  for (int i = 0; i < 3; ++i) {
    out->max_block_dim[i] = p.maxThreadsDim[i];
    out->max_grid_dim[i] = p.maxGridSize[i];
  }
  out->shared_mem_per_block = static_cast<int>(p.sharedMemPerBlock);
  out->warp_size = p.warpSize;
  out->multiprocessor_count = p.multiProcessorCount;
  out->clock_rate_khz = p.clockRate;
  out->memory_clock_rate_khz = p.memoryClockRate;
  out->memory_bus_width_bits = p.memoryBusWidth;
  out->l2_cache_size = p.l2CacheSize;
  out->compute_major = p.major;
  out->compute_minor = p.minor;
  out->max_registers_per_block = p.regsPerBlock;
  return SAREK_HIP_OK;
}

int sarek_hip_device_info_size(void) { return static_cast<int>(sizeof(sarek_hip_device_info)); }

int sarek_hip_device_set_current(int device) {
  SAREK_HIP_TRY(hipSetDevice(device));
  return SAREK_HIP_OK;
}

int sarek_hip_device_get_current(int *device) {
  if (!device) return fail(SAREK_HIP_E_INVALID_ARG, "device_get_current: NULL out pointer");
  SAREK_HIP_TRY(hipGetDevice(device));
  return SAREK_HIP_OK;
}

int sarek_hip_device_synchronize(void) {
  SAREK_HIP_TRY(hipDeviceSynchronize());
  return SAREK_HIP_OK;
}

int sarek_hip_mem_get_info(size_t *free_bytes, size_t *total_bytes) {
  if (!free_bytes || !total_bytes) return fail(SAREK_HIP_E_INVALID_ARG, "mem_get_info: NULL out pointer");
  SAREK_HIP_TRY(hipMemGetInfo(free_bytes, total_bytes));
  return SAREK_HIP_OK;
}

int sarek_hip_driver_version(int *version) {
  if (!version) return fail(SAREK_HIP_E_INVALID_ARG, "driver_version: NULL out pointer");
  SAREK_HIP_TRY(hipDriverGetVersion(version));
  return SAREK_HIP_OK;
}

int sarek_hip_mem_alloc(void **dptr, size_t bytes) {
  if (!dptr) return fail(SAREK_HIP_E_INVALID_ARG, "mem_alloc: NULL out pointer");
  *dptr = nullptr;
  // A zero-length vector still needs a distinct, freeable handle.
  SAREK_HIP_TRY(hipMalloc(dptr, bytes ? bytes : 1));
  std::lock_guard<std::mutex> lock(g_mu);
  g_live_allocs.insert(*dptr);
  return SAREK_HIP_OK;
}

int sarek_hip_mem_free(void *dptr) {
  if (!dptr) return SAREK_HIP_OK;
  {
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_live_allocs.find(dptr);
    if (it == g_live_allocs.end()) return SAREK_HIP_OK;  // already freed (or not ours): no-op
    g_live_allocs.erase(it);
  }
  SAREK_HIP_TRY(hipFree(dptr));
  return SAREK_HIP_OK;
}

int sarek_hip_memcpy_dtod(void *dst_device, const void *src_device, size_t bytes) {
  if (bytes == 0) return SAREK_HIP_OK;
  if (!dst_device || !src_device) return fail(SAREK_HIP_E_INVALID_ARG, "memcpy_dtod: NULL pointer");
  SAREK_HIP_TRY(hipMemcpy(dst_device, src_device, bytes, hipMemcpyDeviceToDevice));
  return SAREK_HIP_OK;
}

int sarek_hip_memset_d8(void *dst_device, unsigned char value, size_t bytes) {
  if (bytes == 0) return SAREK_HIP_OK;
  if (!dst_device) return fail(SAREK_HIP_E_INVALID_ARG, "memset_d8: NULL pointer");
  SAREK_HIP_TRY(hipMemset(dst_device, value, bytes));
  return SAREK_HIP_OK;
}

int sarek_hip_stream_create(sarek_hip_stream *out) {
  if (!out) return fail(SAREK_HIP_E_INVALID_ARG, "stream_create: NULL out pointer");
  hipStream_t s;
  SAREK_HIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *out = s;
  return SAREK_HIP_OK;
}

int sarek_hip_stream_destroy(sarek_hip_stream s) {
  if (!s) return SAREK_HIP_OK;
  SAREK_HIP_TRY(hipStreamDestroy(as_stream(s)));
  return SAREK_HIP_OK;
}

int sarek_hip_stream_synchronize(sarek_hip_stream s) {
  SAREK_HIP_TRY(hipStreamSynchronize(as_stream(s)));
  return SAREK_HIP_OK;
}

int sarek_hip_event_create(sarek_hip_event *out) {
  if (!out) return fail(SAREK_HIP_E_INVALID_ARG, "event_create: NULL out pointer");
  hipEvent_t e;
  SAREK_HIP_TRY(hipEventCreate(&e));
  *out = e;
  return SAREK_HIP_OK;
}

int sarek_hip_event_destroy(sarek_hip_event e) {
  if (!e) return SAREK_HIP_OK;
  SAREK_HIP_TRY(hipEventDestroy(reinterpret_cast<hipEvent_t>(e)));
  return SAREK_HIP_OK;
}

int sarek_hip_event_record(sarek_hip_event e, sarek_hip_stream s) {
  if (!e) return fail(SAREK_HIP_E_INVALID_ARG, "event_record: NULL event");
  SAREK_HIP_TRY(hipEventRecord(reinterpret_cast<hipEvent_t>(e), as_stream(s)));
  return SAREK_HIP_OK;
}

int sarek_hip_event_synchronize(sarek_hip_event e) {
  if (!e) return fail(SAREK_HIP_E_INVALID_ARG, "event_synchronize: NULL event");
  SAREK_HIP_TRY(hipEventSynchronize(reinterpret_cast<hipEvent_t>(e)));
  return SAREK_HIP_OK;
}

int sarek_hip_event_elapsed_ms(sarek_hip_event start, sarek_hip_event stop, float *ms) {
  if (!start || !stop || !ms) return fail(SAREK_HIP_E_INVALID_ARG, "event_elapsed_ms: NULL argument");
  SAREK_HIP_TRY(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start),
                                    reinterpret_cast<hipEvent_t>(stop)));
  return SAREK_HIP_OK;
}

int sarek_hip_profiler_start(void) {
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wdeprecated-declarations"
  if (hipProfilerStart() != hipSuccess) (void)hipGetLastError();
#pragma clang diagnostic pop
  return SAREK_HIP_OK;
}

int sarek_hip_profiler_stop(void) {
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wdeprecated-declarations"
  if (hipProfilerStop() != hipSuccess) (void)hipGetLastError();
#pragma clang diagnostic pop
  return SAREK_HIP_OK;
}

int sarek_hip_kernel_compile(const char *source, const char *kernel_name, sarek_hip_kernel *out,
                             char *log, size_t log_len) {
  return compile_impl(source, kernel_name, out, log, log_len);
}

int sarek_hip_kernel_compile_cached(const char *source, const char *kernel_name,
                                    sarek_hip_kernel *out, char *log, size_t log_len) {
  if (!source || !kernel_name || !out)
    return fail(SAREK_HIP_E_INVALID_ARG, "kernel_compile_cached: NULL argument");
  int dev = 0;
  SAREK_HIP_TRY(hipGetDevice(&dev));
  const size_t len = std::strlen(source);
  const uint64_t key = hash_text(source, len) ^ (static_cast<uint64_t>(dev) << 56);
  auto find = [&]() -> sarek_hip_kernel {
    auto it = g_kernel_cache.find(key);
    if (it == g_kernel_cache.end()) return nullptr;
    for (const CachedKernel &c : it->second)
      if (c.dev == dev && c.source.size() == len && c.name == kernel_name &&
          std::memcmp(c.source.data(), source, len) == 0)
        return c.kernel;
    return nullptr;
  };
  {
    std::lock_guard<std::mutex> lock(g_mu);
    if (sarek_hip_kernel hit = find()) {
      *out = hit;
      if (log && log_len) log[0] = '\0';
      return SAREK_HIP_OK;
    }
  }
  sarek_hip_kernel k = nullptr;
  int rc = compile_impl(source, kernel_name, &k, log, log_len);
  if (rc != SAREK_HIP_OK) return rc;
  k->cached = true;
  std::lock_guard<std::mutex> lock(g_mu);
  if (sarek_hip_kernel other = find()) {  // another thread compiled the same source meanwhile
    (void)hipModuleUnload(k->module);
    delete k;
    *out = other;
    return SAREK_HIP_OK;
  }
  g_kernel_cache[key].push_back({dev, kernel_name, std::string(source, len), k});
  *out = k;
  return SAREK_HIP_OK;
}

int sarek_hip_kernel_clear_cache(void) {
  std::lock_guard<std::mutex> lock(g_mu);
  g_kernel_cache_generation.fetch_add(1, std::memory_order_release);
  for (auto &bucket : g_kernel_cache)
    for (CachedKernel &c : bucket.second) {
      (void)hipModuleUnload(c.kernel->module);
      delete c.kernel;
    }
  g_kernel_cache.clear();
  return SAREK_HIP_OK;
}

int sarek_hip_kernel_destroy(sarek_hip_kernel k) {
  if (!k || k->cached) return SAREK_HIP_OK;  // cached kernels live until clear_cache
  hipError_t e = hipModuleUnload(k->module);
  delete k;
  return check_hip(e, "hipModuleUnload");
}

int sarek_hip_kernel_launch(sarek_hip_kernel k, const unsigned grid[3], const unsigned block[3],
                            unsigned shared_mem_bytes, sarek_hip_stream stream, void **params,
                            int n_params) {
  if (!k || !grid || !block) return fail(SAREK_HIP_E_INVALID_ARG, "kernel_launch: NULL argument");
  if (n_params > 0 && !params) return fail(SAREK_HIP_E_INVALID_ARG, "kernel_launch: NULL params");
  for (int i = 0; i < 3; ++i)
    if (grid[i] == 0 || block[i] == 0)
      return fail(SAREK_HIP_E_INVALID_ARG, "kernel_launch: zero grid or block dimension");
  // A launch that asks for more dynamic LDS than a kernel gets by default (?shared_mem of Execute.run_vectors above
  // 48 KiB; a CU has 160 KiB) needs the kernel's limit raised first, once per kernel and size.
  if (shared_mem_bytes > k->dynamic_lds_allowed.load(std::memory_order_acquire)) {
    SAREK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(k->function),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(shared_mem_bytes)));
    k->dynamic_lds_allowed.store(shared_mem_bytes, std::memory_order_release);
  }
  SAREK_HIP_TRY(hipModuleLaunchKernel(k->function, grid[0], grid[1], grid[2], block[0], block[1],
                                      block[2], shared_mem_bytes, as_stream(stream), params,
                                      nullptr));
  return SAREK_HIP_OK;
}
}
