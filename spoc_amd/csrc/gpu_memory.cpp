// Bookkeeping of the device memory that vectors hold, and the retry of an allocation after the host
// has released what it no longer reaches (sarek/core/Gpu_memory.ml:20-141).  In the reference this
// is backend-agnostic OCaml called from Transfer.ensure_buffer / free_buffer / free_all_buffers
// (Transfer.ml:184,218,359,375) and from the finaliser of a vector; a host without OCaml gets it here,
// driven by the native Vector layer.  The garbage collector's part is a callback: the host language
// registers what "collect now" means for it.
#include <atomic>
#include <string>

#include "common.hpp"
#include "gpu_memory.hpp"
#include "sarek_hip.h"

namespace sarek_hip {
namespace {

std::atomic<bool> g_auto_gc{true};                       // Gpu_memory.auto_gc
std::atomic<int64_t> g_allocated{0}, g_peak{0};          // allocated_bytes, peak_bytes
std::atomic<int64_t> g_allocs{0}, g_frees{0}, g_gc_frees{0}, g_gc_freed_bytes{0}, g_retries{0};
std::atomic<sarek_hip_reclaim_fn> g_reclaim{nullptr};
std::atomic<void *> g_reclaim_ctx{nullptr};

void reclaim(int attempt) {
  if (sarek_hip_reclaim_fn fn = g_reclaim.load()) fn(g_reclaim_ctx.load(), attempt);
}

}  // namespace

void track_gc_free(int64_t bytes) {                      // Gpu_memory.register_finalizer's body, per buffer
  g_gc_frees.fetch_add(1);
  g_gc_freed_bytes.fetch_add(bytes);
  g_allocated.fetch_sub(bytes);
}

}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" {

void sarek_hip_gpu_memory_set_auto_gc(int enabled) { g_auto_gc.store(enabled != 0); }
int sarek_hip_gpu_memory_get_auto_gc(void) { return g_auto_gc.load() ? 1 : 0; }

void sarek_hip_gpu_memory_track_alloc(int64_t bytes) {
  g_allocs.fetch_add(1);
  const int64_t current = g_allocated.fetch_add(bytes) + bytes;
  int64_t peak = g_peak.load();
  while (current > peak && !g_peak.compare_exchange_weak(peak, current)) {
  }
}

void sarek_hip_gpu_memory_track_free(int64_t bytes) {
  g_frees.fetch_add(1);
  g_allocated.fetch_sub(bytes);
}

int64_t sarek_hip_gpu_memory_usage(void) { return g_allocated.load(); }
int64_t sarek_hip_gpu_memory_peak_usage(void) { return g_peak.load(); }

int sarek_hip_gpu_memory_stats(sarek_hip_gpu_memory_stats_t *out) {
  if (!out) return fail(SAREK_HIP_E_INVALID_ARG, "gpu_memory_stats: NULL result");
  out->current_bytes = g_allocated.load();
  out->peak_bytes = g_peak.load();
  out->alloc_count = g_allocs.load();
  out->free_count = g_frees.load();
  out->gc_free_count = g_gc_frees.load();
  out->gc_freed_bytes = g_gc_freed_bytes.load();
  out->retry_count = g_retries.load();
  return SAREK_HIP_OK;
}

void sarek_hip_gpu_memory_reset_stats(void) {
  for (auto *c : {&g_allocated, &g_peak, &g_allocs, &g_frees, &g_gc_frees, &g_gc_freed_bytes, &g_retries}) c->store(0);
}

void sarek_hip_gpu_memory_set_reclaim(sarek_hip_reclaim_fn fn, void *ctx) {
  g_reclaim_ctx.store(ctx);
  g_reclaim.store(fn);
}

void sarek_hip_gpu_memory_trigger_gc(void) { reclaim(1); }

// Gpu_memory.with_retry: up to three attempts, the host's collector between them (first a full
// collection, then a compaction), and the FIRST failure is the one reported.
int sarek_hip_gpu_memory_with_retry(sarek_hip_attempt_fn attempt, void *ctx) {
  if (!attempt) return fail(SAREK_HIP_E_INVALID_ARG, "gpu_memory_with_retry: NULL function");
  int first = attempt(ctx);
  if (first == SAREK_HIP_OK || !g_auto_gc.load()) return first;
  const std::string first_message = last_error_slot();
  for (int round = 1; round <= 2; ++round) {
    g_retries.fetch_add(1);
    reclaim(round);
    if (attempt(ctx) == SAREK_HIP_OK) return SAREK_HIP_OK;
  }
  last_error_slot() = first_message;
  return first;
}

}  // extern "C"
