// Host <-> device copies behind Memory.host_ptr_to_device / device_to_host_ptr
// (sarek/core/Transfer.ml:228-333 hands over the vector's whole host block, a pageable
// Bigarray, and expects the copy to be complete on return).
//
// A pageable block cannot be read by the DMA engines, so the driver's own hipMemcpy
// bounces it through one pinned buffer on one thread: 29 GB/s up and 17 GB/s down on an
// MI355X box whose PCIe link carries 57.6 GB/s from pinned memory.  Large copies are
// therefore cut into chunks and handled by a few host threads, each with two pinned
// staging slots and a stream of its own: while the DMA engine drains one slot the thread
// fills the other, and several threads together copy faster than the link.  Measured with
// 4 threads: 55 GB/s up and 46-55 GB/s down at 1 GiB, 41 / 32 GB/s at 16 MiB.
//
// Blocks the caller allocated with sarek_hip_host_alloc are pinned already and go to the
// DMA engines directly.
#include <algorithm>
#include <condition_variable>
#include <cstring>
#include <mutex>
#include <cstdint>
#include <thread>
#include <vector>

#include "common.hpp"
#include "tunables.hpp"

namespace sarek_hip {
namespace {

constexpr int kMaxThreads = 16;
constexpr int kMaxDevices = 64;
constexpr size_t kMinChunk = 1 << 20;
// Sizes from which the staged copy beats the driver's (measured, MI355X box, PCIe 5 x16).
constexpr int64_t kMinUploadKib = 12 << 10, kMinDownloadKib = 2 << 10;

struct Lane {                 // one host thread's share of the staging pool
  hipStream_t stream = nullptr;
  char *slot[2] = {nullptr, nullptr};
  hipEvent_t drained[2] = {nullptr, nullptr};   // the DMA out of / into the slot has finished
};

struct Pool {                 // per device; lives until the process ends
  std::vector<Lane> lanes;
  size_t chunk = 0;
};

Pool g_pools[kMaxDevices];

void release(Pool &p) {
  for (Lane &l : p.lanes) {
    if (l.stream) (void)hipStreamDestroy(l.stream);
    for (int b = 0; b < 2; ++b) {
      if (l.slot[b]) (void)hipHostFree(l.slot[b]);
      if (l.drained[b]) (void)hipEventDestroy(l.drained[b]);
    }
  }
  p.lanes.clear();
  p.chunk = 0;
}

// Pool of `threads` lanes with `chunk`-byte slots on the current device (rebuilt when a
// tunable changed the shape).  Called by the one staged copy in progress.
int prepare(Pool &p, int threads, size_t chunk) {
  if (static_cast<int>(p.lanes.size()) == threads && p.chunk == chunk) return SAREK_HIP_OK;
  release(p);
  p.lanes.resize(threads);
  p.chunk = chunk;
  for (Lane &l : p.lanes) {
    int st = check_hip(hipStreamCreateWithFlags(&l.stream, hipStreamNonBlocking), "staging stream");
    for (int b = 0; b < 2 && st == SAREK_HIP_OK; ++b) {
      st = check_hip(hipHostMalloc(reinterpret_cast<void **>(&l.slot[b]), chunk, hipHostMallocDefault),
                     "staging slot (pinned host memory)");
      if (st == SAREK_HIP_OK)
        st = check_hip(hipEventCreateWithFlags(&l.drained[b], hipEventDisableTiming), "staging event");
    }
    if (st != SAREK_HIP_OK) {
      release(p);
      return st;
    }
  }
  return SAREK_HIP_OK;
}

// Chunks lane, lane + T, lane + 2T ... of the copy, alternating between the lane's two slots.
hipError_t lane_upload(Lane &l, int lane, int T, size_t chunk, char *dev, const char *host, size_t bytes) {
  const size_t nchunks = (bytes + chunk - 1) / chunk;
  int k = 0;
  for (size_t c = lane; c < nchunks; c += T, ++k) {
    const int b = k & 1;
    const size_t off = c * chunk, len = std::min(chunk, bytes - off);
    hipError_t e;
    if (k >= 2 && (e = hipEventSynchronize(l.drained[b])) != hipSuccess) return e;
    std::memcpy(l.slot[b], host + off, len);
    if ((e = hipMemcpyAsync(dev + off, l.slot[b], len, hipMemcpyHostToDevice, l.stream)) != hipSuccess) return e;
    if ((e = hipEventRecord(l.drained[b], l.stream)) != hipSuccess) return e;
  }
  return hipStreamSynchronize(l.stream);
}

hipError_t lane_download(Lane &l, int lane, int T, size_t chunk, char *host, const char *dev, size_t bytes) {
  const size_t nchunks = (bytes + chunk - 1) / chunk;
  size_t held_off[2] = {0, 0}, held_len[2] = {0, 0};   // what each slot holds for the host copy
  auto unload = [&](int b) -> hipError_t {
    if (held_len[b] == 0) return hipSuccess;
    hipError_t e = hipEventSynchronize(l.drained[b]);
    if (e != hipSuccess) return e;
    std::memcpy(host + held_off[b], l.slot[b], held_len[b]);
    held_len[b] = 0;
    return hipSuccess;
  };
  int k = 0;
  for (size_t c = lane; c < nchunks; c += T, ++k) {
    const int b = k & 1;
    const size_t off = c * chunk, len = std::min(chunk, bytes - off);
    hipError_t e;
    if ((e = unload(b)) != hipSuccess) return e;
    if ((e = hipMemcpyAsync(l.slot[b], dev + off, len, hipMemcpyDeviceToHost, l.stream)) != hipSuccess) return e;
    if ((e = hipEventRecord(l.drained[b], l.stream)) != hipSuccess) return e;
    held_off[b] = off;
    held_len[b] = len;
  }
  hipError_t e = unload(k & 1);                  // the older of the two slots first
  if (e == hipSuccess) e = unload((k + 1) & 1);
  if (e != hipSuccess) (void)hipStreamSynchronize(l.stream);   // leave no DMA in flight into the slots
  return e;
}

bool is_pinned(const void *host) {
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, host) != hipSuccess) {
    (void)hipGetLastError();          // an ordinary malloc'd block: not an error for the caller
    return false;
  }
  return attr.type == hipMemoryTypeHost;
}

// The helper threads of the staged copies.  They are started on first use, sleep between
// copies and are never joined: the object is allocated once and left alone at process
// exit, so a thread that is still parked then touches nothing that has been destroyed.
struct Job {
  bool upload;
  char *dst;
  const char *src;
  size_t bytes, chunk;
  int T, dev;
  Pool *pool;
};

hipError_t run_lane(const Job &j, int lane) {
  hipError_t e = hipSetDevice(j.dev);
  if (e != hipSuccess) return e;
  Lane &l = j.pool->lanes[lane];
  return j.upload ? lane_upload(l, lane, j.T, j.chunk, j.dst, j.src, j.bytes)
                  : lane_download(l, lane, j.T, j.chunk, j.dst, j.src, j.bytes);
}

struct Crew {
  std::mutex mu;
  std::condition_variable wake, finished;
  uint64_t generation = 0;
  int pending = 0;
  int started = 0;                       // helper threads so far; helper i serves lane i + 1
  Job job{};
  hipError_t results[kMaxThreads] = {};

  void helper(int lane, uint64_t seen) {
    for (;;) {
      Job j;
      {
        std::unique_lock<std::mutex> lock(mu);
        wake.wait(lock, [&] { return generation != seen; });
        seen = generation;
        if (lane >= job.T) continue;
        j = job;
      }
      const hipError_t e = run_lane(j, lane);
      std::lock_guard<std::mutex> lock(mu);
      results[lane] = e;
      if (--pending == 0) finished.notify_one();
    }
  }

  // Runs lanes 0..T-1 of `j` (lane 0 on the calling thread) and returns the first failure.
  hipError_t run(const Job &j) {
    {
      std::lock_guard<std::mutex> lock(mu);
      for (; started < j.T - 1; ++started)
        std::thread(&Crew::helper, this, started + 1, generation).detach();
      job = j;
      pending = j.T - 1;
      ++generation;
    }
    wake.notify_all();
    const hipError_t mine = run_lane(j, 0);
    std::unique_lock<std::mutex> lock(mu);
    finished.wait(lock, [&] { return pending == 0; });
    if (mine != hipSuccess) return mine;
    for (int lane = 1; lane < j.T; ++lane)
      if (results[lane] != hipSuccess) return results[lane];
    return hipSuccess;
  }
};

Crew &crew() {
  static Crew *c = new Crew;             // never deleted, see above
  return *c;
}
std::mutex g_crew_busy;                  // one staged copy at a time (all devices share the crew)

int staged_copy(bool upload, void *dst, const void *src, size_t bytes, const char *what) {
  const void *host = upload ? src : dst;
  const int threads = static_cast<int>(
      std::clamp<int64_t>(tunable("transfer.threads", 4), 0, kMaxThreads));
  const size_t slot = static_cast<size_t>(std::clamp<int64_t>(tunable("transfer.chunk_kib", 8192), 1024, 1 << 20)) << 10;
  const size_t least = static_cast<size_t>(std::max<int64_t>(
      upload ? tunable("transfer.min_up_kib", kMinUploadKib) : tunable("transfer.min_down_kib", kMinDownloadKib), 0)) << 10;
  int dev = 0;
  SAREK_HIP_TRY(hipGetDevice(&dev));
  if (threads == 0 || bytes < least || bytes < 2 * kMinChunk || dev >= kMaxDevices || is_pinned(host)) {
    SAREK_HIP_TRY(hipMemcpy(dst, src, bytes, upload ? hipMemcpyHostToDevice : hipMemcpyDeviceToHost));
    return SAREK_HIP_OK;
  }
  // The first chunk's host copy and the last chunk's DMA are not overlapped with anything,
  // so a short copy is cut finer than a long one: about 8 chunks per thread, but no finer
  // than 1 MiB (below that the per-chunk calls cost more than the DMA they start).
  const size_t chunk = std::clamp((bytes / (8 * static_cast<size_t>(threads)) + kMinChunk - 1) / kMinChunk * kMinChunk,
                                  kMinChunk, slot);
  // hipMemcpy orders itself after everything the default stream was given; the staging
  // streams do not, so wait for the device first (earlier kernels may read or write `dst`/`src`).
  SAREK_HIP_TRY(hipDeviceSynchronize());
  std::lock_guard<std::mutex> lock(g_crew_busy);
  Pool &pool = g_pools[dev];
  const int st = prepare(pool, threads, slot);
  if (st != SAREK_HIP_OK) return st;
  Job job{upload, static_cast<char *>(dst), static_cast<const char *>(src), bytes, chunk,
          static_cast<int>(std::min<size_t>(threads, (bytes + chunk - 1) / chunk)), dev, &pool};
  return check_hip(crew().run(job), what);
}

}  // namespace
}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" {

int sarek_hip_memcpy_htod(void *dst_device, const void *src_host, size_t bytes) {
  if (bytes == 0) return SAREK_HIP_OK;
  if (!dst_device || !src_host) return fail(SAREK_HIP_E_INVALID_ARG, "memcpy_htod: NULL pointer");
  return staged_copy(true, dst_device, src_host, bytes, "memcpy_htod");
}

int sarek_hip_memcpy_dtoh(void *dst_host, const void *src_device, size_t bytes) {
  if (bytes == 0) return SAREK_HIP_OK;
  if (!dst_host || !src_device) return fail(SAREK_HIP_E_INVALID_ARG, "memcpy_dtoh: NULL pointer");
  return staged_copy(false, dst_host, src_device, bytes, "memcpy_dtoh");
}

int sarek_hip_host_alloc(void **host_ptr, size_t bytes) {
  if (!host_ptr) return fail(SAREK_HIP_E_INVALID_ARG, "host_alloc: NULL out pointer");
  *host_ptr = nullptr;
  SAREK_HIP_TRY(hipHostMalloc(host_ptr, bytes ? bytes : 1, hipHostMallocDefault));
  return SAREK_HIP_OK;
}

int sarek_hip_mem_alloc_zero_copy(void *host_ptr, size_t bytes, void **dptr, int *supported) {
  if (!dptr || !supported) return fail(SAREK_HIP_E_INVALID_ARG, "alloc_zero_copy: NULL out pointer");
  *dptr = nullptr;
  *supported = 0;
  (void)bytes;
  if (!host_ptr || !is_pinned(host_ptr)) return SAREK_HIP_OK;      // None: the caller allocates and copies
  void *alias = nullptr;
  if (hipHostGetDevicePointer(&alias, host_ptr, 0) != hipSuccess || !alias) {
    (void)hipGetLastError();
    return SAREK_HIP_OK;
  }
  *dptr = alias;
  *supported = 1;
  return SAREK_HIP_OK;
}

int sarek_hip_host_free(void *host_ptr) {
  if (!host_ptr) return SAREK_HIP_OK;
  SAREK_HIP_TRY(hipHostFree(host_ptr));
  return SAREK_HIP_OK;
}

}  // extern "C"
