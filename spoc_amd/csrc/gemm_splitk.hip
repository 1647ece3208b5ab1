// What the GEMMs share when a product with few tiles and a long K is cut along K over several workgroups per tile:
// device memory for the partial M x N planes, and the kernel that adds them up.
#include <map>
#include <mutex>
#include <utility>

#include "common.hpp"
#include "gemm_common.hpp"

namespace sarek_hip {
namespace {

typedef __attribute__((ext_vector_type(4))) float f32x4_t;

// Adds the `splits` partial planes into C, plane 0 first: a fixed order, so the result does not depend on which
// workgroup finished when.  mn is a multiple of 4 and both pointers are 16-byte aligned (the callers' conditions).
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ partials, float *__restrict__ C,
                                                            int64_t mn, int splits) {
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
  if (i >= mn) return;
  f32x4_t acc = *reinterpret_cast<const f32x4_t *>(partials + i);
  for (int s = 1; s < splits; ++s) acc += *reinterpret_cast<const f32x4_t *>(partials + s * mn + i);
  *reinterpret_cast<f32x4_t *>(C + i) = acc;
}

}  // namespace

// One block of kSplitWorkspaceBytes per (device, stream), allocated at the first call that wants one on that stream and
// kept until the process ends (never grown or freed, so a pointer handed out stays good whatever other threads do):
// calls on different streams never share one, calls on one stream are ordered by it.  nullptr (the caller then works
// without one: no K split, row sums by atomicAdd) for a stream under capture -- a recorded graph would carry the
// block's address to wherever it is replayed, next to eager calls or other replays that use the same block --, past 16
// streams, or when the allocation fails.
float *splitk_workspace(hipStream_t st) {
  static std::mutex mu;
  static std::map<std::pair<int, hipStream_t>, void *> blocks;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(mu);
  auto it = blocks.find({dev, st});
  if (it != blocks.end()) return static_cast<float *>(it->second);
  if (blocks.size() >= 16) return nullptr;
  void *p = nullptr;
  if (hipMalloc(&p, kSplitWorkspaceBytes) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  blocks[{dev, st}] = p;
  return static_cast<float *>(p);
}

int launch_splitk_reduce(const float *partials, float *c, int64_t mn, int splits, hipStream_t st) {
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3(static_cast<unsigned>((mn / 4 + 255) / 256)), dim3(256), 0, st, partials,
                     c, mn, splits);
  return check_launch("split-K reduction launch");
}

}  // namespace sarek_hip
