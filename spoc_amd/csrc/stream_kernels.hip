// Bandwidth-bound kernels of the sarek-hip hot path for gfx950 (wave64):
// stream triad, fused triad+sum, block-256 sum / dot product, the double fold of
// partials and the f32 -> bf16/fp16 input casts.
//
// Design: every global access is a 128-bit (float4) coalesced load or store marked
// non-temporal (nothing is re-read), each thread keeps 8 independent 128-bit loads in
// flight, and the grid is "one shot": one 256-thread workgroup per 4096 elements and no
// grid-stride loop, which measured ~8 % faster on MI355X than any persistent-grid shape
// (the hardware dispatcher balances the 8 XCDs better than a fixed stride does).  Sums go
// lane -> DPP wave reduction -> LDS across the waves of a block -> one f32 partial per
// block -> a fold kernel in double (fixed order; long folds: 256 workgroups, the last to finish adds
// their sums).  Folding inside the triad
// kernel ("last workgroup to arrive") was measured and rejected: on this multi-XCD chip a
// device-scope fence writes back a whole L2 (7x slower) and publishing the partials with
// device-scope atomics instead still cost 25 % of the bandwidth.
#include <atomic>
#include <map>
#include <mutex>
#include <utility>

#include "common.hpp"
#include "tunables.hpp"

namespace sarek_hip {
namespace {

constexpr int kBlock = 256;   // threads per workgroup (4 waves)
constexpr int kUnroll = 4;    // float4 per thread
constexpr int kChunk = kBlock * kUnroll;   // float4 per workgroup (4096 elements)

// ---- wave64 sum by DPP -------------------------------------------------------
template <int Ctrl>
__device__ __forceinline__ float dpp_add(float v) {
  int iv = __builtin_bit_cast(int, v);
  int sh = __builtin_amdgcn_update_dpp(0, iv, Ctrl, 0xF, 0xF, true);
  return v + __builtin_bit_cast(float, sh);
}

// Sum over the 64 lanes of a wave; the result is valid in every lane.
__device__ __forceinline__ float wave_sum(float v) {
  v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x141>(v);  // row_half_mirror: lane i <-> 7-i within each 8 lanes: sums of 8
  v = dpp_add<0x140>(v);  // row_mirror: sums of 16, valid in all 16 lanes of a row
  int iv = __builtin_bit_cast(int, v);
  float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0));
  float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16));
  float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32));
  float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
  return (r0 + r1) + (r2 + r3);
}

// The same for a double: both halves moved by the same lane pattern.
template <int Ctrl>
__device__ __forceinline__ double dpp_add(double v) {
  const long long bits = __builtin_bit_cast(long long, v);
  const int lo = __builtin_amdgcn_update_dpp(0, static_cast<int>(bits), Ctrl, 0xF, 0xF, true);
  const int hi = __builtin_amdgcn_update_dpp(0, static_cast<int>(bits >> 32), Ctrl, 0xF, 0xF, true);
  const long long moved = (static_cast<long long>(hi) << 32) | static_cast<unsigned int>(lo);
  return v + __builtin_bit_cast(double, moved);
}
__device__ __forceinline__ double readlane(double v, int lane) {
  const long long bits = __builtin_bit_cast(long long, v);
  const int lo = __builtin_amdgcn_readlane(static_cast<int>(bits), lane);
  const int hi = __builtin_amdgcn_readlane(static_cast<int>(bits >> 32), lane);
  return __builtin_bit_cast(double, (static_cast<long long>(hi) << 32) | static_cast<unsigned int>(lo));
}
// Sum over the 64 lanes of a wave in a fixed order; every lane of the wave takes part, the result is valid in all.
__device__ __forceinline__ double wave_sum(double v) {
  v = dpp_add<0xB1>(v);
  v = dpp_add<0x4E>(v);
  v = dpp_add<0x141>(v);
  v = dpp_add<0x140>(v);
  return (readlane(v, 0) + readlane(v, 16)) + (readlane(v, 32) + readlane(v, 48));
}

// Sum over a 256-thread block; valid in thread 0.
__device__ __forceinline__ float block_sum(float v) {
  __shared__ float wave_part[kBlock / 64];
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) wave_part[wave] = v;
  __syncthreads();
  float r = 0.f;
  if (threadIdx.x == 0) r = (wave_part[0] + wave_part[1]) + (wave_part[2] + wave_part[3]);
  return r;
}

// One triad element with the Native backend's rounding: operands widen to double,
// the product of two binary32 values is exact in double, one double addition, one
// rounding to binary32.
__device__ __forceinline__ float triad1(float b, float c, double s) {
  return static_cast<float>(static_cast<double>(b) + static_cast<double>(c) * s);
}

__device__ __forceinline__ float4 triad4(float4 b, float4 c, double s) {
  return make_float4(triad1(b.x, c.x, s), triad1(b.y, c.y, s), triad1(b.z, c.z, s),
                     triad1(b.w, c.w, s));
}

typedef float f32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 ldg_nt(const float4 *p) {
  f32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(p));
  return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void stg_nt(float4 *p, float4 v) {
  f32x4_t w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, reinterpret_cast<f32x4_t *>(p));
}

// What a triad launch leaves besides `a`.
enum : int {
  SUM_NONE = 0,
  SUM_WORKGROUP = 1,   // partials[g] = f32 sum of workgroup g's 4096 elements
  SUM_BLOCK256 = 2     // partials[j] = f32 sum of a[256j .. 256j+255], the reference's block-256 kernel's output
};

// a = b + c*s.  Workgroup g owns float4 [g*kChunk, (g+1)*kChunk); the last one also takes
// the (n & 3) scalar tail.  Each float4 slot of a wave (64 lanes x 4 elements) is one 256-element
// block of the reference's tree kernel, so SUM_BLOCK256 needs one wave reduction per load and no
// LDS; its lane and wave order is block256_kernel's, the results are the same bits.
// Runs: 0 = a wave's float4 slots lie a workgroup's width apart (one KiB every four KiB); 1 = a wave owns
// four consecutive KiB, so its four block sums are neighbours and leave as one 16-byte store by lane 0
// (measured at n = 2^28: 506 against 515 us for four 4-byte stores per wave; the plain triad 501).
template <int Sum, bool NtLoad = true, int Runs = 0>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(8, 8))) void triad_kernel(float *__restrict__ a,
                                                       const float *__restrict__ b,
                                                       const float *__restrict__ c, float s,
                                                       int64_t n, float *__restrict__ partials) {
  const double sd = static_cast<double>(s);
  const int64_t n4 = n >> 2;
  float4 *a4 = reinterpret_cast<float4 *>(a);
  const float4 *b4 = reinterpret_cast<const float4 *>(b);
  const float4 *c4 = reinterpret_cast<const float4 *>(c);
  constexpr int kStep = Runs ? 64 : kBlock;   // float4 between two slots of a thread
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kChunk +
                       (Runs ? (threadIdx.x >> 6) * (64 * kUnroll) + (threadIdx.x & 63) : threadIdx.x);
  const bool full = base + (kUnroll - 1) * kStep < n4;
  float4 r[kUnroll];
  // SUM_BLOCK256: the scalar tail's share of the block that holds it.  It starts at -0, the one value whose addition
  // changes nothing: a block of 256 elements that are all -0 sums to -0, as in block256_kernel.
  float extra[kUnroll];
  if (full) {
    float4 bv[kUnroll], cv[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) bv[u] = NtLoad ? ldg_nt(b4 + base + u * kStep) : b4[base + u * kStep];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) cv[u] = NtLoad ? ldg_nt(c4 + base + u * kStep) : c4[base + u * kStep];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      r[u] = triad4(bv[u], cv[u], sd);
      extra[u] = -0.f;
    }
  } else {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t i = base + u * kStep;
      r[u] = i < n4 ? triad4(b4[i], c4[i], sd) : make_float4(0.f, 0.f, 0.f, 0.f);
      extra[u] = -0.f;
      if (Sum == SUM_BLOCK256 && i == n4) {
        // the lane whose float4 slot holds the end of the vector takes the one to three elements there
        for (int64_t e = n4 << 2; e < n; ++e) {
          const float v = triad1(b[e], c[e], sd);
          a[e] = v;
          extra[u] += v;
        }
      }
    }
  }
  // scalar tail: at most three elements, taken by the first threads of the last workgroup
  float tail = 0.f;
  const int64_t ti = (n4 << 2) + threadIdx.x;
  const bool has_tail = Sum != SUM_BLOCK256 && blockIdx.x == gridDim.x - 1 && ti < n;
  if (has_tail) tail = triad1(b[ti], c[ti], sd);

  // the stores go out first: the sums below are register work that needs nothing from memory
  if (full) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) stg_nt(a4 + base + u * kStep, r[u]);
  } else {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t i = base + u * kStep;
      if (i < n4) a4[i] = r[u];
    }
  }
  if (has_tail) a[ti] = tail;

  if (Sum == SUM_WORKGROUP) {
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      acc.x += r[u].x; acc.y += r[u].y; acc.z += r[u].z; acc.w += r[u].w;
    }
    float t = block_sum(((acc.x + acc.y) + (acc.z + acc.w)) + tail);
    if (threadIdx.x == 0) partials[blockIdx.x] = t;
  }
  if (Sum == SUM_BLOCK256 && Runs == 0) {
    const int64_t nblocks = (n + 255) >> 8;
    const int64_t j0 = static_cast<int64_t>(blockIdx.x) * (kChunk / 64) + (threadIdx.x >> 6);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const float t = wave_sum(((r[u].x + r[u].y) + (r[u].z + r[u].w)) + extra[u]);
      const int64_t j = j0 + u * (kBlock / 64);
      if ((threadIdx.x & 63) == 0 && j < nblocks) partials[j] = t;
    }
  }
  if (Sum == SUM_BLOCK256 && Runs != 0) {
    static_assert(kUnroll == 4, "four block sums per wave leave as one float4");
    const int64_t nblocks = (n + 255) >> 8;
    const int wave = threadIdx.x >> 6;
    float t[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) t[u] = wave_sum(((r[u].x + r[u].y) + (r[u].z + r[u].w)) + extra[u]);
    const int64_t j0 = static_cast<int64_t>(blockIdx.x) * (kChunk / 64) + wave * kUnroll;
    if ((threadIdx.x & 63) == 0) {
      if (j0 + kUnroll <= nblocks) {
        *reinterpret_cast<float4 *>(partials + j0) = make_float4(t[0], t[1], t[2], t[3]);
      } else {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
          if (j0 + u < nblocks) partials[j0 + u] = t[u];
      }
    }
  }
}

// Unaligned-pointer fallback: one element per thread, grid-stride.
template <bool WithSum>
__global__ __launch_bounds__(kBlock) void triad_scalar_kernel(float *__restrict__ a,
                                                              const float *__restrict__ b,
                                                              const float *__restrict__ c,
                                                              float s, int64_t n,
                                                              float *__restrict__ partials) {
  const double sd = static_cast<double>(s);
  float acc = 0.f;
  const int64_t step = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += step) {
    float r = triad1(b[i], c[i], sd);
    a[i] = r;
    acc += r;
  }
  if (WithSum) {
    float t = block_sum(acc);
    if (threadIdx.x == 0) partials[blockIdx.x] = t;
  }
}

// Double sum of x[0..count) by one 1024-thread block, valid in every thread.  Each thread takes float4
// pieces at a stride of 1024 pieces, eight loads in flight, then the wave's lanes are added by lane moves
// and the sixteen waves' sums through LDS; the summation order is fixed by (count, the pointer's
// alignment, thread layout) only.
__device__ __forceinline__ double fold_block(const float *__restrict__ x, int64_t count) {
  __shared__ double sh[16];
  double acc = 0.0;
  const bool vec = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
  const int64_t n4 = vec ? count >> 2 : 0;
  const float4 *p4 = reinterpret_cast<const float4 *>(x);
  int64_t i = threadIdx.x;
  for (; i + 7 * 1024 < n4; i += 8 * 1024) {
    float4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = p4[i + u * 1024];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      acc += (static_cast<double>(v[u].x) + static_cast<double>(v[u].y)) +
             (static_cast<double>(v[u].z) + static_cast<double>(v[u].w));
  }
  for (; i < n4; i += 1024) {
    float4 v = p4[i];
    acc += (static_cast<double>(v.x) + static_cast<double>(v.y)) +
           (static_cast<double>(v.z) + static_cast<double>(v.w));
  }
  for (int64_t j = (n4 << 2) + threadIdx.x; j < count; j += 1024) acc += static_cast<double>(x[j]);
  // across the lanes of a wave by lane moves (no LDS, no barrier), then the sixteen waves' sums in wave order
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = acc;
  __syncthreads();
  double total = 0.0;
#pragma unroll
  for (int w = 0; w < 16; ++w) total += sh[w];
  return total;
}

// *out = sum of partials[0..count) accumulated in double by one block.
__global__ __launch_bounds__(1024) void fold_kernel(const float *__restrict__ partials,
                                                    int64_t count, double *__restrict__ out) {
  const double t = fold_block(partials, count);
  if (threadIdx.x == 0) *out = t;
}

// Long inputs in one launch: workgroup g sums the piece [g*piece, (g+1)*piece) into slot->stage[g] and takes a
// ticket; the workgroup that takes the last one adds the stage up in index order (a fixed order whichever
// workgroup that is) and puts the ticket counter back to zero for the next launch.  `piece` is a multiple of
// 4, so every workgroup sees its piece at the alignment of the whole.  The stage values cross the device as
// device-scope atomic stores and loads, ordered by the ticket's release / acquire: in a kernel this small the
// L2s hold next to nothing that the release has to write back.
constexpr int kFoldGroups = 256;
struct FoldSlot {
  double stage[kFoldGroups];
  unsigned ticket;
  unsigned unused[63];
};
// The 256 stage values, one in each of the first 256 threads: four waves add theirs by lane moves, then the four sums
// in wave order.  Valid in thread 0.
__device__ __forceinline__ double fold_stage(double v) {
  __shared__ double last_sums[kFoldGroups / 64];
  if (threadIdx.x < kFoldGroups) {   // four whole waves
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) last_sums[threadIdx.x >> 6] = v;
  }
  __syncthreads();
  return (last_sums[0] + last_sums[1]) + (last_sums[2] + last_sums[3]);
}
__global__ __launch_bounds__(1024) void fold_onepass_kernel(const float *__restrict__ partials, int64_t count,
                                                            int64_t piece, FoldSlot *__restrict__ slot,
                                                            double *__restrict__ out) {
  const int64_t lo = static_cast<int64_t>(blockIdx.x) * piece;
  const int64_t len = lo >= count ? 0 : (count - lo < piece ? count - lo : piece);
  const double t = fold_block(partials + lo, len);
  __shared__ bool last;
  if (threadIdx.x == 0) {
    __hip_atomic_store(&slot->stage[blockIdx.x], t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned before = __hip_atomic_fetch_add(&slot->ticket, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    last = before == gridDim.x - 1;
  }
  __syncthreads();
  if (!last) return;
  const double v = threadIdx.x < kFoldGroups
                       ? __hip_atomic_load(&slot->stage[threadIdx.x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                       : 0.0;
  const double total = fold_stage(v);
  if (threadIdx.x == 0) {
    *out = total;
    __hip_atomic_store(&slot->ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// The 256 pieces of a long fold through one workgroup, for aligned pieces of at most K * 4096 elements (K 128-bit
// loads per thread and piece): 8 / K pieces at a time, their loads asked for while the pieces before them are added
// up.  Thread t adds what fold_block's thread t adds to its running sum, in its order, and the wave's lanes are
// added as there; the sixteen wave sums of every piece wait in LDS (32 KiB) for one barrier at the end, so no wave
// waits for another on the way, and thread g then adds piece g's sixteen in wave order: stage[g] gets fold_block's
// bits for piece g.
template <int K>
__device__ __forceinline__ void fold_pieces_batched(const float *__restrict__ partials, int64_t count, int64_t piece,
                                                    double (*wave_sums)[16], double *stage) {
  constexpr int B = 8 / K;    // pieces per batch: eight 128-bit loads per thread in flight, which 128 registers hold
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  auto length_of = [&](int g) {
    const int64_t lo = static_cast<int64_t>(g) * piece;
    return lo >= count ? int64_t{0} : (count - lo < piece ? count - lo : piece);
  };
  float4 next[B * K];
  // all pieces but the last ones are whole: a batch that lies inside the input has one length, known beforehand
  const int64_t whole_n4 = piece >> 2;
  const float4 *const base4 = reinterpret_cast<const float4 *>(partials);
  auto whole = [&](int b) { return static_cast<int64_t>(b + 1) * B * piece <= count; };
  auto load_batch = [&](int b) {
    if (whole(b)) {
      const float4 *p4 = base4 + static_cast<int64_t>(b) * B * whole_n4 + t;
#pragma unroll
      for (int q = 0; q < B; ++q)
#pragma unroll
        for (int k = 0; k < K; ++k)
          next[q * K + k] = t + k * 1024 < whole_n4 ? p4[q * whole_n4 + k * 1024] : make_float4(0.f, 0.f, 0.f, 0.f);
      return;
    }
#pragma unroll
    for (int q = 0; q < B; ++q) {
      const int g = b * B + q;
      const int64_t n4 = length_of(g) >> 2;
      const float4 *p4 = reinterpret_cast<const float4 *>(partials + static_cast<int64_t>(g) * piece);
#pragma unroll
      for (int k = 0; k < K; ++k) next[q * K + k] = t + k * 1024 < n4 ? p4[t + k * 1024] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };
  load_batch(0);
  for (int b = 0; b < kFoldGroups / B; ++b) {
    double acc[B];
    const bool all_whole = whole(b);
#pragma unroll
    for (int q = 0; q < B; ++q) {
      const int g = b * B + q;
      const int64_t len = all_whole ? piece : length_of(g), n4 = len >> 2;
      acc[q] = 0.0;
#pragma unroll
      for (int k = 0; k < K; ++k)
        if (t + k * 1024 < n4) {
          const float4 v = next[q * K + k];
          acc[q] += (static_cast<double>(v.x) + static_cast<double>(v.y)) + (static_cast<double>(v.z) + static_cast<double>(v.w));
        }
      // the last, short four of the whole input
      if (!all_whole && (n4 << 2) + t < len)
        acc[q] += static_cast<double>(partials[static_cast<int64_t>(g) * piece + (n4 << 2) + t]);
    }
    if (b + 1 < kFoldGroups / B) load_batch(b + 1);
#pragma unroll
    for (int q = 0; q < B; ++q) {
      const double s = wave_sum(acc[q]);
      if (lane == 0) wave_sums[b * B + q][wave] = s;
    }
  }
  __syncthreads();
  if (t < kFoldGroups) {
    double total = 0.0;
#pragma unroll
    for (int w = 0; w < 16; ++w) total += wave_sums[t][w];
    stage[t] = total;
  }
  __syncthreads();
}

// The same sum with no stage outside the workgroup: one workgroup takes the 256 pieces itself and keeps their sums
// in LDS.  Piece by piece and in the last step it adds what fold_onepass_kernel adds, in that order, so a long fold
// gives the same bits whether or not it had a stage (a launch recorded into a graph, or a stream that came when every
// slot was taken, has none).  Aligned folds of up to 2^22 partials take the batched walk above; longer or unaligned
// ones go through fold_block piece by piece.
__global__ __launch_bounds__(1024) void fold_pieces_kernel(const float *__restrict__ partials, int64_t count,
                                                           int64_t piece, double *__restrict__ out) {
  __shared__ double stage[kFoldGroups];
  __shared__ double wave_sums[kFoldGroups][16];
  const bool aligned = (reinterpret_cast<uintptr_t>(partials) & 15u) == 0;
  if (aligned && piece <= 4096) {
    fold_pieces_batched<1>(partials, count, piece, wave_sums, stage);
  } else if (aligned && piece <= 8192) {
    fold_pieces_batched<2>(partials, count, piece, wave_sums, stage);
  } else if (aligned && piece <= 16384) {
    fold_pieces_batched<4>(partials, count, piece, wave_sums, stage);
  } else {
    for (int g = 0; g < kFoldGroups; ++g) {
      const int64_t lo = static_cast<int64_t>(g) * piece;
      const int64_t len = lo >= count ? 0 : (count - lo < piece ? count - lo : piece);
      const double t = fold_block(partials + lo, len);
      if (threadIdx.x == 0) stage[g] = t;
      __syncthreads();   // fold_block's own LDS is free again, stage[g] is written
    }
  }
  const double total = fold_stage(threadIdx.x < kFoldGroups ? stage[threadIdx.x] : 0.0);
  if (threadIdx.x == 0) *out = total;
}

// Per-256-element-block kernels: out[j] = reduction of in[256j .. 256j+255].  A wave takes
// kBlocksPerWave consecutive blocks (8 KiB of each input) in one shot, all loads issued
// before the first use, non-temporal; the grid has one wave per such group, no loop.
constexpr int kBlocksPerWave = 8;

// Sum (or, Dot, sum of x[i]*y[i]), zero padded past n.  Each lane folds its four elements,
// the wave sum is f32; the summation order differs from the reference's halving tree,
// which its own checks allow for (1e-3 relative on the folded total).
template <bool Dot>
__global__ __launch_bounds__(kBlock) void block256_kernel(const float *__restrict__ x,
                                                          const float *__restrict__ y,
                                                          float *__restrict__ out, int64_t n,
                                                          int64_t nblocks) {
  constexpr int U = kBlocksPerWave;
  const int lane = threadIdx.x & 63;
  const int64_t j0 = (static_cast<int64_t>(blockIdx.x) * (kBlock / 64) + (threadIdx.x >> 6)) * U;
  if (j0 >= nblocks) return;
  float r[U];
  if ((j0 + U) * 256 <= n) {
    float4 xv[U], yv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) xv[u] = ldg_nt(reinterpret_cast<const float4 *>(x + (j0 + u) * 256) + lane);
    if (Dot) {
#pragma unroll
      for (int u = 0; u < U; ++u) yv[u] = ldg_nt(reinterpret_cast<const float4 *>(y + (j0 + u) * 256) + lane);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float v = Dot ? (xv[u].x * yv[u].x + xv[u].y * yv[u].y) + (xv[u].z * yv[u].z + xv[u].w * yv[u].w)
                          : (xv[u].x + xv[u].y) + (xv[u].z + xv[u].w);
      r[u] = wave_sum(v);
    }
    if (lane == 0) {
      // j0 is a multiple of 8: with `out` on a 16-byte boundary the eight sums leave as two 16-byte stores
      if ((reinterpret_cast<uintptr_t>(out) & 15u) == 0) {
        float4 *o4 = reinterpret_cast<float4 *>(out + j0);
        o4[0] = make_float4(r[0], r[1], r[2], r[3]);
        o4[1] = make_float4(r[4], r[5], r[6], r[7]);
      } else {
#pragma unroll
        for (int u = 0; u < U; ++u) out[j0 + u] = r[u];
      }
    }
    return;
  }
  // the group that holds the end of the input
  for (int u = 0; u < U && j0 + u < nblocks; ++u) {
    const int64_t i = (j0 + u) * 256 + lane * 4;
    float t[4];
    for (int e = 0; e < 4; ++e) t[e] = i + e < n ? (Dot ? x[i + e] * y[i + e] : x[i + e]) : 0.f;
    float v = (t[0] + t[1]) + (t[2] + t[3]);   // the pairing of the full groups above
    v = wave_sum(v);
    if (lane == 0) out[j0 + u] = v;
  }
}

// out[j] = the value the reference's halving tree
// (benchmarks/bench_reduction_max.ml:18-100: sdata[tid] = gid < n ? in[gid] : pad, then for
// half = 128..1 "if sdata[tid+half] > sdata[tid] then sdata[tid] <- sdata[tid+half]")
// leaves in sdata[0].  The same pairs are compared in the same order with the same
// strict ">" (lane l holds elements l, l+64, l+128, l+192 of the block), so NaNs and
// signed zeros come out as from the tree.
__device__ __forceinline__ float take_greater(float a, float b) { return b > a ? b : a; }

__device__ __forceinline__ float tree_max_of_block(float v0, float v1, float v2, float v3) {
  v0 = take_greater(v0, v2);   // half = 128: (l, l+128), (l+64, l+192)
  v1 = take_greater(v1, v3);
  float m = take_greater(v0, v1);  // half = 64
#pragma unroll
  for (int half = 32; half >= 1; half >>= 1) {
    const float other = __shfl_down(m, half, 64);
    m = take_greater(m, other);    // only lanes < half matter from here on
  }
  return m;                        // valid in lane 0
}

// The stream triad and the block-256 maximum of its output in one pass (the element-wise kernel of bench_stream_triad.ml
// or bench_vector_add.ml followed by bench_reduction_max.ml's tree).  Layout as triad_kernel's Runs form: a wave owns four
// consecutive KiB, lane l of a slot holds elements 4l .. 4l+3 of that slot's 256-element block.  The tree's comparisons
// are made in the tree's order with its strict ">" -- halves 128 .. 4 pair lane l with lanes l+32 .. l+1 component by
// component, halves 2 and 1 pair the four components of lane 0 -- so NaNs and signed zeros come out as from the tree.
// Elements past n count as `pad`, as in the reference kernel.
template <bool NtLoad>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(8, 8))) void triad_block256_max_kernel(
    float *__restrict__ a, const float *__restrict__ b, const float *__restrict__ c, float s, int64_t n, float pad,
    float *__restrict__ block_max) {
  static_assert(kUnroll == 4, "four block maxima per wave leave as one float4");
  const double sd = static_cast<double>(s);
  const int64_t n4 = n >> 2;
  float4 *a4 = reinterpret_cast<float4 *>(a);
  const float4 *b4 = reinterpret_cast<const float4 *>(b);
  const float4 *c4 = reinterpret_cast<const float4 *>(c);
  constexpr int kStep = 64;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kChunk + wave * (64 * kUnroll) + lane;
  const bool full = base + (kUnroll - 1) * kStep < n4;   // the same for all lanes of a wave up to the slot that holds n
  float4 r[kUnroll];
  if (full) {
    float4 bv[kUnroll], cv[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) bv[u] = NtLoad ? ldg_nt(b4 + base + u * kStep) : b4[base + u * kStep];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) cv[u] = NtLoad ? ldg_nt(c4 + base + u * kStep) : c4[base + u * kStep];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      r[u] = triad4(bv[u], cv[u], sd);
      stg_nt(a4 + base + u * kStep, r[u]);
    }
  } else {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t i = base + u * kStep;
      if (i < n4) {
        r[u] = triad4(b4[i], c4[i], sd);
        a4[i] = r[u];
      } else {
        // the slot that holds the end of the vector takes its one to three elements; everything past n is pad
        float t[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int64_t k = (i << 2) + e;
          t[e] = pad;
          if (k < n) {
            t[e] = triad1(b[k], c[k], sd);
            a[k] = t[e];
          }
        }
        r[u] = make_float4(t[0], t[1], t[2], t[3]);
      }
    }
  }
  const int64_t nblocks = (n + 255) >> 8;
  float m[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    float4 v = r[u];
#pragma unroll
    for (int half = 32; half >= 1; half >>= 1) {   // tree halves 128 .. 4: element e against e + 4 * half
      v.x = take_greater(v.x, __shfl_down(v.x, half, 64));
      v.y = take_greater(v.y, __shfl_down(v.y, half, 64));
      v.z = take_greater(v.z, __shfl_down(v.z, half, 64));
      v.w = take_greater(v.w, __shfl_down(v.w, half, 64));
    }
    m[u] = take_greater(take_greater(v.x, v.z), take_greater(v.y, v.w));   // halves 2 and 1 (lane 0)
  }
  if (lane != 0) return;
  const int64_t j0 = static_cast<int64_t>(blockIdx.x) * (kChunk / 64) + wave * kUnroll;
  if (j0 + kUnroll <= nblocks && (reinterpret_cast<uintptr_t>(block_max) & 15u) == 0) {
    *reinterpret_cast<float4 *>(block_max + j0) = make_float4(m[0], m[1], m[2], m[3]);
  } else {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      if (j0 + u < nblocks) block_max[j0 + u] = m[u];
  }
}

__global__ __launch_bounds__(kBlock) void block256_max_kernel(const float *__restrict__ x,
                                                              float *__restrict__ out, int64_t n,
                                                              int64_t nblocks, float pad) {
  constexpr int U = kBlocksPerWave;
  const int lane = threadIdx.x & 63;
  const int64_t j0 = (static_cast<int64_t>(blockIdx.x) * (kBlock / 64) + (threadIdx.x >> 6)) * U;
  if (j0 >= nblocks) return;
  const bool full = (j0 + U) * 256 <= n;
  float v[U][4];
#pragma unroll
  for (int u = 0; u < U; ++u)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int64_t i = (j0 + u) * 256 + lane + 64 * q;
      v[u][q] = (full || i < n) ? __builtin_nontemporal_load(x + (i < n ? i : 0)) : pad;
    }
  float m[U];
#pragma unroll
  for (int u = 0; u < U; ++u) m[u] = tree_max_of_block(v[u][0], v[u][1], v[u][2], v[u][3]);
  if (lane != 0) return;
  if (j0 + U <= nblocks && (reinterpret_cast<uintptr_t>(out) & 15u) == 0) {
    float4 *o4 = reinterpret_cast<float4 *>(out + j0);   // j0 is a multiple of 8
    o4[0] = make_float4(m[0], m[1], m[2], m[3]);
    o4[1] = make_float4(m[4], m[5], m[6], m[7]);
  } else {
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (j0 + u < nblocks) out[j0 + u] = m[u];
  }
}

// f32 -> bf16 bits, round to nearest even; NaN stays a quiet NaN.
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  if ((u & 0x7F800000u) == 0x7F800000u) {
    if (u & 0x007FFFFFu) u |= 0x00400000u;
    return static_cast<uint16_t>(u >> 16);
  }
  u += 0x7FFFu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ uint16_t f32_to_f16_rne(float f) {
  _Float16 h = static_cast<_Float16>(f);  // v_cvt_f16_f32: round to nearest even
  return __builtin_bit_cast(uint16_t, h);
}

template <bool Bf16>
__global__ __launch_bounds__(kBlock) void cast16_kernel(const float *__restrict__ in,
                                                        uint16_t *__restrict__ out, int64_t n) {
  const int64_t step = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += step)
    out[i] = Bf16 ? f32_to_bf16_rne(in[i]) : f32_to_f16_rne(in[i]);
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Load policy for `input_bytes` of input.  Inputs that together fit the 256 MB last-level
// cache may still be there (the producer's output, the previous launch's input): plain loads
// hit it, non-temporal ones go round it (measured: triad 7.1 vs 6.6 TB/s at 3 x 120 MB).
// Larger inputs come from HBM whatever the policy and non-temporal loads keep them out of
// the way of the stores (6.4 vs 5.8 TB/s at 3 x 1 GiB).  The read-only block-256 kernels have
// no store stream to protect and measured the same or better with non-temporal loads at
// every size, so they always use them.  Tunable "stream.nt" forces 0 / 1.
inline bool streams_from_hbm(int64_t input_bytes) {
  const int64_t forced = tunable("stream.nt", -1);
  return forced >= 0 ? forced != 0 : input_bytes > (int64_t{256} << 20);
}

// Workgroups (= f32 partials) of the triad kernels for n elements.
inline int64_t triad_blocks(int64_t n) {
  return ceil_div(n > 0 ? n : 1, static_cast<int64_t>(kChunk) * 4);
}

int launch_fold(const float *partials, int64_t count, double *sum_out, hipStream_t st);

int launch_triad(float *a, const float *b, const float *c, float s, int64_t n, float *partials,
                 double *sum_out, bool with_sum, hipStream_t st) {
  // The 128-bit accesses need no 16-byte alignment on this hardware (a vector that starts anywhere on a 4-byte boundary
  // costs the kernel about 7 % at n = 2^28, where the element-per-thread kernel costs 57 %); stream.force_scalar keeps
  // the scalar kernel reachable.
  const bool vec = tunable("stream.force_scalar", 0) == 0;
  const int64_t blocks64 = triad_blocks(n);
  if (blocks64 > 0x7FFFFFFF) return fail(SAREK_HIP_E_INVALID_ARG, "triad: vector too long");
  const unsigned blocks = static_cast<unsigned>(blocks64);
  if (vec) {
    const bool nt = streams_from_hbm(n * 8);
    if (with_sum) {
      if (nt) hipLaunchKernelGGL((triad_kernel<SUM_WORKGROUP, true>), dim3(blocks), dim3(kBlock), 0, st, a, b, c, s, n, partials);
      else hipLaunchKernelGGL((triad_kernel<SUM_WORKGROUP, false>), dim3(blocks), dim3(kBlock), 0, st, a, b, c, s, n, partials);
      int rc = check_launch("triad kernel launch");
      if (rc != SAREK_HIP_OK) return rc;
      return launch_fold(partials, blocks64, sum_out, st);
    }
    if (nt) hipLaunchKernelGGL((triad_kernel<SUM_NONE, true>), dim3(blocks), dim3(kBlock), 0, st, a, b, c, s, n, partials);
    else hipLaunchKernelGGL((triad_kernel<SUM_NONE, false>), dim3(blocks), dim3(kBlock), 0, st, a, b, c, s, n, partials);
    return check_launch("triad kernel launch");
  }
  // one element per thread on a capped grid, then a separate fold
  const unsigned sblocks = blocks < 8192u ? blocks : 8192u;
  if (with_sum) {
    hipLaunchKernelGGL(triad_scalar_kernel<true>, dim3(sblocks), dim3(kBlock), 0, st, a, b, c, s, n, partials);
    int rc = check_launch("triad kernel launch");
    if (rc != SAREK_HIP_OK) return rc;
    return launch_fold(partials, (int64_t)sblocks, sum_out, st);
  }
  hipLaunchKernelGGL(triad_scalar_kernel<false>, dim3(sblocks), dim3(kBlock), 0, st, a, b, c, s, n, partials);
  return check_launch("triad kernel launch");
}

__global__ void store_f64_kernel(double *p, double v) { *p = v; }

}  // namespace
}  // namespace sarek_hip

// Partials of sarek_hip_triad_sum_f32_static: one f32 per triad workgroup (4096 elements), room
// for vectors of up to 2^31 elements; 2 MiB of every device the library runs on, held until the
// process ends.  In host code this name is only a handle for hipGetSymbolAddress: kernels get the
// per-device address kept in g_scratch_addr.
constexpr int64_t kScratchFloats = int64_t{1} << 19;
static __device__ __align__(256) float scratch[kScratchFloats];

// Stages of long folds: kFoldSlots slots of one double per workgroup of fold_onepass_kernel and a ticket counter
// (36 KiB per device).  The counters start at zero (the image's initial value) and every launch leaves its own at zero.
constexpr int kFoldSlots = 16;
static __device__ __align__(256) sarek_hip::FoldSlot fold_slots[kFoldSlots];

namespace sarek_hip {
namespace {
constexpr int kMaxDevices = 64;
std::atomic<float *> g_scratch_addr[kMaxDevices];
std::atomic<FoldSlot *> g_fold_slots_addr[kMaxDevices];

bool capturing(hipStream_t st) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &status) != hipSuccess) {
    (void)hipGetLastError();
    return true;   // treated as the cautious case
  }
  return status != hipStreamCaptureStatusNone;
}

// Device address of a file-scope __device__ array on the current device, looked up once per
// device: every device holds its own copy of the array at its own address.  The lookup is not
// allowed while `st` records a graph; a device whose address is not known yet is then refused.
template <typename T>
int address_on_current_device(std::atomic<T *> *table, const void *symbol, const char *what, hipStream_t st, T **out) {
  int dev = 0;
  SAREK_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(SAREK_HIP_E_UNSUPPORTED, "%s: device ordinal %d beyond %d", what, dev, kMaxDevices);
  T *p = table[dev].load(std::memory_order_acquire);
  if (!p) {
    if (capturing(st))
      return fail(SAREK_HIP_E_UNSUPPORTED,
                  "%s: first use on device %d under stream capture (call it once outside a capture first)", what,
                  dev);
    SAREK_HIP_TRY(hipGetSymbolAddress(reinterpret_cast<void **>(&p), symbol));
    if (!p) return fail(SAREK_HIP_E_UNSUPPORTED, "%s: no device address for the library's own array", what);
    table[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return SAREK_HIP_OK;
}

int scratch_on_current_device(hipStream_t st, float **out) {
  return address_on_current_device(g_scratch_addr, HIP_SYMBOL(scratch), "triad_sum_static", st, out);
}

// The stage slot of (current device, st): a stream keeps the slot it got first, so folds on one stream follow each
// other through the same slot and folds on different streams never share one.  nullptr when all slots of the device
// are taken by other streams (a slot stays with its stream's handle for the life of the process): the caller then
// folds with one workgroup, which needs no stage.
FoldSlot *fold_slot_for(hipStream_t st) {
  FoldSlot *slots = nullptr;
  if (address_on_current_device(g_fold_slots_addr, HIP_SYMBOL(fold_slots), "fold_partials", st, &slots) != SAREK_HIP_OK) {
    last_error_slot().clear();
    return nullptr;
  }
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  static std::mutex mu;
  static std::map<std::pair<int, hipStream_t>, int> taken;   // (device, stream) -> slot
  static int used[kMaxDevices] = {};
  std::lock_guard<std::mutex> lock(mu);
  auto it = taken.find({dev, st});
  if (it != taken.end()) return slots + it->second;
  if (used[dev] >= kFoldSlots) return nullptr;
  const int slot = used[dev]++;
  taken[{dev, st}] = slot;
  return slots + slot;
}

// Folds shorter than this run as one workgroup; longer ones as 256 workgroups whose last one adds their sums up.
constexpr int64_t kFoldOnePassFrom = int64_t{1} << 17;

int launch_fold(const float *partials, int64_t count, double *sum_out, hipStream_t st) {
  // a launch recorded into a graph may be replayed on any stream, next to anything: it gets no shared stage
  if (count < kFoldOnePassFrom) {
    hipLaunchKernelGGL(fold_kernel, dim3(1), dim3(1024), 0, st, partials, count, sum_out);
    return check_launch("fold kernel launch");
  }
  const int64_t piece = ceil_div(ceil_div(count, kFoldGroups), 4) * 4;
  FoldSlot *slot = capturing(st) ? nullptr : fold_slot_for(st);
  if (!slot) {
    hipLaunchKernelGGL(fold_pieces_kernel, dim3(1), dim3(1024), 0, st, partials, count, piece, sum_out);
    return check_launch("fold kernel launch");
  }
  hipLaunchKernelGGL(fold_onepass_kernel, dim3(kFoldGroups), dim3(1024), 0, st, partials, count, piece, slot, sum_out);
  return check_launch("fold kernel launch");
}
}  // namespace
}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" {

int sarek_hip_triad_f32(float *a, const float *b, const float *c, float s, int64_t n,
                        sarek_hip_stream stream) {
  if (n < 0) return fail(SAREK_HIP_E_INVALID_ARG, "triad: negative length %lld", (long long)n);
  if (n > 0 && (!a || !b || !c)) return fail(SAREK_HIP_E_INVALID_ARG, "triad: NULL vector");
  if (n == 0) return SAREK_HIP_OK;
  return launch_triad(a, b, c, s, n, nullptr, nullptr, false, as_stream(stream));
}

int64_t sarek_hip_triad_sum_workspace_floats(int64_t n) { return n <= 0 ? 1 : triad_blocks(n); }

int sarek_hip_triad_sum_f32(float *a, const float *b, const float *c, float s, int64_t n,
                            float *partials, int64_t partials_len, double *sum_out,
                            sarek_hip_stream stream) {
  if (n < 0) return fail(SAREK_HIP_E_INVALID_ARG, "triad_sum: negative length %lld", (long long)n);
  if (!sum_out) return fail(SAREK_HIP_E_INVALID_ARG, "triad_sum: NULL sum_out");
  if (n > 0 && (!a || !b || !c || !partials))
    return fail(SAREK_HIP_E_INVALID_ARG, "triad_sum: NULL vector or workspace");
  const int64_t blocks = n == 0 ? 0 : triad_blocks(n);
  if (partials_len < blocks)
    return fail(SAREK_HIP_E_WORKSPACE, "triad_sum: workspace holds %lld floats, %lld needed",
                (long long)partials_len, (long long)blocks);
  hipStream_t st = as_stream(stream);
  if (n == 0) {
    hipLaunchKernelGGL(store_f64_kernel, dim3(1), dim3(1), 0, st, sum_out, 0.0);
    return check_launch("triad_sum empty launch");
  }
  return launch_triad(a, b, c, s, n, partials, sum_out, true, st);
}

int64_t sarek_hip_triad_sum_static_max_n(void) { return kScratchFloats * kChunk * 4; }

int sarek_hip_triad_sum_f32_static(float *a, const float *b, const float *c, float s, int64_t n,
                                   double *sum_out, sarek_hip_stream stream) {
  if (n < 0) return fail(SAREK_HIP_E_INVALID_ARG, "triad_sum_static: negative length %lld", (long long)n);
  if (!sum_out) return fail(SAREK_HIP_E_INVALID_ARG, "triad_sum_static: NULL sum_out");
  if (n > 0 && (!a || !b || !c)) return fail(SAREK_HIP_E_INVALID_ARG, "triad_sum_static: NULL vector");
  if (n > sarek_hip_triad_sum_static_max_n())
    return fail(SAREK_HIP_E_WORKSPACE,
                "triad_sum_static: %lld elements, the built-in partials array serves at most %lld "
                "(use sarek_hip_triad_sum_f32 with a workspace)",
                (long long)n, (long long)sarek_hip_triad_sum_static_max_n());
  hipStream_t st = as_stream(stream);
  if (n == 0) {
    hipLaunchKernelGGL(store_f64_kernel, dim3(1), dim3(1), 0, st, sum_out, 0.0);
    return check_launch("triad_sum_static empty launch");
  }
  // Every workgroup stores its partial before the fold reads exactly those: nothing has to start at zero.
  float *partials = nullptr;
  int rc = scratch_on_current_device(st, &partials);
  if (rc != SAREK_HIP_OK) return rc;
  return launch_triad(a, b, c, s, n, partials, sum_out, true, st);
}

int sarek_hip_fold_partials_f64(const float *partials, int64_t count, double *sum_out,
                                sarek_hip_stream stream) {
  if (count < 0 || !sum_out || (count > 0 && !partials))
    return fail(SAREK_HIP_E_INVALID_ARG, "fold_partials: bad arguments");
  return launch_fold(partials, count, sum_out, as_stream(stream));
}

int sarek_hip_triad_block256_sum_f32(float *a, const float *b, const float *c, float s, int64_t n,
                                     float *block_sums, sarek_hip_stream stream) {
  if (n < 0) return fail(SAREK_HIP_E_INVALID_ARG, "triad_block256_sum: negative length %lld", (long long)n);
  if (n == 0) return SAREK_HIP_OK;
  if (!a || !b || !c || !block_sums) return fail(SAREK_HIP_E_INVALID_ARG, "triad_block256_sum: NULL vector");
  const int64_t blocks64 = triad_blocks(n);
  if (blocks64 > 0x7FFFFFFF) return fail(SAREK_HIP_E_INVALID_ARG, "triad_block256_sum: vector too long");
  const dim3 grid(static_cast<unsigned>(blocks64));
  hipStream_t st = as_stream(stream);
  const bool nt = streams_from_hbm(n * 8);
  // block sums that are not 16-byte aligned cannot leave as float4: the layout with 4-byte stores
  const bool runs = aligned16(block_sums) && tunable("triad.block_sum_runs", 1) != 0;
  if (runs) {
    if (nt) hipLaunchKernelGGL((triad_kernel<SUM_BLOCK256, true, 1>), grid, dim3(kBlock), 0, st, a, b, c, s, n, block_sums);
    else hipLaunchKernelGGL((triad_kernel<SUM_BLOCK256, false, 1>), grid, dim3(kBlock), 0, st, a, b, c, s, n, block_sums);
  } else if (nt) {
    hipLaunchKernelGGL((triad_kernel<SUM_BLOCK256, true>), grid, dim3(kBlock), 0, st, a, b, c, s, n, block_sums);
  } else {
    hipLaunchKernelGGL((triad_kernel<SUM_BLOCK256, false>), grid, dim3(kBlock), 0, st, a, b, c, s, n, block_sums);
  }
  return check_launch("triad + block-256 sum kernel launch");
}

int sarek_hip_triad_block256_max_f32(float *a, const float *b, const float *c, float s, int64_t n, float pad,
                                     float *block_max, sarek_hip_stream stream) {
  if (n < 0) return fail(SAREK_HIP_E_INVALID_ARG, "triad_block256_max: negative length %lld", (long long)n);
  if (n == 0) return SAREK_HIP_OK;
  if (!a || !b || !c || !block_max) return fail(SAREK_HIP_E_INVALID_ARG, "triad_block256_max: NULL vector");
  const int64_t blocks64 = triad_blocks(n);
  if (blocks64 > 0x7FFFFFFF) return fail(SAREK_HIP_E_INVALID_ARG, "triad_block256_max: vector too long");
  const dim3 grid(static_cast<unsigned>(blocks64));
  hipStream_t st = as_stream(stream);
  if (streams_from_hbm(n * 8))
    hipLaunchKernelGGL(triad_block256_max_kernel<true>, grid, dim3(kBlock), 0, st, a, b, c, s, n, pad, block_max);
  else
    hipLaunchKernelGGL(triad_block256_max_kernel<false>, grid, dim3(kBlock), 0, st, a, b, c, s, n, pad, block_max);
  return check_launch("triad + block-256 max kernel launch");
}

static int launch_block256(const float *x, const float *y, float *out, int64_t n, bool dot,
                           hipStream_t st) {
  if (n < 0) return fail(SAREK_HIP_E_INVALID_ARG, "block256: negative length");
  if (n == 0) return SAREK_HIP_OK;
  if (!x || !out || (dot && !y)) return fail(SAREK_HIP_E_INVALID_ARG, "block256: NULL vector");
  const int64_t nblocks = ceil_div(n, 256);
  const int64_t wg = ceil_div(nblocks, (kBlock / 64) * kBlocksPerWave);
  if (wg > 0x7FFFFFFF) return fail(SAREK_HIP_E_INVALID_ARG, "block256: input too long for one launch");
  if (dot)
    hipLaunchKernelGGL(block256_kernel<true>, dim3((unsigned)wg), dim3(kBlock), 0, st, x, y, out, n, nblocks);
  else
    hipLaunchKernelGGL(block256_kernel<false>, dim3((unsigned)wg), dim3(kBlock), 0, st, x, y, out, n, nblocks);
  return check_launch("block256 kernel launch");
}

int sarek_hip_reduce_sum_block256_f32(const float *in, float *out, int64_t n,
                                      sarek_hip_stream stream) {
  return launch_block256(in, nullptr, out, n, false, as_stream(stream));
}

int sarek_hip_dot_block256_f32(const float *a, const float *b, float *out, int64_t n,
                               sarek_hip_stream stream) {
  return launch_block256(a, b, out, n, true, as_stream(stream));
}

int sarek_hip_reduce_max_block256_f32(const float *in, float *out, int64_t n, float pad,
                                      sarek_hip_stream stream) {
  if (n < 0) return fail(SAREK_HIP_E_INVALID_ARG, "block256 max: negative length");
  if (n == 0) return SAREK_HIP_OK;
  if (!in || !out) return fail(SAREK_HIP_E_INVALID_ARG, "block256 max: NULL vector");
  const int64_t nblocks = ceil_div(n, 256);
  const int64_t wg = ceil_div(nblocks, (kBlock / 64) * kBlocksPerWave);
  if (wg > 0x7FFFFFFF) return fail(SAREK_HIP_E_INVALID_ARG, "block256 max: input too long for one launch");
  hipLaunchKernelGGL(block256_max_kernel, dim3((unsigned)wg), dim3(kBlock), 0, as_stream(stream), in,
                     out, n, nblocks, pad);
  return check_launch("block256 max kernel launch");
}

static int launch_cast(const float *in, uint16_t *out, int64_t n, bool bf16, hipStream_t st) {
  if (n < 0 || (n > 0 && (!in || !out))) return fail(SAREK_HIP_E_INVALID_ARG, "cast: bad arguments");
  if (n == 0) return SAREK_HIP_OK;
  int64_t wg = ceil_div(n, kBlock);
  if (wg > 256 * 32) wg = 256 * 32;
  if (bf16)
    hipLaunchKernelGGL(cast16_kernel<true>, dim3((unsigned)wg), dim3(kBlock), 0, st, in, out, n);
  else
    hipLaunchKernelGGL(cast16_kernel<false>, dim3((unsigned)wg), dim3(kBlock), 0, st, in, out, n);
  return check_launch("cast kernel launch");
}

int sarek_hip_cast_f32_to_bf16(const float *in, uint16_t *out, int64_t n, sarek_hip_stream stream) {
  return launch_cast(in, out, n, true, as_stream(stream));
}

int sarek_hip_cast_f32_to_f16(const float *in, uint16_t *out, int64_t n, sarek_hip_stream stream) {
  return launch_cast(in, out, n, false, as_stream(stream));
}
}
