// Histograms of int32 keys and the scatter of a radix-sort pass for gfx950: the hand-written
// counterparts of the generated kernels of benchmarks/bench_histogram.ml:54-84 (bin = key mod
// num_bins) and of benchmarks/bench_radix_sort.ml:82-137 (bin = (key >> shift) & mask; counting,
// then scattering) in the reference.
//
// The reference's kernels give every 256-thread block one pass over 256 keys and then 256
// atomic adds on the global histogram: 4 bytes read per key and one global atomic per key, all
// of them on the same 256 addresses, which is what bounds them (measured: 54 GB/s of keys).
// Here a workgroup walks many keys, counts them in per-wave histograms in LDS (crowded bins by
// one add per wave), and touches the global histogram once per bin at its end: HBM-bound at
// 4 bytes per key.  Integer adds
// commute, so the counts are those of the reference's kernel bit for bit.
#include "common.hpp"
#include "tunables.hpp"

namespace sarek_hip {
namespace {

typedef int i32x4_t __attribute__((ext_vector_type(4)));

constexpr int kBins = 256;          // the reference's shared array has 256 slots
constexpr int kThreads = 1024;      // 16 waves per workgroup
constexpr int kWaves = kThreads / 64;
constexpr int kUnroll = 4;          // 16-byte loads in flight per thread
constexpr int kRounds = 4;          // bins a crowded pass counts wave-wide before it goes key by key
constexpr int kCrowd = 8;           // lanes of a wave on one bin from which one add counts them all

struct ModBin {       // bench_histogram.ml:72: key mod num_bins (C remainder: sign of the key)
  int bins;
  __device__ int operator()(int key) const { return key % bins; }
};
struct ModPow2Bin {   // the same for num_bins a power of two, without the division
  unsigned low;
  __device__ int operator()(int key) const {
    const unsigned k = static_cast<unsigned>(key);
    return key >= 0 ? static_cast<int>(k & low) : -static_cast<int>((0u - k) & low);
  }
};
struct DigitBin {     // bench_radix_sort.ml:101: (key >> shift) & mask, `>>` as the generated code has it
  int shift, mask;
  __device__ int operator()(int key) const { return (key >> shift) & mask; }
};

// histogram[b] += #{ i < n : bin(keys[i]) == b } for 0 <= b < bins (bins <= 256).  A key whose bin
// falls outside [0, bins) is not counted (the reference's kernel indexes its shared array with it).
// keys at any alignment (the 128-bit loads need none beyond the element's); workgroup g takes the 16-byte groups g, g + G, g + 2G, ... in steps
// of kThreads, the last workgroup also the n & 3 trailing keys.
template <class Bin>
__global__ __launch_bounds__(kThreads) void histogram_kernel(int *__restrict__ histogram,
                                                            const int *__restrict__ keys, int64_t n, int bins,
                                                            Bin bin) {
  __shared__ int counts[kWaves][kBins];
  int *mine = counts[threadIdx.x >> 6];
  for (int i = threadIdx.x; i < kWaves * kBins; i += kThreads) (&counts[0][0])[i] = 0;
  __syncthreads();

  // One LDS add per key costs as many cycles as lanes of the wave share an address: 64 for keys that
  // are all alike, about 5 for keys spread over 256 bins.  So each pass over kUnroll loads first looks
  // at one key per lane; when a bin is crowded there (kCrowd lanes or more), the pass counts by
  // `crowded_pass`, otherwise key by key.
  const int lane = threadIdx.x & 63;
  auto in_range = [&](int b) { return static_cast<unsigned>(b) < static_cast<unsigned>(bins); };
  auto plain = [&](int key) {
    const int b = bin(key);
    if (in_range(b)) atomicAdd(&mine[b], 1);
  };
  // kRounds rounds of: take the bin of the first lane that still has a key to count in slot `round`, count
  // the lanes of all kUnroll * 4 slots that hold it (wave-wide masks and bit counts, scalar work), add
  // that number once.  What is left after the rounds is added key by key.
  auto crowded_pass = [&](const i32x4_t (&v)[kUnroll]) {
    constexpr int kSlots = kUnroll * 4;
    int b[kSlots];
    unsigned long long live[kSlots];
#pragma unroll
    for (int j = 0; j < kSlots; ++j) {
      b[j] = bin(v[j >> 2][j & 3]);
      live[j] = __ballot(in_range(b[j]));
    }
#pragma unroll
    for (int round = 0; round < kRounds; ++round) {
      if (live[round] == 0) continue;                  // the same for every lane of the wave
      const int first = __builtin_amdgcn_readlane(b[round], __ffsll(live[round]) - 1);
      int tally = 0;
#pragma unroll
      for (int j = 0; j < kSlots; ++j) {
        const unsigned long long same = live[j] & __ballot(b[j] == first);
        tally += __popcll(same);
        live[j] &= ~same;
      }
      if (lane == 0) atomicAdd(&mine[first], tally);
    }
#pragma unroll
    for (int j = 0; j < kSlots; ++j)
      if ((live[j] >> lane) & 1) atomicAdd(&mine[b[j]], 1);
  };
  auto any_crowd = [&](int key) {    // the same for every lane of the wave
    const int b = bin(key);
    const unsigned long long alive = __ballot(in_range(b));
    const int first = __builtin_amdgcn_readlane(b, (__ffsll(alive) - 1) & 63);
    return __popcll(alive & __ballot(b == first)) >= kCrowd;
  };
  const int64_t n4 = n >> 2;
  const int64_t step = static_cast<int64_t>(gridDim.x) * kThreads;
  int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const i32x4_t *k4 = reinterpret_cast<const i32x4_t *>(keys);
  // every lane of a wave makes the same number of passes: the masks above span the whole wave
  const int64_t wave_i = i - lane;
  int64_t w = wave_i;
  for (; w + 63 + (kUnroll - 1) * step < n4; w += kUnroll * step, i += kUnroll * step) {
    i32x4_t v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) v[u] = __builtin_nontemporal_load(k4 + i + u * step);
    if (any_crowd(v[0].x)) {
      crowded_pass(v);
    } else {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        plain(v[u].x);
        plain(v[u].y);
        plain(v[u].z);
        plain(v[u].w);
      }
    }
  }
  for (; i < n4; i += step) {
    const i32x4_t v = __builtin_nontemporal_load(k4 + i);
    plain(v.x);
    plain(v.y);
    plain(v.z);
    plain(v.w);
  }
  const int64_t ti = (n4 << 2) + threadIdx.x;
  if (blockIdx.x == gridDim.x - 1 && ti < n) plain(keys[ti]);
  __syncthreads();

  if (threadIdx.x < bins) {
    int total = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) total += counts[w][threadIdx.x];
    if (total != 0) atomicAdd(&histogram[threadIdx.x], total);
  }
}

// ---- one radix-sort pass: scatter ---------------------------------------------------------------
// benchmarks/bench_radix_sort.ml:120-137: every key takes the next free position of its digit,
//     pos = atomic_add_global(counters[digit], 1); output[pos] = key,
// one global atomic per key on 256 addresses (measured: 22.6 ms for 50M keys).  The order of the
// keys inside a digit's range is whatever order the atomics happen in.  Here a workgroup ranks a
// tile of keys inside LDS, takes its range of every digit with ONE global atomic per digit, orders
// the tile by digit in LDS and writes each digit's run to consecutive addresses: an order the
// reference's kernel can produce too (all keys of a workgroup arriving together), counters left
// exactly as it leaves them.  8 bytes per key.  What is left of the atomics still sets the pace below
// HBM speed: the 256 counters share eight cache lines, and the L2 retires about one 4-byte atomic per
// clock and line (15 ns per tile, whatever the tile size; 64-bit atomics on counter pairs cost the same).
// out_len guards the stores: a position outside [0, out_len) (counters that do not leave room for the
// keys) is skipped, where the reference's kernel would write out of bounds.  The tile (Threads * Keys
// keys) is staged in dynamic LDS.
template <int Threads, int Keys>
__global__ __launch_bounds__(Threads) void radix_scatter_kernel(int *__restrict__ out, int64_t out_len,
                                                                int *__restrict__ counters,
                                                                const int *__restrict__ keys, int64_t n, int shift,
                                                                int mask) {
  constexpr int kTile = Threads * Keys;
  extern __shared__ int stage[];    // kTile keys, ordered by digit
  __shared__ int count[kBins];      // keys of the tile per digit
  __shared__ int start[kBins];      // first slot of the digit in `stage` (exclusive scan of count)
  __shared__ int base[kBins];       // position in `out` of the digit's first key of this tile, less its slot
  __shared__ int wave_total[kBins / 64];
  const int t = threadIdx.x, lane = t & 63;
  const int64_t tile = static_cast<int64_t>(blockIdx.x) * kTile;
  const int valid = n - tile < kTile ? static_cast<int>(n - tile) : kTile;
  if (t < kBins) count[t] = 0;
  __syncthreads();

  // slot j of thread t is key tile + (j / 4 * Threads + t) * 4 + j % 4: 16-byte loads
  int key[Keys], rank[Keys];
  if (valid == kTile) {
    const i32x4_t *k4 = reinterpret_cast<const i32x4_t *>(keys + tile);
#pragma unroll
    for (int u = 0; u < Keys / 4; ++u) {
      const i32x4_t v = __builtin_nontemporal_load(k4 + u * Threads + t);
      key[4 * u] = v.x;
      key[4 * u + 1] = v.y;
      key[4 * u + 2] = v.z;
      key[4 * u + 3] = v.w;
    }
  } else {
#pragma unroll
    for (int j = 0; j < Keys; ++j) {
      const int at = ((j >> 2) * Threads + t) * 4 + (j & 3);
      key[j] = at < valid ? keys[tile + at] : 0;
    }
  }
  auto in_tile = [&](int j) { return ((j >> 2) * Threads + t) * 4 + (j & 3) < valid; };
#pragma unroll
  for (int j = 0; j < Keys; ++j)
    rank[j] = in_tile(j) ? atomicAdd(&count[(key[j] >> shift) & mask], 1) : 0;
  __syncthreads();

  if (t < kBins) {
    const int c = count[t];
    int incl = c;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o);
      if (lane >= o) incl += up;
    }
    if (lane == 63) wave_total[t >> 6] = incl;
    start[t] = incl - c;                       // within the wave; the waves before are added below
    base[t] = c != 0 ? atomicAdd(&counters[t], c) : 0;
  }
  __syncthreads();
  if (t < kBins) {
    int before = 0;
    for (int w = 0; w < (t >> 6); ++w) before += wave_total[w];
    start[t] += before;
    base[t] -= start[t];                       // slot s of digit t goes to out[base[t] + s]
  }
  __syncthreads();

#pragma unroll
  for (int j = 0; j < Keys; ++j)
    if (in_tile(j)) stage[start[(key[j] >> shift) & mask] + rank[j]] = key[j];
  __syncthreads();

  for (int s = t; s < valid; s += Threads) {
    const int k = stage[s];
    const int d = (k >> shift) & mask;
    const int64_t pos = static_cast<int64_t>(base[d]) + s;
    if (pos >= 0 && pos < out_len) out[pos] = k;
  }
}

template <int Threads, int Keys>
int launch_scatter(int *out, int64_t out_len, int *counters, const int *keys, int64_t n, int shift, int mask,
                   hipStream_t st) {
  constexpr int kTile = Threads * Keys;
  constexpr int kLds = kTile * 4;
  static_assert(Threads >= kBins && Threads % 64 == 0 && Keys % 4 == 0, "tile shape");
  const int64_t tiles = ceil_div(n, static_cast<int64_t>(kTile));
  if (tiles > 0x7FFFFFFF) return fail(SAREK_HIP_E_INVALID_ARG, "radix scatter: vector too long for one launch");
  auto kern = radix_scatter_kernel<Threads, Keys>;
  static bool attr_done[16] = {};
  int dev = 0;
  SAREK_HIP_TRY(hipGetDevice(&dev));
  if (dev >= 0 && dev < 16 && !attr_done[dev]) {
    SAREK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, kLds));
    attr_done[dev] = true;
  }
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(tiles)), dim3(Threads), kLds, st, out, out_len, counters,
                     keys, n, shift, mask);
  return check_launch("radix scatter kernel launch");
}

int compute_units() {
  static const int cus = [] {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
      v = 256;
    return v;
  }();
  return cus;
}

template <class Bin>
int launch(int *histogram, const int *keys, int64_t n, int bins, Bin bin, hipStream_t st) {
  // one workgroup per 64 KiB of keys until every CU has `per_cu` of them
  const int64_t per_cu = tunable("histogram.per_cu", 1);
  const int64_t cap = static_cast<int64_t>(compute_units()) * (per_cu < 1 ? 1 : per_cu);
  int64_t groups = ceil_div(n, static_cast<int64_t>(kThreads) * 16);
  if (groups > cap) groups = cap;
  if (groups < 1) groups = 1;
  hipLaunchKernelGGL(histogram_kernel<Bin>, dim3(static_cast<unsigned>(groups)), dim3(kThreads), 0, st, histogram,
                     keys, n, bins, bin);
  return check_launch("histogram kernel launch");
}

int check_common(const char *what, const int *histogram, const int *keys, int64_t n) {
  if (n < 0) return fail(SAREK_HIP_E_INVALID_ARG, "%s: negative length %lld", what, (long long)n);
  if (n > 0 && (!histogram || !keys)) return fail(SAREK_HIP_E_INVALID_ARG, "%s: NULL vector", what);
  return SAREK_HIP_OK;
}

}  // namespace
}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" {

int sarek_hip_histogram_i32(int32_t *histogram, const int32_t *keys, int64_t n, int num_bins,
                            sarek_hip_stream stream) {
  if (const int rc = check_common("histogram", histogram, keys, n)) return rc;
  if (num_bins < 1 || num_bins > kBins)
    return fail(SAREK_HIP_E_INVALID_ARG, "histogram: %d bins, 1 to %d are supported", num_bins, kBins);
  if (n == 0) return SAREK_HIP_OK;
  if ((num_bins & (num_bins - 1)) == 0)
    return launch(histogram, keys, n, num_bins, ModPow2Bin{static_cast<unsigned>(num_bins - 1)}, as_stream(stream));
  return launch(histogram, keys, n, num_bins, ModBin{num_bins}, as_stream(stream));
}

int sarek_hip_radix_histogram_i32(int32_t *histogram, const int32_t *keys, int64_t n, int shift, int mask,
                                  sarek_hip_stream stream) {
  if (const int rc = check_common("radix histogram", histogram, keys, n)) return rc;
  if (shift < 0 || shift > 31)
    return fail(SAREK_HIP_E_INVALID_ARG, "radix histogram: shift %d outside 0..31", shift);
  if (mask < 0 || mask >= kBins)
    return fail(SAREK_HIP_E_INVALID_ARG, "radix histogram: mask %d outside 0..%d", mask, kBins - 1);
  if (n == 0) return SAREK_HIP_OK;
  return launch(histogram, keys, n, kBins, DigitBin{shift, mask}, as_stream(stream));
}

int sarek_hip_radix_scatter_i32(int32_t *out, int64_t out_len, int32_t *counters, const int32_t *keys, int64_t n,
                                int shift, int mask, sarek_hip_stream stream) {
  if (const int rc = check_common("radix scatter", counters, keys, n)) return rc;
  if (out_len < 0) return fail(SAREK_HIP_E_INVALID_ARG, "radix scatter: negative output length");
  if (n > 0 && !out) return fail(SAREK_HIP_E_INVALID_ARG, "radix scatter: NULL vector");
  if (shift < 0 || shift > 31)
    return fail(SAREK_HIP_E_INVALID_ARG, "radix scatter: shift %d outside 0..31", shift);
  if (mask < 0 || mask >= kBins)
    return fail(SAREK_HIP_E_INVALID_ARG, "radix scatter: mask %d outside 0..%d", mask, kBins - 1);
  if (n == 0) return SAREK_HIP_OK;
  hipStream_t st = as_stream(stream);
  // Measured on MI355X: 16384-key tiles from about 4M keys on (half the global atomics of 8192-key tiles:
  // 95 against 142 us at 50M keys), 8192-key tiles below (more workgroups than CUs sooner), 32768-key tiles
  // from 2^27 keys on (573 against 648 us at 2^28 keys; 111 against 100 us at 50M).
  int64_t shape = tunable("radix_scatter.tile", 0);
  if (shape == 0) shape = n >= (int64_t{1} << 27) ? 4 : n >= (int64_t{1} << 22) ? 2 : 1;
  switch (shape) {
    case 1: return launch_scatter<512, 16>(out, out_len, counters, keys, n, shift, mask, st);
    case 2: return launch_scatter<1024, 16>(out, out_len, counters, keys, n, shift, mask, st);
    case 3: return launch_scatter<512, 32>(out, out_len, counters, keys, n, shift, mask, st);
    case 4: return launch_scatter<1024, 32>(out, out_len, counters, keys, n, shift, mask, st);
    default: return launch_scatter<512, 16>(out, out_len, counters, keys, n, shift, mask, st);
  }
}

}  // extern "C"
