// Plugin-level entry points: what Hip_plugin.run_source does for an external or
// generated kernel (compile cached, bind the run_source_arg list, launch on the
// default stream; sarek-cuda/Cuda_plugin.ml:174-220), plus the hand-kernel dispatch:
// a source that starts with "// sarek-hip-specialise: <tag>" is served by the matching
// hand-written kernel when the caller's launch geometry covers the whole problem the
// way the generated kernel assumes; otherwise the text is JIT-compiled as it stands.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "common.hpp"
#include "host/map_fuse.hpp"
#include "plugin.hpp"

namespace sarek_hip {

const char *const kSpecialiseMarker = "// sarek-hip-specialise: ";

namespace {

int g_specialise = -1;  // -1: read the environment on first use
thread_local std::string t_last_path = "none";

bool specialisation_enabled() {
  if (g_specialise < 0) {
    const char *e = std::getenv("SAREK_HIP_SPECIALISE");
    g_specialise = (e && e[0] == '0') ? 0 : 1;
  }
  return g_specialise == 1;
}

std::string read_tag(const char *source) {
  const size_t ml = std::strlen(kSpecialiseMarker);
  // skip leading whitespace / blank lines
  while (*source == ' ' || *source == '\n' || *source == '\r' || *source == '\t') ++source;
  if (std::strncmp(source, kSpecialiseMarker, ml) != 0) return "";
  const char *p = source + ml;
  const char *e = p;
  while (*e && *e != '\n' && *e != '\r' && *e != ' ') ++e;
  return std::string(p, e);
}

// A tag counts only on a text this library wrote: a library kernel's own text, or a text that
// generate_source produced here after the recogniser matched its IR.  A caller's program that merely
// starts with the same line is compiled and run as written.
bool tag_is_ours(const std::string &tag, const char *source) {
  if (is_library_kernel_name(tag)) return is_library_kernel_text(tag, source);
  return is_generated_tagged_text(source);
}

bool is_buf(const sarek_hip_arg &a) { return a.kind == SAREK_HIP_ARG_BUFFER; }
bool is_i32(const sarek_hip_arg &a) { return a.kind == SAREK_HIP_ARG_INT32; }
bool is_f32(const sarek_hip_arg &a) { return a.kind == SAREK_HIP_ARG_FLOAT32; }

// Argument shape of a generated kernel: each vector parameter is a buffer followed by
// its int32 length (Execute.expand_to_run_source_args, sarek/sarek/Execute.ml:197-216).
bool vec_at(const sarek_hip_arg *args, int n_args, int i) {
  return i + 1 < n_args && is_buf(args[i]) && is_i32(args[i + 1]) && args[i].buffer != nullptr;
}

int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// [p, p + n) and [q, q + n) (floats) share an element without being the same range.  Element-wise
// kernels give the same result in place as out of place; a shifted overlap is a race in the
// generated kernel and is left to it.
bool shifted_overlap(const void *p, const void *q, int64_t n) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p), b = reinterpret_cast<uintptr_t>(q);
  const uintptr_t bytes = static_cast<uintptr_t>(n) * 4;
  return a != b && a < b + bytes && b < a + bytes;
}

// Byte ranges [p, p + pb) and [q, q + qb) share a byte.
bool ranges_meet(const void *p, int64_t pb, const void *q, int64_t qb) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p), b = reinterpret_cast<uintptr_t>(q);
  return a < b + static_cast<uintptr_t>(qb) && b < a + static_cast<uintptr_t>(pb);
}

// A 1-D launch with at least `threads` threads.
bool covers_1d(const int block[3], const int grid[3], int64_t threads) {
  return block[1] == 1 && block[2] == 1 && grid[1] == 1 && grid[2] == 1 &&
         static_cast<int64_t>(block[0]) * grid[0] >= threads;
}

// An element-wise kernel (tag map_f32) rebuilt in the stream kernels' shape: 128-bit accesses, four loads per input
// in flight per thread, the kernel's own expression on every element; with `red` (the arguments of a block-256 sum
// launched right after it on the vector it writes) the sums leave in the same pass.  The text is compiled once per
// kernel and variant.  Returns 1 when the launch (or the pair) was served, 0 to fall back.
// The compiled kernel of one variant of a rebuilt text, built at the first launch that wants it and kept in the
// kernel's entry; nullptr when the text does not compile (a name of the kernel's that means something else in HIP, say:
// no reason to fail the launch, the generated kernel is still there).
sarek_hip_kernel rebuilt_kernel(MapEntry &e, int reduce, bool nt, uint32_t pad_bits, const char *entry_point) {
  std::lock_guard<std::mutex> lock(e.mu);
  const uint64_t generation = kernel_cache_generation();
  if (e.cache_generation != generation) {   // the compile cache was emptied: the handles kept here are gone
    e.built.clear();
    e.cache_generation = generation;
  }
  for (const MapEntry::Built &b : e.built)
    if (b.reduce == reduce && b.nt == nt && b.pad_bits == pad_bits) return static_cast<sarek_hip_kernel>(b.kernel);
  const std::string text = reduce < 0 ? (e.m.is_max ? ir::tree_max_source(e.m) : ir::tree_sum_source(e.m, nt))
                                      : ir::map_source(e.m, reduce, nt, pad_bits);
  sarek_hip_kernel k = nullptr;
  thread_local std::vector<char> log(16384);
  if (text.empty() || sarek_hip_kernel_compile_cached(text.c_str(), entry_point, &k, log.data(), log.size()) != SAREK_HIP_OK) {
    k = nullptr;
    last_error_slot().clear();   // the launch goes on with the generated text: the compiler's message is not its error
  }
  if (e.built.size() < 64) e.built.push_back({reduce, nt, pad_bits, k});
  return k;
}

int try_map(const char *source, const int block[3], const int grid[3], const sarek_hip_arg *a, int na,
            const sarek_hip_arg *red, int nred, const int rblock[3], const int rgrid[3], int *rc, bool red_is_max = false,
            uint32_t pad_bits = 0) {
  const std::shared_ptr<MapEntry> entry = find_generated_map(source);
  if (!entry) return 0;
  const ir::MapKernel &m = entry->m;
  struct Slot {
    union {
      void *p;
      int32_t i32;
      float f32;
    };
  };
  constexpr int kMaxParams = 24;
  if (m.params.size() + 1 > kMaxParams) return 0;
  Slot slots[kMaxParams];
  void *params[kMaxParams];
  int64_t lengths[kMaxParams];
  int ai = 0;
  for (size_t i = 0; i < m.params.size(); ++i) {
    lengths[i] = 0;
    switch (m.params[i].kind) {
      case ir::MapKernel::Param::Vec:
        if (!vec_at(a, na, ai)) return 0;
        slots[i].p = a[ai].buffer;
        lengths[i] = a[ai].length;
        ai += 2;
        break;
      case ir::MapKernel::Param::F32:
        if (ai >= na || !is_f32(a[ai])) return 0;
        slots[i].f32 = a[ai++].f32;
        break;
      case ir::MapKernel::Param::I32:
        if (ai >= na || !is_i32(a[ai])) return 0;
        slots[i].i32 = a[ai++].i32;
        break;
    }
    params[i] = &slots[i];
  }
  if (ai != na) return 0;
  const int64_t n = slots[m.n].i32;
  if (n <= 0 || n > 0x7FFFFFFF - 4096 || !covers_1d(block, grid, n)) return 0;
  if (lengths[m.out] < n) return 0;
  for (int in : m.inputs)
    if (lengths[in] < n || shifted_overlap(slots[m.out].p, slots[in].p, n)) return 0;
  const int64_t nblocks = cdiv(n, 256);
  void *partials = nullptr;
  if (red) {
    if (nred != 5 || !vec_at(red, nred, 0) || !vec_at(red, nred, 2) || !is_i32(red[4]) || red[4].i32 != n) return 0;
    if (rblock[0] != 256 || rblock[1] != 1 || rblock[2] != 1 || rgrid[1] != 1 || rgrid[2] != 1 || rgrid[0] != nblocks)
      return 0;
    if (red[0].buffer != slots[m.out].p || red[0].length < n || red[2].length < nblocks) return 0;
    if (ranges_meet(red[2].buffer, nblocks * 4, slots[m.out].p, n * 4)) return 0;
    for (int in : m.inputs)
      if (ranges_meet(red[2].buffer, nblocks * 4, slots[in].p, n * 4)) return 0;
    partials = red[2].buffer;
  }
  // inputs that together fit the 256 MB last-level cache may still be there: plain loads; larger ones go past it
  const bool nt = static_cast<int64_t>(m.inputs.size()) * n * 4 > (int64_t{256} << 20);
  const int reduce = !red ? 0 : red_is_max ? 2 : 1;
  sarek_hip_kernel k = rebuilt_kernel(*entry, reduce, nt, red_is_max ? pad_bits : 0, "sarek_map");
  if (!k) return 0;
  Slot part;
  part.p = partials;
  params[m.params.size()] = &part;
  const unsigned g[3] = {static_cast<unsigned>(cdiv(n, 4096)), 1, 1}, b[3] = {256, 1, 1};
  *rc = sarek_hip_kernel_launch(k, g, b, 0, nullptr, params, static_cast<int>(m.params.size()) + 1);
  return 1;
}

// A block-256 tree sum or maximum with an element-wise expression in front (tags tree_sum_map_f32, tree_max_map_f32),
// rebuilt in the hand block-256 kernel's shape.  Same conditions as for the plain tree: 256-thread blocks, exactly ceil(n / 256) of them.
int try_tree_map(const char *source, const int block[3], const int grid[3], const sarek_hip_arg *a, int na, int *rc) {
  const std::shared_ptr<MapEntry> entry = find_generated_map(source);
  if (!entry) return 0;
  const ir::MapKernel &m = entry->m;
  struct Slot {
    union {
      void *p;
      int32_t i32;
      float f32;
    };
  };
  constexpr int kMaxParams = 24;
  if (m.params.size() > kMaxParams) return 0;
  Slot slots[kMaxParams];
  void *params[kMaxParams];
  int64_t lengths[kMaxParams];
  int ai = 0;
  for (size_t i = 0; i < m.params.size(); ++i) {
    lengths[i] = 0;
    switch (m.params[i].kind) {
      case ir::MapKernel::Param::Vec:
        if (!vec_at(a, na, ai)) return 0;
        slots[i].p = a[ai].buffer;
        lengths[i] = a[ai].length;
        ai += 2;
        break;
      case ir::MapKernel::Param::F32:
        if (ai >= na || !is_f32(a[ai])) return 0;
        slots[i].f32 = a[ai++].f32;
        break;
      case ir::MapKernel::Param::I32:
        if (ai >= na || !is_i32(a[ai])) return 0;
        slots[i].i32 = a[ai++].i32;
        break;
    }
    params[i] = &slots[i];
  }
  if (ai != na) return 0;
  const int64_t n = slots[m.n].i32;
  if (n <= 0 || n > 0x7FFFFFFF - 8192) return 0;
  if (block[0] != 256 || block[1] != 1 || block[2] != 1 || grid[1] != 1 || grid[2] != 1) return 0;
  const int64_t nblocks = cdiv(n, 256);
  if (grid[0] != nblocks || lengths[m.out] < nblocks) return 0;
  for (int in : m.inputs)
    if (lengths[in] < n || ranges_meet(slots[m.out].p, nblocks * 4, slots[in].p, n * 4)) return 0;
  // the hand block-256 kernels read past the caches at every size
  sarek_hip_kernel k = rebuilt_kernel(*entry, -1, true, 0, "sarek_tree");
  if (!k) return 0;
  const unsigned g[3] = {static_cast<unsigned>(cdiv(nblocks, 32)), 1, 1}, b[3] = {256, 1, 1};
  *rc = sarek_hip_kernel_launch(k, g, b, 0, nullptr, params, static_cast<int>(m.params.size()));
  return 1;
}

// Returns 1 when the call was served by a hand kernel (status in *rc), 0 to fall back.
int try_specialised(const std::string &tag, const int block[3], const int grid[3],
                    const sarek_hip_arg *args, int n_args, int *rc) {
  if (tag == "matmul_tiled_f32") {
    // (a, len, b, len, c, len, m, n, k); block 16x16, grid covering the whole C.
    if (n_args != 9 || !vec_at(args, n_args, 0) || !vec_at(args, n_args, 2) ||
        !vec_at(args, n_args, 4) || !is_i32(args[6]) || !is_i32(args[7]) || !is_i32(args[8]))
      return 0;
    const int64_t m = args[6].i32, n = args[7].i32, k = args[8].i32;
    if (m <= 0 || n <= 0 || k <= 0) return 0;
    if (block[0] != 16 || block[1] != 16 || block[2] != 1) return 0;
    if (grid[0] < cdiv(n, 16) || grid[1] < cdiv(m, 16) || grid[2] != 1) return 0;
    if (args[0].length < m * k || args[2].length < k * n || args[4].length < m * n) return 0;
    // C written over A or B is a race in the generated kernel: left to it
    if (ranges_meet(args[4].buffer, m * n * 4, args[0].buffer, m * k * 4) ||
        ranges_meet(args[4].buffer, m * n * 4, args[2].buffer, k * n * 4))
      return 0;
    *rc = sarek_hip_gemm_f32(static_cast<const float *>(args[0].buffer),
                             static_cast<const float *>(args[2].buffer),
                             static_cast<float *>(args[4].buffer), (int)m, (int)n, (int)k, nullptr);
    return 1;
  }
  if (tag == "stream_triad_f32") {
    // (a, len, b, len, c, len, scalar, n); 1-D launch with at least n threads.
    if (n_args != 8 || !vec_at(args, n_args, 0) || !vec_at(args, n_args, 2) ||
        !vec_at(args, n_args, 4) || !is_f32(args[6]) || !is_i32(args[7]))
      return 0;
    const int64_t n = args[7].i32;
    if (n < 0) return 0;
    if (block[1] != 1 || block[2] != 1 || grid[1] != 1 || grid[2] != 1) return 0;
    if (static_cast<int64_t>(block[0]) * grid[0] < n) return 0;
    if (args[0].length < n || args[2].length < n || args[4].length < n) return 0;
    // in place (a is b or c) is element-wise and fine; a shifted overlap is a race in the generated kernel
    if (shifted_overlap(args[0].buffer, args[2].buffer, n) || shifted_overlap(args[0].buffer, args[4].buffer, n))
      return 0;
    *rc = sarek_hip_triad_f32(static_cast<float *>(args[0].buffer),
                              static_cast<const float *>(args[2].buffer),
                              static_cast<const float *>(args[4].buffer), args[6].f32, n, nullptr);
    return 1;
  }
  if (tag == "vector_add_f32") {
    // (a, len, b, len, c, len, n): c[i] = a[i] + b[i], i < n.  The triad kernel with scalar 1:
    // a + b*1 in double, rounded once, is the f32 sum.
    if (n_args != 7 || !vec_at(args, n_args, 0) || !vec_at(args, n_args, 2) || !vec_at(args, n_args, 4) ||
        !is_i32(args[6]))
      return 0;
    const int64_t n = args[6].i32;
    if (n < 0 || !covers_1d(block, grid, n)) return 0;
    if (args[0].length < n || args[2].length < n || args[4].length < n) return 0;
    if (shifted_overlap(args[4].buffer, args[0].buffer, n) || shifted_overlap(args[4].buffer, args[2].buffer, n))
      return 0;
    *rc = sarek_hip_triad_f32(static_cast<float *>(args[4].buffer), static_cast<const float *>(args[0].buffer),
                              static_cast<const float *>(args[2].buffer), 1.0f, n, nullptr);
    return 1;
  }
  if (tag == "vector_copy_f32") {
    // (a, len, b, len, n): b[i] = a[i], i < n
    if (n_args != 5 || !vec_at(args, n_args, 0) || !vec_at(args, n_args, 2) || !is_i32(args[4])) return 0;
    const int64_t n = args[4].i32;
    if (n < 0 || !covers_1d(block, grid, n)) return 0;
    if (args[0].length < n || args[2].length < n) return 0;
    if (shifted_overlap(args[2].buffer, args[0].buffer, n)) return 0;
    *rc = sarek_hip_copy_f32(static_cast<float *>(args[2].buffer), static_cast<const float *>(args[0].buffer), n,
                             nullptr);
    return 1;
  }
  if (tag == "matmul_naive_f32") {
    // (a, len, b, len, c, len, m, n, k); one thread per element of C, row = tid / n, col = tid mod n
    if (n_args != 9 || !vec_at(args, n_args, 0) || !vec_at(args, n_args, 2) ||
        !vec_at(args, n_args, 4) || !is_i32(args[6]) || !is_i32(args[7]) || !is_i32(args[8]))
      return 0;
    const int64_t m = args[6].i32, n = args[7].i32, k = args[8].i32;
    if (m <= 0 || n <= 0 || k <= 0 || m * n > 0x7FFFFFFF) return 0;
    if (!covers_1d(block, grid, m * n)) return 0;
    if (args[0].length < m * k || args[2].length < k * n || args[4].length < m * n) return 0;
    if (ranges_meet(args[4].buffer, m * n * 4, args[0].buffer, m * k * 4) ||
        ranges_meet(args[4].buffer, m * n * 4, args[2].buffer, k * n * 4))
      return 0;
    *rc = sarek_hip_gemm_f32(static_cast<const float *>(args[0].buffer),
                             static_cast<const float *>(args[2].buffer),
                             static_cast<float *>(args[4].buffer), (int)m, (int)n, (int)k, nullptr);
    return 1;
  }
  if (tag == "transpose_naive_f32" || tag == "transpose_tiled_f32") {
    // (input, len, output, len, width, height): output[c * height + r] = input[r * width + c]
    if (n_args != 6 || !vec_at(args, n_args, 0) || !vec_at(args, n_args, 2) || !is_i32(args[4]) ||
        !is_i32(args[5]))
      return 0;
    const int64_t w = args[4].i32, h = args[5].i32;
    if (w <= 0 || h <= 0 || w * h > 0x7FFFFFFF) return 0;
    if (tag == "transpose_naive_f32") {
      if (!covers_1d(block, grid, w * h)) return 0;
    } else {
      // 16 x 16 tiles; block x walks input columns, block y input rows
      if (block[0] != 16 || block[1] != 16 || block[2] != 1 || grid[2] != 1) return 0;
      if (grid[0] < cdiv(w, 16) || grid[1] < cdiv(h, 16)) return 0;
    }
    if (args[0].length < w * h || args[2].length < w * h) return 0;
    const uintptr_t in = reinterpret_cast<uintptr_t>(args[0].buffer),
                    out = reinterpret_cast<uintptr_t>(args[2].buffer), bytes = static_cast<uintptr_t>(w * h) * 4;
    if (in < out + bytes && out < in + bytes) return 0;   // overlapping matrices: leave it to the generated code
    *rc = sarek_hip_transpose_f32(static_cast<const float *>(args[0].buffer), static_cast<float *>(args[2].buffer),
                                  (int)w, (int)h, nullptr);
    return 1;
  }
  if (tag == "stencil_2d_f32" || tag == "conv2d_f32") {
    // (input, len, output, len, width, height).  The stencil's threads are the cells of a 2-D launch, the
    // filter's the cells in row-major order of a 1-D one; a launch that does not reach every cell computes
    // only those it reaches and is left to the generated code, like grids that overlap (cells read their
    // neighbours).
    if (n_args != 6 || !vec_at(args, n_args, 0) || !vec_at(args, n_args, 2) || !is_i32(args[4]) ||
        !is_i32(args[5]))
      return 0;
    const int64_t w = args[4].i32, h = args[5].i32;
    if (w <= 0 || h <= 0 || w * h > 0x7FFFFFFF) return 0;
    const bool stencil = tag[0] == 's';
    if (stencil) {
      if (block[2] != 1 || grid[2] != 1) return 0;
      if (static_cast<int64_t>(block[0]) * grid[0] < w || static_cast<int64_t>(block[1]) * grid[1] < h) return 0;
    } else if (!covers_1d(block, grid, w * h)) {
      return 0;
    }
    if (args[0].length < w * h || args[2].length < w * h) return 0;
    if (ranges_meet(args[0].buffer, w * h * 4, args[2].buffer, w * h * 4)) return 0;
    const float *in = static_cast<const float *>(args[0].buffer);
    float *out = static_cast<float *>(args[2].buffer);
    *rc = stencil ? sarek_hip_stencil_2d_f32(in, out, (int)w, (int)h, nullptr)
                  : sarek_hip_conv2d_f32(in, out, (int)w, (int)h, nullptr);
    return 1;
  }
  if (tag == "histogram_i32" || tag == "radix_histogram_i32") {
    // (input, len, histogram, len, n, num_bins) or (input, len, histogram, len, n, shift, mask).  Each block
    // clears and merges the bins below its own size, so a block at least as wide as the bin range makes the
    // launch a plain histogram of the keys its threads reach.
    const bool radix = tag[0] == 'r';
    if (n_args != (radix ? 7 : 6) || !vec_at(args, n_args, 0) || !vec_at(args, n_args, 2)) return 0;
    for (int i = 4; i < n_args; ++i)
      if (!is_i32(args[i])) return 0;
    if (block[1] != 1 || block[2] != 1 || grid[1] != 1 || grid[2] != 1) return 0;
    const int64_t reach = static_cast<int64_t>(block[0]) * grid[0];
    const int64_t n = args[4].i32 < reach ? args[4].i32 : reach;
    const int bins = radix ? 256 : args[5].i32;
    if (n < 0 || bins < 1 || bins > 256 || block[0] < bins) return 0;
    // up to a shift of 24 the eight digit bits are key bits whichever way `shr` fills from the left
    // (the reference's GPU code has `>>` on int, its Native backend Int32.shift_right_logical)
    if (radix && (args[5].i32 < 0 || args[5].i32 > 24 || args[6].i32 < 0 || args[6].i32 > 255)) return 0;
    if (args[0].length < n || args[2].length < bins) return 0;
    const uintptr_t in = reinterpret_cast<uintptr_t>(args[0].buffer), hist = reinterpret_cast<uintptr_t>(args[2].buffer);
    if (in < hist + static_cast<uintptr_t>(bins) * 4 && hist < in + static_cast<uintptr_t>(n) * 4) return 0;
    *rc = radix ? sarek_hip_radix_histogram_i32(static_cast<int32_t *>(args[2].buffer),
                                                static_cast<const int32_t *>(args[0].buffer), n, args[5].i32,
                                                args[6].i32, nullptr)
                : sarek_hip_histogram_i32(static_cast<int32_t *>(args[2].buffer),
                                          static_cast<const int32_t *>(args[0].buffer), n, bins, nullptr);
    return 1;
  }
  if (tag == "radix_scatter_i32") {
    // (input, len, output, len, counters, len, n, shift, mask): each key of the threads' reach takes the next
    // position of its digit
    if (n_args != 9 || !vec_at(args, n_args, 0) || !vec_at(args, n_args, 2) || !vec_at(args, n_args, 4) ||
        !is_i32(args[6]) || !is_i32(args[7]) || !is_i32(args[8]))
      return 0;
    if (block[1] != 1 || block[2] != 1 || grid[1] != 1 || grid[2] != 1) return 0;
    const int64_t reach = static_cast<int64_t>(block[0]) * grid[0];
    const int64_t n = args[6].i32 < reach ? args[6].i32 : reach;
    const int shift = args[7].i32, mask = args[8].i32;
    if (n < 0 || shift < 0 || shift > 24 || mask < 0 || mask > 255) return 0;
    if (args[0].length < n || args[2].length < 0 || args[4].length < mask + 1) return 0;
    const uintptr_t in = reinterpret_cast<uintptr_t>(args[0].buffer), out = reinterpret_cast<uintptr_t>(args[2].buffer),
                    cnt = reinterpret_cast<uintptr_t>(args[4].buffer);
    const uintptr_t in_b = static_cast<uintptr_t>(n) * 4, out_b = static_cast<uintptr_t>(args[2].length) * 4,
                    cnt_b = static_cast<uintptr_t>(mask + 1) * 4;
    auto meet = [](uintptr_t a, uintptr_t ab, uintptr_t b, uintptr_t bb) { return a < b + bb && b < a + ab; };
    if (meet(in, in_b, out, out_b) || meet(in, in_b, cnt, cnt_b) || meet(out, out_b, cnt, cnt_b)) return 0;
    *rc = sarek_hip_radix_scatter_i32(static_cast<int32_t *>(args[2].buffer), args[2].length,
                                      static_cast<int32_t *>(args[4].buffer),
                                      static_cast<const int32_t *>(args[0].buffer), n, shift, mask, nullptr);
    return 1;
  }
  if (tag == "reduce_sum_block256_f32" || tag == "dot_block256_f32") {
    const bool dot = tag[0] == 'd';
    const int nv = dot ? 3 : 2;
    if (n_args != 2 * nv + 1) return 0;
    for (int v = 0; v < nv; ++v)
      if (!vec_at(args, n_args, 2 * v)) return 0;
    if (!is_i32(args[2 * nv])) return 0;
    const int64_t n = args[2 * nv].i32;
    if (n < 0) return 0;
    // the generated kernel's tree is written for exactly 256 threads per block
    if (block[0] != 256 || block[1] != 1 || block[2] != 1 || grid[1] != 1 || grid[2] != 1) return 0;
    const int64_t nblocks = cdiv(n, 256);
    // blocks past ceil(n/256) would store zeros; only take over when the grid is exact
    if (grid[0] != nblocks) return 0;
    if (args[2 * (nv - 1)].length < nblocks) return 0;
    for (int v = 0; v < nv - 1; ++v) {
      if (args[2 * v].length < n) return 0;
    }
    if (dot)
      *rc = sarek_hip_dot_block256_f32(static_cast<const float *>(args[0].buffer),
                                       static_cast<const float *>(args[2].buffer),
                                       static_cast<float *>(args[4].buffer), n, nullptr);
    else
      *rc = sarek_hip_reduce_sum_block256_f32(static_cast<const float *>(args[0].buffer),
                                              static_cast<float *>(args[2].buffer), n, nullptr);
    return 1;
  }
  if (tag.compare(0, 24, "reduce_max_block256_f32:") == 0 && tag.size() == 32) {
    // (input, len, output, len, n); the fill value travels in the tag as f32 bits
    char *end = nullptr;
    const unsigned long bits = std::strtoul(tag.c_str() + 24, &end, 16);
    if (*end != 0) return 0;
    const uint32_t b32 = static_cast<uint32_t>(bits);
    float pad;
    std::memcpy(&pad, &b32, 4);
    if (n_args != 5 || !vec_at(args, n_args, 0) || !vec_at(args, n_args, 2) || !is_i32(args[4])) return 0;
    const int64_t n = args[4].i32;
    if (n < 0) return 0;
    if (block[0] != 256 || block[1] != 1 || block[2] != 1 || grid[1] != 1 || grid[2] != 1) return 0;
    const int64_t nblocks = cdiv(n, 256);
    if (grid[0] != nblocks || args[2].length < nblocks || args[0].length < n) return 0;
    *rc = sarek_hip_reduce_max_block256_f32(static_cast<const float *>(args[0].buffer),
                                            static_cast<float *>(args[2].buffer), n, pad, nullptr);
    return 1;
  }
  // ---- the library kernels (texts from sarek_hip_library_kernel_source) -----------------------
  if (tag == "gemm_bf16" || tag == "gemm_f16") {
    // (a, len, b, len, c, len, m, n, k); a, b: 2-byte elements; 2-D launch, one thread per element of C
    if (n_args != 9 || !vec_at(args, n_args, 0) || !vec_at(args, n_args, 2) || !vec_at(args, n_args, 4) ||
        !is_i32(args[6]) || !is_i32(args[7]) || !is_i32(args[8]))
      return 0;
    const int64_t m = args[6].i32, n = args[7].i32, k = args[8].i32;
    if (m <= 0 || n <= 0 || k <= 0) return 0;
    if (block[2] != 1 || grid[2] != 1) return 0;
    if (static_cast<int64_t>(block[0]) * grid[0] < n || static_cast<int64_t>(block[1]) * grid[1] < m) return 0;
    if (args[0].length < m * k || args[2].length < k * n || args[4].length < m * n) return 0;
    if (ranges_meet(args[4].buffer, m * n * 4, args[0].buffer, m * k * 2) ||
        ranges_meet(args[4].buffer, m * n * 4, args[2].buffer, k * n * 2))
      return 0;
    auto fn = tag == "gemm_bf16" ? sarek_hip_gemm_bf16 : sarek_hip_gemm_f16;
    *rc = fn(static_cast<const uint16_t *>(args[0].buffer), static_cast<const uint16_t *>(args[2].buffer),
             static_cast<float *>(args[4].buffer), (int)m, (int)n, (int)k, nullptr);
    return 1;
  }
  if (tag == "gemm_f16_bias_relu_rowsum") {
    // (a, len, b, len, bias, len, y, len, rowsum, len, m, n, k); 1-D launch, workgroups take whole rows
    if (n_args != 13) return 0;
    for (int v = 0; v < 5; ++v)
      if (!vec_at(args, n_args, 2 * v)) return 0;
    if (!is_i32(args[10]) || !is_i32(args[11]) || !is_i32(args[12])) return 0;
    const int64_t m = args[10].i32, n = args[11].i32, k = args[12].i32;
    if (m <= 0 || n <= 0 || k <= 0) return 0;
    if (block[1] != 1 || block[2] != 1 || grid[1] != 1 || grid[2] != 1) return 0;
    if (args[0].length < m * k || args[2].length < k * n || args[4].length < n || args[6].length < m * n ||
        args[8].length < m)
      return 0;
    const void *ptr[5] = {args[0].buffer, args[2].buffer, args[4].buffer, args[6].buffer, args[8].buffer};
    const int64_t bytes[5] = {m * k * 2, k * n * 2, n * 4, m * n * 4, m * 4};
    for (int out = 3; out < 5; ++out)          // y and rowsum against everything else
      for (int other = 0; other < 5; ++other)
        if (other != out && ranges_meet(ptr[out], bytes[out], ptr[other], bytes[other])) return 0;
    *rc = sarek_hip_gemm_f16_bias_relu_rowsum(static_cast<const uint16_t *>(args[0].buffer),
                                              static_cast<const uint16_t *>(args[2].buffer),
                                              static_cast<const float *>(args[4].buffer),
                                              static_cast<float *>(args[6].buffer),
                                              static_cast<float *>(args[8].buffer), (int)m, (int)n, (int)k, nullptr);
    return 1;
  }
  if (tag == "triad_sum_f32") {
    // (a, len, b, len, c, len, sum (f64), len, scalar, n); one 1-D workgroup of a power-of-two size
    if (n_args != 10 || !vec_at(args, n_args, 0) || !vec_at(args, n_args, 2) || !vec_at(args, n_args, 4) ||
        !vec_at(args, n_args, 6) || !is_f32(args[8]) || !is_i32(args[9]))
      return 0;
    const int64_t n = args[9].i32;
    if (n < 0) return 0;
    if (grid[0] != 1 || grid[1] != 1 || grid[2] != 1 || block[1] != 1 || block[2] != 1) return 0;
    if (block[0] > 1024 || (block[0] & (block[0] - 1)) != 0) return 0;
    if (args[0].length < n || args[2].length < n || args[4].length < n || args[6].length < 1) return 0;
    if (shifted_overlap(args[0].buffer, args[2].buffer, n) || shifted_overlap(args[0].buffer, args[4].buffer, n))
      return 0;
    for (int v = 0; v < 3; ++v)
      if (ranges_meet(args[6].buffer, 8, args[2 * v].buffer, n * 4)) return 0;
    if (reinterpret_cast<uintptr_t>(args[6].buffer) % 8 != 0) return 0;
    // n is an int32: always within what the library's own partials array serves
    *rc = sarek_hip_triad_sum_f32_static(static_cast<float *>(args[0].buffer),
                                         static_cast<const float *>(args[2].buffer),
                                         static_cast<const float *>(args[4].buffer), args[8].f32, n,
                                         static_cast<double *>(args[6].buffer), nullptr);
    return 1;
  }
  return 0;
}

// The pair `stream triad, then the block-256 sum of the triad's output`, both recognised from IR,
// served by one pass over the data.  Conditions: each launch alone would be taken over (same
// checks as above), the sum reads exactly the vector the triad writes, over the same n, and its
// output lies apart from the triad's three vectors.
int try_specialised_pair(const std::string &tag0, const int block0[3], const int grid0[3],
                         const sarek_hip_arg *a0, int n0, const std::string &tag1, const int block1[3],
                         const int grid1[3], const sarek_hip_arg *a1, int n1, int *rc) {
  // the reduction: the block-256 sum (input, len, output, len, n) or the block-256 maximum, same arguments, whose
  // fill value travels in the tag as f32 bits
  const bool is_sum = tag1 == "reduce_sum_block256_f32";
  const bool is_max = tag1.compare(0, 24, "reduce_max_block256_f32:") == 0 && tag1.size() == 32;
  if (!is_sum && !is_max) return 0;
  float pad = 0.f;
  if (is_max) {
    char *end = nullptr;
    const unsigned long bits = std::strtoul(tag1.c_str() + 24, &end, 16);
    if (*end != 0) return 0;
    const uint32_t b32 = static_cast<uint32_t>(bits);
    std::memcpy(&pad, &b32, 4);
  }
  // the element-wise producer: the stream triad (a, len, b, len, c, len, scalar, n), a = b + scalar * c, or the vector
  // add (a, len, b, len, c, len, n), c = a + b, which is the triad with scalar 1 (one rounding of the exact sum)
  int out, in0, in1;
  float scalar;
  int64_t n;
  if (tag0 == "stream_triad_f32") {
    if (n0 != 8 || !is_f32(a0[6]) || !is_i32(a0[7])) return 0;
    out = 0, in0 = 2, in1 = 4, scalar = a0[6].f32, n = a0[7].i32;
  } else if (tag0 == "vector_add_f32") {
    if (n0 != 7 || !is_i32(a0[6])) return 0;
    out = 4, in0 = 0, in1 = 2, scalar = 1.0f, n = a0[6].i32;
  } else {
    return 0;
  }
  if (!vec_at(a0, n0, 0) || !vec_at(a0, n0, 2) || !vec_at(a0, n0, 4)) return 0;
  if (n1 != 5 || !vec_at(a1, n1, 0) || !vec_at(a1, n1, 2) || !is_i32(a1[4])) return 0;
  if (n <= 0 || a1[4].i32 != n) return 0;
  if (!covers_1d(block0, grid0, n)) return 0;
  if (a0[0].length < n || a0[2].length < n || a0[4].length < n) return 0;
  if (shifted_overlap(a0[out].buffer, a0[in0].buffer, n) || shifted_overlap(a0[out].buffer, a0[in1].buffer, n)) return 0;
  const int64_t nblocks = cdiv(n, 256);
  if (block1[0] != 256 || block1[1] != 1 || block1[2] != 1 || grid1[1] != 1 || grid1[2] != 1) return 0;
  if (grid1[0] != nblocks) return 0;
  if (a1[0].buffer != a0[out].buffer || a1[0].length < n || a1[2].length < nblocks) return 0;
  for (int v = 0; v < 3; ++v) {
    if (ranges_meet(a1[2].buffer, nblocks * 4, a0[2 * v].buffer, n * 4)) return 0;
  }
  if (is_sum)
    *rc = sarek_hip_triad_block256_sum_f32(static_cast<float *>(a0[out].buffer), static_cast<const float *>(a0[in0].buffer),
                                           static_cast<const float *>(a0[in1].buffer), scalar, n,
                                           static_cast<float *>(a1[2].buffer), nullptr);
  else
    *rc = sarek_hip_triad_block256_max_f32(static_cast<float *>(a0[out].buffer), static_cast<const float *>(a0[in0].buffer),
                                           static_cast<const float *>(a0[in1].buffer), scalar, n, pad,
                                           static_cast<float *>(a1[2].buffer), nullptr);
  return 1;
}

// An element-wise kernel followed by the block-256 sum or maximum (fill value in the tag, as f32 bits) of its output
int try_map_pair(const sarek_hip_launch &l0, const std::string &tag1, const sarek_hip_launch &l1, int *rc) {
  if (tag1 == "reduce_sum_block256_f32")
    return try_map(l0.source, l0.block, l0.grid, l0.args, l0.n_args, l1.args, l1.n_args, l1.block, l1.grid, rc);
  if (tag1.compare(0, 24, "reduce_max_block256_f32:") == 0 && tag1.size() == 32) {
    char *end = nullptr;
    const unsigned long bits = std::strtoul(tag1.c_str() + 24, &end, 16);
    if (*end != 0) return 0;
    return try_map(l0.source, l0.block, l0.grid, l0.args, l0.n_args, l1.args, l1.n_args, l1.block, l1.grid, rc, true,
                   static_cast<uint32_t>(bits));
  }
  return 0;
}

}  // namespace

}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" {

int sarek_hip_set_specialisation(int enabled) {
  g_specialise = enabled ? 1 : 0;
  return SAREK_HIP_OK;
}

const char *sarek_hip_last_run_path(void) { return t_last_path.c_str(); }

int sarek_hip_run_sources(const sarek_hip_launch *launches, int n_launches, int *device_launches, int *completed) {
  if (device_launches) *device_launches = 0;
  if (completed) *completed = 0;
  if (n_launches < 0 || (n_launches > 0 && !launches))
    return fail(SAREK_HIP_E_INVALID_ARG, "run_sources: NULL or negative argument");
  std::string path;
  for (int i = 0; i < n_launches; ++i) {
    const sarek_hip_launch &l0 = launches[i];
    int served = 0;
    if (i + 1 < n_launches && specialisation_enabled() && l0.source && launches[i + 1].source && l0.args &&
        launches[i + 1].args) {
      // two launches one hand-written kernel computes in a single pass over the data
      const sarek_hip_launch &l1 = launches[i + 1];
      const bool langs_ok = (l0.lang == SAREK_HIP_LANG_HIP_SOURCE || l0.lang == SAREK_HIP_LANG_CUDA_SOURCE) &&
                            (l1.lang == SAREK_HIP_LANG_HIP_SOURCE || l1.lang == SAREK_HIP_LANG_CUDA_SOURCE);
      const std::string tag0 = read_tag(l0.source), tag1 = read_tag(l1.source);
      int rc = SAREK_HIP_OK;
      if (langs_ok && !tag0.empty() && !tag1.empty() && tag_is_ours(tag0, l0.source) && tag_is_ours(tag1, l1.source) &&
          (tag0 == "map_f32"
               ? try_map_pair(l0, tag1, l1, &rc)
               : try_specialised_pair(tag0, l0.block, l0.grid, l0.args, l0.n_args, tag1, l1.block, l1.grid, l1.args,
                                      l1.n_args, &rc))) {
        if (rc != SAREK_HIP_OK) return rc;
        path += (path.empty() ? "" : ";") + tag0 + "+" + tag1;
        served = 2;
      }
    }
    if (!served) {
      const int rc = sarek_hip_run_source(l0.source, l0.lang, l0.kernel_name, l0.block, l0.grid, l0.shared_mem_bytes,
                                          l0.args, l0.n_args);
      if (rc != SAREK_HIP_OK) return rc;
      path += (path.empty() ? "" : ";") + t_last_path;
      served = 1;
    }
    i += served - 1;
    if (device_launches) ++*device_launches;
    if (completed) *completed += served;
  }
  t_last_path = path.empty() ? "none" : path;
  return SAREK_HIP_OK;
}

int sarek_hip_run_source(const char *source, int lang, const char *kernel_name, const int block[3],
                         const int grid[3], int shared_mem_bytes, const sarek_hip_arg *args,
                         int n_args) {
  t_last_path = "none";
  if (!source || !kernel_name || !block || !grid || n_args < 0 || (n_args > 0 && !args))
    return fail(SAREK_HIP_E_INVALID_ARG, "run_source: NULL or negative argument");
  switch (lang) {
    case SAREK_HIP_LANG_HIP_SOURCE:
    case SAREK_HIP_LANG_CUDA_SOURCE:
      break;
    case SAREK_HIP_LANG_OPENCL_SOURCE:
      return fail(SAREK_HIP_E_UNSUPPORTED, "HIP backend does not support OpenCL_Source");
    case SAREK_HIP_LANG_PTX:
      return fail(SAREK_HIP_E_UNSUPPORTED, "HIP backend does not support PTX");
    case SAREK_HIP_LANG_SPIR_V:
      return fail(SAREK_HIP_E_UNSUPPORTED, "HIP backend does not support SPIR_V");
    case SAREK_HIP_LANG_GLSL_SOURCE:
      return fail(SAREK_HIP_E_UNSUPPORTED, "HIP backend does not support GLSL_Source");
    default:
      return fail(SAREK_HIP_E_INVALID_ARG, "run_source: unknown source language %d", lang);
  }
  for (int i = 0; i < 3; ++i)
    if (block[i] <= 0 || grid[i] <= 0)
      return fail(SAREK_HIP_E_INVALID_ARG, "run_source: block and grid dimensions must be positive");
  if (shared_mem_bytes < 0)
    return fail(SAREK_HIP_E_INVALID_ARG, "run_source: negative shared memory size");

  if (specialisation_enabled()) {
    std::string tag = read_tag(source);
    if (!tag.empty() && !tag_is_ours(tag, source)) tag.clear();
    if (!tag.empty()) {
      int rc = SAREK_HIP_OK;
      if (tag == "map_f32"            ? try_map(source, block, grid, args, n_args, nullptr, 0, nullptr, nullptr, &rc)
          : tag == "tree_sum_map_f32" || tag == "tree_max_map_f32" ? try_tree_map(source, block, grid, args, n_args, &rc)
                                      : try_specialised(tag, block, grid, args, n_args, &rc)) {
        t_last_path = tag;
        return rc;
      }
    }
  }

  sarek_hip_kernel k = nullptr;
  thread_local std::vector<char> log(16384);        // compile log, filled on a failed compile only
  int rc = sarek_hip_kernel_compile_cached(source, kernel_name, &k, log.data(), log.size());
  if (rc != SAREK_HIP_OK) return rc;

  // Parameter block: one slot per argument, kept alive until the launch call returns.
  struct Slot {
    union {
      void *p;
      int32_t i32;
      int64_t i64;
      float f32;
      double f64;
    };
  };
  constexpr int kInline = 32;                        // launches with more arguments take the heap
  Slot inline_slots[kInline];
  void *inline_params[kInline];
  std::vector<Slot> heap_slots;
  std::vector<void *> heap_params;
  Slot *slots = inline_slots;
  void **params = inline_params;
  if (n_args > kInline) {
    heap_slots.resize(n_args);
    heap_params.resize(n_args);
    slots = heap_slots.data();
    params = heap_params.data();
  }
  for (int i = 0; i < n_args; ++i) {
    switch (args[i].kind) {
      case SAREK_HIP_ARG_BUFFER: slots[i].p = args[i].buffer; break;
      case SAREK_HIP_ARG_INT32: slots[i].i32 = args[i].i32; break;
      case SAREK_HIP_ARG_INT64: slots[i].i64 = args[i].i64; break;
      case SAREK_HIP_ARG_FLOAT32: slots[i].f32 = args[i].f32; break;
      case SAREK_HIP_ARG_FLOAT64: slots[i].f64 = args[i].f64; break;
      default:
        return fail(SAREK_HIP_E_INVALID_ARG, "run_source: argument %d has unknown kind %d", i,
                    args[i].kind);
    }
    params[i] = &slots[i];
  }
  const unsigned g[3] = {(unsigned)grid[0], (unsigned)grid[1], (unsigned)grid[2]};
  const unsigned b[3] = {(unsigned)block[0], (unsigned)block[1], (unsigned)block[2]};
  rc = sarek_hip_kernel_launch(k, g, b, (unsigned)shared_mem_bytes, nullptr, params, n_args);
  if (rc == SAREK_HIP_OK) t_last_path = "jit";
  return rc;
}
}
