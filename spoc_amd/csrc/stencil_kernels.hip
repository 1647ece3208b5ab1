// The reference's two 2-D neighbourhood kernels, hand-written for gfx950: the five-point mean of
// benchmarks/bench_stencil_2d.ml:43-58 and the 3 x 3 box filter of benchmarks/bench_conv2d.ml:49-77.
// Both are HBM-bound at 8 bytes per cell (every input cell read once, every output cell written once).  The
// generated kernels fetch five or nine scalars per cell and leave the reuse to the caches; here a wave owns a strip
// of 256 columns (four per lane, 128-bit accesses), walks a band of rows down it with the last three input rows of
// its columns in registers, and takes the columns next to a lane's four from the neighbouring lanes by wave
// shuffles (from memory at the two ends of the strip), so a row is fetched once per band plus the band's two halo
// rows, which the band above or below has just brought into the L2.  The four waves of a workgroup take four
// neighbouring strips, 4 KiB of every row in one piece (four bands of one strip instead: 10-15 % slower).  The
// arithmetic is the Native backend's: the operands widened to double, added in the order the kernel text adds them,
// divided in double, rounded once at the store.
#include "common.hpp"
#include "tunables.hpp"

namespace sarek_hip {
namespace {

typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr int kBlock = 256;   // four waves: four neighbouring strips of one band
constexpr int kStrip = 256;   // columns of a strip: 64 lanes x 4

// A lane's four cells of one input row (columns x0 .. x0 + 3) with the cells left and right of them; cells outside
// the row read as 0 and are never used.
struct Row {
  float c[6];   // c[0] = column x0 - 1, c[1..4] = columns x0 .. x0 + 3, c[5] = column x0 + 4
};

__device__ __forceinline__ Row load_row(const float *__restrict__ in, int w, int y, int x0, int lane) {
  Row q;
  const float *p = in + static_cast<int64_t>(y) * w + x0;
  if (x0 + 3 < w) {
    // element alignment is all a 128-bit load needs; a plain load: the halo rows are read again from the L2
    // (non-temporal loads: 4-12 % slower)
    const f32x4_t t = *reinterpret_cast<const f32x4_t *>(p);
    q.c[1] = t.x, q.c[2] = t.y, q.c[3] = t.z, q.c[4] = t.w;
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) q.c[1 + j] = x0 + j < w ? p[j] : 0.f;
  }
  q.c[0] = __shfl_up(q.c[4], 1, 64);
  q.c[5] = __shfl_down(q.c[1], 1, 64);
  if (lane == 0) q.c[0] = x0 > 0 ? p[-1] : 0.f;
  if (lane == 63) q.c[5] = x0 + 4 < w ? p[4] : 0.f;
  return q;
}

// Output row y from input rows y - 1 (a), y (b), y + 1 (c); 1 <= y <= h - 2.
template <bool Box>
__device__ __forceinline__ void emit_row(float *__restrict__ out, int w, int y, int x0, const Row &a, const Row &b,
                                         const Row &c) {
  if (x0 >= w) return;
  float res[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = j + 1;
    if constexpr (Box) {
      // p00 + p01 + p02 + p10 + p11 + p12 + p20 + p21 + p22, left to right (bench_conv2d.ml:62-75)
      double s = static_cast<double>(a.c[i - 1]) + static_cast<double>(a.c[i]);
      s = s + static_cast<double>(a.c[i + 1]);
      s = s + static_cast<double>(b.c[i - 1]);
      s = s + static_cast<double>(b.c[i]);
      s = s + static_cast<double>(b.c[i + 1]);
      s = s + static_cast<double>(c.c[i - 1]);
      s = s + static_cast<double>(c.c[i]);
      s = s + static_cast<double>(c.c[i + 1]);
      res[j] = static_cast<float>(s / 9.0);
    } else {
      // (up + down + left + right + center) / 5 (bench_stencil_2d.ml:52-58)
      double s = static_cast<double>(a.c[i]) + static_cast<double>(c.c[i]);
      s = s + static_cast<double>(b.c[i - 1]);
      s = s + static_cast<double>(b.c[i + 1]);
      s = s + static_cast<double>(b.c[i]);
      res[j] = static_cast<float>(s / 5.0);
    }
  }
  float *p = out + static_cast<int64_t>(y) * w + x0;
  if constexpr (Box) {
    // the first and the last column are written as 0
    if (x0 == 0) res[0] = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (x0 + j == w - 1) res[j] = 0.f;
    if (x0 + 3 < w) {
      __builtin_nontemporal_store(f32x4_t{res[0], res[1], res[2], res[3]}, reinterpret_cast<f32x4_t *>(p));
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (x0 + j < w) p[j] = res[j];
    }
  } else {
    // the first and the last column keep what they hold
    if (x0 >= 1 && x0 + 3 <= w - 2) {
      __builtin_nontemporal_store(f32x4_t{res[0], res[1], res[2], res[3]}, reinterpret_cast<f32x4_t *>(p));
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (x0 + j >= 1 && x0 + j <= w - 2) p[j] = res[j];
    }
  }
}

__device__ __forceinline__ void zero_row(float *__restrict__ out, int w, int y, int x0) {
  float *p = out + static_cast<int64_t>(y) * w + x0;
  if (x0 + 3 < w) {
    __builtin_nontemporal_store(f32x4_t{0.f, 0.f, 0.f, 0.f}, reinterpret_cast<f32x4_t *>(p));
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (x0 + j < w) p[j] = 0.f;
  }
}

// Box = false: output[y][x] = (up + down + left + right + center) / 5 for 0 < x < w - 1, 0 < y < h - 1, the border
// untouched.  Box = true: the mean of the 3 x 3 cells round (x, y) there, 0 on the border.  4 * blockIdx.x + wave is
// the strip, blockIdx.y the band of `rows` output rows.  Every lane of a wave stays in the loop (the shuffles need
// them all); lanes past the last column neither load nor store.  Two rows are asked for before either is used, so
// a wave has 2 KiB of loads in flight (four rows: the same speed with more registers).
template <bool Box>
__global__ __launch_bounds__(kBlock) void neighbourhood_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                               int w, int h, int rows) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  constexpr int U = 2;
  const int strip = blockIdx.x * (kBlock / 64) + wave;
  const int x0 = strip * kStrip + lane * 4;
  const int64_t y_begin64 = static_cast<int64_t>(blockIdx.y) * rows;
  if (y_begin64 >= h || strip * kStrip >= w) return;   // whole waves leave together; the kernel has no barrier
  const int y_begin = static_cast<int>(y_begin64);
  const int y_end = y_begin + rows < h ? y_begin + rows : h;
  if constexpr (Box) {
    if (x0 < w) {
      if (y_begin == 0) zero_row(out, w, 0, x0);
      if (y_end == h && h > 1) zero_row(out, w, h - 1, x0);
    }
  }
  const int ys = y_begin > 1 ? y_begin : 1;
  const int ye = y_end < h - 1 ? y_end : h - 1;
  if (ys >= ye) return;
  Row win[U + 2];   // input rows y - 1 .. y + U
  win[0] = load_row(in, w, ys - 1, x0, lane);
  win[1] = load_row(in, w, ys, x0, lane);
  int y = ys;
  for (; y + U <= ye; y += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) win[2 + u] = load_row(in, w, y + 1 + u, x0, lane);
#pragma unroll
    for (int u = 0; u < U; ++u) emit_row<Box>(out, w, y + u, x0, win[u], win[u + 1], win[u + 2]);
    win[0] = win[U];
    win[1] = win[U + 1];
  }
  for (; y < ye; ++y) {
    win[2] = load_row(in, w, y + 1, x0, lane);
    emit_row<Box>(out, w, y, x0, win[0], win[1], win[2]);
    win[0] = win[1];
    win[1] = win[2];
  }
}

template <bool Box>
int launch_neighbourhood(const char *what, const float *in, float *out, int width, int height,
                         sarek_hip_stream stream) {
  if (width < 0 || height < 0) return fail(SAREK_HIP_E_INVALID_ARG, "%s: negative shape %d x %d", what, width, height);
  if (width == 0 || height == 0) return SAREK_HIP_OK;
  // (a strip may reach 1023 columns past the width: those column numbers must still fit an int)
  if (static_cast<int64_t>(width) * height > 0x7FFFFFFF || width > 0x7FFFFFFF - 1024)
    return fail(SAREK_HIP_E_INVALID_ARG, "%s: %d x %d cells exceed the kernel's int32 indices", what, width, height);
  if (!in || !out) return fail(SAREK_HIP_E_INVALID_ARG, "%s: NULL grid", what);
  const uintptr_t pi = reinterpret_cast<uintptr_t>(in), po = reinterpret_cast<uintptr_t>(out);
  const uintptr_t bytes = static_cast<uintptr_t>(width) * height * 4;
  if (pi < po + bytes && po < pi + bytes)
    return fail(SAREK_HIP_E_INVALID_ARG, "%s: input and output overlap (cells read their neighbours)", what);
  if (!Box && (width < 3 || height < 3)) return SAREK_HIP_OK;   // no interior: nothing is written
  // Rows per band.  Short bands win although they fetch more halo rows (those hit in the L2): 4 rows, or 8 for grids
  // of at most 2^24 cells that still make 4096 waves with them (measured on 1024^2 ... 32768 x 8192 and ragged
  // shapes: 16 and 32 rows are 5-20 % slower on most, and which of 4 and 8 is ahead changes with the shape by a few
  // per cent).  stencil.rows: 0 = this rule.
  const int strips = (width + kStrip - 1) / kStrip;
  int rows = static_cast<int>(tunable("stencil.rows", 0));
  if (rows <= 0)
    rows = static_cast<int64_t>(width) * height <= (1 << 24) && static_cast<int64_t>(height) * strips / 8 >= 4096 ? 8 : 4;
  const int64_t bands = (static_cast<int64_t>(height) + rows - 1) / rows;
  if (bands > 65535) {   // a very tall grid: taller bands
    rows = static_cast<int>((static_cast<int64_t>(height) + 65534) / 65535);
    rows += rows & 1;
  }
  const dim3 grid((strips + kBlock / 64 - 1) / (kBlock / 64),
                  static_cast<unsigned>((static_cast<int64_t>(height) + rows - 1) / rows));
  hipLaunchKernelGGL((neighbourhood_kernel<Box>), grid, dim3(kBlock), 0, as_stream(stream), in, out, width, height,
                     rows);
  return check_launch(what);
}

}  // namespace
}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" {

int sarek_hip_stencil_2d_f32(const float *input, float *output, int width, int height, sarek_hip_stream stream) {
  return launch_neighbourhood<false>("stencil_2d kernel launch", input, output, width, height, stream);
}

int sarek_hip_conv2d_f32(const float *input, float *output, int width, int height, sarek_hip_stream stream) {
  return launch_neighbourhood<true>("conv2d kernel launch", input, output, width, height, stream);
}

}  // extern "C"
