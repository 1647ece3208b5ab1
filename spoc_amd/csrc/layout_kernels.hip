// Pure data-movement kernels for gfx950: vector copy and matrix transpose, the hand-written
// counterparts of the generated kernels of benchmarks/bench_vector_copy.ml:21-27,
// benchmarks/bench_transpose.ml and benchmarks/bench_transpose_tiled.ml in the reference.
// Both are HBM-bound at 8 bytes per element (one read, one write): 128-bit non-temporal
// accesses, every load of a thread issued before its first store, one-shot grids.
#include "common.hpp"
#include "tunables.hpp"

namespace sarek_hip {
namespace {

typedef float f32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4_t ldg_nt(const float *p) {
  return __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(p));
}
__device__ __forceinline__ void stg_nt(float *p, f32x4_t v) {
  __builtin_nontemporal_store(v, reinterpret_cast<f32x4_t *>(p));
}

constexpr int kBlock = 256;
// An input no larger than this may still be in the last-level cache (256 MB on MI355X) when
// the kernel starts: then plain loads hit there and non-temporal ones would go round it.
constexpr int64_t kLastLevelCacheBytes = int64_t{256} << 20;

// ---- copy ------------------------------------------------------------------------------
constexpr int kCopyUnroll = 8;                                  // float4 per thread
constexpr int kCopyChunk = kBlock * kCopyUnroll * 4;            // elements per workgroup (8192)

// dst[i] = src[i], i < n.  Workgroup g owns elements [g*kCopyChunk, (g+1)*kCopyChunk); the
// last one also takes the (n & 3) scalar tail.  NtLoad: the source is read past the caches
// (right when it comes from HBM anyway; wrong when it still sits in the 256 MB last-level
// cache from whoever produced it).
template <bool NtLoad>
__global__ __launch_bounds__(kBlock) void copy_kernel(float *__restrict__ dst, const float *__restrict__ src,
                                                      int64_t n) {
  auto load = [](const float *p) { return NtLoad ? ldg_nt(p) : *reinterpret_cast<const f32x4_t *>(p); };
  const int64_t n4 = n >> 2;
  const int64_t base = static_cast<int64_t>(blockIdx.x) * (kCopyChunk / 4) + threadIdx.x;
  if (base + (kCopyUnroll - 1) * kBlock < n4) {
    f32x4_t v[kCopyUnroll];
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u) v[u] = load(src + 4 * (base + u * kBlock));
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u) stg_nt(dst + 4 * (base + u * kBlock), v[u]);
  } else {
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u) {
      const int64_t i = base + u * kBlock;
      if (i < n4) stg_nt(dst + 4 * i, load(src + 4 * i));
    }
  }
  const int64_t ti = (n4 << 2) + threadIdx.x;
  if (blockIdx.x == gridDim.x - 1 && ti < n) dst[ti] = src[ti];
}

// 4-byte aligned vectors.
__global__ __launch_bounds__(kBlock) void copy_scalar_kernel(float *__restrict__ dst,
                                                             const float *__restrict__ src, int64_t n) {
  const int64_t step = static_cast<int64_t>(gridDim.x) * kBlock;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += step) dst[i] = src[i];
}

// ---- transpose -------------------------------------------------------------------------
// in: `height` rows of `width` floats; out[c * height + r] = in[r * width + c].
constexpr int kTile = 64;

// Workgroup -> tile.  order 0: tiles along an input row are consecutive workgroups (their
// reads are neighbours); order 1: tiles along an input column are (their writes are).
__device__ __forceinline__ void tile_of(int order, int tiles_c, int tiles_r, int &tr, int &tc) {
  int b = blockIdx.x;
  if (order >= 2) {
    // workgroup ids are dealt round-robin to the 8 XCDs: give each XCD one contiguous run of tiles
    const int nb = tiles_c * tiles_r, xcd = b % 8, slot = b / 8;
    b = xcd * (nb / 8) + (xcd < nb % 8 ? xcd : nb % 8) + slot;
    order -= 2;
  }
  if (order == 0) {
    tr = b / tiles_c;
    tc = b - tr * tiles_c;
  } else {
    tc = b / tiles_r;
    tr = b - tc * tiles_r;
  }
}

// 64 x 64 tile through LDS: 16 lanes read 256 contiguous bytes of an input row, the tile is
// kept with a row pitch of 65 words (both the row-wise stores and the column-wise loads then
// touch 64 different banks per wave), and 16 lanes write 256 contiguous bytes of an output
// row.  The matrices may start on any 4-byte boundary.  Ragged: width or height is not a multiple of 4, so rows start
// at any 4-byte offset too (the 128-bit accesses do not mind) and the pieces that straddle the end of a row go
// element by element.
template <int TR, bool NtLoad, bool NtStore, bool Ragged>
__global__ __launch_bounds__(kBlock) void transpose_lds_kernel(const float *__restrict__ in,
                                                               float *__restrict__ out, int width, int height,
                                                               int tiles_c, int tiles_r, int order) {
  __shared__ float tile[TR][kTile + 1];
  int tr, tc;
  tile_of(order, tiles_c, tiles_r, tr, tc);
  const int t = threadIdx.x, q = t & 15, p = t >> 4;
  const int64_t r0 = static_cast<int64_t>(tr) * TR, c0 = static_cast<int64_t>(tc) * kTile;
  constexpr int NL = TR / 16;            // loads per thread
  f32x4_t v[NL];
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int64_t r = r0 + p + 16 * i, c = c0 + 4 * q;
    const float *src = in + r * width + c;
    if (r < height && (Ragged ? c + 3 < width : c < width)) {
      v[i] = NtLoad ? ldg_nt(src) : *reinterpret_cast<const f32x4_t *>(src);
    } else {
      v[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if constexpr (Ragged) {
        if (r < height) {
#pragma unroll
          for (int j = 0; j < 3; ++j)
            if (c + j < width) v[i][j] = src[j];
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < NL; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) tile[p + 16 * i][4 * q + j] = v[i][j];
  __syncthreads();
  // an output row holds TR floats of this tile: TR/4 lanes per row, 256 / (TR/4) rows per pass
  constexpr int LPR = TR / 4, RPP = kBlock / LPR;
  const int oq = t % LPR, op = t / LPR;
#pragma unroll
  for (int i = 0; i < kTile / RPP; ++i) {
    const int oc = op + RPP * i;                     // input column = output row within the tile
    const int64_t orow = c0 + oc, ocol = r0 + 4 * oq;
    if (orow < width && ocol < height) {
      const f32x4_t w = {tile[4 * oq][oc], tile[4 * oq + 1][oc], tile[4 * oq + 2][oc], tile[4 * oq + 3][oc]};
      float *dst = out + orow * height + ocol;
      if (Ragged && ocol + 3 >= height) {
#pragma unroll
        for (int j = 0; j < 3; ++j)
          if (ocol + j < height) dst[j] = w[j];
      } else if (NtStore) {
        stg_nt(dst, w);
      } else {
        *reinterpret_cast<f32x4_t *>(dst) = w;
      }
    }
  }
}

// The same tile without LDS: a thread takes a 4 x 4 block (four 128-bit loads from four
// consecutive input rows), transposes it in registers and stores four 128-bit pieces into
// four consecutive output rows.  Eight lanes cover 128 contiguous bytes on either side.
__global__ __launch_bounds__(kBlock) void transpose_reg_kernel(const float *__restrict__ in,
                                                               float *__restrict__ out, int width, int height,
                                                               int tiles_c, int tiles_r, int order) {
  int tr, tc;
  tile_of(order, tiles_c, tiles_r, tr, tc);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // wave w owns the 32 x 32 quadrant (w >> 1, w & 1); lane -> 4 x 4 block (lane >> 3, lane & 7)
  const int64_t r = static_cast<int64_t>(tr) * kTile + 32 * (wave >> 1) + 4 * (lane >> 3);
  const int64_t c = static_cast<int64_t>(tc) * kTile + 32 * (wave & 1) + 4 * (lane & 7);
  if (r >= height || c >= width) return;
  f32x4_t v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = ldg_nt(in + (r + i) * width + c);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const f32x4_t w = {v[0][j], v[1][j], v[2][j], v[3][j]};
    stg_nt(out + (c + j) * height + r, w);
  }
}

// Any shape and alignment: 32 x 32 tile through LDS, one element per access.
__global__ __launch_bounds__(kBlock) void transpose_scalar_kernel(const float *__restrict__ in,
                                                                  float *__restrict__ out, int width,
                                                                  int height, int tiles_c) {
  __shared__ float tile[32][33];
  const int tr = blockIdx.x / tiles_c, tc = blockIdx.x - tr * tiles_c;
  const int x = threadIdx.x & 31, y = threadIdx.x >> 5;   // 8 rows per pass
  const int64_t r0 = static_cast<int64_t>(tr) * 32, c0 = static_cast<int64_t>(tc) * 32;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t r = r0 + y + 8 * i, c = c0 + x;
    if (r < height && c < width) tile[y + 8 * i][x] = in[r * width + c];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t orow = c0 + y + 8 * i, ocol = r0 + x;
    if (orow < width && ocol < height) out[orow * height + ocol] = tile[x][y + 8 * i];
  }
}


}  // namespace
}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" {

int sarek_hip_copy_f32(float *dst, const float *src, int64_t n, sarek_hip_stream stream) {
  if (n < 0) return fail(SAREK_HIP_E_INVALID_ARG, "copy: negative length %lld", (long long)n);
  if (n == 0) return SAREK_HIP_OK;
  if (!dst || !src) return fail(SAREK_HIP_E_INVALID_ARG, "copy: NULL vector");
  const int64_t blocks = ceil_div(n, static_cast<int64_t>(kCopyChunk));
  if (blocks > 0x7FFFFFFF) return fail(SAREK_HIP_E_INVALID_ARG, "copy: vector too long for one launch");
  // the 128-bit accesses need no alignment beyond the element's; copy.force_scalar keeps the other kernel reachable
  if (tunable("copy.force_scalar", 0) == 0) {
    int64_t nt = tunable("copy.nt", -1);
    if (nt < 0) nt = n * 4 > kLastLevelCacheBytes;
    if (nt)
      hipLaunchKernelGGL(copy_kernel<true>, dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0,
                         as_stream(stream), dst, src, n);
    else
      hipLaunchKernelGGL(copy_kernel<false>, dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0,
                         as_stream(stream), dst, src, n);
  } else {
    const unsigned sblocks = blocks < 8192 ? static_cast<unsigned>(blocks) : 8192u;
    hipLaunchKernelGGL(copy_scalar_kernel, dim3(sblocks), dim3(kBlock), 0, as_stream(stream), dst, src, n);
  }
  return check_launch("copy kernel launch");
}

int sarek_hip_transpose_f32(const float *in, float *out, int width, int height, sarek_hip_stream stream) {
  if (width < 0 || height < 0)
    return fail(SAREK_HIP_E_INVALID_ARG, "transpose: negative shape %d x %d", width, height);
  if (width == 0 || height == 0) return SAREK_HIP_OK;
  if (!in || !out) return fail(SAREK_HIP_E_INVALID_ARG, "transpose: NULL matrix");
  if (in == out) return fail(SAREK_HIP_E_INVALID_ARG, "transpose: in-place transposition is not supported");
  hipStream_t st = as_stream(stream);
  if (tunable("transpose.force_scalar", 0) == 0) {
    const bool ragged = width % 4 != 0 || height % 4 != 0;
    // Measured on MI355X: 128-row tiles; an input that fits the last-level cache is best read
    // with plain loads and with each XCD walking its own run of tiles (order 3), a larger one
    // with non-temporal loads and neighbouring workgroups writing neighbouring pieces (order 1); a larger one whose
    // rows start off 16 bytes (ragged) with plain accesses and order 3 (4.2 against 3.3-3.6 TB/s at 16383 x 16385 and
    // 12001 x 20003).
    const bool cached = static_cast<int64_t>(width) * height * 4 <= kLastLevelCacheBytes;
    const int rows = tunable("transpose.rows", 128) == 64 ? 64 : 128;
    const int tiles_c = (width + kTile - 1) / kTile;
    const int64_t variant = tunable("transpose.variant", 0);
    int64_t nt = tunable("transpose.nt", -1);
    if (nt < 0) nt = cached ? 2 : ragged ? 0 : 3;
    const bool lds = variant == 0 || ragged;   // the register-only kernel takes whole 4 x 4 blocks
    const int tiles_r = (height + (lds ? rows : kTile) - 1) / (lds ? rows : kTile);
    const int64_t tiles = static_cast<int64_t>(tiles_c) * tiles_r;
    if (tiles > 0x7FFFFFFF) return fail(SAREK_HIP_E_INVALID_ARG, "transpose: matrix too large for one launch");
    int order = static_cast<int>(tunable("transpose.order", -1));
    if (order < 0) order = cached || ragged ? 3 : 1;
#define SAREK_TRANSPOSE(TR, NL, NS)                                                                              \
  do {                                                                                                             \
    if (ragged)                                                                                                    \
      hipLaunchKernelGGL((transpose_lds_kernel<TR, NL, NS, true>), dim3(static_cast<unsigned>(tiles)), dim3(kBlock), \
                         0, st, in, out, width, height, tiles_c, tiles_r, order);                                  \
    else                                                                                                           \
      hipLaunchKernelGGL((transpose_lds_kernel<TR, NL, NS, false>), dim3(static_cast<unsigned>(tiles)),            \
                         dim3(kBlock), 0, st, in, out, width, height, tiles_c, tiles_r, order);                    \
  } while (0)
    if (lds) {
      if (rows == 64) {
        if (nt == 3) SAREK_TRANSPOSE(64, true, true);
        else if (nt == 1) SAREK_TRANSPOSE(64, true, false);
        else if (nt == 2) SAREK_TRANSPOSE(64, false, true);
        else SAREK_TRANSPOSE(64, false, false);
      } else {
        if (nt == 3) SAREK_TRANSPOSE(128, true, true);
        else if (nt == 1) SAREK_TRANSPOSE(128, true, false);
        else if (nt == 2) SAREK_TRANSPOSE(128, false, true);
        else SAREK_TRANSPOSE(128, false, false);
      }
    } else {
      hipLaunchKernelGGL(transpose_reg_kernel, dim3(static_cast<unsigned>(tiles)), dim3(kBlock), 0, st, in, out,
                         width, height, tiles_c, tiles_r, order);
    }
#undef SAREK_TRANSPOSE
  } else {
    const int tiles_c = (width + 31) / 32, tiles_r = (height + 31) / 32;
    const int64_t tiles = static_cast<int64_t>(tiles_c) * tiles_r;
    if (tiles > 0x7FFFFFFF) return fail(SAREK_HIP_E_INVALID_ARG, "transpose: matrix too large for one launch");
    hipLaunchKernelGGL(transpose_scalar_kernel, dim3(static_cast<unsigned>(tiles)), dim3(kBlock), 0, st, in, out,
                       width, height, tiles_c);
  }
  return check_launch("transpose kernel launch");
}

}  // extern "C"
