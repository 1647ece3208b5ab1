// f32 GEMM for gfx950 on v_mfma_f32_32x32x2_f32 (f32 in, f32 accumulate).
//
// C[M x N] = A[M x K] . B[K x N], all row-major.  Replaces the 16x16 LDS-tiled kernel
// Sarek generates for its tiled matrix multiply: same result up to f32 summation
// order, computed on the matrix cores.
//
// Tiling: one workgroup (512 threads = 8 waves, 2 along M x 4 along N) owns a
// 256 x 256 tile of C and walks K in slabs of 32.  Each wave owns 128 x 64 = 4 x 2
// MFMA tiles of 32 x 32.  LDS holds two stages of (A slab [256][32], rows padded to
// 36 floats; B slab [32][256]).
//
// Operand fetch: the MFMA consumes, per step, k = {k_lo, k_hi} with lanes 0-31 feeding
// k_lo and lanes 32-63 feeding k_hi.  Any assignment of real k indices to (step, half)
// is valid as long as A and B agree, so each lane (m, h) reads FOUR consecutive k of
// its A row with one ds_read_b128 (k = 8*kk + 4h + j, j = 0..3) and uses them over
// four MFMA steps; the matching B values are row 8*kk + 4h + j, column n (ds_read_b32,
// bank-conflict free because n is contiguous).
#include "common.hpp"
#include "tunables.hpp"

namespace sarek_hip {
namespace {

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int BM = 256, BN = 256, BK = 32;
constexpr int THREADS = 512;
constexpr int NUM_XCD = 8;   // XCDs of an MI355X; workgroup ids are dealt to them round-robin
constexpr int A_STRIDE = BK + 4;            // floats per A row in LDS (36)
constexpr int B_STRIDE = BN;                // floats per B row in LDS
constexpr int A_FLOATS = BM * A_STRIDE;     // 9216
constexpr int B_FLOATS = BK * B_STRIDE;     // 8192
constexpr int STAGE_FLOATS = A_FLOATS + B_FLOATS;
constexpr int LDS_BYTES = 2 * STAGE_FLOATS * 4;  // 139264

__global__ __launch_bounds__(THREADS) void gemm_f32_kernel(const float *__restrict__ A,
                                                           const float *__restrict__ B,
                                                           float *__restrict__ C, int M, int N,
                                                           int K, int tiles_m, int tiles_n, int xcd_remap) {
  extern __shared__ __attribute__((aligned(16))) float lds_f[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 2, wn = wave & 3;
  const int lm = lane & 31, lh = lane >> 5;

  // Workgroup -> tile.  The hardware deals consecutive workgroup ids round-robin to the
  // 8 XCDs (each with its own L2), so ids are first regrouped to give every XCD one
  // contiguous run of tiles, and the run is walked in bands of GROUP tile-rows, column by
  // column: the ~32 tiles an XCD has in flight then form a compact GROUP x 4 patch that
  // moves through K together and shares A row-panels and B column-panels in that L2.
  const int nblocks = tiles_m * tiles_n;
  const int xcd = blockIdx.x % NUM_XCD, slot = blockIdx.x / NUM_XCD;
  int tile = xcd * (nblocks / NUM_XCD) + min(xcd, nblocks % NUM_XCD) + slot;
  if (xcd_remap == 0) tile = blockIdx.x;
  const int GROUP = xcd_remap > 1 ? xcd_remap : 8;   // tile-rows per raster band
  const int per_group = GROUP * tiles_n;
  const int g = tile / per_group;
  const int rows_in_group = min(GROUP, tiles_m - g * GROUP);
  const int in_g = tile - g * per_group;
  const int tm = g * GROUP + in_g % rows_in_group;
  const int tn = in_g / rows_in_group;
  const int m0 = tm * BM, n0 = tn * BN;

  f32x4 ra[4], rb[4];
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  // A slab: 256 rows x 8 chunks of 4 floats; B slab: 32 rows x 64 chunks of 4 floats.
  auto load_slab = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + THREADS * i;
      const int row = c >> 3, kc = (c & 7) * 4;
      const int gr = m0 + row, gk = k0 + kc;
      ra[i] = (gr < M && gk < K)
                  ? *reinterpret_cast<const f32x4 *>(A + static_cast<int64_t>(gr) * K + gk)
                  : zero4;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + THREADS * i;
      const int kr = c >> 6, nc = (c & 63) * 4;
      const int gk = k0 + kr, gn = n0 + nc;
      rb[i] = (gk < K && gn < N)
                  ? *reinterpret_cast<const f32x4 *>(B + static_cast<int64_t>(gk) * N + gn)
                  : zero4;
    }
  };
  auto store_slab = [&](int stage) {
    float *sa = lds_f + stage * STAGE_FLOATS;
    float *sb = sa + A_FLOATS;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + THREADS * i;
      *reinterpret_cast<f32x4 *>(sa + (c >> 3) * A_STRIDE + (c & 7) * 4) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + THREADS * i;
      *reinterpret_cast<f32x4 *>(sb + (c >> 6) * B_STRIDE + (c & 63) * 4) = rb[i];
    }
  };

  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int a_off = (wm * 128 + lm) * A_STRIDE + lh * 4;   // + i*32*A_STRIDE + kk*8
  const int b_off = (lh * 4) * B_STRIDE + wn * 64 + lm;     // + (kk*8 + j)*B_STRIDE + jn*32

  const int nslabs = (K + BK - 1) / BK;
  load_slab(0);
  store_slab(0);
  __syncthreads();

  for (int s = 0; s < nslabs; ++s) {
    const int cur = s & 1;
    if (s + 1 < nslabs) load_slab((s + 1) * BK);
    const float *sa = lds_f + cur * STAGE_FLOATS;
    const float *sb = sa + A_FLOATS;
#pragma unroll
    for (int kk = 0; kk < BK / 8; ++kk) {
      f32x4 af[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        af[i] = *reinterpret_cast<const f32x4 *>(sa + a_off + i * 32 * A_STRIDE + kk * 8);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float bf[2];
#pragma unroll
        for (int jn = 0; jn < 2; ++jn) bf[jn] = sb[b_off + (kk * 8 + j) * B_STRIDE + jn * 32];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int jn = 0; jn < 2; ++jn)
            acc[i][jn] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][j], bf[jn], acc[i][jn], 0, 0, 0);
      }
    }
    if (s + 1 < nslabs) store_slab(cur ^ 1);
    __syncthreads();
  }

  // Accumulator layout: register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4,
  // column l%32 of its 32 x 32 tile.
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = m0 + wm * 128 + i * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
#pragma unroll
      for (int jn = 0; jn < 2; ++jn) {
        const int col = n0 + wn * 64 + jn * 32 + lm;
        if (row < M && col < N) C[static_cast<int64_t>(row) * N + col] = acc[i][jn][r];
      }
    }
}

// Any shape, any alignment: one thread per C element, f32 FMA in k order.
__global__ __launch_bounds__(256) void gemm_f32_simple_kernel(const float *__restrict__ A,
                                                              const float *__restrict__ B,
                                                              float *__restrict__ C, int M, int N,
                                                              int K) {
  const int col = blockIdx.x * 64 + (threadIdx.x & 63);
  const int row = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (row >= M || col >= N) return;
  float acc = 0.f;
  for (int k = 0; k < K; ++k)
    acc = fmaf(A[static_cast<int64_t>(row) * K + k], B[static_cast<int64_t>(k) * N + col], acc);
  C[static_cast<int64_t>(row) * N + col] = acc;
}

}  // namespace
}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" int sarek_hip_gemm_f32(const float *a, const float *b, float *c, int m, int n, int k,
                                  sarek_hip_stream stream) {
  if (m <= 0 || n <= 0 || k <= 0)
    return fail(SAREK_HIP_E_INVALID_ARG, "gemm_f32: m, n, k must be positive (got %d %d %d)", m, n, k);
  if (!a || !b || !c) return fail(SAREK_HIP_E_INVALID_ARG, "gemm_f32: NULL matrix");
  hipStream_t st = as_stream(stream);
  const bool vec_ok = (k % 4 == 0) && (n % 4 == 0) &&
                      (reinterpret_cast<uintptr_t>(a) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(b) % 16 == 0);
  if (vec_ok && tunable("gemm_f32.force_simple", 0) == 0) {
    static bool attr_done = false;
    if (!attr_done) {
      SAREK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_f32_kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
      attr_done = true;
    }
    const int tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
    hipLaunchKernelGGL(gemm_f32_kernel, dim3(tiles_m * tiles_n), dim3(THREADS), LDS_BYTES, st, a, b,
                       c, m, n, k, tiles_m, tiles_n, (int)tunable("gemm.xcd_remap", 1));
  } else {
    hipLaunchKernelGGL(gemm_f32_simple_kernel, dim3((n + 63) / 64, (m + 3) / 4), dim3(256), 0, st,
                       a, b, c, m, n, k);
  }
  return check_launch("gemm_f32 kernel launch");
}
