// 16-bit-input (bf16 / fp16), f32-accumulate GEMM for gfx950 on v_mfma_f32_32x32x16,
// with an optional fused epilogue  y = relu(acc + bias[col]),  rowsum[row] += y.
//
// C[M x N] = A[M x K] . B[K x N], all row-major.
//
// Tiling: one workgroup (512 threads = 8 waves, 2 along M x 4 along N) owns a
// 256 x 256 tile of C and walks K in slabs of 64.  Each wave owns 128 x 64 of the
// tile = 4 x 2 MFMA tiles of 32 x 32 (128 accumulator registers).
//
// LDS holds two stages of (A slab [256][64], B slab [64][256]).  A rows are padded
// to 144 bytes so the eight 16-byte reads of consecutive rows fall in distinct
// banks; B rows are padded to 544 bytes so the four rows touched by one transposing
// read fall in distinct banks.
//
// Operand fetch:
//   A: lane (m = lane%32, h = lane/32) needs k = 8h..8h+7 of row m: one ds_read_b128.
//   B: lane (n = lane%32, h) needs k = 8h..8h+7 of column n.  B is n-contiguous in
//      LDS, so the column is gathered by ds_read_b64_tr_b16: within each group of
//      16 lanes, lane i supplies the address of 4 consecutive n of row (i/4) at
//      n-offset 4*(i%4), and receives column i of that 4 x 16 block (its 4 rows).
//      Two such reads (rows 0-3 and 4-7 of the lane's k range) give the 8 k values.
//
// Global -> LDS goes through registers with 16-byte loads; the next slab's loads are
// issued before the MFMA work of the current slab and written to the other LDS stage
// after it (one barrier per slab).
#include "common.hpp"
#include "tunables.hpp"

namespace sarek_hip {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

#define LDS_PTR __attribute__((address_space(3)))

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int THREADS = 512;
constexpr int A_STRIDE = BK * 2 + 16;   // bytes per A row in LDS (144)
constexpr int B_STRIDE = BN * 2 + 32;   // bytes per B row in LDS (544)
constexpr int A_BYTES = BM * A_STRIDE;  // 36864
constexpr int B_BYTES = BK * B_STRIDE;  // 34816
constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
constexpr int LDS_BYTES = 2 * STAGE_BYTES;  // 143360

enum { EPI_STORE = 0, EPI_BIAS_RELU_ROWSUM = 1 };

template <bool Bf16>
__device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (Bf16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// ds_read_b64_tr_b16 at byte offset `off` of the dynamic LDS block.
__device__ __forceinline__ u32x2 lds_read_tr16(const char *lds, int off) {
  auto p = (LDS_PTR bf16x4 *)(lds + off);
  bf16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(p);
  return __builtin_bit_cast(u32x2, v);
}

// Sum over the 32 lanes of each half-wave; valid in every lane of the half.
__device__ __forceinline__ float half_wave_sum(float v) {
  for (int off = 16; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

template <bool Bf16, int Epi>
__global__ __launch_bounds__(THREADS) void gemm16_kernel(const uint16_t *__restrict__ A,
                                                         const uint16_t *__restrict__ B,
                                                         float *__restrict__ C,
                                                         const float *__restrict__ bias,
                                                         float *__restrict__ rowsum, int M, int N,
                                                         int K, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 2, wn = wave & 3;  // 2 x 4 waves
  const int lm = lane & 31, lh = lane >> 5;

  // Tile raster: groups of 8 tile-rows walk the N direction together so the tiles
  // resident at one time share A row-panels and B column-panels in L2.
  int tile = blockIdx.x;
  constexpr int GROUP = 8;
  const int per_group = GROUP * tiles_n;
  const int g = tile / per_group;
  const int rows_in_group = min(GROUP, tiles_m - g * GROUP);
  const int in_g = tile - g * per_group;
  const int tm = g * GROUP + in_g % rows_in_group;
  const int tn = in_g / rows_in_group;
  const int m0 = tm * BM, n0 = tn * BN;

  // ---- global -> register staging --------------------------------------------
  // A slab: 256 rows x 8 chunks of 16 B; chunk c = tid + 512*i -> row c/8, chunk c%8.
  // B slab: 64 rows x 32 chunks of 16 B; chunk c = tid + 512*i -> row c/32, chunk c%32.
  u32x4 ra[4], rb[4];
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  auto load_slab = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + THREADS * i;
      const int row = c >> 3, kc = (c & 7) * 8;
      const int gr = m0 + row, gk = k0 + kc;
      ra[i] = (gr < M && gk < K)
                  ? *reinterpret_cast<const u32x4 *>(A + static_cast<int64_t>(gr) * K + gk)
                  : zero4;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + THREADS * i;
      const int kr = c >> 5, nc = (c & 31) * 8;
      const int gk = k0 + kr, gn = n0 + nc;
      rb[i] = (gk < K && gn < N)
                  ? *reinterpret_cast<const u32x4 *>(B + static_cast<int64_t>(gk) * N + gn)
                  : zero4;
    }
  };
  auto store_slab = [&](int stage) {
    char *sa = lds + stage * STAGE_BYTES;
    char *sb = sa + A_BYTES;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + THREADS * i;
      *reinterpret_cast<u32x4 *>(sa + (c >> 3) * A_STRIDE + (c & 7) * 16) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + THREADS * i;
      *reinterpret_cast<u32x4 *>(sb + (c >> 5) * B_STRIDE + (c & 31) * 16) = rb[i];
    }
  };

  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Per-lane LDS offsets that do not depend on the K slab.
  const int a_off = (wm * 128 + lm) * A_STRIDE + lh * 16;  // + i*32*A_STRIDE + kk*32
  // transposing read: group of 16 lanes, lane i in group: row i/4, n offset 4*(i%4)
  const int li = lane & 15;
  const int b_off = (lh * 8 + (li >> 2)) * B_STRIDE +
                    (wn * 64 + ((lane >> 4) & 1) * 16 + (li & 3) * 4) * 2;  // + j*64 + kk*16*B_STRIDE

  const int nslabs = (K + BK - 1) / BK;
  load_slab(0);
  store_slab(0);
  __syncthreads();

  for (int s = 0; s < nslabs; ++s) {
    const int cur = s & 1;
    if (s + 1 < nslabs) load_slab((s + 1) * BK);
    const char *sa = lds + cur * STAGE_BYTES;
    const char *sb = sa + A_BYTES;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      u32x4 af[4], bf[2];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        af[i] = *reinterpret_cast<const u32x4 *>(sa + a_off + i * 32 * A_STRIDE + kk * 32);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int off = A_BYTES + cur * STAGE_BYTES + b_off + j * 64 + kk * 16 * B_STRIDE;
        u32x2 lo = lds_read_tr16(lds, off);
        u32x2 hi = lds_read_tr16(lds, off + 4 * B_STRIDE);
        bf[j] = u32x4{lo.x, lo.y, hi.x, hi.y};
      }
      (void)sb;
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mfma<Bf16>(af[i], bf[j], acc[i][j]);
    }
    if (s + 1 < nslabs) store_slab(cur ^ 1);
    __syncthreads();
  }

  // ---- epilogue ----------------------------------------------------------------
  // Accumulator layout of the 32x32 MFMA: register r of lane l holds
  // row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the tile.
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = m0 + wm * 128 + i * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
      float rs = 0.f;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int col = n0 + wn * 64 + j * 32 + lm;
        float v = acc[i][j][r];
        if (Epi == EPI_BIAS_RELU_ROWSUM) {
          v += (col < N) ? bias[col] : 0.f;
          v = v > 0.f ? v : 0.f;
          if (col < N) rs += v;
        }
        if (row < M && col < N) C[static_cast<int64_t>(row) * N + col] = v;
      }
      if (Epi == EPI_BIAS_RELU_ROWSUM) {
        rs = half_wave_sum(rs);
        if (lm == 0 && row < M) atomicAdd(rowsum + row, rs);
      }
    }
  }
}

// Any shape, any alignment: one thread per C element, f32 accumulate in k order.
template <bool Bf16, int Epi>
__global__ __launch_bounds__(256) void gemm16_simple_kernel(const uint16_t *__restrict__ A,
                                                            const uint16_t *__restrict__ B,
                                                            float *__restrict__ C,
                                                            const float *__restrict__ bias,
                                                            float *__restrict__ rowsum, int M,
                                                            int N, int K) {
  const int col = blockIdx.x * 64 + (threadIdx.x & 63);
  const int row = blockIdx.y * 4 + (threadIdx.x >> 6);
  float acc = 0.f;
  if (row < M && col < N) {
    for (int k = 0; k < K; ++k) {
      const uint16_t ab = A[static_cast<int64_t>(row) * K + k];
      const uint16_t bb = B[static_cast<int64_t>(k) * N + col];
      float af, bf;
      if (Bf16) {
        af = __builtin_bit_cast(float, static_cast<uint32_t>(ab) << 16);
        bf = __builtin_bit_cast(float, static_cast<uint32_t>(bb) << 16);
      } else {
        af = static_cast<float>(__builtin_bit_cast(_Float16, ab));
        bf = static_cast<float>(__builtin_bit_cast(_Float16, bb));
      }
      acc = fmaf(af, bf, acc);
    }
    if (Epi == EPI_BIAS_RELU_ROWSUM) {
      acc += bias[col];
      acc = acc > 0.f ? acc : 0.f;
    }
    C[static_cast<int64_t>(row) * N + col] = acc;
  }
  if (Epi == EPI_BIAS_RELU_ROWSUM) {
    float rs = (row < M && col < N) ? acc : 0.f;
    for (int off = 32; off >= 1; off >>= 1) rs += __shfl_xor(rs, off, 64);
    if ((threadIdx.x & 63) == 0 && row < M) atomicAdd(rowsum + row, rs);
  }
}

__global__ void zero_f32_kernel(float *p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

template <bool Bf16, int Epi>
int launch_gemm16(const uint16_t *a, const uint16_t *b, float *c, const float *bias, float *rowsum,
                  int m, int n, int k, hipStream_t st) {
  if (m <= 0 || n <= 0 || k <= 0)
    return fail(SAREK_HIP_E_INVALID_ARG, "gemm16: m, n, k must be positive (got %d %d %d)", m, n, k);
  if (!a || !b || !c) return fail(SAREK_HIP_E_INVALID_ARG, "gemm16: NULL matrix");
  if (Epi == EPI_BIAS_RELU_ROWSUM) {
    if (!bias || !rowsum) return fail(SAREK_HIP_E_INVALID_ARG, "gemm16: NULL bias or rowsum");
    hipLaunchKernelGGL(zero_f32_kernel, dim3((m + 255) / 256), dim3(256), 0, st, rowsum, m);
    int rc = check_launch("rowsum clear launch");
    if (rc != SAREK_HIP_OK) return rc;
  }
  // The MFMA kernel issues 16-byte loads: rows of A and B must keep 16-byte alignment.
  const bool vec_ok = (k % 8 == 0) && (n % 8 == 0) &&
                      (reinterpret_cast<uintptr_t>(a) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(b) % 16 == 0);
  if (vec_ok && tunable("gemm16.force_simple", 0) == 0) {
    static bool attr_done[2][2] = {{false, false}, {false, false}};
    auto kern = gemm16_kernel<Bf16, Epi>;
    if (!attr_done[Bf16][Epi]) {
      SAREK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
      attr_done[Bf16][Epi] = true;
    }
    const int tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(THREADS), LDS_BYTES, st, a, b, c, bias,
                       rowsum, m, n, k, tiles_m, tiles_n);
  } else {
    auto kern = gemm16_simple_kernel<Bf16, Epi>;
    hipLaunchKernelGGL(kern, dim3((n + 63) / 64, (m + 3) / 4), dim3(256), 0, st, a, b, c, bias,
                       rowsum, m, n, k);
  }
  return check_launch("gemm16 kernel launch");
}

}  // namespace
}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" {

int sarek_hip_gemm_bf16(const uint16_t *a, const uint16_t *b, float *c, int m, int n, int k,
                        sarek_hip_stream stream) {
  return launch_gemm16<true, EPI_STORE>(a, b, c, nullptr, nullptr, m, n, k, as_stream(stream));
}

int sarek_hip_gemm_f16(const uint16_t *a, const uint16_t *b, float *c, int m, int n, int k,
                       sarek_hip_stream stream) {
  return launch_gemm16<false, EPI_STORE>(a, b, c, nullptr, nullptr, m, n, k, as_stream(stream));
}

int sarek_hip_gemm_f16_bias_relu_rowsum(const uint16_t *a, const uint16_t *b, const float *bias,
                                        float *y, float *rowsum, int m, int n, int k,
                                        sarek_hip_stream stream) {
  return launch_gemm16<false, EPI_BIAS_RELU_ROWSUM>(a, b, y, bias, rowsum, m, n, k,
                                                    as_stream(stream));
}
}
