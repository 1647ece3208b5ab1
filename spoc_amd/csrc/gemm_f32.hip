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
#include <type_traits>
#include <utility>

#include <algorithm>

#include "common.hpp"
#include "gemm_common.hpp"
#include "tunables.hpp"

namespace sarek_hip {
namespace {

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int BM = 256, BN = 256, BK = 32;
constexpr int THREADS = 512;
constexpr int A_STRIDE = BK + 4;            // floats per A row in LDS (36)
constexpr int B_STRIDE = BN;                // floats per B row in LDS
constexpr int A_FLOATS = BM * A_STRIDE;     // 9216
constexpr int B_FLOATS = BK * B_STRIDE;     // 8192
constexpr int STAGE_FLOATS = A_FLOATS + B_FLOATS;
constexpr int LDS_BYTES = 2 * STAGE_FLOATS * 4;  // 139264

__global__ __launch_bounds__(THREADS) void gemm_f32_staged_kernel(const float *__restrict__ A,
                                                           const float *__restrict__ B,
                                                           float *__restrict__ C, int M, int N,
                                                           int K, int tiles_m, int tiles_n, int xcd_remap) {
  extern __shared__ __attribute__((aligned(16))) float lds_f[];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 2, wn = wave & 3;
  const int lm = lane & 31, lh = lane >> 5;

  int tm, tn;
  tile_of_block(tiles_m, tiles_n, xcd_remap, tm, tn);
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

// ---- direct-to-LDS ring kernel ------------------------------------------------------
// Tile = (32*TI*WMW) x (32*TJ*WNW), WMW x WNW waves, each wave TI x TJ MFMA tiles of 32 x 32.
// K slabs of BKT stream through NS LDS stages by global_load_lds_dwordx4 (no staging
// registers, no ds_write); the pipeline is the one of the 16-bit GEMM: DMA of slab s+NS
// issued after the barrier inside slab s, barrier before the last k-step of a slab, next
// slab's first fragments fetched under that step's MFMAs.
//
// k-step = 8 k.  A: lane (m, h) reads k = 8kk+4h .. +3 of its row with one ds_read_b128 and
// feeds them to four MFMA steps j; B: for step j the lane reads row 8kk+4h+j at columns
// TJ*lane .. TJ*lane+TJ-1 of the wave's span (one ds_read of TJ floats): MFMA tile jn of the
// wave therefore holds columns {TJ*l + jn}, and in the epilogue every lane owns TJ adjacent
// columns of C, stored as one vector.
//
// LDS (64 banks x 4 B): A rows of 64 B: slot ^= (row>>2)&3, rows of 128 B: slot ^= (row>>1)&7
// (16-lane phases of ds_read_b128).  B reads are contiguous across lanes; only for TJ = 1
// the two half-waves (rows r, r+4) would meet modulo 256 B, so rows with bit 2 set are
// stored with their 128-byte halves swapped.
//
// Ragged = false: N % 4 == 0, K % BKT == 0, A, B and C 16-byte aligned.  Ragged = true: any N, any K >= BKT (or a multiple of
// 4 below it), any alignment.  A lane whose offset lies outside the buffer resource's range brings zeros into LDS, the range
// is checked per dword and the address needs no alignment beyond the element's, so B rows that must not count are a per-lane
// choice between the usual offset and one past the range, B's range ends with its last element, pieces past column N bring
// the next row's elements into columns that are never stored, and C is stored element by element.
template <int TI, int TJ, int WMW, int WNW, int BKT, int NS, bool Ragged = false>
__global__ __launch_bounds__(64 * WMW * WNW) void gemm_f32_dma_kernel(
    const float *__restrict__ A, const float *__restrict__ B, float *__restrict__ C, int M, int N,
    int K, int tiles_m, int tiles_n, int xcd_remap, unsigned long long *probe, int k_chunk,
    float *__restrict__ partials) {
  typedef __attribute__((ext_vector_type(TJ))) float bvec_t;
  constexpr int BMT = 32 * TI * WMW, BNT = 32 * TJ * WNW, NWAVES = WMW * WNW;
  constexpr int KK = BKT / 8;
  constexpr int A_ROW = BKT * 4, A_CHUNKS = A_ROW / 16, A_ROWS_PER_DMA = 1024 / A_ROW;
  constexpr int B_ROW = BNT * 4, B_CHUNKS = B_ROW / 16, B_ROWS_PER_DMA = 1024 / B_ROW;
  constexpr int A_BYTES_S = BMT * A_ROW, B_BYTES_S = BKT * B_ROW;
  constexpr int A_DMA = A_BYTES_S / 1024 / NWAVES, B_DMA = B_BYTES_S / 1024 / NWAVES;
  static_assert(A_DMA >= 1 && B_DMA >= 1 && A_DMA * 1024 * NWAVES == A_BYTES_S &&
                    B_DMA * 1024 * NWAVES == B_BYTES_S, "slab does not split over the waves");
  static_assert(A_ROW == 64 || A_ROW == 128, "BKT must be 16 or 32");
  static_assert(B_ROW <= 1024 && NS * (A_BYTES_S + B_BYTES_S) <= 160 * 1024, "LDS layout");
  static_assert((NS - 1) * (A_DMA + B_DMA) < 64, "vmcnt range");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WNW, wn = wave % WNW;
  const int lm = lane & 31, lh = lane >> 5;
  int tm, tn;
  tile_of_block(tiles_m, tiles_n, xcd_remap, tm, tn);
  const int m0 = tm * BMT, n0 = tn * BNT;
  long long probe_c0 = 0, probe_t0 = 0;
  if (kMeasureBuild && probe) {
    probe_c0 = clock64();
    probe_t0 = wall_clock64();
  }

  auto a_swz = [](int row) { return A_CHUNKS == 8 ? ((row >> 1) & 7) : ((row >> 2) & 3); };
  auto b_swz = [](int row) { return TJ == 1 ? (((row >> 2) & 1) << 3) : 0; };

  // DMA sources: uniform 64-bit base + per-lane 32-bit byte offset.  Rows past M and columns
  // past N are clamped to valid addresses; what they produce is never stored.
  uint32_t a_off[A_DMA], b_off[B_DMA];
#pragma unroll
  for (int i = 0; i < A_DMA; ++i) {
    const int q = wave + NWAVES * i;
    const int row_t = q * A_ROWS_PER_DMA + lane / A_CHUNKS;
    const int row = min(row_t, M - 1 - m0);
    a_off[i] = (static_cast<uint32_t>(row) * K + (((lane % A_CHUNKS) ^ a_swz(row_t)) << 2)) * 4u;
  }
#pragma unroll
  for (int i = 0; i < B_DMA; ++i) {
    const int q = wave + NWAVES * i;
    const int brow = q * B_ROWS_PER_DMA + lane / B_CHUNKS;
    const int chunk = (lane % B_CHUNKS) ^ b_swz(brow);
    const int col = Ragged ? n0 + chunk * 4 : min(n0 + chunk * 4, N - 4);
    b_off[i] = (static_cast<uint32_t>(brow) * N + col) * 4u;
  }
  // K cut over gridDim.y workgroups per tile: this one takes k0 .. k0 + k_len - 1 and writes its partial tile to its
  // own M x N plane of `partials`, which a second kernel adds up in a fixed order
  const int k0 = blockIdx.y * k_chunk;
  const int k_len = min(k_chunk, K - k0);
  if (gridDim.y > 1) C = partials + static_cast<int64_t>(blockIdx.y) * M * N;
  const char *a_base = reinterpret_cast<const char *>(A + static_cast<int64_t>(m0) * K + k0);
  const char *b_base = reinterpret_cast<const char *>(B + static_cast<int64_t>(k0) * N);
  const int64_t b_slab_bytes = static_cast<int64_t>(BKT) * N * 4;
  const int nslabs = (k_len + BKT - 1) / BKT;
  // The end of K inside the last slab.  With K >= BKT the last slab is moved back to end at K (its A pieces then hold
  // nothing but elements of their own row, at whatever alignment) and the B rows it shares with the slab before it
  // are the ones left out; with a single slab (K < BKT, K % 4 == 0) the A pieces and B rows past K are.  A lane's k
  // piece is the same for all its A transfers: rows NWAVES * A_ROWS_PER_DMA apart share the swizzle.
  const int k_tail = k_len - (nslabs - 1) * BKT;
  const bool move_last = Ragged && k_len >= BKT && k_tail != BKT;
  const int k_last = move_last ? k_len - BKT : (nslabs - 1) * BKT;   // first k of the last slab, from k0
  const bool a_lane_in_k =
      !Ragged || move_last || (((lane % A_CHUNKS) ^ a_swz(wave * A_ROWS_PER_DMA + lane / A_CHUNKS)) << 2) < k_tail;
  bool b_lane_in_k[B_DMA];
#pragma unroll
  for (int i = 0; i < B_DMA; ++i) {
    const int brow = (wave + NWAVES * i) * B_ROWS_PER_DMA + lane / B_CHUNKS;
    b_lane_in_k[i] = !Ragged || (move_last ? brow >= BKT - k_tail : brow < k_tail);
  }
  const char *b_end = reinterpret_cast<const char *>(B) + static_cast<int64_t>(K) * N * 4;
  constexpr uint32_t kOutOfRange = 0x80000000u;

  f32x16 acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // A wave with a single MFMA tile would feed every MFMA the result of the one before; it keeps a second
  // accumulator for the odd MFMA steps instead (two independent chains), added to the first at the end.
  constexpr bool kTwoChains = TI * TJ == 1;
  f32x16 acc_odd;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc_odd[r] = 0.f;

  const int a_row = wm * 32 * TI + lm;
  int a_addr0 = a_row * A_ROW + ((lh ^ a_swz(a_row)) << 4);           // ^ (kk << 5), + i*32*A_ROW
  int b_addr0 = (4 * lh) * B_ROW + (((wn * 32 * TJ + TJ * lm) * 4) ^ (TJ == 1 ? (lh << 7) : 0));

  // A: one resource for the tile's row panel, the slab selects a scalar byte offset.
  // B: the resource is rebased to the slab's first row (keeps every offset below 2^31).
  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(a_base, 0x80000000u);
  auto issue = [&](char *sa, char *sb, int slab) {
    const int sl = min(slab, nslabs - 1);   // the tail re-issues the last slab: constant vmcnt
    const bool whole = !Ragged || slab < nslabs - 1;
    const char *b_src = whole ? b_base + sl * b_slab_bytes : b_base + static_cast<int64_t>(k_last) * N * 4;
    const int64_t b_left = b_end - b_src;
    const __amdgpu_buffer_rsrc_t b_rsrc =
        make_rsrc(b_src, Ragged && b_left < 0x80000000ll ? static_cast<uint32_t>(b_left) : kOutOfRange);
    const uint32_t a_so = static_cast<uint32_t>(whole ? sl * BKT : k_last) * 4u;
#pragma unroll
    for (int i = 0; i < A_DMA; ++i)
      dma16(a_rsrc, (whole || a_lane_in_k) ? a_off[i] : kOutOfRange, a_so, sa + (wave + NWAVES * i) * 1024);
#pragma unroll
    for (int i = 0; i < B_DMA; ++i)
      dma16(b_rsrc, (whole || b_lane_in_k[i]) ? b_off[i] : kOutOfRange, 0u, sb + (wave + NWAVES * i) * 1024);
  };
  auto load_frags = [&](const char *sa, const char *sb, int kk, f32x4 (&af)[TI], bvec_t (&bf)[4]) {
    const char *pa = sa + (a_addr0 ^ (kk << 5));
#pragma unroll
    for (int i = 0; i < TI; ++i) af[i] = *reinterpret_cast<const f32x4 *>(pa + i * 32 * A_ROW);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      bf[j] = *reinterpret_cast<const bvec_t *>(sb + b_addr0 + (kk * 8 + j) * B_ROW);
  };
  auto mfma_step = [&](f32x4 (&af)[TI], bvec_t (&bf)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int jn = 0; jn < TJ; ++jn) {
          if (kTwoChains && (j & 1))
            acc_odd = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][j], bf[j][jn], acc_odd, 0, 0, 0);
          else
            acc[i][jn] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][j], bf[j][jn], acc[i][jn], 0, 0, 0);
        }
  };
  // Issue order inside one k-step: behind each of the first MFMAs go the DMA instructions
  // of this k-step (NV of them; unpinned, the compiler bunches them in front of the first
  // MFMA, where their issue time leaves the pipe idle) and the LDS reads of the next
  // step's fragments.
  auto interleave = [](auto nv_c) {
    constexpr int NV = decltype(nv_c)::value;
    constexpr int READS = TI + 4, MFMAS = 4 * TI * TJ;
    constexpr int GROUPS = READS < MFMAS ? READS : MFMAS;
    constexpr int PER = (READS + GROUPS - 1) / GROUPS, VPER = (NV + GROUPS - 1) / GROUPS;
    [&]<int... Gs>(std::integer_sequence<int, Gs...>) {
      (([] {
         __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);    // 1 MFMA
         if constexpr (Gs * VPER < NV)                         // DMA instructions
           __builtin_amdgcn_sched_group_barrier(0x020, (NV - Gs * VPER) < VPER ? (NV - Gs * VPER) : VPER, 0);
         __builtin_amdgcn_sched_group_barrier(0x100, PER, 0);  // DS reads
       }()),
       ...);
    }(std::make_integer_sequence<int, GROUPS>{});
    if (MFMAS > GROUPS) __builtin_amdgcn_sched_group_barrier(0x008, MFMAS - GROUPS, 0);
    __builtin_amdgcn_sched_barrier(0);
  };

  f32x4 af[2][TI];
  bvec_t bf[2][4];

  auto slab = [&](char *ca, char *cb, const char *na, const char *nb, int s) {
    asm volatile("" : "+v"(a_addr0), "+v"(b_addr0));   // keep per-stage addresses out of registers
#pragma unroll
    for (int kk = 0; kk + 1 < KK; ++kk) {
      load_frags(ca, cb, kk + 1, af[(kk + 1) & 1], bf[(kk + 1) & 1]);
      mfma_step(af[kk & 1], bf[kk & 1]);
      interleave(std::integral_constant<int, 0>{});
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0((NS - 2) * (A_DMA + B_DMA)));
    barrier_no_fence();
    issue(ca, cb, s + NS);
    load_frags(na, nb, 0, af[0], bf[0]);
    mfma_step(af[(KK - 1) & 1], bf[(KK - 1) & 1]);
    interleave(std::integral_constant<int, A_DMA + B_DMA>{});
  };

  issue(lds_ring<0, A_BYTES_S>, lds_ring<1, B_BYTES_S>, 0);
  issue(lds_ring<2, A_BYTES_S>, lds_ring<3, B_BYTES_S>, 1);
  if constexpr (NS == 4) {
    issue(lds_ring<4, A_BYTES_S>, lds_ring<5, B_BYTES_S>, 2);
    issue(lds_ring<6, A_BYTES_S>, lds_ring<7, B_BYTES_S>, 3);
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0((NS - 1) * (A_DMA + B_DMA)));
  barrier_no_fence();
  load_frags(lds_ring<0, A_BYTES_S>, lds_ring<1, B_BYTES_S>, 0, af[0], bf[0]);
  __builtin_amdgcn_sched_barrier(0);

  auto ring_slab = [&](auto st_c, int s) {
    constexpr int st = decltype(st_c)::value;
    constexpr int nx = (st + 1) % NS;
    slab(lds_ring<2 * st, A_BYTES_S>, lds_ring<2 * st + 1, B_BYTES_S>, lds_ring<2 * nx, A_BYTES_S>,
         lds_ring<2 * nx + 1, B_BYTES_S>, s);
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  const int full = nslabs - nslabs % NS;
  for (int s = 0; s < full; s += NS) {
    ring_slab(I0{}, s);
    ring_slab(I1{}, s + 1);
    if constexpr (NS == 4) {
      ring_slab(I2{}, s + 2);
      ring_slab(I3{}, s + 3);
    }
  }
  if (full < nslabs) ring_slab(I0{}, full);
  if constexpr (NS == 4) {
    if (full + 1 < nslabs) ring_slab(I1{}, full + 1);
    if (full + 2 < nslabs) ring_slab(I2{}, full + 2);
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));   // drain the redundant tail DMA
  if constexpr (kTwoChains) {
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[0][0][r] += acc_odd[r];
  }

  // Epilogue: register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4 of its 32-row tile and
  // columns TJ*(l%32) .. +TJ-1 of the wave's span (one per MFMA tile jn).
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = m0 + wm * 32 * TI + i * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
      const int col = n0 + wn * 32 * TJ + TJ * lm;
      if constexpr (Ragged) {
#pragma unroll
        for (int jn = 0; jn < TJ; ++jn)
          if (row < M && col + jn < N) C[static_cast<int64_t>(row) * N + col + jn] = acc[i][jn][r];
      } else if (row < M && col < N) {
        bvec_t v;
#pragma unroll
        for (int jn = 0; jn < TJ; ++jn) v[jn] = acc[i][jn][r];
        *reinterpret_cast<bvec_t *>(C + static_cast<int64_t>(row) * N + col) = v;
      }
    }
  if (kMeasureBuild && probe && tid == 0) {
    probe[2 * blockIdx.x] = static_cast<unsigned long long>(clock64() - probe_c0);
    probe[2 * blockIdx.x + 1] = static_cast<unsigned long long>(wall_clock64() - probe_t0);
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

namespace {
// Tile choice by a cost model of the launch: a CU holds `occ` workgroups of a tile shape at once (LDS ring), tiles run
// in rounds of cus*occ, a workgroup that shares its CU takes occ times as long, and the tail round runs unshared when it
// fits one workgroup per CU.  `eff` is the MFMA issue efficiency measured for each shape.
int gemm_f32_tile_for(int m, int n) {
  auto ntiles = [&](int t) { return static_cast<int64_t>((m + t - 1) / t) * ((n + t - 1) / t); };
  static const int cus = [] {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
      v = 256;
    return v;
  }();
  auto cost = [&](int t, int occ, double eff) {
    const int64_t tiles = ntiles(t), slots = static_cast<int64_t>(cus) * occ;
    const int64_t full = tiles / slots, rest = tiles % slots;
    const double rounds = static_cast<double>(full) * occ + (rest == 0 ? 0 : rest <= cus ? 1 : occ);
    return rounds * t * t / eff;
  };
  const double c256 = cost(256, 1, 1.0), c128 = cost(128, 2, 0.95), c64 = cost(64, 2, 0.80);
  return (c256 <= c128 && c256 <= c64) ? 256 : (c128 <= c64 ? 128 : 64);
}

// K pieces for a product on the 64 x 64 tile; 1 = whole.  One such tile per CU runs at the rate of its MFMAs (0.45 us per
// K = 32 slab, measured; two on a CU share the pipes), so pieces help while CUs are idle; against that stand the second
// launch (5 us) and the partial planes (0.65 us per MiB).  The count in {2, 4, 8, 16} with the lowest estimate is taken
// if it is a tenth below the whole product's.  gemm_f32.split_k: 0 = this rule, 1 = never, n >= 2 forces n.
int splitk_f32_for(int m, int n, int k) {
  const int64_t forced = tunable("gemm_f32.split_k", 0);
  if (forced == 1 || (static_cast<int64_t>(m) * n) % 4 != 0 || k % 32 != 0) return 1;
  static const int cus = [] {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
      v = 256;
    return v;
  }();
  const int64_t tiles = static_cast<int64_t>((m + 63) / 64) * ((n + 63) / 64);
  const double plane_mib = static_cast<double>(m) * n * 4 / (1 << 20);
  const int64_t fit = static_cast<int64_t>(static_cast<double>(kSplitWorkspaceBytes >> 20) / plane_mib);
  int64_t splits = 1;
  if (forced >= 2) {
    splits = std::min<int64_t>({forced, static_cast<int64_t>(k / 32), fit});
  } else {
    auto estimate = [&](int64_t s) {
      const double rounds = static_cast<double>((tiles * s + cus - 1) / cus);
      return 8.0 + static_cast<double>(k) / 32 / s * 0.45 * rounds + (s > 1 ? 5.0 + s * plane_mib * 0.65 : 0.0);
    };
    double best = estimate(1) * 0.9;
    for (int64_t s = 2; s <= 16; s *= 2) {
      if (k / s < 256 || s > fit) break;
      if (estimate(s) < best) best = estimate(s), splits = s;
    }
  }
  if (splits < 2) return 1;
  const int chunk = static_cast<int>(((k / 32 + splits - 1) / splits) * 32);
  return (k + chunk - 1) / chunk;
}
}  // namespace

extern "C" int sarek_hip_gemm_f32_k_splits(int m, int n, int k) {
  if (m < 1 || n < 1 || k < 1) return 1;
  // the split belongs to the 64 x 64 tile, which the launcher takes where its cost model says so
  const int64_t forced_tile = tunable("gemm_f32.tile", 0);
  if (forced_tile != 0 && forced_tile != 64) return 1;
  if (forced_tile == 0 && gemm_f32_tile_for(m, n) != 64) return 1;
  return splitk_f32_for(m, n, k);
}

extern "C" int sarek_hip_gemm_f32(const float *a, const float *b, float *c, int m, int n, int k,
                                  sarek_hip_stream stream) {
  if (m <= 0 || n <= 0 || k <= 0)
    return fail(SAREK_HIP_E_INVALID_ARG, "gemm_f32: m, n, k must be positive (got %d %d %d)", m, n, k);
  if (!a || !b || !c) return fail(SAREK_HIP_E_INVALID_ARG, "gemm_f32: NULL matrix");
  hipStream_t st = as_stream(stream);
  // The direct-to-LDS kernels take any shape and alignment in their Ragged form, except a K below one slab that is
  // not a multiple of 4; the aligned form is the faster one where it applies.
  const bool aligned = (k % 4 == 0) && (reinterpret_cast<uintptr_t>(a) % 16 == 0) &&
                       (reinterpret_cast<uintptr_t>(b) % 16 == 0);
  const bool ab_ok = aligned || k >= 32;   // the ragged form needs no alignment once K fills a slab
  const int remap = (int)tunable("gemm.xcd_remap", 1);
  // DMA offsets are 32-bit: 256 rows of A and 32 rows of B must span less than 2 GiB
  const bool offsets_ok = static_cast<int64_t>(k) * 256 * 4 < 0x7FFFFFFF &&
                          static_cast<int64_t>(n) * 32 * 4 < 0x7FFFFFFF;
  if (ab_ok && offsets_ok && tunable("gemm_f32.force_simple", 0) == 0 && tunable("gemm_f32.force_staged", 0) == 0) {
    const bool ragged = !aligned || n % 4 != 0 || k % 32 != 0 || reinterpret_cast<uintptr_t>(c) % 16 != 0;
    auto ntiles = [&](int t) { return static_cast<int64_t>((m + t - 1) / t) * ((n + t - 1) / t); };
    int tile = (int)tunable("gemm_f32.tile", 0);
    if (tile == 0) tile = gemm_f32_tile_for(m, n);
    // K cut over idle CUs for the 64 x 64 tile (few tiles, long K): whole slabs per piece, planes added 16 bytes at a time
    int splits = 1;
    float *partials = nullptr;
    if (tile == 64 && k % 32 == 0 && reinterpret_cast<uintptr_t>(c) % 16 == 0) {
      splits = splitk_f32_for(m, n, k);
      if (splits > 1) partials = splitk_workspace(st);
      if (!partials) splits = 1;
    }
    const int k_chunk = splits > 1 ? ((k / 32 + splits - 1) / splits) * 32 : k;
#define SAREK_LAUNCH_F32(T, TI, TJ, WMW, WNW, BKT, RAGGED)                                         \
  hipLaunchKernelGGL((gemm_f32_dma_kernel<TI, TJ, WMW, WNW, BKT, 4, RAGGED>),                     \
                     dim3((unsigned)ntiles(T), splits), dim3(64 * WMW * WNW), 0, st, a, b, c, m, n, k, \
                     (m + T - 1) / T, (n + T - 1) / T, remap, splits > 1 ? nullptr : clock_probe(ntiles(T)), k_chunk, \
                     partials)
    if (ragged) {
      if (tile == 256) SAREK_LAUNCH_F32(256, 4, 2, 2, 4, 16, true);
      else if (tile == 128) SAREK_LAUNCH_F32(128, 2, 2, 2, 2, 16, true);
      else SAREK_LAUNCH_F32(64, 1, 1, 2, 2, 32, true);
    } else {
      if (tile == 256) SAREK_LAUNCH_F32(256, 4, 2, 2, 4, 16, false);
      else if (tile == 128) SAREK_LAUNCH_F32(128, 2, 2, 2, 2, 16, false);
      else SAREK_LAUNCH_F32(64, 1, 1, 2, 2, 32, false);
    }
#undef SAREK_LAUNCH_F32
    const int rc = check_launch("gemm_f32 kernel launch");
    if (rc != SAREK_HIP_OK || splits == 1) return rc;
    return launch_splitk_reduce(partials, c, static_cast<int64_t>(m) * n, splits, st);
  }
  if (aligned && n % 4 == 0 && tunable("gemm_f32.force_simple", 0) == 0) {
    static bool attr_done = false;
    if (!attr_done) {
      SAREK_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_f32_staged_kernel),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
      attr_done = true;
    }
    const int tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
    hipLaunchKernelGGL(gemm_f32_staged_kernel, dim3(tiles_m * tiles_n), dim3(THREADS), LDS_BYTES, st, a, b,
                       c, m, n, k, tiles_m, tiles_n, remap);
  } else {
    hipLaunchKernelGGL(gemm_f32_simple_kernel, dim3((n + 63) / 64, (m + 3) / 4), dim3(256), 0, st,
                       a, b, c, m, n, k);
  }
  return check_launch("gemm_f32 kernel launch");
}
