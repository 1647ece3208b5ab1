// 16-bit-input (bf16 / fp16), f32-accumulate GEMM for gfx950 on v_mfma_f32_16x16x32,
// with an optional fused epilogue  y = relu(acc + bias[col]),  rowsum[row] = sum of y over the row.
//
// C[M x N] = A[M x K] . B[K x N], all row-major.
//
// Kernels:
//   gemm16_m16_kernel: one workgroup owns a 256 x 256 tile of C and walks K in slabs; 8 waves (2 along M x 4 along
//     N, two per SIMD), each owning 128 x 64 = 8 x 4 MFMA tiles of 16 x 16 (128 accumulator registers).  One
//     workgroup per CU (LDS bound), 8192^3 = 1024 tiles = 4 per CU.  Global -> LDS by buffer_load_dwordx4 ... lds,
//     which writes the 64 lanes' 16-byte pieces to 1 KiB of consecutive LDS with no register staging and no ds_write
//     (the buffer form: the global_load form of the same transfer slows MFMA issue down).  Rows cannot be padded that
//     way, so bank conflicts are removed by an XOR swizzle applied on the global-address side (which chunk a lane
//     fetches) and again by the readers.  A streams through a ring of 2 LDS stages of K = 64 (whole 128-byte lines
//     per request), B through a ring of 4 slabs of K = 32 (128 KiB in all): a stage is refilled as soon as the
//     barrier inside the slab that read it last has passed.  B is n-contiguous in LDS (as in global memory): a lane's
//     column fragment is gathered by ds_read_b64_tr_b16.
//   gemm16_m16_small_kernel: the same pipeline on a 128 x 128 tile (4 waves), two workgroups per CU, for products
//     that do not fill the chip with large tiles; K split over several workgroups per tile where tiles are few.
//   gemm16_simple_kernel: any shape and alignment, one thread per C element (K below one LDS stage that is not a
//     multiple of 8, or operands whose 256-row / 64-row panels span 2 GiB).
//   gemm16_last_column_kernel: column N-1 of an odd N.
// A build with -DSAREK_HIP_MEASURE (libsarek_hip_measure.so, for bench.py --measure-build) also holds gemm16_dma_kernel,
// the same pipeline on v_mfma_f32_32x32x16 in several ring and wave shapes, and variants of both MFMA kernels that leave
// parts of the K loop out: what the power and ablation studies were measured with.  The product library has none of them.
#include <algorithm>
#include <map>
#include <mutex>
#include <type_traits>
#include <utility>

#include "common.hpp"
#include "gemm_common.hpp"
#include "tunables.hpp"

namespace sarek_hip {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

constexpr int BM = 256, BN = 256, BK = 64;

enum { EPI_STORE = 0, EPI_BIAS_RELU_ROWSUM = 1 };


// ds_read_b64_tr_b16 at byte offset `off` of the dynamic LDS block.
__device__ __forceinline__ u32x2 lds_read_tr16(const char *lds, int off) {
  auto p = (LDS_PTR bf16x4 *)(lds + off);
  bf16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(p);
  return __builtin_bit_cast(u32x2, v);
}

// ---- what the direct-to-LDS kernels share -----------------------------------------
// A moves in stages of BKA k (ring of NA), B in slabs of BKB k (ring of NB); RA = BKA / BKB
// B slabs consume one A stage.  Default: BKA = 64, NA = 2, BKB = 32, NB = 4.  A rows are
// K-contiguous in memory, so a 32-wide A slab would touch half of each 128-byte line and
// the next slab the other half (two L1 -> L2 requests per line: a third more requests
// over the whole kernel, and the address path stalls on them); with 64-wide A stages
// every request is a whole line, while B, whose rows are N-contiguous (512 bytes of a row
// per tile), keeps the finer slabs and the deeper ring.  One barrier per B slab.
// TJ: 32-column MFMA tiles per wave along N.  TJ = 2: 8 waves (2 x 4) of 128 x 64, two
// per SIMD; TJ = 4: 4 waves (2 x 2) of 128 x 128, one per SIMD with the 256 accumulator
// registers in the AGPR half of the register file (fewer LDS bytes read per flop).
//
// Order of a wave's transfers (what vmcnt counts): top of slab j: B(j-1+NB), into the stage
// slab j-1 used; after the barrier of slab j: the A stage that slab j was the last to read.
constexpr int dma_allowed_in_flight(int I, int RA, int NA, int NB, int DA, int DB, int slabs_per_barrier = 1) {
  // Transfers that may still be in flight at the barrier of slab s = I (mod period) once
  // everything slab s+1 reads has landed: those issued after the later of B(s+1) and the
  // A stage that slab s+1 starts (if it starts one).  Event 2j = top of slab j, 2j+1 = its
  // barrier.  With a barrier in every other slab only (slabs_per_barrier = 2: the top of slab j
  // issues B(j-2+NB), and the barrier of an odd slab s covers what slabs s+1 and s+2 read) the
  // later B slab is B(s+2), issued at the top of slab s+4-NB.
  const int s = I + 64 * RA * NA * NB;
  int need = slabs_per_barrier == 2 ? 2 * (s + 4 - NB) : 2 * (s + 2 - NB);
  if ((s + 1) % RA == 0) {
    const int ev = 2 * (s + RA - RA * NA) + 1;
    if (ev > need) need = ev;
  }
  int count = 0;
  for (int e = need + 1; e < 2 * s + 1; ++e) {
    const int j = e / 2;
    if (e % 2 == 0) count += DB;
    else if (j % RA == RA - 1) count += DA;
  }
  return count;
}
constexpr int lcm_int(int a, int b) {
  int m = a;
  while (m % b != 0) m += a;
  return m;
}

#ifdef SAREK_HIP_MEASURE
template <bool Bf16>
__device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (Bf16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// Writes one wave's 128 x (32*TJ) accumulator block.  Accumulator layout of the 32x32 MFMA:
// register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its tile.
//
// Fused form: y = relu(acc + bias[col]) is stored, and the row sums of the workgroup's
// 256 x 256 tile are formed before anything goes to memory:
//   1. per lane: sum over its TJ columns -> 64 values, one per row the lane touches
//      (index q = 16*i + r);
//   2. across the 32 lanes of a half-wave (which share those 64 rows) by a halving
//      butterfly: at the step with lane mask m a lane keeps one half of its values and
//      receives the partner's sums for that half, so 32+16+8+4+2 exchanges leave lane lm
//      with the sums of rows q = 2*lm and 2*lm+1;
//   3. across the WN waves that share the rows through `scratch` (LDS, WN x 256 floats; all
//      waves must be done with the LDS ring: barriers inside), then one atomicAdd per row.
template <int Epi, int TJ, bool NoStore = false>
__device__ __forceinline__ void epilogue(f32x16 (&acc)[4][TJ], float *__restrict__ C,
                                         const float *__restrict__ bias,
                                         float *__restrict__ rowsum, int M, int N, int m0,
                                         int wm, int wn, int col0, int lm, int lh,
                                         float *scratch) {
  constexpr int WN = 8 / TJ;
  const int row0 = m0 + wm * 128;
  float bj[TJ];
  bool cok[TJ];
#pragma unroll
  for (int j = 0; j < TJ; ++j) {
    const int col = col0 + j * 32 + lm;
    cok[j] = col < N;
    bj[j] = (Epi == EPI_BIAS_RELU_ROWSUM && cok[j]) ? bias[col] : 0.f;
  }
  float rs[64];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = row0 + i * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
      float sum = 0.f;
#pragma unroll
      for (int j = 0; j < TJ; ++j) {
        float v = acc[i][j][r];
        if (Epi == EPI_BIAS_RELU_ROWSUM) {
          v += bj[j];
          v = v > 0.f ? v : 0.f;
          sum += cok[j] ? v : 0.f;
        }
        // NoStore (measurement only): the compare keeps the values alive, nothing is written
        if (row < M && cok[j] && (!NoStore || v == 1.2345e30f)) C[static_cast<int64_t>(row) * N + col0 + j * 32 + lm] = v;
      }
      rs[i * 16 + r] = sum;
    }
  }
  if constexpr (Epi == EPI_BIAS_RELU_ROWSUM) {
#pragma unroll
    for (int step = 0; step < 5; ++step) {
      const int m = 16 >> step, half = 32 >> step;
      const bool up = (lm & m) != 0;
#pragma unroll
      for (int q = 0; q < half; ++q) {
        const float send = up ? rs[q] : rs[q + half];
        const float keep = up ? rs[q + half] : rs[q];
        rs[q] = keep + __shfl_xor(send, m, 64);
      }
    }
    // lane lm now holds rows q = 2*lm + e (e = 0, 1) of its half-wave's row set
    __syncthreads();  // every wave has left the K loop: the LDS ring is free
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int q = 2 * lm + e, i = q >> 4, r = q & 15;
      scratch[wn * 256 + wm * 128 + i * 32 + 8 * (r >> 2) + 4 * lh + (r & 3)] = rs[e];
    }
    __syncthreads();
    const int t = threadIdx.x;
    if (t < 256 && m0 + t < M) {
      float total = 0.f;
#pragma unroll
      for (int w = 0; w < WN; ++w) total += scratch[w * 256 + t];
      atomicAdd(rowsum + m0 + t, total);
    }
  }
}

// Ablate (measurement only, results are wrong by construction; tunable gemm16.ablate): bit 0 leaves the
// global -> LDS transfers out of the K loop (the ring keeps what the prologue put there), bit 1 the LDS
// fragment reads (every MFMA reuses the first fragments), bit 2 makes every workgroup fetch the panels of
// tile (0, 0) (the same global -> LDS transfers, all served by the L2s: no traffic past them), bit 3 leaves the
// stores of C out.  What remains
// shows what each part of the loop costs in cycles and, under the package power limit, in clock.
template <bool Bf16, int Epi, int BKA, int BKB, int NA, int NB, int TJ, int Ablate = 0>
__global__ __launch_bounds__(64 * 2 * (8 / TJ)) void gemm16_dma_kernel(const uint16_t *__restrict__ A,
                                                             const uint16_t *__restrict__ B,
                                                             float *__restrict__ C,
                                                             const float *__restrict__ bias,
                                                             float *__restrict__ rowsum, int M,
                                                             int N, int K, int tiles_m,
                                                             int tiles_n, int xcd_remap,
                                                             unsigned long long *probe) {
  constexpr int KKB = BKB / 16;                // MFMA k-steps per B slab
  constexpr int RA = BKA / BKB;                // B slabs per A stage
  constexpr int A_ROW = BKA * 2;               // bytes per A row in LDS (unpadded)
  constexpr int A_ROWS_PER_DMA = 1024 / A_ROW; // rows one wave-wide DMA fills
  constexpr int A_CHUNKS = A_ROW / 16;
  constexpr int A_BYTES_S = BM * A_ROW, B_BYTES_S = BKB * BN * 2;
  constexpr int WN = 8 / TJ;                   // waves along N (4 or 2); 2 along M
  constexpr int NWAVES = 2 * WN;
  constexpr int DA = A_BYTES_S / 1024 / NWAVES;   // transfers per wave and A stage
  constexpr int DB = B_BYTES_S / 1024 / NWAVES;   // transfers per wave and B slab
  constexpr int P = lcm_int(NB, RA * NA);         // slabs after which the stage pattern repeats
  static_assert(KKB >= 2 && KKB % 2 == 0 && BKA % BKB == 0, "slab shapes");
  static_assert(NA >= 2 && NB >= 2 && RA * (NA - 1) >= 1, "ring depths");
  static_assert(NA * A_BYTES_S + NB * B_BYTES_S <= 160 * 1024, "LDS ring too large");
  static_assert((NB - 1) * DB + NA * DA < 64, "vmcnt range");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int lm = lane & 31, lh = lane >> 5;
  int tm, tn;
  tile_of_block(tiles_m, tiles_n, xcd_remap, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int m0_src = (Ablate & 4) ? 0 : m0, n0_src = (Ablate & 4) ? 0 : n0;
  long long probe_c0 = 0, probe_t0 = 0;
  if (kMeasureBuild && probe) {
    probe_c0 = clock64();
    probe_t0 = wall_clock64();
  }

  // Swizzles (XOR on the 16-byte slot index within a row).  The LDS of this chip serves
  // 256 bytes per clock (64 banks x 4 bytes): a ds_read_b128 is served 16 lanes at a time
  // and a ds_read_b64_tr_b16 32 lanes at a time, and a phase is conflict free when its
  // pieces fall on distinct positions modulo 256 bytes.
  //   A, 128-byte rows: 16 consecutive rows read the same chunk c; row parity picks the
  //      128-byte half, so the slot must differ over rows of equal parity:
  //      slot = c ^ ((row >> 1) & 7).   A, 64-byte rows: slot = c ^ ((row >> 2) & 3).
  //   B, 512-byte rows: a phase reads 4 rows x two 32-byte pieces (n halves); rows are
  //      spread 64 bytes apart: slot = c ^ ((row & 3) << 2).
  auto a_swz = [](int row) { return A_CHUNKS == 8 ? ((row >> 1) & 7) : ((row >> 2) & 3); };

  // ---- DMA source addresses (stage / slab 0) ---------------------------------------
  // A: wave-instruction q = wave + NWAVES*i fills rows q*R .. q*R+R-1 (R = A_ROWS_PER_DMA);
  //    lane l -> row q*R + l/A_CHUNKS, LDS slot l%A_CHUNKS, global chunk slot ^ a_swz(row).
  // B: instruction q fills rows 2q, 2q+1; lane l -> row 2q + l/32, slot l%32,
  //    global chunk slot ^ ((row & 3) << 2).
  // Rows past M and columns past N are clamped to valid addresses: what they produce is
  // never stored.
  // Addresses are (uniform 64-bit base) + (per-lane 32-bit byte offset), the form the
  // hardware takes as scalar base + vector offset, so only one register per DMA is kept.
  uint32_t a_off[DA], b_off[DB];
#pragma unroll
  for (int i = 0; i < DA; ++i) {
    const int q = wave + NWAVES * i;
    const int arow_t = q * A_ROWS_PER_DMA + lane / A_CHUNKS;
    const int arow = min(arow_t, M - 1 - m0_src);
    a_off[i] = (static_cast<uint32_t>(arow) * K + (((lane % A_CHUNKS) ^ a_swz(arow_t)) << 3)) * 2u;
  }
#pragma unroll
  for (int i = 0; i < DB; ++i) {
    const int q = wave + NWAVES * i;
    const int brow = 2 * q + (lane >> 5);
    const int bchunk = (lane & 31) ^ ((brow & 3) << 2);
    const int bcol = min(n0_src + bchunk * 8, N - 8);
    b_off[i] = (static_cast<uint32_t>(brow) * N + bcol) * 2u;
  }
  const char *a_base = reinterpret_cast<const char *>(A + static_cast<int64_t>(m0_src) * K);
  const char *b_base = reinterpret_cast<const char *>(B);
  const int64_t b_slab_bytes = static_cast<int64_t>(BKB) * N * 2;
  const int nslabs = K / BKB, nstages = K / BKA;

  f32x16 acc[4][TJ];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // ---- fragment read offsets ------------------------------------------------------
  // A: row = wm*128 + i*32 + lm, chunk = 2*ka + lh (ka = k-step within the stage),
  //    slot = chunk ^ a_swz(row).  Since 2*ka and lh occupy different bits,
  //    slot = (lh ^ a_swz) ^ 2*ka: the address for k-step ka is one base XOR (ka << 5),
  //    and i*32 rows is a constant offset.
  // B (transposing read): 16-lane group g16 = lane/16: n half = g16 & 1, k half = lh; lane li
  //    supplies row (li>>2) of its 4-row block and the 8 bytes at n offset 4*(li&3).  Rows
  //    kb*16 + lh*8 + {0..3} and +4 share (row & 3) = li>>2, so the swizzle XOR is the same
  //    for both reads; j*64 bytes only touches bit 6, i.e. another XOR.
  const int a_row = wm * 128 + lm;
  int a_addr0 = a_row * A_ROW + ((lh ^ a_swz(a_row)) << 4);
  const int li = lane & 15;
  const int b_r = li >> 2;
  int b_addr0 = (lh * 8 + b_r) * 512 +
                (((wn * (32 * TJ) + ((lane >> 4) & 1) * 16) * 2 + (li & 3) * 8) ^ (b_r << 6));

  // Indices past the end are clamped: the tail keeps issuing (redundant) DMA into stages
  // nobody reads any more, so that the count of outstanding transfers per wave follows the
  // same pattern in every iteration.
  // A: one resource for the tile's row panel, the stage selects a scalar byte offset.
  // B: the resource is rebased to the slab's first row (keeps every offset below 2^31).
  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(a_base, 0x80000000u);
  auto issue_a = [&](char *sa, int stage) {
    if (stage >= NA && (Ablate & 1)) return;
    const uint32_t a_so = static_cast<uint32_t>(min(stage, nstages - 1)) * (BKA * 2);
#pragma unroll
    for (int i = 0; i < DA; ++i) dma16(a_rsrc, a_off[i], a_so, sa + (wave + NWAVES * i) * 1024);
  };
  auto issue_b = [&](char *sb, int slab) {
    if (slab >= NB && (Ablate & 1)) return;
    const int sl = min(slab, nslabs - 1);
    const __amdgpu_buffer_rsrc_t b_rsrc = make_rsrc(b_base + sl * b_slab_bytes, 0x80000000u);
#pragma unroll
    for (int i = 0; i < DB; ++i) dma16(b_rsrc, b_off[i], 0u, sb + (wave + NWAVES * i) * 1024);
  };
  // ka: k-step within the A stage, kb: k-step within the B slab
  bool frags_loaded = false;
  auto load_frags = [&](const char *sa, const char *sb, int ka, int kb, u32x4 (&af)[4], u32x4 (&bf)[TJ]) {
    if ((Ablate & 2) && frags_loaded) return;
    const char *pa = sa + (a_addr0 ^ (ka << 5));
#pragma unroll
    for (int i = 0; i < 4; ++i)
      af[i] = *reinterpret_cast<const u32x4 *>(pa + i * 32 * A_ROW);
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
      // j*64 bytes: with TJ = 4 the wave's 256-byte column span is 256-byte aligned, so
      // adding j*64 never carries into the bits the swizzle touches differently
      const int off = (b_addr0 ^ (j << 6)) + kb * 16 * 512;
      u32x2 lo = lds_read_tr16(sb, off);
      u32x2 hi = lds_read_tr16(sb, off + 4 * 512);
      bf[j] = u32x4{lo.x, lo.y, hi.x, hi.y};
    }
  };
  auto mfma_step = [&](u32x4 (&af)[4], u32x4 (&bf)[TJ]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < TJ; ++j) acc[i][j] = mfma<Bf16>(af[i], bf[j], acc[i][j]);
  };
  // Issue order inside one k-step: an MFMA goes first, then behind each following MFMA
  // one DMA instruction (NV of them belong to this k-step) and two LDS reads of the next
  // step's fragments; the remaining MFMAs cover the read latency.  Left to itself the
  // compiler bunches the DMA instructions in front of the first MFMA, where their issue
  // time (and any back-pressure from the address path) leaves the MFMA pipe idle: pinning
  // them behind MFMAs took 6 % (8 waves) to 9 % (4 waves) off the cycle count.
  auto interleave = [](auto nv_c) {
    constexpr int NV = decltype(nv_c)::value;
    constexpr int READS = 4 + 2 * TJ, MFMAS = 4 * TJ;
    constexpr int G = READS / 2, SLOTS = NV > G ? NV : G;
    static_assert(SLOTS + 1 <= MFMAS, "not enough MFMAs to hide the issues behind");
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                // 1 MFMA
#pragma unroll
    for (int g = 0; g < SLOTS; ++g) {
      if (g < NV) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // 1 VMEM read (DMA)
      if (g < G) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);   // 2 DS reads
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, MFMAS - 1 - SLOTS, 0);
    __builtin_amdgcn_sched_barrier(0);
  };

  u32x4 af[2][4], bf[2][TJ];

  // One B slab; I = its index modulo P fixes every stage at compile time (each stage is
  // its own array, so the compiler does not order DMA into one stage against reads of
  // another).  After the barrier every wave is done reading the slab's B stage, which the
  // next slab's top refills, and, on the last slab of an A stage, that stage, which is
  // refilled at once.  The barrier sits before the last k-step, whose MFMAs cover the
  // first fragment reads of the next slab.
  auto slab = [&](auto ic, int s) {
    constexpr int I = decltype(ic)::value;
    constexpr int In = (I + 1) % P;
    constexpr int ia = (I / RA) % NA, ib = I % NB, ibp = (I + NB - 1) % NB;
    constexpr int ian = (In / RA) % NA, ibn = In % NB;
    constexpr int ka0 = (I % RA) * KKB, ka0n = (In % RA) * KKB;
    // Keep the per-stage LDS addresses from being hoisted out of the K loop (they would
    // occupy a register per stage and k-step): the bases are made opaque once per slab.
    asm volatile("" : "+v"(a_addr0), "+v"(b_addr0));
#pragma unroll
    for (int kk = 0; kk + 1 < KKB; ++kk) {
      if (kk == 0) issue_b(lds_ring<20 + ibp, B_BYTES_S>, s - 1 + NB);
      load_frags(lds_ring<10 + ia, A_BYTES_S>, lds_ring<20 + ib, B_BYTES_S>, ka0 + kk + 1, kk + 1,
                 af[(kk + 1) & 1], bf[(kk + 1) & 1]);
      mfma_step(af[kk & 1], bf[kk & 1]);
      if (kk == 0) interleave(std::integral_constant<int, DB>{});
      else interleave(std::integral_constant<int, 0>{});
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(dma_allowed_in_flight(I, RA, NA, NB, DA, DB)));
    barrier_no_fence();
    if constexpr (I % RA == RA - 1) issue_a(lds_ring<10 + ia, A_BYTES_S>, s / RA + NA);
    load_frags(lds_ring<10 + ian, A_BYTES_S>, lds_ring<20 + ibn, B_BYTES_S>, ka0n, 0, af[0], bf[0]);
    mfma_step(af[(KKB - 1) & 1], bf[(KKB - 1) & 1]);
    interleave(std::integral_constant<int, (I % RA == RA - 1) ? DA : 0>{});
  };

  // prologue: fill both rings except the last B stage (the top of slab 0 issues it) and
  // wait for all of it, so that from here on a wave never has more in flight than the
  // steady-state pattern assumes
  [&]<int... Is>(std::integer_sequence<int, Is...>) {
    (issue_a(lds_ring<10 + Is, A_BYTES_S>, Is), ...);
  }(std::make_integer_sequence<int, NA>{});
  [&]<int... Is>(std::integer_sequence<int, Is...>) {
    (issue_b(lds_ring<20 + Is, B_BYTES_S>, Is), ...);
  }(std::make_integer_sequence<int, NB - 1>{});
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
  barrier_no_fence();
  load_frags(lds_ring<10, A_BYTES_S>, lds_ring<20, B_BYTES_S>, 0, 0, af[0], bf[0]);
  if (Ablate & 2) {
    load_frags(lds_ring<10, A_BYTES_S>, lds_ring<20, B_BYTES_S>, 1, 1, af[1], bf[1]);
    frags_loaded = true;
  }
  __builtin_amdgcn_sched_barrier(0);

  // Whole periods first (no exits inside a period, which keeps the accumulators in
  // place), then the remaining nslabs % P slabs.
  const int full = nslabs - nslabs % P;
  for (int s = 0; s < full; s += P) {
    [&]<int... Is>(std::integer_sequence<int, Is...>) {
      (slab(std::integral_constant<int, Is>{}, s + Is), ...);
    }(std::make_integer_sequence<int, P>{});
  }
  [&]<int... Is>(std::integer_sequence<int, Is...>) {
    ((full + Is < nslabs ? slab(std::integral_constant<int, Is>{}, full + Is) : (void)0), ...);
  }(std::make_integer_sequence<int, P - 1>{});
  // drain the (redundant) tail DMA before the LDS is released
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
  epilogue<Epi, TJ, (Ablate & 8) != 0>(acc, C, bias, rowsum, M, N, m0, wm, wn, n0 + wn * (32 * TJ), lm, lh,
                                       reinterpret_cast<float *>(lds_ring<10, A_BYTES_S>));
  if (kMeasureBuild && probe && tid == 0) {
    probe[2 * blockIdx.x] = static_cast<unsigned long long>(clock64() - probe_c0);
    probe[2 * blockIdx.x + 1] = static_cast<unsigned long long>(wall_clock64() - probe_t0);
  }
}

#endif  // SAREK_HIP_MEASURE

// ---- direct-to-LDS kernel on v_mfma_f32_16x16x32 ---------------------------------------
// The same tile, rings and transfers as gemm16_dma_kernel<.., 64, 32, 2, 4, 2> (256 x 256 per workgroup, 8 waves
// of 128 x 64, A in 2 stages of K = 64, B in 4 slabs of K = 32, one barrier per B slab), but the products go
// through the 16 x 16 x 32 instruction: 8 x 4 accumulator tiles of 16 x 16 per wave instead of 4 x 2 of 32 x 32.
// On N(0, 0.02) data under the package power limit a bare stream of the 16 x 16 x 32 instruction runs 17 % faster
// than one of the 32 x 32 x 16 instruction (2.09 against 1.79 PFLOP/s; on zeros both reach 2.45): it writes half as
// many accumulator values per flop.  The LDS bytes read per flop are the same (the wave tile is).
//
// Operands: lane (m = lane%16, g = lane/16) supplies k = 8g..8g+7 of row m (A) / column m (B) and receives
// rows 4g..4g+3 of column m of the 16 x 16 result.
//   A: one ds_read_b128 per 16-row tile: chunk 4*ks + g of the row (ks = the B slab's place in the A stage).
//   B: two ds_read_b64_tr_b16 per 16-column tile: rows 8g + {0..3} and 8g + {4..7} of the slab, 16 columns.
//      A 32-lane phase of that read holds two k groups (rows r and r + 8): the B swizzle of the 32 x 32 kernel
//      (slot ^= (row & 3) << 2, rows 64 bytes apart) is extended by slot ^= ((row >> 3) & 1) << 1, which puts
//      the second group on the other 32-byte half of each 64-byte piece.
// A slab is worked in two units of 16 MFMAs (rows 0-63 of the wave tile, then rows 64-127, same B fragments);
// the barrier sits between them, and the second unit covers the fragment reads of the next slab.
template <bool Bf16>
__device__ __forceinline__ f32x4_t mfma16(u32x4 a, u32x4 b, f32x4_t c) {
  if constexpr (Bf16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                   0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                  0, 0);
}

// Writes one wave's (16*TI) x 64 block held as TI x 4 tiles of 16 x 16 (register r of lane l: row 4*(l/16) + r, column
// l%16 of its tile); TI = 8 in the 256 x 256 workgroup tile (2 x 4 waves), 4 in the 128 x 128 one (2 x 2 waves).
// Fused form as in `epilogue`: per lane the sum over its four columns for each of its 4*TI rows, a halving butterfly
// over the 16 lanes that share those rows (with TI = 8: 16+8+4+2 exchanges leave lane m with rows 2m, 2m+1 of the 32;
// with TI = 4: 8+4+2+1 leave it with row m of the 16), the WNW waves along N through LDS.  The tile's sum of row r then
// goes to rs_plane[r] when the launch has planes (one per tile column, added up in tile order by
// rowsum_fold_kernel: the same bits on every run), else to rowsum[r] by atomicAdd.
template <int Epi, int TI = 8, int WNW = 4>
__device__ __forceinline__ void epilogue16(f32x4_t (&acc)[TI][4], float *__restrict__ C, const float *__restrict__ bias,
                                           float *__restrict__ rowsum, float *__restrict__ rs_plane, int M, int N, int ld,
                                           int m0, int wm, int wn, int col0, int l16, int g, float *scratch) {
  constexpr int WROWS = 16 * TI, TROWS = 2 * WROWS, NV = 4 * TI, E = NV / 16;
  static_assert(TI == 8 || TI == 4, "wave tiles of 128 or 64 rows");
  static_assert(WNW == 4 || WNW == 2, "four or two waves along N");
  const int row0 = m0 + wm * WROWS;
  float bj[4];
  bool cok[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int col = col0 + j * 16 + l16;
    cok[j] = col < N;
    bj[j] = (Epi == EPI_BIAS_RELU_ROWSUM && cok[j]) ? bias[col] : 0.f;
  }
  float rs[NV];
#pragma unroll
  for (int i = 0; i < TI; ++i) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = row0 + i * 16 + 4 * g + r;
      float sum = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float v = acc[i][j][r];
        if (Epi == EPI_BIAS_RELU_ROWSUM) {
          v += bj[j];
          v = v > 0.f ? v : 0.f;
          sum += cok[j] ? v : 0.f;
        }
        if (row < M && cok[j]) C[static_cast<int64_t>(row) * ld + col0 + j * 16 + l16] = v;
      }
      rs[i * 4 + r] = sum;
    }
  }
  if constexpr (Epi == EPI_BIAS_RELU_ROWSUM) {
#pragma unroll
    for (int step = 0; step < 4; ++step) {
      const int m = 8 >> step, half = (NV / 2) >> step;
      const bool up = (l16 & m) != 0;
#pragma unroll
      for (int q = 0; q < half; ++q) {
        // both values in registers before the selects: otherwise the compiler turns the selects into one
        // lane-indexed read of rs[] (a compare-and-select chain over all its registers per value)
        float lo = rs[q], hi = rs[q + half];
        asm volatile("" : "+v"(lo), "+v"(hi));
        const float send = up ? lo : hi;
        const float keep = up ? hi : lo;
        rs[q] = keep + __shfl_xor(send, m, 64);
      }
    }
    // lane l16 now holds rows q = E*l16 + e (e < E) of its 16-lane group's 4*TI rows: tile q/4, register q%4
    __syncthreads();  // every wave has left the K loop: the LDS ring is free
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int q = E * l16 + e;
      scratch[wn * TROWS + wm * WROWS + (q >> 2) * 16 + 4 * g + (q & 3)] = rs[e];
    }
    __syncthreads();
    const int t = threadIdx.x;
    if (t < TROWS && m0 + t < M) {
      float total;
      if constexpr (WNW == 4) total = (scratch[t] + scratch[TROWS + t]) + (scratch[2 * TROWS + t] + scratch[3 * TROWS + t]);
      else total = scratch[t] + scratch[TROWS + t];
      if (rs_plane) rs_plane[m0 + t] = total;
      else atomicAdd(rowsum + m0 + t, total);
    }
  }
}

template <bool Bf16, int Epi, int Ablate = 0, bool Ragged = false, bool HalfBarriers = false>
__global__ __launch_bounds__(512) void gemm16_m16_kernel(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
                                                         float *__restrict__ C, const float *__restrict__ bias,
                                                         float *__restrict__ rowsum, int M, int N, int K, int tiles_m,
                                                         int tiles_n, int xcd_remap, unsigned long long *probe, int ld,
                                                         float *__restrict__ rs_planes) {
  // HalfBarriers: one barrier per A stage (K = 64) instead of one per B slab (K = 32).  A transfer may then only
  // overwrite the slab before the previous one (the waves are a whole stage apart at most), so the top of slab j
  // issues B(j - 2 + NB) and the ring is two slabs deeper, 160 KiB of LDS in all.
  constexpr int BKA = 64, BKB = 32, NA = 2, NB = HalfBarriers ? 6 : 4;
  constexpr int BEHIND = HalfBarriers ? 2 : 1;   // the slab whose stage the top of a slab refills lies this far back
  constexpr int RA = BKA / BKB;                  // B slabs per A stage
  static_assert(!HalfBarriers || RA == 2, "the barrier sits in the second slab of an A stage");
  constexpr int A_ROW = BKA * 2, A_CHUNKS = A_ROW / 16, A_ROWS_PER_DMA = 1024 / A_ROW;
  constexpr int A_BYTES_S = BM * A_ROW, B_BYTES_S = BKB * BN * 2;
  constexpr int NWAVES = 8, WN = 4;
  constexpr int DA = A_BYTES_S / 1024 / NWAVES, DB = B_BYTES_S / 1024 / NWAVES;
  constexpr int P = lcm_int(NB, RA * NA);
  static_assert(P % 2 == 0, "the B fragment buffers alternate by slab parity");
  static_assert((NB - 1) * DB + NA * DA < 64, "vmcnt range");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int l16 = lane & 15, g = lane >> 4;
  int tm, tn;
  tile_of_block(tiles_m, tiles_n, xcd_remap, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  long long probe_c0 = 0, probe_t0 = 0;
  if (kMeasureBuild && probe) {
    probe_c0 = clock64();
    probe_t0 = wall_clock64();
  }
  auto a_swz = [](int row) { return (row >> 1) & 7; };
  auto b_swz = [](int row) { return ((row & 3) << 2) | (((row >> 3) & 1) << 1); };

  // DMA sources (rows past M clamped: what they bring is never stored)
  uint32_t a_off[DA], b_off[DB];
#pragma unroll
  for (int i = 0; i < DA; ++i) {
    const int q = wave + NWAVES * i;
    const int arow_t = q * A_ROWS_PER_DMA + lane / A_CHUNKS;
    const int arow = min(arow_t, M - 1 - m0);
    a_off[i] = (static_cast<uint32_t>(arow) * K + (((lane % A_CHUNKS) ^ a_swz(arow_t)) << 3)) * 2u;
  }
#pragma unroll
  for (int i = 0; i < DB; ++i) {
    const int q = wave + NWAVES * i;
    const int brow = 2 * q + (lane >> 5);
    const int bchunk = (lane & 31) ^ b_swz(brow);
    // Ragged: columns past N are fetched as they lie (the next row's, or zeros past the end of B: the range of the
    // buffer resource is exact) and never stored, and rows need no 16-byte alignment (ld may be odd); otherwise
    // (N % 8 == 0) the pieces past N are clamped onto the last one
    const int bcol = Ragged ? n0 + bchunk * 8 : min(n0 + bchunk * 8, N - 8);
    b_off[i] = (static_cast<uint32_t>(brow) * ld + bcol) * 2u;
  }
  const char *a_base = reinterpret_cast<const char *>(A + static_cast<int64_t>(m0) * K);
  const char *b_base = reinterpret_cast<const char *>(B);
  const int64_t b_slab_bytes = static_cast<int64_t>(BKB) * ld * 2;
  // Ragged: K need not fill the last A stage.  A lane whose offset lies outside the buffer resource's range brings
  // zeros into LDS, so k that must not count are a per-lane choice between the usual offset and one past the range.
  // From one whole stage on (K >= 64) the last stage is moved back to end at K: its A pieces then hold nothing but
  // elements of their own rows, at whatever alignment, and the B rows it shares with the stage before it are the
  // lanes sent out of range, in the first of its two slabs and, past 32 shared rows, in the second.  Below one stage
  // (K % 8 == 0) the A pieces and B rows past K are.  A lane's k piece is the same for all its transfers of a stage
  // (rows 16 apart share the swizzle).
  const int nstages = (K + BKA - 1) / BKA;
  const bool move_last = Ragged && K >= BKA && K % BKA != 0;
  const int nslabs = move_last ? RA * nstages : (K + BKB - 1) / BKB;
  const int k_tail_a = K - (nstages - 1) * BKA, k_tail_b = K - (nslabs - 1) * BKB;   // single stage
  const int shared_k = nstages * BKA - K;                                               // moved stage
  const bool a_lane_in_k = !Ragged || move_last ||
                           (((lane % A_CHUNKS) ^ a_swz(wave * A_ROWS_PER_DMA + lane / A_CHUNKS)) << 3) < k_tail_a;
  bool b_in_last[DB], b_in_prev[DB];   // the lanes that count in the last slab and in the one before it
#pragma unroll
  for (int i = 0; i < DB; ++i) {
    const int brow = 2 * (wave + NWAVES * i) + (lane >> 5);
    b_in_last[i] = !Ragged || (move_last ? brow + BKB >= shared_k : brow < k_tail_b);
    b_in_prev[i] = !move_last || brow >= shared_k;
  }
  const char *b_end = b_base + (static_cast<int64_t>(K - 1) * ld + N) * 2;   // the end of row K-1's N columns
  constexpr uint32_t kOutOfRange = 0x80000000u;

  f32x4_t acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

  // fragment read offsets.  A: row wm*128 + 16*i + l16, slot (4*ks + g) ^ swz = ((g ^ swz) ^ 4*ks): one base,
  // XOR (ks << 6), + i * 2 KiB (16 rows leave the swizzle unchanged).  B: row 8g + li/4 (+4), the 8 bytes at
  // column offset 4*(li%4) of the 16-column tile; tile j is an XOR with j << 5 (32 bytes).
  const int a_row = wm * 128 + l16;
  int a_addr0 = a_row * A_ROW + ((g ^ a_swz(a_row)) << 4);
  const int b_r = l16 >> 2;
  int b_addr0 = (g * 8 + b_r) * 512 + ((wn * 128 + (l16 & 3) * 8) ^ ((b_r << 6) | ((g & 1) << 5)));

  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(a_base, 0x80000000u);
  auto issue_a = [&](char *sa, int stage) {
    if (stage >= NA && (Ablate & 1)) return;
    const bool whole = stage < nstages - 1;
    const uint32_t a_so = static_cast<uint32_t>(!whole && move_last ? K - BKA : min(stage, nstages - 1) * BKA) * 2u;
#pragma unroll
    for (int i = 0; i < DA; ++i)
      dma16(a_rsrc, (!Ragged || whole || a_lane_in_k) ? a_off[i] : kOutOfRange, a_so, sa + (wave + NWAVES * i) * 1024);
  };
  // B slabs are issued in order 0, 1, 2, ...: the source of the next one is a running pointer (two scalar adds per
  // slab instead of a 64-bit multiply) that stops at the last slab, which the tail of the K loop re-issues into
  // stages nobody reads any more so that the count of outstanding transfers follows the same pattern throughout
  const char *b_src = b_base;
  int b_next = 0;
  auto issue_b = [&](char *sb, int slab) {
    if (slab >= NB && (Ablate & 1)) return;
    (void)slab;   // == b_next
    const bool last = b_next >= nslabs - 1, prev = b_next == nslabs - 2;
    if (move_last && prev) b_src = b_base + static_cast<int64_t>(K - BKA) * ld * 2;
    const int64_t b_left = b_end - b_src;
    const __amdgpu_buffer_rsrc_t b_rsrc =
        make_rsrc(b_src, Ragged && b_left < 0x80000000ll ? static_cast<uint32_t>(b_left) : kOutOfRange);
#pragma unroll
    for (int i = 0; i < DB; ++i)
      dma16(b_rsrc, (!Ragged || (last ? b_in_last[i] : prev ? b_in_prev[i] : true)) ? b_off[i] : kOutOfRange, 0u,
            sb + (wave + NWAVES * i) * 1024);
    ++b_next;
    if (b_next < nslabs) b_src += b_slab_bytes;
  };
  // half: rows 0-63 (0) or 64-127 (1) of the wave tile
  bool frags_loaded = false;
  auto load_a = [&](const char *sa, int ks, int half, u32x4 (&af)[4]) {
    if ((Ablate & 2) && frags_loaded) return;
    const char *pa = sa + (a_addr0 ^ (ks << 6)) + half * (64 * A_ROW);
#pragma unroll
    for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const u32x4 *>(pa + i * 16 * A_ROW);
  };
  auto load_b = [&](const char *sb, u32x4 (&bf)[4]) {
    if ((Ablate & 2) && frags_loaded) return;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int off = b_addr0 ^ (j << 5);
      u32x2 lo = lds_read_tr16(sb, off);
      u32x2 hi = lds_read_tr16(sb, off + 4 * 512);
      bf[j] = u32x4{lo.x, lo.y, hi.x, hi.y};
    }
  };
  // MFMAs First .. First+Count-1 of a slab's 32, in the order (row tile i, column tile j); row tiles 0-3 take their
  // A fragments from af[0], 4-7 from af[1]
  auto mfma_range = [&](auto first_c, auto count_c, u32x4 (&af)[2][4], u32x4 (&bf)[4]) {
    constexpr int First = decltype(first_c)::value, Count = decltype(count_c)::value;
    [&]<int... Ts>(std::integer_sequence<int, Ts...>) {
      ((acc[(First + Ts) / 4][(First + Ts) % 4] = mfma16<Bf16>(af[(First + Ts) / 16][((First + Ts) / 4) % 4],
                                                              bf[(First + Ts) % 4],
                                                              acc[(First + Ts) / 4][(First + Ts) % 4])),
       ...);
    }(std::make_integer_sequence<int, Count>{});
  };
  // Issue order: the T = NV + READS other instructions (DMA, LDS reads) go one each behind MFMAs spread evenly over
  // the MFMAS of the section, the DMA instructions evenly among the reads.  (A 16 x 16 x 32 MFMA occupies the pipe for
  // 16 cycles: two reads and a DMA instruction behind one MFMA, the 32 x 32 kernel's pattern, do not fit in its shadow
  // and cost 8 % of the cycle count.)
  auto spread = [](auto nv_c, auto reads_c, auto mfmas_c) {
    constexpr int NV = decltype(nv_c)::value, READS = decltype(reads_c)::value, MFMAS = decltype(mfmas_c)::value;
    constexpr int T = NV + READS;
    static_assert(T <= MFMAS, "one instruction per MFMA at most");
    [&]<int... Ms>(std::integer_sequence<int, Ms...>) {
      (([] {
         __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
         // item k sits behind MFMA (k * MFMAS) / T
         constexpr int k = (Ms * T + MFMAS - 1) / MFMAS;          // first item at or after this MFMA
         if constexpr (k < T && (k * MFMAS) / T == Ms) {
           if constexpr (NV > 0 && (k * NV) / T != ((k + 1) * NV) / T) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
           else __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
         }
       }()),
       ...);
    }(std::make_integer_sequence<int, MFMAS>{});
    __builtin_amdgcn_sched_barrier(0);
  };
  auto load_a1 = [&](const char *sa, int ks, int half, int i, u32x4 &af) {
    if ((Ablate & 2) && frags_loaded) return;
    af = *reinterpret_cast<const u32x4 *>(sa + (a_addr0 ^ (ks << 6)) + half * (64 * A_ROW) + i * 16 * A_ROW);
  };
  u32x4 af[2][4], bf[2][4];   // af: [half], bf: [slab parity]

  auto slab = [&](auto ic, int s) {
    constexpr int I = decltype(ic)::value;
    constexpr int In = (I + 1) % P;
    constexpr int ia = (I / RA) % NA, ib = I % NB, ibp = (I + NB - BEHIND) % NB;
    constexpr int ian = (In / RA) % NA, ibn = In % NB;
    constexpr int ks = I % RA, ksn = In % RA;
    (void)ib;
    asm volatile("" : "+v"(a_addr0), "+v"(b_addr0));
    issue_b(lds_ring<20 + ibp, B_BYTES_S>, s - BEHIND + NB);
    load_a(lds_ring<10 + ia, A_BYTES_S>, ks, 1, af[1]);
    mfma_range(std::integral_constant<int, 0>{}, std::integral_constant<int, 16>{}, af, bf[I & 1]);
    spread(std::integral_constant<int, DB>{}, std::integral_constant<int, 4>{}, std::integral_constant<int, 16>{});
    if constexpr (!HalfBarriers || I % RA == RA - 1) {
      __builtin_amdgcn_s_waitcnt(
          waitcnt_vm_lgkm0(dma_allowed_in_flight(I, RA, NA, NB, DA, DB, HalfBarriers ? 2 : 1)));
      barrier_no_fence();
    }
    if constexpr (I % RA == RA - 1) issue_a(lds_ring<10 + ia, A_BYTES_S>, s / RA + NA);
    // the next slab's fragments in the order its first MFMAs need them: A tile 0, the four B tiles, A tiles 1-3.
    // (The barrier was also tried after 8 and after 12 MFMAs, with the low-half A registers reloaded behind their
    // last readers: 1 % slower.)
    load_a1(lds_ring<10 + ian, A_BYTES_S>, ksn, 0, 0, af[0][0]);
    load_b(lds_ring<20 + ibn, B_BYTES_S>, bf[In & 1]);
    load_a1(lds_ring<10 + ian, A_BYTES_S>, ksn, 0, 1, af[0][1]);
    load_a1(lds_ring<10 + ian, A_BYTES_S>, ksn, 0, 2, af[0][2]);
    load_a1(lds_ring<10 + ian, A_BYTES_S>, ksn, 0, 3, af[0][3]);
    mfma_range(std::integral_constant<int, 16>{}, std::integral_constant<int, 16>{}, af, bf[I & 1]);
    spread(std::integral_constant<int, (I % RA == RA - 1) ? DA : 0>{}, std::integral_constant<int, 12>{},
           std::integral_constant<int, 16>{});
  };

  [&]<int... Is>(std::integer_sequence<int, Is...>) {
    (issue_a(lds_ring<10 + Is, A_BYTES_S>, Is), ...);
  }(std::make_integer_sequence<int, NA>{});
  [&]<int... Is>(std::integer_sequence<int, Is...>) {
    (issue_b(lds_ring<20 + Is, B_BYTES_S>, Is), ...);
  }(std::make_integer_sequence<int, NB - BEHIND>{});
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
  barrier_no_fence();
  load_a(lds_ring<10, A_BYTES_S>, 0, 0, af[0]);
  load_b(lds_ring<20, B_BYTES_S>, bf[0]);
  if (Ablate & 2) {
    load_a(lds_ring<10, A_BYTES_S>, 0, 1, af[1]);
    load_b(lds_ring<20, B_BYTES_S>, bf[1]);
    frags_loaded = true;
  }
  __builtin_amdgcn_sched_barrier(0);

  const int full = nslabs - nslabs % P;
  for (int s = 0; s < full; s += P) {
    [&]<int... Is>(std::integer_sequence<int, Is...>) {
      (slab(std::integral_constant<int, Is>{}, s + Is), ...);
    }(std::make_integer_sequence<int, P>{});
  }
  [&]<int... Is>(std::integer_sequence<int, Is...>) {
    ((full + Is < nslabs ? slab(std::integral_constant<int, Is>{}, full + Is) : (void)0), ...);
  }(std::make_integer_sequence<int, P - 1>{});
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));   // drain the (redundant) tail DMA before the LDS is released
  epilogue16<Epi>(acc, C, bias, rowsum, rs_planes ? rs_planes + static_cast<int64_t>(tn) * M : nullptr, M, N, ld, m0, wm, wn,
                  n0 + wn * 64, l16, g, reinterpret_cast<float *>(lds_ring<10, A_BYTES_S>));
  if (kMeasureBuild && probe && tid == 0) {
    probe[2 * blockIdx.x] = static_cast<unsigned long long>(clock64() - probe_c0);
    probe[2 * blockIdx.x + 1] = static_cast<unsigned long long>(wall_clock64() - probe_t0);
  }
}

#ifdef SAREK_HIP_MEASURE
// The 256 x 256 tile with 4 waves (2 x 2) of 128 x 128 = 8 x 8 MFMA tiles, one wave per SIMD with its 256 accumulator
// registers in the AGPR half of the register file: the same rings, transfers and LDS layout as gemm16_m16_kernel, two
// thirds of its LDS fragment bytes (a wave reads 128 rows of A and 128 columns of B per k where two waves of 128 x 64
// read 256 and 128).  Left to the compiler, the 64 accumulator tiles do not stay in place (the MFMA builtin came out
// with different source and destination registers and two AGPR <-> VGPR copies per MFMA), so the MFMAs are written
// as asm with the accumulator tied to itself, and with them the issue order: memory instructions do not move across a
// volatile asm, so each LDS read and each transfer sits behind the MFMA it is written after.  A slab is 64 MFMAs per
// wave: row tiles 0-3 before the barrier with the slab's last four A fragments and its 4 B transfers behind every
// fourth MFMA, row tiles 4-7 after it with the next slab's 20 fragment reads (and, every other slab, the 8 transfers of
// an A stage) one behind each MFMA.  Aligned shapes, plain store.  Measurement build only (tunable gemm16.waves = 4):
// with every instruction where it was meant to be it takes 0.766 ms for the bf16 8192^3 product where the 8-wave kernel
// takes 0.744 in the same run -- a higher clock (1.68 against 1.59 GHz), fewer of its cycles used: with one wave per SIMD
// nothing fills the pipe while that wave waits at the slab's barrier.
template <bool Bf16>
__device__ __forceinline__ void mfma16_in_place(u32x4 a, u32x4 b, f32x4_t &c) {
  if constexpr (Bf16) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

template <bool Bf16>
__global__ __launch_bounds__(256) void gemm16_m16w4_kernel(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
                                                           float *__restrict__ C, int M, int N, int K, int tiles_m,
                                                           int tiles_n, int xcd_remap, int ld) {
  constexpr int BKA = 64, BKB = 32, NA = 2, NB = 4;
  constexpr int RA = BKA / BKB;
  constexpr int A_ROW = BKA * 2, A_CHUNKS = A_ROW / 16, A_ROWS_PER_DMA = 1024 / A_ROW;
  constexpr int A_BYTES_S = BM * A_ROW, B_BYTES_S = BKB * BN * 2;
  constexpr int NWAVES = 4, WN = 2;
  constexpr int DA = A_BYTES_S / 1024 / NWAVES, DB = B_BYTES_S / 1024 / NWAVES;   // 8, 4
  constexpr int P = lcm_int(NB, RA * NA);
  static_assert(P % 2 == 0 && DA == 8 && DB == 4, "the issue tables below are written for these counts");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int l16 = lane & 15, g = lane >> 4;
  int tm, tn;
  tile_of_block(tiles_m, tiles_n, xcd_remap, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  auto a_swz = [](int row) { return (row >> 1) & 7; };
  auto b_swz = [](int row) { return ((row & 3) << 2) | (((row >> 3) & 1) << 1); };

  uint32_t a_off[DA], b_off[DB];
#pragma unroll
  for (int i = 0; i < DA; ++i) {
    const int q = wave + NWAVES * i;
    const int arow_t = q * A_ROWS_PER_DMA + lane / A_CHUNKS;
    const int arow = min(arow_t, M - 1 - m0);
    a_off[i] = (static_cast<uint32_t>(arow) * K + (((lane % A_CHUNKS) ^ a_swz(arow_t)) << 3)) * 2u;
  }
#pragma unroll
  for (int i = 0; i < DB; ++i) {
    const int q = wave + NWAVES * i;
    const int brow = 2 * q + (lane >> 5);
    const int bchunk = (lane & 31) ^ b_swz(brow);
    b_off[i] = (static_cast<uint32_t>(brow) * ld + min(n0 + bchunk * 8, N - 8)) * 2u;
  }
  const char *a_base = reinterpret_cast<const char *>(A + static_cast<int64_t>(m0) * K);
  const int64_t b_slab_bytes = static_cast<int64_t>(BKB) * ld * 2;
  const int nstages = K / BKA, nslabs = K / BKB;

  f32x4_t acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

  const int a_row = wm * 128 + l16;
  int a_addr0 = a_row * A_ROW + ((g ^ a_swz(a_row)) << 4);
  const int b_r = l16 >> 2;
  int b_addr0 = (g * 8 + b_r) * 512 + ((wn * 256 + (l16 & 3) * 8) ^ ((b_r << 6) | ((g & 1) << 5)));

  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(a_base, 0x80000000u);
  // transfer i of A stage `stage` / of the next B slab (the tail of the K loop re-issues the last ones into stages
  // nobody reads any more, so the count of transfers in flight keeps its pattern)
  auto dma_a = [&](char *sa, int stage, int i) __attribute__((always_inline)) {
    dma16(a_rsrc, a_off[i], static_cast<uint32_t>(min(stage, nstages - 1) * BKA) * 2u, sa + (wave + NWAVES * i) * 1024);
  };
  const char *b_src = reinterpret_cast<const char *>(B);
  int b_next = 0;
  auto dma_b = [&](char *sb, int i) __attribute__((always_inline)) {
    dma16(make_rsrc(b_src, 0x80000000u), b_off[i], 0u, sb + (wave + NWAVES * i) * 1024);
  };
  auto b_advance = [&]() __attribute__((always_inline)) {
    ++b_next;
    if (b_next < nslabs) b_src += b_slab_bytes;
  };
  auto read_a = [&](const char *sa, int ks, int half, int i, u32x4 &af) __attribute__((always_inline)) {
    af = *reinterpret_cast<const u32x4 *>(sa + (a_addr0 ^ (ks << 6)) + half * (64 * A_ROW) + i * 16 * A_ROW);
  };
  // half h (0: rows 8g+0..3, 1: rows 8g+4..7) of column tile j
  auto read_b = [&](const char *sb, int j, int h, u32x2 &out) __attribute__((always_inline)) { out = lds_read_tr16(sb, (b_addr0 ^ (j << 5)) + h * 4 * 512); };

  u32x4 af[2][4];    // [half of the wave tile's rows]
  u32x2 bh[2][8][2]; // [slab parity][column tile][k half]
  auto bfrag = [&](int par, int j) __attribute__((always_inline)) { return u32x4{bh[par][j][0].x, bh[par][j][0].y, bh[par][j][1].x, bh[par][j][1].y}; };

  auto slab = [&](auto ic, int s) __attribute__((always_inline)) {
    constexpr int I = decltype(ic)::value;
    constexpr int In = (I + 1) % P;
    constexpr int ia = (I / RA) % NA, ibp = (I + NB - 1) % NB;
    constexpr int ian = (In / RA) % NA, ibn = In % NB;
    constexpr int ks = I % RA, ksn = In % RA;
    constexpr bool refill_a = I % RA == RA - 1;
    asm volatile("" : "+v"(a_addr0), "+v"(b_addr0));
    // rows 0-63: MFMA t = 8 i + j; behind every fourth one of the slab's last four A fragments or one of the four
    // transfers of B slab s - 1 + NB
    [&]<int... Ts>(std::integer_sequence<int, Ts...>) {
      (([&]() __attribute__((always_inline)) {
         mfma16_in_place<Bf16>(af[0][Ts / 8], bfrag(I & 1, Ts % 8), acc[Ts / 8][Ts % 8]);
         if constexpr (Ts % 8 == 0) read_a(lds_ring<10 + ia, A_BYTES_S>, ks, 1, Ts / 8, af[1][Ts / 8]);
         if constexpr (Ts % 8 == 4) dma_b(lds_ring<20 + ibp, B_BYTES_S>, Ts / 8);
       }()),
       ...);
    }(std::make_integer_sequence<int, 32>{});
    b_advance();
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(dma_allowed_in_flight(I, RA, NA, NB, DA, DB)));
    barrier_no_fence();
    // rows 64-127, and behind them the next slab's fragments in the order its first MFMAs need them (A tile 0, the
    // eight B tiles, A tiles 1-3: 20 reads) and, after the last slab of an A stage, the 8 transfers that refill it
    [&]<int... Ts>(std::integer_sequence<int, Ts...>) {
      (([&]() __attribute__((always_inline)) {
         mfma16_in_place<Bf16>(af[1][Ts / 8], bfrag(I & 1, Ts % 8), acc[4 + Ts / 8][Ts % 8]);
         if constexpr (Ts == 0) read_a(lds_ring<10 + ian, A_BYTES_S>, ksn, 0, 0, af[0][0]);
         else if constexpr (Ts <= 16) read_b(lds_ring<20 + ibn, B_BYTES_S>, (Ts - 1) / 2, (Ts - 1) % 2, bh[In & 1][(Ts - 1) / 2][(Ts - 1) % 2]);
         else if constexpr (Ts <= 19) read_a(lds_ring<10 + ian, A_BYTES_S>, ksn, 0, Ts - 16, af[0][Ts - 16]);
         if constexpr (refill_a && Ts >= 20 && Ts < 28) dma_a(lds_ring<10 + ia, A_BYTES_S>, s / RA + NA, Ts - 20);
       }()),
       ...);
    }(std::make_integer_sequence<int, 32>{});
  };

  // prologue: fill both rings except the last B stage (the top of slab 0 issues it) and wait for all of it
  [&]<int... Is>(std::integer_sequence<int, Is...>) {
    (([&] {
       _Pragma("unroll") for (int i = 0; i < DA; ++i) dma_a(lds_ring<10 + Is, A_BYTES_S>, Is, i);
     }()),
     ...);
  }(std::make_integer_sequence<int, NA>{});
  [&]<int... Is>(std::integer_sequence<int, Is...>) {
    (([&] {
       _Pragma("unroll") for (int i = 0; i < DB; ++i) dma_b(lds_ring<20 + Is, B_BYTES_S>, i);
       b_advance();
     }()),
     ...);
  }(std::make_integer_sequence<int, NB - 1>{});
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
  barrier_no_fence();
#pragma unroll
  for (int i = 0; i < 4; ++i) read_a(lds_ring<10, A_BYTES_S>, 0, 0, i, af[0][i]);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    read_b(lds_ring<20, B_BYTES_S>, j, 0, bh[0][j][0]);
    read_b(lds_ring<20, B_BYTES_S>, j, 1, bh[0][j][1]);
  }
  __builtin_amdgcn_sched_barrier(0);

  const int full = nslabs - nslabs % P;
  for (int s = 0; s < full; s += P) {
    [&]<int... Is>(std::integer_sequence<int, Is...>) {
      (slab(std::integral_constant<int, Is>{}, s + Is), ...);
    }(std::make_integer_sequence<int, P>{});
  }
  [&]<int... Is>(std::integer_sequence<int, Is...>) {
    ((full + Is < nslabs ? slab(std::integral_constant<int, Is>{}, full + Is) : (void)0), ...);
  }(std::make_integer_sequence<int, P - 1>{});
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));   // drain the (redundant) tail DMA before the LDS is released
  // the compiler does not know that the asm above are matrix instructions whose results land some cycles after issue
  asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
  // register r of lane (l16, g) of tile (i, j): row 16 i + 4 g + r, column 16 j + l16 of the wave's 128 x 128
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = m0 + wm * 128 + i * 16 + 4 * g + r;
      if (row >= M) continue;
      float *crow = C + static_cast<int64_t>(row) * ld + n0 + wn * 128 + l16;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (n0 + wn * 128 + j * 16 + l16 < N) crow[j * 16] = acc[i][j][r];
    }
}

#endif  // SAREK_HIP_MEASURE

// The same pipeline on a 128 x 128 workgroup tile, for products whose 256 x 256 tiles would leave most CUs idle:
// 4 waves (2 x 2) of 64 x 64 = 4 x 4 tiles of v_mfma_f32_16x16x32, A in 3 stages of K = 64 and B in 4 slabs of K = 32
// (80 KiB of LDS: two workgroups per CU fill its 160 KiB).  A small tile needs twice the operand bytes per flop and has
// a quarter of the MFMA work per slab to cover their latency with, so the ring depth is what its speed hangs on: the
// third A stage (transfers 4 slabs ahead instead of 2) is worth 3-7 %, and two resident workgroups run at twice the
// rate of one.  B rows are 256 bytes here; they start on bank 0 like the 512-byte
// rows of the large tile, so the same XOR swizzle keeps the transposing reads free of bank conflicts.  A slab is 16 MFMAs:
// rows 0-31 of the wave tile before the barrier, rows 32-63 after it with the next slab's 12 fragment reads (and, every
// other slab, the 4 transfers of an A stage) behind them; fragments are double-buffered by slab parity.
template <bool Bf16, int Epi, bool Ragged = false>
__global__ __launch_bounds__(256) void gemm16_m16_small_kernel(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
                                                               float *__restrict__ C, const float *__restrict__ bias,
                                                               float *__restrict__ rowsum, int M, int N, int K, int tiles_m,
                                                               int tiles_n, int xcd_remap, unsigned long long *probe,
                                                               int k_chunk, float *__restrict__ partials, int ld,
                                                               float *__restrict__ rs_planes) {
  constexpr int SBM = 128, SBN = 128;
  constexpr int BKA = 64, BKB = 32, NA = 3, NB = 4;
  constexpr int RA = BKA / BKB;
  constexpr int A_ROW = BKA * 2, A_CHUNKS = A_ROW / 16, A_ROWS_PER_DMA = 1024 / A_ROW;
  constexpr int B_ROW = SBN * 2, B_CHUNKS = B_ROW / 16, B_ROWS_PER_DMA = 1024 / B_ROW;
  constexpr int A_BYTES_S = SBM * A_ROW, B_BYTES_S = BKB * B_ROW;
  constexpr int NWAVES = 4, WN = 2;
  constexpr int DA = A_BYTES_S / 1024 / NWAVES, DB = B_BYTES_S / 1024 / NWAVES;
  constexpr int P = lcm_int(NB, RA * NA);
  static_assert(P % 2 == 0, "the fragment buffers alternate by slab parity");
  static_assert(2 * (NA * A_BYTES_S + NB * B_BYTES_S) <= 160 * 1024, "two workgroups per CU");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int l16 = lane & 15, g = lane >> 4;
  int tm, tn;
  tile_of_block(tiles_m, tiles_n, xcd_remap, tm, tn);
  const int m0 = tm * SBM, n0 = tn * SBN;
  long long probe_c0 = 0, probe_t0 = 0;
  if (kMeasureBuild && probe) {
    probe_c0 = clock64();
    probe_t0 = wall_clock64();
  }
  auto a_swz = [](int row) { return (row >> 1) & 7; };
  auto b_swz = [](int row) { return ((row & 3) << 2) | (((row >> 3) & 1) << 1); };

  // DMA sources (rows past M and columns past N clamped: what they bring is never stored)
  uint32_t a_off[DA], b_off[DB];
#pragma unroll
  for (int i = 0; i < DA; ++i) {
    const int q = wave + NWAVES * i;
    const int arow_t = q * A_ROWS_PER_DMA + lane / A_CHUNKS;
    const int arow = min(arow_t, M - 1 - m0);
    a_off[i] = (static_cast<uint32_t>(arow) * K + (((lane % A_CHUNKS) ^ a_swz(arow_t)) << 3)) * 2u;
  }
#pragma unroll
  for (int i = 0; i < DB; ++i) {
    const int q = wave + NWAVES * i;
    const int brow = q * B_ROWS_PER_DMA + lane / B_CHUNKS;
    const int bchunk = (lane % B_CHUNKS) ^ b_swz(brow);
    // Ragged: columns past N are fetched as they lie (the next row's, or zeros past the end of B: the range of the
    // buffer resource is exact) and never stored, and rows need no 16-byte alignment (ld may be odd); otherwise
    // (N % 8 == 0) the pieces past N are clamped onto the last one
    const int bcol = Ragged ? n0 + bchunk * 8 : min(n0 + bchunk * 8, N - 8);
    b_off[i] = (static_cast<uint32_t>(brow) * ld + bcol) * 2u;
  }
  // K split over gridDim.y workgroups per tile (plain store only): this one takes k0 .. k0 + k_len - 1 and writes its
  // partial tile to its own M x N plane of `partials`, which a second kernel adds up in a fixed order
  const int k0 = blockIdx.y * k_chunk;
  const int k_len = min(k_chunk, K - k0);
  if (gridDim.y > 1) C = partials + static_cast<int64_t>(blockIdx.y) * M * ld;
  const char *a_base = reinterpret_cast<const char *>(A + static_cast<int64_t>(m0) * K + k0);
  const int64_t b_slab_bytes = static_cast<int64_t>(BKB) * ld * 2;
  // Ragged: K need not fill the last A stage.  A lane whose offset lies outside the buffer resource's range brings
  // zeros into LDS, so k that must not count are a per-lane choice between the usual offset and one past the range.
  // From one whole stage on (K >= 64) the last stage is moved back to end at K: its A pieces then hold nothing but
  // elements of their own rows, at whatever alignment, and the B rows it shares with the stage before it are the
  // lanes sent out of range, in the first of its two slabs and, past 32 shared rows, in the second.  Below one stage
  // (K % 8 == 0) the A pieces and B rows past K are.  A lane's k piece is the same for all its transfers of a stage
  // (rows 16 apart share the swizzle).
  const int nstages = (k_len + BKA - 1) / BKA;
  const bool move_last = Ragged && k_len >= BKA && k_len % BKA != 0;
  const int nslabs = move_last ? RA * nstages : (k_len + BKB - 1) / BKB;
  const int k_tail_a = k_len - (nstages - 1) * BKA, k_tail_b = k_len - (nslabs - 1) * BKB;   // single stage
  const int shared_k = nstages * BKA - k_len;                                               // moved stage
  const bool a_lane_in_k = !Ragged || move_last ||
                           (((lane % A_CHUNKS) ^ a_swz(wave * A_ROWS_PER_DMA + lane / A_CHUNKS)) << 3) < k_tail_a;
  bool b_in_last[DB], b_in_prev[DB];   // the lanes that count in the last slab and in the one before it
#pragma unroll
  for (int i = 0; i < DB; ++i) {
    const int brow = (wave + NWAVES * i) * B_ROWS_PER_DMA + lane / B_CHUNKS;
    b_in_last[i] = !Ragged || (move_last ? brow + BKB >= shared_k : brow < k_tail_b);
    b_in_prev[i] = !move_last || brow >= shared_k;
  }
  const char *b_end = reinterpret_cast<const char *>(B) + (static_cast<int64_t>(K - 1) * ld + N) * 2;
  constexpr uint32_t kOutOfRange = 0x80000000u;

  f32x4_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

  const int a_row = wm * 64 + l16;
  int a_addr0 = a_row * A_ROW + ((g ^ a_swz(a_row)) << 4);
  const int b_r = l16 >> 2;
  int b_addr0 = (g * 8 + b_r) * B_ROW + ((wn * 128 + (l16 & 3) * 8) ^ ((b_r << 6) | ((g & 1) << 5)));

  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(a_base, 0x80000000u);
  auto issue_a = [&](char *sa, int stage) {
    const bool whole = stage < nstages - 1;
    const uint32_t a_so = static_cast<uint32_t>(!whole && move_last ? k_len - BKA : min(stage, nstages - 1) * BKA) * 2u;
#pragma unroll
    for (int i = 0; i < DA; ++i)
      dma16(a_rsrc, (!Ragged || whole || a_lane_in_k) ? a_off[i] : kOutOfRange, a_so, sa + (wave + NWAVES * i) * 1024);
  };
  // B slabs go out in order; the source is a running pointer that stops at the last slab (the tail of the K loop
  // re-issues it into stages nobody reads any more, so the count of transfers in flight keeps its pattern)
  const char *b_src = reinterpret_cast<const char *>(B + static_cast<int64_t>(k0) * ld);
  int b_next = 0;
  auto issue_b = [&](char *sb) {
    const bool last = b_next >= nslabs - 1, prev = b_next == nslabs - 2;
    if (move_last && prev) b_src = reinterpret_cast<const char *>(B + static_cast<int64_t>(k0 + k_len - BKA) * ld);
    const int64_t b_left = b_end - b_src;
    const __amdgpu_buffer_rsrc_t b_rsrc =
        make_rsrc(b_src, Ragged && b_left < 0x80000000ll ? static_cast<uint32_t>(b_left) : kOutOfRange);
#pragma unroll
    for (int i = 0; i < DB; ++i)
      dma16(b_rsrc, (!Ragged || (last ? b_in_last[i] : prev ? b_in_prev[i] : true)) ? b_off[i] : kOutOfRange, 0u,
            sb + (wave + NWAVES * i) * 1024);
    ++b_next;
    if (b_next < nslabs) b_src += b_slab_bytes;
  };
  auto load_a1 = [&](const char *sa, int ks, int i, u32x4 &af) {
    af = *reinterpret_cast<const u32x4 *>(sa + (a_addr0 ^ (ks << 6)) + i * 16 * A_ROW);
  };
  auto load_b = [&](const char *sb, u32x4 (&bf)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int off = b_addr0 ^ (j << 5);
      u32x2 lo = lds_read_tr16(sb, off);
      u32x2 hi = lds_read_tr16(sb, off + 4 * B_ROW);
      bf[j] = u32x4{lo.x, lo.y, hi.x, hi.y};
    }
  };
  // MFMAs First .. First+Count-1 of a slab's 16, in the order (row tile i, column tile j)
  auto mfma_range = [&](auto first_c, auto count_c, u32x4 (&af)[4], u32x4 (&bf)[4]) {
    constexpr int First = decltype(first_c)::value, Count = decltype(count_c)::value;
    [&]<int... Ts>(std::integer_sequence<int, Ts...>) {
      ((acc[(First + Ts) / 4][(First + Ts) % 4] =
            mfma16<Bf16>(af[(First + Ts) / 4], bf[(First + Ts) % 4], acc[(First + Ts) / 4][(First + Ts) % 4])),
       ...);
    }(std::make_integer_sequence<int, Count>{});
  };
  // Issue order: the T = NV + READS other instructions (DMA, LDS reads) go behind the MFMAs of the section, item k behind
  // MFMA (k * MFMAS) / T (two per MFMA where T > MFMAS), the DMA instructions evenly among the reads
  auto spread = [](auto nv_c, auto reads_c, auto mfmas_c) {
    constexpr int NV = decltype(nv_c)::value, READS = decltype(reads_c)::value, MFMAS = decltype(mfmas_c)::value;
    constexpr int T = NV + READS;
    [&]<int... Ms>(std::integer_sequence<int, Ms...>) {
      (([] {
         __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
         constexpr int k0 = (Ms * T + MFMAS - 1) / MFMAS, k1 = ((Ms + 1) * T + MFMAS - 1) / MFMAS;
         [&]<int... Ks>(std::integer_sequence<int, Ks...>) {
           (([] {
              constexpr int k = k0 + Ks;
              if constexpr (NV > 0 && (k * NV) / T != ((k + 1) * NV) / T) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
              else __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }()),
            ...);
         }(std::make_integer_sequence<int, (k1 < T ? k1 : T) - (k0 < T ? k0 : T)>{});
       }()),
       ...);
    }(std::make_integer_sequence<int, MFMAS>{});
    __builtin_amdgcn_sched_barrier(0);
  };
  u32x4 af[2][4], bf[2][4];   // [slab parity]

  auto slab = [&](auto ic, int s) {
    constexpr int I = decltype(ic)::value;
    constexpr int In = (I + 1) % P;
    constexpr int ia = (I / RA) % NA, ibp = (I + NB - 1) % NB;
    constexpr int ian = (In / RA) % NA, ibn = In % NB;
    constexpr int ksn = In % RA;
    asm volatile("" : "+v"(a_addr0), "+v"(b_addr0));
    issue_b(lds_ring<40 + ibp, B_BYTES_S>);
    mfma_range(std::integral_constant<int, 0>{}, std::integral_constant<int, 8>{}, af[I & 1], bf[I & 1]);
    spread(std::integral_constant<int, DB>{}, std::integral_constant<int, 0>{}, std::integral_constant<int, 8>{});
    __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(dma_allowed_in_flight(I, RA, NA, NB, DA, DB)));
    barrier_no_fence();
    if constexpr (I % RA == RA - 1) issue_a(lds_ring<30 + ia, A_BYTES_S>, s / RA + NA);
    // the next slab's fragments in the order its first MFMAs need them
    load_a1(lds_ring<30 + ian, A_BYTES_S>, ksn, 0, af[In & 1][0]);
    load_b(lds_ring<40 + ibn, B_BYTES_S>, bf[In & 1]);
    load_a1(lds_ring<30 + ian, A_BYTES_S>, ksn, 1, af[In & 1][1]);
    load_a1(lds_ring<30 + ian, A_BYTES_S>, ksn, 2, af[In & 1][2]);
    load_a1(lds_ring<30 + ian, A_BYTES_S>, ksn, 3, af[In & 1][3]);
    mfma_range(std::integral_constant<int, 8>{}, std::integral_constant<int, 8>{}, af[I & 1], bf[I & 1]);
    spread(std::integral_constant<int, (I % RA == RA - 1) ? DA : 0>{}, std::integral_constant<int, 12>{},
           std::integral_constant<int, 8>{});
  };

  // prologue: fill both rings except the last B stage (the top of slab 0 issues it) and wait for all of it
  [&]<int... Is>(std::integer_sequence<int, Is...>) {
    (issue_a(lds_ring<30 + Is, A_BYTES_S>, Is), ...);
  }(std::make_integer_sequence<int, NA>{});
  [&]<int... Is>(std::integer_sequence<int, Is...>) {
    (issue_b(lds_ring<40 + Is, B_BYTES_S>), ...);
  }(std::make_integer_sequence<int, NB - 1>{});
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));
  barrier_no_fence();
#pragma unroll
  for (int i = 0; i < 4; ++i) load_a1(lds_ring<30, A_BYTES_S>, 0, i, af[0][i]);
  load_b(lds_ring<40, B_BYTES_S>, bf[0]);
  __builtin_amdgcn_sched_barrier(0);

  const int full = nslabs - nslabs % P;
  for (int s = 0; s < full; s += P) {
    [&]<int... Is>(std::integer_sequence<int, Is...>) {
      (slab(std::integral_constant<int, Is>{}, s + Is), ...);
    }(std::make_integer_sequence<int, P>{});
  }
  [&]<int... Is>(std::integer_sequence<int, Is...>) {
    ((full + Is < nslabs ? slab(std::integral_constant<int, Is>{}, full + Is) : (void)0), ...);
  }(std::make_integer_sequence<int, P - 1>{});
  __builtin_amdgcn_s_waitcnt(waitcnt_vm_lgkm0(0));   // drain the (redundant) tail DMA before the LDS is released
  epilogue16<Epi, 4, WN>(acc, C, bias, rowsum, rs_planes ? rs_planes + static_cast<int64_t>(tn) * M : nullptr, M, N, ld, m0,
                         wm, wn, n0 + wn * 64, l16, g, reinterpret_cast<float *>(lds_ring<30, A_BYTES_S>));
  if (kMeasureBuild && probe && tid == 0) {
    probe[2 * blockIdx.x] = static_cast<unsigned long long>(clock64() - probe_c0);
    probe[2 * blockIdx.x + 1] = static_cast<unsigned long long>(wall_clock64() - probe_t0);
  }
}

// Any shape, any alignment: one thread per C element, f32 accumulate in k order.
template <bool Bf16, int Epi>
__global__ __launch_bounds__(256) void gemm16_simple_kernel(const uint16_t *__restrict__ A,
                                                            const uint16_t *__restrict__ B,
                                                            float *__restrict__ C,
                                                            const float *__restrict__ bias,
                                                            float *__restrict__ rowsum, int M,
                                                            int N, int K, float *__restrict__ rs_planes) {
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
    if ((threadIdx.x & 63) == 0 && row < M) {
      if (rs_planes) rs_planes[static_cast<int64_t>(blockIdx.x) * M + row] = rs;   // one plane per 64 columns
      else atomicAdd(rowsum + row, rs);
    }
  }
}

__global__ void zero_f32_kernel(float *p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

// rowsum[r] = the per-tile-column sums planes[t * m + r], t = 0 .. count-1, added in that order in double and rounded
// once: the order is the tiles', not the order they finished in, so a product gives the same row sums on every run.
__global__ __launch_bounds__(64) void rowsum_fold_kernel(const float *__restrict__ planes, int count, int m,
                                                         float *__restrict__ rowsum) {
  const int r = blockIdx.x * 64 + threadIdx.x;
  if (r >= m) return;
  double acc = 0.0;
  // sixteen planes' values are asked for before the first is added (the loads are what takes the time: a row has one
  // thread), the additions keep the planes' order
  int t = 0;
  for (; t + 16 <= count; t += 16) {
    float v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) v[u] = planes[static_cast<int64_t>(t + u) * m + r];
#pragma unroll
    for (int u = 0; u < 16; ++u) acc += static_cast<double>(v[u]);
  }
  for (; t < count; ++t) acc += static_cast<double>(planes[static_cast<int64_t>(t) * m + r]);
  rowsum[r] = static_cast<float>(acc);
}

// Whether the 128 x 128 tile beats the 256 x 256 one.  Measured on MI355X: large tiles run in rounds of one per CU;
// small tiles in rounds of two per CU, and such a round takes 0.6-0.65 of a large tile's time whether the CUs hold one
// or two of them (2048^3: 64 large tiles 44.6 us, 256 small ones 28.8; 4096^3: 105 against 127 us).  The small tile is
// taken when that estimate is at least a tenth ahead (with every CU busy on a long K its extra operand traffic costs
// clock under the power limit: 4096 x 2048 x 8192 gains 9 % where the estimate says 35 %).
inline bool small_tile_wins(int m, int n) {
  static const int cus = [] {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
      v = 256;
    return v;
  }();
  const int64_t large = static_cast<int64_t>((m + 255) / 256) * ((n + 255) / 256);
  const int64_t small = static_cast<int64_t>((m + 127) / 128) * ((n + 127) / 128);
  const double cost_large = static_cast<double>((large + cus - 1) / cus);
  const double cost_small = 0.65 * static_cast<double>((small + 2 * cus - 1) / (2 * cus));
  return cost_small < 0.9 * cost_large;
}

// Column N-1 of C for an odd N, one wave per row: the direct-to-LDS kernels fetch B in pairs of 16-bit elements, and
// with rows an odd number of elements apart the pair that holds B[K-1][N-1] ends two bytes past B, so they compute
// the N-1 columns before it (their buffer range ends right in front of that pair) and this kernel the last one, with
// the same epilogue.  Lane l takes k = l, l + 64, ...; the 64 partial sums are added in a fixed tree.
template <bool Bf16, int Epi>
__global__ __launch_bounds__(256) void gemm16_last_column_kernel(const uint16_t *__restrict__ A,
                                                                 const uint16_t *__restrict__ B, float *__restrict__ C,
                                                                 const float *__restrict__ bias, float *__restrict__ rowsum,
                                                                 int M, int N, int K, float *__restrict__ rs_plane) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;   // whole waves leave together
  auto widen = [](uint16_t bits) {
    if constexpr (Bf16) return __uint_as_float(static_cast<uint32_t>(bits) << 16);
    else return static_cast<float>(__builtin_bit_cast(_Float16, bits));
  };
  const uint16_t *a = A + static_cast<int64_t>(row) * K;
  const uint16_t *b = B + (N - 1);
  float sum = 0.f;
  for (int k = lane; k < K; k += 64) sum += widen(a[k]) * widen(b[static_cast<int64_t>(k) * N]);
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) sum += __shfl_xor(sum, m, 64);
  if (lane == 0) {
    if constexpr (Epi == EPI_BIAS_RELU_ROWSUM) {
      sum += bias[N - 1];
      sum = sum > 0.f ? sum : 0.f;
      if (rs_plane) rs_plane[row] = sum;
      else atomicAdd(rowsum + row, sum);
    }
    C[static_cast<int64_t>(row) * N + N - 1] = sum;
  }
}

// K splits of the 128 x 128 kernel for a plain product with few tiles and a long K; 1 = no split.  A tile's K loop is
// bound by the latency of its transfers (0.19 us per K = 32 slab with one or two workgroups on a CU, measured), so
// cutting K over idle CUs shortens it; against that stand the second launch (5 us) and the partial planes, which cost
// 0.65 us per MiB to write and add up.  The count in {2, 4, 8, 16} with the lowest estimate is taken if it is a tenth
// below the unsplit one; every piece is at least 256 of K and the planes fit kSplitWorkspaceBytes.
// gemm16.split_k: 0 = this rule, 1 = never, n >= 2 forces n where the shape allows it.
int splitk_for(int m, int n, int k) {
  const int64_t tiles = static_cast<int64_t>((m + 127) / 128) * ((n + 127) / 128);
  const int64_t forced = tunable("gemm16.split_k", 0);
  // the planes are added 16 bytes at a time; a last piece below one stage needs K % 8 == 0
  if (forced == 1 || (static_cast<int64_t>(m) * n) % 4 != 0 || k % 8 != 0) return 1;
  static const int cus = [] {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
      v = 256;
    return v;
  }();
  const double plane_mib = static_cast<double>(m) * n * 4 / (1 << 20);
  const int64_t fit = static_cast<int64_t>(static_cast<double>(kSplitWorkspaceBytes >> 20) / plane_mib);
  int64_t splits = 1;
  if (forced >= 2) {
    splits = std::min<int64_t>({forced, static_cast<int64_t>(k / 64), fit});
  } else {
    auto estimate = [&](int64_t s) {
      const double slabs = static_cast<double>(k) / 32 / s;
      return 8.0 + slabs * 0.19 * (tiles * s > cus ? 1.15 : 1.0) + (s > 1 ? 5.0 + s * plane_mib * 0.65 : 0.0);
    };
    double best = estimate(1) * 0.9;
    for (int64_t s = 2; s <= 16; s *= 2) {
      if (tiles * s > 2 * cus || k / s < 256 || s > fit) break;
      if (estimate(s) < best) best = estimate(s), splits = s;
    }
  }
  if (splits < 2) return 1;
  // whole K = 64 stages per piece; the count follows from the piece so that none is empty
  const int chunk = static_cast<int>((((k + 63) / 64 + splits - 1) / splits) * 64);
  return (k + chunk - 1) / chunk;
}

// The kernel on v_mfma_f32_16x16x32 with nothing switched off: what a call gets unless, in the measurement build, a sweep
// knob says otherwise.
inline bool gemm16_default_kernel() {
#ifdef SAREK_HIP_MEASURE
  return tunable("gemm16.ring", 0) == 0 && tunable("gemm16.tj", 2) == 2 && tunable("gemm16.mfma", 16) == 16 &&
         tunable("gemm16.ablate", 0) == 0;
#else
  return true;
#endif
}

// The workgroup tile of the direct-to-LDS kernels for this shape under the present tunables (256 or 128), or 0 when
// the shape goes to the simple kernel (pointer alignment, which can also send a call there, is not a property of the
// shape and is not looked at).
int gemm16_tile_for(int m, int n, int k) {
  if (m < 1 || n < 1 || k < 1) return 0;
  if (tunable("gemm16.force_simple", 0) != 0) return 0;
  // transfer offsets are 32-bit: 256 rows of A and 64 rows of B must span less than 2 GiB
  const bool offsets_ok = static_cast<int64_t>(k) * 256 * 2 < 0x7FFFFFFF && static_cast<int64_t>(n) * 64 * 2 < 0x7FFFFFFF;
  if (!offsets_ok) return 0;
  if (gemm16_default_kernel()) {
    // any N; any K from one LDS stage (64) on, below that the multiples of 8
    if (k < 64 && k % 8 != 0) return 0;
    // gemm16.tile: 256 | 128 forces the tile, 0 (default) picks by the tile counts
    const int tile = (int)tunable("gemm16.tile", 0);
    return (tile == 128 || (tile == 0 && small_tile_wins(m, n))) ? 128 : 256;
  }
  // measurement build: the 32 x 32 x 16 kernel and the ablated variants take whole K = 64 stages and 16-byte rows of B
  return (n % 8 == 0 && k % BK == 0) ? 256 : 0;
}

#ifdef SAREK_HIP_MEASURE
// The measurement build's kernels: the 32 x 32 x 16 pipeline in its ring and wave shapes, and both MFMA kernels with parts
// of the K loop left out (gemm16.ablate; the results are then wrong by construction).  Plain store, aligned shapes only.
template <bool Bf16>
int launch_gemm16_measure(const uint16_t *a, const uint16_t *b, float *c, int m, int n, int k, hipStream_t st) {
  const bool ok = k % 8 == 0 && n % 8 == 0 && k % BK == 0 && reinterpret_cast<uintptr_t>(a) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(b) % 16 == 0 && static_cast<int64_t>(k) * 256 * 2 < 0x7FFFFFFF &&
                  static_cast<int64_t>(n) * 64 * 2 < 0x7FFFFFFF;
  if (!ok)
    return fail(SAREK_HIP_E_UNSUPPORTED, "gemm16 measurement kernels: N %% 8 == 0, K %% 64 == 0 and 16-byte aligned A, B only");
  const int tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
  const int remap = (int)tunable("gemm.xcd_remap", 1);
  // gemm16.mfma: 16 = the kernel on the 16 x 16 x 32 instruction (ring 0 and tj 2 only), 32 = 32 x 32 x 16.
  // gemm16.ring 0 = A in K=64 stages x2 + B in K=32 slabs x4, 4 = both in K=32 slabs x4, 2 = both in K=64 slabs x2;
  // gemm16.tj 2 | 4
  const int ring = (int)tunable("gemm16.ring", 0), tj = (int)tunable("gemm16.tj", 2);
  const dim3 grid(tiles_m * tiles_n);
  unsigned long long *probe = clock_probe(static_cast<int64_t>(tiles_m) * tiles_n);
  float *const none = nullptr;
#define SAREK_LAUNCH_DMA(BKA, BKB, NA, NB, TJ)                                                      \
  hipLaunchKernelGGL((gemm16_dma_kernel<Bf16, EPI_STORE, BKA, BKB, NA, NB, TJ>), grid,                \
                     dim3(64 * 2 * (8 / TJ)), 0, st, a, b, c, none, none, m, n, k, tiles_m,           \
                     tiles_n, remap, probe)
  const int ablate = (int)tunable("gemm16.ablate", 0);
  const bool m16 = ring == 0 && tj == 2 && tunable("gemm16.mfma", 16) == 16;
  if (m16 && ablate >= 1 && ablate <= 3 && Bf16) {
    // 1: no transfers in the K loop, 2: no fragment reads, 3: neither
    if constexpr (Bf16) {
#define SAREK_LAUNCH_M16_ABLATED(AB)                                                                        \
  hipLaunchKernelGGL((gemm16_m16_kernel<true, EPI_STORE, AB>), grid, dim3(512), 0, st, a, b, c, none, none, m, n, k, \
                     tiles_m, tiles_n, remap, probe, n, none)
      if (ablate == 1) SAREK_LAUNCH_M16_ABLATED(1);
      else if (ablate == 2) SAREK_LAUNCH_M16_ABLATED(2);
      else SAREK_LAUNCH_M16_ABLATED(3);
#undef SAREK_LAUNCH_M16_ABLATED
    }
    return check_launch("gemm16 kernel launch");
  }
  if (m16)
    return fail(SAREK_HIP_E_UNSUPPORTED, "gemm16.ablate with the 16 x 16 x 32 kernel: 1..3, bf16 (4 and 8: gemm16.mfma=32)");
  if (ablate != 0) {
    if (!Bf16 || ring != 0 || tj != 2 || ablate < 1 || (ablate > 4 && ablate != 8))
      return fail(SAREK_HIP_E_UNSUPPORTED, "gemm16.ablate is for the default bf16 shape only (1..4, 8)");
    if constexpr (Bf16) {
#define SAREK_LAUNCH_ABLATED(AB)                                                                    \
  hipLaunchKernelGGL((gemm16_dma_kernel<true, EPI_STORE, 64, 32, 2, 4, 2, AB>), grid, dim3(512), 0, st, a, b, c, \
                     none, none, m, n, k, tiles_m, tiles_n, remap, probe)
      if (ablate == 1) SAREK_LAUNCH_ABLATED(1);
      else if (ablate == 2) SAREK_LAUNCH_ABLATED(2);
      else if (ablate == 3) SAREK_LAUNCH_ABLATED(3);
      else if (ablate == 8) SAREK_LAUNCH_ABLATED(8);
      else SAREK_LAUNCH_ABLATED(4);
#undef SAREK_LAUNCH_ABLATED
    }
    return check_launch("gemm16 kernel launch");
  }
  if (ring == 4 && tj == 2) SAREK_LAUNCH_DMA(32, 32, 4, 4, 2);
  else if (ring == 4) SAREK_LAUNCH_DMA(32, 32, 4, 4, 4);
  else if (ring == 2 && tj == 2) SAREK_LAUNCH_DMA(64, 64, 2, 2, 2);
  else if (ring == 2) SAREK_LAUNCH_DMA(64, 64, 2, 2, 4);
  else if (tj == 4) SAREK_LAUNCH_DMA(64, 32, 2, 4, 4);
  else SAREK_LAUNCH_DMA(64, 32, 2, 4, 2);
#undef SAREK_LAUNCH_DMA
  return check_launch("gemm16 kernel launch");
}
#endif  // SAREK_HIP_MEASURE

template <bool Bf16, int Epi>
int launch_gemm16(const uint16_t *a, const uint16_t *b, float *c, const float *bias, float *rowsum,
                  int m, int n, int k, hipStream_t st) {
  if (m <= 0 || n <= 0 || k <= 0)
    return fail(SAREK_HIP_E_INVALID_ARG, "gemm16: m, n, k must be positive (got %d %d %d)", m, n, k);
  if (!a || !b || !c) return fail(SAREK_HIP_E_INVALID_ARG, "gemm16: NULL matrix");
  if (Epi == EPI_BIAS_RELU_ROWSUM && (!bias || !rowsum)) return fail(SAREK_HIP_E_INVALID_ARG, "gemm16: NULL bias or rowsum");
#ifdef SAREK_HIP_MEASURE
  if (!gemm16_default_kernel()) {
    if constexpr (Epi == EPI_STORE) return launch_gemm16_measure<Bf16>(a, b, c, m, n, k, st);
    else return fail(SAREK_HIP_E_UNSUPPORTED, "gemm16 measurement kernels: plain store only");
  }
#endif
  // The kernels on v_mfma_f32_16x16x32 (256 x 256 or 128 x 128 tile) take any N, any K of at least one LDS stage and
  // any alignment of A and B in their Ragged form; below one stage K must be a multiple of 8 and A and B 16-byte aligned.
  const int tile_choice = gemm16_tile_for(m, n, k);
  const bool ab16 = reinterpret_cast<uintptr_t>(a) % 16 == 0 && reinterpret_cast<uintptr_t>(b) % 16 == 0;
  const bool tiled = tile_choice != 0 && (k >= 64 || ab16);
  // an odd N: the tiled kernel takes the first N - 1 columns of the N-strided matrices, a matrix-vector kernel the last
  const int nm = n - (n & 1);

  // Row sums: every tile column (every 64 columns of the simple kernel, and the last column of an odd N) leaves its
  // share of each row in a plane of its own, and rowsum_fold_kernel adds the planes in column order, in double, with one
  // rounding: the same bits on every run.  The planes live in the stream's workspace block; a call that has none (under
  // stream capture, past the sixteenth stream, planes beyond the block's size) adds with atomicAdd in arrival order.
  float *planes = nullptr;
  int n_planes = 0;
  if constexpr (Epi == EPI_BIAS_RELU_ROWSUM) {
    n_planes = !tiled ? (n + 63) / 64 : (nm > 0 ? (nm + tile_choice - 1) / tile_choice : 0) + (n & 1);
    if (static_cast<int64_t>(n_planes) * m * 4 <= static_cast<int64_t>(kSplitWorkspaceBytes)) planes = splitk_workspace(st);
    if (!planes) {
      hipLaunchKernelGGL(zero_f32_kernel, dim3((m + 255) / 256), dim3(256), 0, st, rowsum, m);
      const int rc = check_launch("rowsum clear launch");
      if (rc != SAREK_HIP_OK) return rc;
    }
  }
  auto finish = [&](int rc) {
    if (rc != SAREK_HIP_OK || !planes) return rc;
    hipLaunchKernelGGL(rowsum_fold_kernel, dim3((m + 63) / 64), dim3(64), 0, st, planes, n_planes, m, rowsum);
    return check_launch("rowsum fold launch");
  };

  if (!tiled) {
    hipLaunchKernelGGL((gemm16_simple_kernel<Bf16, Epi>), dim3((n + 63) / 64, (m + 3) / 4), dim3(256), 0, st, a, b, c, bias,
                       rowsum, m, n, k, planes);
    return finish(check_launch("gemm16 kernel launch"));
  }
  const bool ragged = n % 8 != 0 || k % 64 != 0 || !ab16;   // the kernels' template flag
  const int remap = (int)tunable("gemm.xcd_remap", 1);
  int rc = SAREK_HIP_OK;
  int tile_planes = 0;
  if (nm > 0 && tile_choice == 128) {
    const int sm = (m + 127) / 128, sn = (nm + 127) / 128;
    tile_planes = sn;
    unsigned long long *sprobe = clock_probe(static_cast<int64_t>(sm) * sn);
    int splits = 1;
    float *partials = nullptr;
    if constexpr (Epi == EPI_STORE) {
      if (reinterpret_cast<uintptr_t>(c) % 16 == 0) splits = splitk_for(m, n, k);
      if (splits > 1) partials = splitk_workspace(st);
      if (!partials) splits = 1;
    }
    if (splits > 1) {
      const int64_t mn = static_cast<int64_t>(m) * n;
      const int chunk = (((k + 63) / 64 + splits - 1) / splits) * 64;
      if (ragged)
        hipLaunchKernelGGL((gemm16_m16_small_kernel<Bf16, Epi, true>), dim3(sm * sn, splits), dim3(256), 0, st, a, b, c,
                           bias, rowsum, m, nm, k, sm, sn, remap, nullptr, chunk, partials, n, planes);
      else
        hipLaunchKernelGGL((gemm16_m16_small_kernel<Bf16, Epi, false>), dim3(sm * sn, splits), dim3(256), 0, st, a, b, c,
                           bias, rowsum, m, nm, k, sm, sn, remap, nullptr, chunk, partials, n, planes);
      rc = check_launch("gemm16 kernel launch");
      if (rc != SAREK_HIP_OK) return rc;
      rc = launch_splitk_reduce(partials, c, mn, splits, st);
    } else {
      if (ragged)
        hipLaunchKernelGGL((gemm16_m16_small_kernel<Bf16, Epi, true>), dim3(sm * sn), dim3(256), 0, st, a, b, c, bias,
                           rowsum, m, nm, k, sm, sn, remap, sprobe, k, nullptr, n, planes);
      else
        hipLaunchKernelGGL((gemm16_m16_small_kernel<Bf16, Epi, false>), dim3(sm * sn), dim3(256), 0, st, a, b, c, bias,
                           rowsum, m, nm, k, sm, sn, remap, sprobe, k, nullptr, n, planes);
      rc = check_launch("gemm16 kernel launch");
    }
  } else if (nm > 0) {
    const int tiles_m = (m + BM - 1) / BM, tiles_n = (nm + BN - 1) / BN;
    tile_planes = tiles_n;
    unsigned long long *probe = clock_probe(static_cast<int64_t>(tiles_m) * tiles_n);
#ifdef SAREK_HIP_MEASURE
    if (Epi == EPI_STORE && !ragged && tunable("gemm16.waves", 8) == 4) {
      hipLaunchKernelGGL((gemm16_m16w4_kernel<Bf16>), dim3(tiles_m * tiles_n), dim3(256), 0, st, a, b, c, m, nm, k, tiles_m,
                         tiles_n, remap, n);
    } else if (!ragged && tunable("gemm16.barriers", 2) == 1) {
      hipLaunchKernelGGL((gemm16_m16_kernel<Bf16, Epi, 0, false, true>), dim3(tiles_m * tiles_n), dim3(512), 0, st, a, b, c,
                         bias, rowsum, m, nm, k, tiles_m, tiles_n, remap, probe, n, planes);
    } else
#endif
    if (ragged)
      hipLaunchKernelGGL((gemm16_m16_kernel<Bf16, Epi, 0, true>), dim3(tiles_m * tiles_n), dim3(512), 0, st, a, b, c, bias,
                         rowsum, m, nm, k, tiles_m, tiles_n, remap, probe, n, planes);
    else
      hipLaunchKernelGGL((gemm16_m16_kernel<Bf16, Epi, 0, false>), dim3(tiles_m * tiles_n), dim3(512), 0, st, a, b, c, bias,
                         rowsum, m, nm, k, tiles_m, tiles_n, remap, probe, n, planes);
    rc = check_launch("gemm16 kernel launch");
  }
  if (rc != SAREK_HIP_OK) return rc;
  if (nm != n) {
    hipLaunchKernelGGL((gemm16_last_column_kernel<Bf16, Epi>), dim3((m + 3) / 4), dim3(256), 0, st, a, b, c, bias, rowsum,
                       m, n, k, planes ? planes + static_cast<int64_t>(tile_planes) * m : nullptr);
    rc = check_launch("gemm16 last-column launch");
  }
  return finish(rc);
}

}  // namespace
}  // namespace sarek_hip

using namespace sarek_hip;

extern "C" {

int sarek_hip_gemm16_tile(int m, int n, int k) { return gemm16_tile_for(m, n, k); }

int sarek_hip_gemm16_k_splits(int m, int n, int k) { return gemm16_tile_for(m, n, k) == 128 ? splitk_for(m, n, k) : 1; }

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
