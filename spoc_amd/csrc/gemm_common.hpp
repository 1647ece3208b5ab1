// Device helpers shared by the GEMM kernels: workgroup -> tile raster, the LDS ring of
// the direct-to-LDS pipelines, DMA and barrier primitives.
#pragma once
#include <hip/hip_runtime.h>

namespace sarek_hip {

// K-split products (gemm_splitk.hip): the per-stream block of device memory for the partial planes and the kernel that
// adds them into C in a fixed order.
constexpr size_t kSplitWorkspaceBytes = 64u << 20;
float *splitk_workspace(hipStream_t st);
int launch_splitk_reduce(const float *partials, float *c, int64_t mn, int splits, hipStream_t st);

namespace {

#define LDS_PTR __attribute__((address_space(3)))

constexpr int NUM_XCD = 8;   // XCDs of an MI355X; workgroup ids are dealt to them round-robin

// Workgroup -> tile.  The hardware deals consecutive workgroup ids round-robin to the
// 8 XCDs (each with its own L2), so ids are first regrouped to give every XCD one
// contiguous run of tiles, and the run is walked in bands of GROUP tile-rows, column by
// column: the ~32 tiles an XCD has in flight then form a compact GROUP x (32 / GROUP) patch that
// moves through K together and shares A row-panels and B column-panels in that L2.
// GROUP = 4 (xcd_remap = 1; a larger xcd_remap sets another height): with 32 x 32 tiles every XCD then owns one
// band of four tile-rows and all eight walk the same column panels of B at the same time, so what one of them
// brings past its L2 the others find in the memory-side cache.  Measured on bf16 products against bands of 8:
// 8192^3 0.729 against 0.740 ms, 8192 x 4096 x 8192 0.365 against 0.374, 16384 x 8192 x 2048 0.442 against 0.474,
// nothing lost on 3072^3, 4096^3, the fp16 epilogue shape and the f32 8192^3 product; bands of 2, 16 or 32 are slower.
__device__ __forceinline__ void tile_of_block(int tiles_m, int tiles_n, int xcd_remap, int &tm,
                                              int &tn) {
  const int GROUP = xcd_remap > 1 ? xcd_remap : 4;   // tile-rows per raster band
  const int nblocks = tiles_m * tiles_n;
  const int xcd = blockIdx.x % NUM_XCD, slot = blockIdx.x / NUM_XCD;
  int tile = xcd * (nblocks / NUM_XCD) + min(xcd, nblocks % NUM_XCD) + slot;
  if (xcd_remap == 0) tile = blockIdx.x;
  const int per_group = GROUP * tiles_n;
  const int g = tile / per_group;
  const int rows_in_group = min(GROUP, tiles_m - g * GROUP);
  const int in_g = tile - g * per_group;
  tm = g * GROUP + in_g % rows_in_group;
  tn = in_g / rows_in_group;
}

// One static LDS array per ring stage and operand: distinct objects, so the compiler can
// tell that the DMA into one stage does not alias the ds_reads of another and need not
// wait for it.
template <int Id, int Bytes>
__shared__ __attribute__((aligned(1024))) char lds_ring[Bytes];

// Global -> LDS DMA: buffer_load_dwordx4 ... lds.  64 lanes x 16 bytes, lane l's piece lands
// at lds_dst + 16*l.  The buffer form (scalar resource + 32-bit lane offset + scalar offset)
// is used on purpose: measured on MI355X, four global_load_lds_dwordx4 per 32 MFMAs cut the
// MFMA issue rate by a third, the same number of buffer_load ... lds cost nothing.
// Offsets at or past `bytes` read as zero (raw buffer range check).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, static_cast<int>(bytes),
                                           0x00020000);
}
// Cache-policy bits stay 0: sc0 / sc1 change nothing measurable for these loads, nt costs 8 % (the
// panels are shared through the L2 by the tiles of a patch, and nt lines leave it early).
__device__ __forceinline__ void dma16(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off,
                                      uint32_t uniform_off, char *lds_dst) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (LDS_PTR void *)lds_dst, 16,
                                           static_cast<int>(lane_off),
                                           static_cast<int>(uniform_off), 0, 0);
}

// s_waitcnt immediate (gfx9 encoding) that waits for vmcnt <= n and lgkmcnt <= 0.
constexpr int waitcnt_vm_lgkm0(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (0 << 8); }

// Workgroup barrier without the fence __syncthreads() carries (which would drain every
// outstanding DMA): callers wait for exactly the DMA they need first.
__device__ __forceinline__ void barrier_no_fence() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

}  // namespace
}  // namespace sarek_hip
