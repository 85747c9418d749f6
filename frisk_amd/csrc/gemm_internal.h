// Internal declarations shared by the kernel translation units, the planner and the C ABI.
#pragma once
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include "frisk_hip.h"

namespace frisk {

struct GemmParams {
  const void* A;
  const void* B;
  void* C;
  const float* scaleA;
  const float* scaleB;
  int64_t lda, ldb, ldc;  // elements
  int M, N, K;
  int tiles_m, tiles_n;
  int group_m, xcd_remap;
  int epilogue, dtype_out, accumulate;
  // K range of a work-group: blockIdx.y walks `split_k` slices of `kt_per_slice` K tiles each.  With more than one
  // slice the kernel writes raw 32-bit accumulators to partial[slice][M][N] and a second kernel sums the slices.
  int split_k, kt_per_slice;
  void* partial;
  // Tail split: the last `tail_tiles` tiles of a grid that is a little more than a whole number of rounds of 256 are
  // each computed by `tail_split` work-groups, `tail_kt` K tiles apiece.  Work-group ids from `tail_from` on are tail
  // units (tile = tail_from + unit / tail_split, slice = unit % tail_split); they leave raw accumulators in
  // partial[slice][tile - tail_from][BM][BN] and a second kernel sums them.  tail_split <= 1: no tail.
  int tail_from, tail_tiles, tail_split, tail_kt;
  int tile_m, tile_n;  // BM, BN of the kernel (for the tail reduction)
  int k_rotate;        // 32-row kernels: work-groups start at different K tiles of their slice and wrap around
};

// Hardware hands consecutive work-group ids to the 8 XCDs round-robin.  Give each XCD a contiguous range of "compact"
// ids, then walk the tile grid in column-major order inside bands of GM tile rows, so the work-groups resident on one
// XCD (one L2) cover a GM x (resident/GM) block of tiles.
__host__ __device__ inline void tile_of_workgroup(int wg, int tiles_m, int tiles_n, int gm, int xcd_remap, int& tm, int& tn) {
  int total = tiles_m * tiles_n;
  int cid = wg;
  if (xcd_remap) {
    int per = total >> 3;
    if (wg < per * 8) cid = (wg & 7) * per + (wg >> 3);
  }
  int band = gm * tiles_n;
  int b = cid / band;
  int first_m = b * gm;
  int rows = tiles_m - first_m < gm ? tiles_m - first_m : gm;
  int in = cid - b * band;
  tm = first_m + in % rows;
  tn = in / rows;
}

// One compiled kernel variant.
struct KernelEntry {
  const char* name;
  int dtype;  // frisk_dtype of A and B
  int transA, transB;
  int bm, bn, bk, wm, wn;
  int stages, stages_b;  // LDS ring depth for A and for B (stages_b >= stages)
  int wk;  // waves splitting the K steps of a tile (1 = none)
  int guard;  // 1: handles any shape / leading dimension (slower staging)
  int splitk;  // 1: compiled with the split-K store path
  int atom;  // rows and columns of the MFMA atom: 32 (32x32xK) or 16 (16x16x2K)
  int edge;  // 1: M and N need not be multiples of the tile (K, and the alignment of rows and pointers, as for the plain kernels)
  int lds_bytes;
  int min_k_tiles;  // fewest K tiles the kernel's loop is written for
  hipError_t (*launch)(const GemmParams&, hipStream_t);
  hipError_t (*prepare)();  // one-time, non-stream set-up of the kernel function (dynamic LDS limit)
};

// sums the split-K slices and applies the epilogue (splitk_reduce.hip)
hipError_t launch_splitk_reduce(const GemmParams& p, int acc_is_int, hipStream_t stream);
// the same for the tiles of a tail split
hipError_t launch_tail_reduce(const GemmParams& p, int acc_is_int, hipStream_t stream);

// defined in kernels_*.hip (two tables per element type: kernels_<type>.hip and kernels_<type>_2.hip)
extern const KernelEntry kKernelsF16[];
extern const int kNumKernelsF16;
extern const KernelEntry kKernelsF16_2[];
extern const int kNumKernelsF16_2;
extern const KernelEntry kKernelsBF16[];
extern const int kNumKernelsBF16;
extern const KernelEntry kKernelsBF16_2[];
extern const int kNumKernelsBF16_2;
extern const KernelEntry kKernelsI8[];
extern const int kNumKernelsI8;
extern const KernelEntry kKernelsI8_2[];
extern const int kNumKernelsI8_2;
extern const KernelEntry kKernelsE4M3[];
extern const int kNumKernelsE4M3;
extern const KernelEntry kKernelsE4M3_2[];
extern const int kNumKernelsE4M3_2;
extern const KernelEntry kKernelsF32[];
extern const int kNumKernelsF32;
extern const KernelEntry kKernelsF32_2[];
extern const int kNumKernelsF32_2;

}  // namespace frisk
