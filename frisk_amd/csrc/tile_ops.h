// Launch helpers of tile_ops.hip, called by the C ABI after argument validation.
#pragma once
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include "frisk_hip.h"

namespace frisk {
// vec_ok: every row of every view starts on a 16-byte boundary (pointers and leading dimensions), so whole
// 16-byte groups may be moved with one access
hipError_t launch_fill(int dtype, void* dst, int64_t rows, int64_t cols, int64_t ld, double value, int vec_ok, hipStream_t s);
hipError_t launch_copy(int src_dtype, const void* src, int64_t src_ld, int dst_dtype, void* dst, int64_t dst_ld, int64_t rows, int64_t cols, int vec_ok,
                       hipStream_t s);
// n0 x n1 tiles of rows x cols, tile (a, b) displaced by a * step0 + b * step1 elements on either side
struct TilePlacement {
  int64_t n0 = 1, n1 = 1, src_step0 = 0, src_step1 = 0, dst_step0 = 0, dst_step1 = 0;
};
hipError_t launch_copy_tiles(int src_dtype, const void* src, int64_t src_ld, int dst_dtype, void* dst, int64_t dst_ld, int64_t rows, int64_t cols,
                             const TilePlacement& tiles, int vec_ok, hipStream_t s);
// the interpreter of frisk.block bodies (elementwise.hip); the descriptor's fields after validation
struct EwParams {
  const void* in[FRISK_EW_MAX_INPUTS];
  void* out;
  int64_t in_row_stride[FRISK_EW_MAX_INPUTS];
  int64_t out_ld, rows, cols;
  int32_t in_dtype[FRISK_EW_MAX_INPUTS], in_col_stride[FRISK_EW_MAX_INPUTS];
  int32_t out_dtype, n_ops;
  int32_t op[FRISK_EW_MAX_OPS], arg[FRISK_EW_MAX_OPS];
  float imm[FRISK_EW_MAX_OPS];
};
// vec_ok: 8 columns per lane through 16-byte accesses (every row of every walked operand and of the output starts on a
// 16-byte boundary and cols is a multiple of 8)
hipError_t launch_elementwise(const EwParams& p, int vec_ok, hipStream_t s);
// slices > 1: the reduced extent is split over that many work-groups through `partial` (slices x kept-extent floats)
int reduce_slices(int dtype, int64_t rows, int64_t cols, int dim);
hipError_t launch_reduce(int dtype, const void* src, int64_t rows, int64_t cols, int64_t ld, int dim, int kind, int clear, void* dst, float* partial, int slices,
                         int vec_ok, hipStream_t s);
// row softmax in base 2 (softmax.hip); rows_aligned: every row of both views starts on a 16-byte boundary
hipError_t launch_softmax_rows(int dtype, const void* src, int64_t sld, void* dst, int64_t dld, int64_t rows, int64_t cols, float scale_log2, float* lse,
                               int rows_aligned, float* partial, int slices, hipStream_t s);
// work-groups a row is split over (1 = not split); a split needs rows * slices * 2 floats of workspace
int softmax_slices(int dtype, int64_t rows, int64_t cols);
}  // namespace frisk
