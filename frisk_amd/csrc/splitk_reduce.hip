// Second pass of a split-K GEMM: sums the raw 32-bit accumulators the K slices
// left in the workspace ([slice][M][N], row length N) and applies what the
// single-pass epilogue applies: integer output as is, otherwise (x * scaleA) *
// scaleB with two separately rounded multiplies, then accumulate-into-C, then
// the conversion to the output type.  A thread owns 4 consecutive columns.
#include <hip/hip_runtime.h>
#include "gemm_internal.h"

namespace frisk {

typedef int r_v4i __attribute__((ext_vector_type(4)));
typedef float r_v4f __attribute__((ext_vector_type(4)));

template <bool INT_ACC> __global__ void __launch_bounds__(256) splitk_reduce_kernel(GemmParams p) {
  const int64_t quads_per_row = (p.N + 3) / 4;
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= quads_per_row * p.M) return;
  const int64_t m = id / quads_per_row, n = (id % quads_per_row) * 4;
  const size_t slice = (size_t)p.M * (size_t)p.N;
  const bool whole = n + 4 <= p.N && (p.N & 3) == 0;  // 16-byte aligned quad inside the row
  int isum[4] = {0, 0, 0, 0};
  float fsum[4] = {0.f, 0.f, 0.f, 0.f};
  const char* src = (const char*)p.partial + ((size_t)m * p.N + n) * 4;
  if (whole) {
    // the slices' quads are fetched eight at a time and then added in slice order: one memory latency per eight slices instead
    // of one per slice (16 slices of a 256 x 256 result: 9.9 -> 4.4 us in a kernel trace), the same sum
    for (int z0 = 0; z0 < p.split_k; z0 += 8) {
      r_v4i t[8];
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (z0 + i < p.split_k) t[i] = *(const r_v4i*)(src + (size_t)(z0 + i) * slice * 4);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (z0 + i >= p.split_k) break;
        for (int e = 0; e < 4; ++e) {
          if (INT_ACC) isum[e] += t[i][e]; else fsum[e] += __builtin_bit_cast(float, (int)t[i][e]);
        }
      }
    }
  } else {
    for (int z = 0; z < p.split_k; ++z, src += slice * 4)
      for (int e = 0; e < 4; ++e) {
        if (n + e >= p.N) break;
        if (INT_ACC) isum[e] += ((const int*)src)[e]; else fsum[e] += ((const float*)src)[e];
      }
  }
  float sa = 1.f, sb[4] = {1.f, 1.f, 1.f, 1.f};
  if (p.epilogue == FRISK_EPI_TENSOR_SCALE) {
    sa = p.scaleA[0];
    for (int e = 0; e < 4; ++e) sb[e] = p.scaleB[0];
  } else if (p.epilogue == FRISK_EPI_ROW_COL_SCALE) {
    sa = p.scaleA[m];
    for (int e = 0; e < 4; ++e) if (n + e < p.N) sb[e] = p.scaleB[n + e];
  }
  const bool accum = p.accumulate != 0;
  for (int e = 0; e < 4; ++e) {
    if (n + e >= p.N) break;
    const int64_t at = m * p.ldc + n + e;
    if (INT_ACC && p.dtype_out == FRISK_I32) {
      int* q = (int*)p.C + at;
      *q = isum[e] + (accum ? *q : 0);
      continue;
    }
    float x = INT_ACC ? (float)isum[e] : fsum[e];
    if (p.epilogue != FRISK_EPI_NONE) x = (x * sa) * sb[e];
    if (p.dtype_out == FRISK_F16) { _Float16* q = (_Float16*)p.C + at; if (accum) x += (float)*q; *q = (_Float16)x; }
    else if (p.dtype_out == FRISK_BF16) { __bf16* q = (__bf16*)p.C + at; if (accum) x += (float)*q; *q = (__bf16)x; }
    else { float* q = (float*)p.C + at; if (accum) x += *q; *q = x; }
  }
}

// The tiles of a tail split: partial[slice][tail tile][BM][BN]; a work-group of 256 lanes per 16 rows of a tile when BN = 256
// (a thread owns 4 consecutive columns), the tile's place in C from the same id mapping as the GEMM kernel's.
template <bool INT_ACC> __global__ void __launch_bounds__(256) tail_reduce_kernel(GemmParams p) {
  const int BM = p.tile_m, BN = p.tile_n;
  const int quads_per_row = BN / 4, quads = BM * quads_per_row;
  const int t = blockIdx.y;
  int tm, tn;
  tile_of_workgroup(p.tail_from + t, p.tiles_m, p.tiles_n, p.group_m, p.xcd_remap, tm, tn);
  const size_t tile_elems = (size_t)BM * BN;
  for (int id = blockIdx.x * 256 + threadIdx.x; id < quads; id += gridDim.x * 256) {
    const int r = id / quads_per_row, c = (id % quads_per_row) * 4;
    const int64_t m = (int64_t)tm * BM + r, n = (int64_t)tn * BN + c;
    int isum[4] = {0, 0, 0, 0};
    float fsum[4] = {0.f, 0.f, 0.f, 0.f};
    r_v4i v[8];  // a tail has 2, 4 or 8 slices: all fetched before the first addition, added in slice order
#pragma unroll
    for (int z = 0; z < 8; ++z)
      if (z < p.tail_split) v[z] = *(const r_v4i*)((const char*)p.partial + (((size_t)z * p.tail_tiles + t) * tile_elems + (size_t)r * BN + c) * 4);
#pragma unroll
    for (int z = 0; z < 8; ++z) {
      if (z >= p.tail_split) break;
      for (int e = 0; e < 4; ++e) {
        if (INT_ACC) isum[e] += v[z][e]; else fsum[e] += __builtin_bit_cast(float, (int)v[z][e]);
      }
    }
    float sa = 1.f, sb[4] = {1.f, 1.f, 1.f, 1.f};
    if (p.epilogue == FRISK_EPI_TENSOR_SCALE) {
      sa = p.scaleA[0];
      for (int e = 0; e < 4; ++e) sb[e] = p.scaleB[0];
    } else if (p.epilogue == FRISK_EPI_ROW_COL_SCALE) {
      sa = p.scaleA[m];
      for (int e = 0; e < 4; ++e) sb[e] = p.scaleB[n + e];
    }
    const bool accum = p.accumulate != 0;
    for (int e = 0; e < 4; ++e) {
      const int64_t at = m * p.ldc + n + e;
      if (INT_ACC && p.dtype_out == FRISK_I32) {
        int* q = (int*)p.C + at;
        *q = isum[e] + (accum ? *q : 0);
        continue;
      }
      float x = INT_ACC ? (float)isum[e] : fsum[e];
      if (p.epilogue != FRISK_EPI_NONE) x = (x * sa) * sb[e];
      if (p.dtype_out == FRISK_F16) { _Float16* q = (_Float16*)p.C + at; if (accum) x += (float)*q; *q = (_Float16)x; }
      else if (p.dtype_out == FRISK_BF16) { __bf16* q = (__bf16*)p.C + at; if (accum) x += (float)*q; *q = (__bf16)x; }
      else { float* q = (float*)p.C + at; if (accum) x += *q; *q = x; }
    }
  }
}

hipError_t launch_tail_reduce(const GemmParams& p, int acc_is_int, hipStream_t stream) {
  const int quads = p.tile_m * p.tile_n / 4;
  const dim3 grid((unsigned)((quads + 1023) / 1024), (unsigned)p.tail_tiles);  // four quads per lane
  if (acc_is_int) hipLaunchKernelGGL(tail_reduce_kernel<true>, grid, dim3(256), 0, stream, p);
  else hipLaunchKernelGGL(tail_reduce_kernel<false>, grid, dim3(256), 0, stream, p);
  return hipGetLastError();
}

hipError_t launch_splitk_reduce(const GemmParams& p, int acc_is_int, hipStream_t stream) {
  const int64_t quads = (((int64_t)p.N + 3) / 4) * p.M;
  const unsigned blocks = (unsigned)((quads + 255) / 256);
  if (acc_is_int) hipLaunchKernelGGL(splitk_reduce_kernel<true>, dim3(blocks), dim3(256), 0, stream, p);
  else hipLaunchKernelGGL(splitk_reduce_kernel<false>, dim3(blocks), dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace frisk
