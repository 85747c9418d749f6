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
  for (int z = 0; z < p.split_k; ++z) {
    const char* src = (const char*)p.partial + (z * slice + (size_t)m * p.N + n) * 4;
    if (whole) {
      if (INT_ACC) { const r_v4i t = *(const r_v4i*)src; for (int e = 0; e < 4; ++e) isum[e] += t[e]; }
      else { const r_v4f t = *(const r_v4f*)src; for (int e = 0; e < 4; ++e) fsum[e] += t[e]; }
    } else {
      for (int e = 0; e < 4; ++e) {
        if (n + e >= p.N) break;
        if (INT_ACC) isum[e] += ((const int*)src)[e]; else fsum[e] += ((const float*)src)[e];
      }
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

hipError_t launch_splitk_reduce(const GemmParams& p, int acc_is_int, hipStream_t stream) {
  const int64_t quads = (((int64_t)p.N + 3) / 4) * p.M;
  const unsigned blocks = (unsigned)((quads + 255) / 256);
  if (acc_is_int) hipLaunchKernelGGL(splitk_reduce_kernel<true>, dim3(blocks), dim3(256), 0, stream, p);
  else hipLaunchKernelGGL(splitk_reduce_kernel<false>, dim3(blocks), dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace frisk
