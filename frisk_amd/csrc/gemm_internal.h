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
};

// One compiled kernel variant.
struct KernelEntry {
  const char* name;
  int dtype;  // frisk_dtype of A and B
  int transA, transB;
  int bm, bn, bk, wm, wn, stages;
  int guard;  // 1: handles any shape / leading dimension (slower staging)
  int lds_bytes;
  hipError_t (*launch)(const GemmParams&, hipStream_t);
};

// defined in kernels_*.hip
extern const KernelEntry kKernelsF16[];
extern const int kNumKernelsF16;
extern const KernelEntry kKernelsBF16[];
extern const int kNumKernelsBF16;
extern const KernelEntry kKernelsI8[];
extern const int kNumKernelsI8;
extern const KernelEntry kKernelsE4M3[];
extern const int kNumKernelsE4M3;
extern const KernelEntry kKernelsF32[];
extern const int kNumKernelsF32;

}  // namespace frisk
