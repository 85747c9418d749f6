// Row softmax in base 2: y[r][j] = 2^(c x[r][j]) / sum_j 2^(c x[r][j]), the kernel the reference sketches as
// @online_softmax (tmp/ir.mlir:21-66): per row, chunks of 1024 go through frisk.copy, frisk.reduce max, a frisk.block
// of exp2(x * cst - max * cst), frisk.reduce sum and a running log-sum (:33-57), then a second sweep writes
// exp2(x * cst - lse) (:58-68).  Here rows of up to 256 groups of 16 bytes (2048 f16) are shared by 1 to 64 lanes of one
// wave and combined by shuffles; longer rows get a work-group of 256 lanes each.  Rows of up to 64 elements per lane are
// read once and held in registers (maximum, exponentials, sum, scaling: one read and one write of HBM per element);
// longer rows take the sketch's two sweeps with a running maximum and sum per lane, the second sweep re-reading x.
// A lane moves 16 bytes at a time where rows start on 16-byte boundaries; groups that are not whole and, in the
// work-group kernels, any view whose row length is not a whole number of groups are walked element by element.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "tile_ops.h"

namespace frisk {
namespace {

typedef unsigned v4u __attribute__((ext_vector_type(4)));

template <int DT> struct SElem;
template <> struct SElem<FRISK_F32> { typedef float T; static __device__ float load(const T& x) { return x; } static __device__ T store(float x) { return x; } };
template <> struct SElem<FRISK_F16> { typedef _Float16 T; static __device__ float load(const T& x) { return (float)x; } static __device__ T store(float x) { return (_Float16)x; } };
template <> struct SElem<FRISK_BF16> { typedef __bf16 T; static __device__ float load(const T& x) { return (float)x; } static __device__ T store(float x) { return (__bf16)x; } };

// (maximum, sum of 2^(v - maximum)) pairs combine associatively
struct MaxSum {
  float m, l;
  __device__ void add(float v) {
    // a masked element (-inf) adds nothing; without the test an all-masked prefix would compute 2^(-inf - -inf)
    if (v == -INFINITY) return;
    if (v > m) { l = l * __builtin_amdgcn_exp2f(m - v) + 1.f; m = v; }
    else l += __builtin_amdgcn_exp2f(v - m);
  }
  __device__ void merge(const MaxSum& o) {
    const float nm = fmaxf(m, o.m);
    // an empty partner has m = -inf, l = 0: its term must not become 0 * 2^(-inf - -inf)
    const float a = m == nm ? l : l * __builtin_amdgcn_exp2f(m - nm), b = o.m == nm ? o.l : o.l * __builtin_amdgcn_exp2f(o.m - nm);
    m = nm;
    l = a + b;
  }
};

__device__ __forceinline__ MaxSum block_merge(MaxSum v, float* lds) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    MaxSum o;
    o.m = __shfl_xor(v.m, off);
    o.l = __shfl_xor(v.l, off);
    v.merge(o);
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) { lds[2 * wave] = v.m; lds[2 * wave + 1] = v.l; }
  __syncthreads();
  MaxSum r = {lds[0], lds[1]};
#pragma unroll
  for (int w = 1; w < 4; ++w) r.merge(MaxSum{lds[2 * w], lds[2 * w + 1]});
  __syncthreads();
  return r;
}

// Longer rows, a work-group each.  NPT > 0: the row fits in NPT 16-byte groups per lane and is kept in registers.  NPT == 0: two sweeps, 16-byte
// groups when `vec`, single elements otherwise.
template <int DT, int NPT>
__global__ void __launch_bounds__(256) softmax_rows_kernel(const typename SElem<DT>::T* src, int64_t sld, typename SElem<DT>::T* dst, int64_t dld, int64_t rows,
                                                           int64_t cols, float c, float* lse, int vec) {
  typedef typename SElem<DT>::T T;
  constexpr int G = 16 / (int)sizeof(T);
  __shared__ float lds[8];
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const T* x = src + r * sld;
    T* y = dst + r * dld;
    if constexpr (NPT > 0) {
      const int64_t groups = cols / G;
      float v[NPT][G];
      float mx = -INFINITY;
#pragma unroll
      for (int q = 0; q < NPT; ++q) {
        const int64_t g = (int64_t)q * 256 + threadIdx.x;
        T in[G];
        if (g < groups) *(v4u*)in = __builtin_nontemporal_load((const v4u*)(x + g * G));
#pragma unroll
        for (int e = 0; e < G; ++e) {
          v[q][e] = g < groups ? SElem<DT>::load(in[e]) * c : -INFINITY;
          mx = fmaxf(mx, v[q][e]);
        }
      }
      const MaxSum top = block_merge(MaxSum{mx, 1.f}, lds);  // only the maximum is used here
      float sum = 0.f;
#pragma unroll
      for (int q = 0; q < NPT; ++q)
#pragma unroll
        for (int e = 0; e < G; ++e) {
          v[q][e] = __builtin_amdgcn_exp2f(v[q][e] - top.m);
          sum += v[q][e];
        }
      const MaxSum all = block_merge(MaxSum{0.f, sum}, lds);  // equal maxima: the sums add
      const float inv = 1.f / all.l;
#pragma unroll
      for (int q = 0; q < NPT; ++q) {
        const int64_t g = (int64_t)q * 256 + threadIdx.x;
        if (g < groups) {
          T out[G];
#pragma unroll
          for (int e = 0; e < G; ++e) out[e] = SElem<DT>::store(v[q][e] * inv);
          __builtin_nontemporal_store(*(const v4u*)out, (v4u*)(y + g * G));
        }
      }
      if (lse && threadIdx.x == 0) lse[r] = top.m + __builtin_amdgcn_logf(all.l);
    } else {
      MaxSum acc = {-INFINITY, 0.f};
      if (vec) {
        for (int64_t g = threadIdx.x; g < cols / G; g += 256) {
          T in[G];
          *(v4u*)in = *(const v4u*)(x + g * G);
#pragma unroll
          for (int e = 0; e < G; ++e) acc.add(SElem<DT>::load(in[e]) * c);
        }
      } else {
        for (int64_t j = threadIdx.x; j < cols; j += 256) acc.add(SElem<DT>::load(x[j]) * c);
      }
      const MaxSum all = block_merge(acc, lds);
      const float ref = all.m + __builtin_amdgcn_logf(all.l);  // log2 of the denominator
      if (vec) {
        for (int64_t g = threadIdx.x; g < cols / G; g += 256) {
          T in[G], out[G];
          *(v4u*)in = *(const v4u*)(x + g * G);
#pragma unroll
          for (int e = 0; e < G; ++e) out[e] = SElem<DT>::store(__builtin_amdgcn_exp2f(SElem<DT>::load(in[e]) * c - ref));
          __builtin_nontemporal_store(*(const v4u*)out, (v4u*)(y + g * G));
        }
      } else {
        for (int64_t j = threadIdx.x; j < cols; j += 256) y[j] = SElem<DT>::store(__builtin_amdgcn_exp2f(SElem<DT>::load(x[j]) * c - ref));
      }
      if (lse && threadIdx.x == 0) lse[r] = ref;
    }
  }
}

// Rows of at most 256 groups of 16 bytes: 2^lanes_log2 <= 64 lanes of one wave share a row, each holding up to NPT groups in
// registers, and combine maximum and sum by shuffles (no LDS, no barrier); a work-group holds 256 >> lanes_log2 rows.  Any
// alignment: a group that is not a whole, aligned 16 bytes is walked element by element.
template <int DT, int NPT>
__global__ void __launch_bounds__(256) softmax_short_rows_kernel(const typename SElem<DT>::T* src, int64_t sld, typename SElem<DT>::T* dst, int64_t dld, int64_t rows,
                                                                 int64_t cols, float c, float* lse, int vec, int lanes_log2) {
  typedef typename SElem<DT>::T T;
  constexpr int G = 16 / (int)sizeof(T);
  const int lanes = 1 << lanes_log2, lane = threadIdx.x & (lanes - 1), rows_per_group = 256 >> lanes_log2;
  const int64_t blocks = (rows + rows_per_group - 1) / rows_per_group;
  for (int64_t rb = blockIdx.x; rb < blocks; rb += gridDim.x) {
    const int64_t r = rb * rows_per_group + (threadIdx.x >> lanes_log2);
    const bool live = r < rows;  // lanes of rows past the end still take part in the shuffles
    const T* x = src + r * sld;
    T* y = dst + r * dld;
    float v[NPT][G];
    bool whole[NPT];
    T in[NPT][G];
#pragma unroll
    for (int q = 0; q < NPT; ++q) {
      const int64_t c0 = (int64_t)(q * lanes + lane) * G;
      whole[q] = live && vec && c0 + G <= cols;
      if (whole[q]) *(v4u*)in[q] = __builtin_nontemporal_load((const v4u*)(x + c0));
    }
    float mx = -INFINITY;
#pragma unroll
    for (int q = 0; q < NPT; ++q) {
      const int64_t c0 = (int64_t)(q * lanes + lane) * G;
#pragma unroll
      for (int e = 0; e < G; ++e) {
        if (whole[q]) v[q][e] = SElem<DT>::load(in[q][e]) * c;
        else v[q][e] = live && c0 + e < cols ? SElem<DT>::load(x[c0 + e]) * c : -INFINITY;
        mx = fmaxf(mx, v[q][e]);
      }
    }
    for (int off = lanes >> 1; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    float sum = 0.f;
#pragma unroll
    for (int q = 0; q < NPT; ++q)
#pragma unroll
      for (int e = 0; e < G; ++e) {
        v[q][e] = __builtin_amdgcn_exp2f(v[q][e] - mx);
        sum += v[q][e];
      }
    for (int off = lanes >> 1; off >= 1; off >>= 1) sum += __shfl_xor(sum, off, 64);
    const float inv = 1.f / sum;
#pragma unroll
    for (int q = 0; q < NPT; ++q) {
      const int64_t c0 = (int64_t)(q * lanes + lane) * G;
      if (whole[q]) {
        T out[G];
#pragma unroll
        for (int e = 0; e < G; ++e) out[e] = SElem<DT>::store(v[q][e] * inv);
        __builtin_nontemporal_store(*(const v4u*)out, (v4u*)(y + c0));
      } else if (live) {
#pragma unroll
        for (int e = 0; e < G; ++e)
          if (c0 + e < cols) y[c0 + e] = SElem<DT>::store(v[q][e] * inv);
      }
    }
    if (lse && live && lane == 0) lse[r] = mx + __builtin_amdgcn_logf(sum);
  }
}

// A few very long rows: a row is dealt to gridDim.y work-groups in runs of 256 groups (neighbouring work-groups read
// neighbouring memory).  First launch: every work-group leaves the (maximum, sum) of its share in partial[row][slice];
// second launch: every work-group merges the row's pairs and writes its share of exp2(x * c - log-sum).  Two reads and
// one write per element, as in the two sweeps above, but on rows x slices work-groups instead of rows.
template <int DT>
__global__ void __launch_bounds__(256) softmax_split_stats_kernel(const typename SElem<DT>::T* src, int64_t sld, int64_t cols, float c, float* partial, int vec) {
  typedef typename SElem<DT>::T T;
  constexpr int G = 16 / (int)sizeof(T);
  __shared__ float lds[8];
  const T* x = src + (int64_t)blockIdx.x * sld;
  MaxSum acc = {-INFINITY, 0.f};
  if (vec) {
    for (int64_t g = (int64_t)blockIdx.y * 256 + threadIdx.x; g < cols / G; g += (int64_t)gridDim.y * 256) {
      T in[G];
      *(v4u*)in = *(const v4u*)(x + g * G);
#pragma unroll
      for (int e = 0; e < G; ++e) acc.add(SElem<DT>::load(in[e]) * c);
    }
  } else {
    for (int64_t j = (int64_t)blockIdx.y * 256 + threadIdx.x; j < cols; j += (int64_t)gridDim.y * 256) acc.add(SElem<DT>::load(x[j]) * c);
  }
  const MaxSum all = block_merge(acc, lds);
  if (threadIdx.x == 0) {
    float* out = partial + ((int64_t)blockIdx.x * gridDim.y + blockIdx.y) * 2;
    out[0] = all.m;
    out[1] = all.l;
  }
}

template <int DT>
__global__ void __launch_bounds__(256) softmax_split_write_kernel(const typename SElem<DT>::T* src, int64_t sld, typename SElem<DT>::T* dst, int64_t dld, int64_t cols,
                                                                  float c, float* lse, const float* partial, int vec) {
  typedef typename SElem<DT>::T T;
  constexpr int G = 16 / (int)sizeof(T);
  __shared__ float lds[8];
  const T* x = src + (int64_t)blockIdx.x * sld;
  T* y = dst + (int64_t)blockIdx.x * dld;
  MaxSum acc = {-INFINITY, 0.f};
  for (int k = threadIdx.x; k < (int)gridDim.y; k += 256) {
    const float* in = partial + ((int64_t)blockIdx.x * gridDim.y + k) * 2;
    acc.merge(MaxSum{in[0], in[1]});
  }
  const MaxSum all = block_merge(acc, lds);
  const float ref = all.m + __builtin_amdgcn_logf(all.l);  // log2 of the denominator
  if (vec) {
    for (int64_t g = (int64_t)blockIdx.y * 256 + threadIdx.x; g < cols / G; g += (int64_t)gridDim.y * 256) {
      T in[G], out[G];
      *(v4u*)in = __builtin_nontemporal_load((const v4u*)(x + g * G));
#pragma unroll
      for (int e = 0; e < G; ++e) out[e] = SElem<DT>::store(__builtin_amdgcn_exp2f(SElem<DT>::load(in[e]) * c - ref));
      __builtin_nontemporal_store(*(const v4u*)out, (v4u*)(y + g * G));
    }
  } else {
    for (int64_t j = (int64_t)blockIdx.y * 256 + threadIdx.x; j < cols; j += (int64_t)gridDim.y * 256)
      y[j] = SElem<DT>::store(__builtin_amdgcn_exp2f(SElem<DT>::load(x[j]) * c - ref));
  }
  if (lse && blockIdx.y == 0 && threadIdx.x == 0) lse[blockIdx.x] = ref;
}

template <int DT> hipError_t launch_typed(const void* src, int64_t sld, void* dst, int64_t dld, int64_t rows, int64_t cols, float c, float* lse, int rows_aligned,
                                          float* partial, int slices, hipStream_t s) {
  typedef typename SElem<DT>::T T;
  constexpr int G = 16 / (int)sizeof(T);
  const int vec = rows_aligned && cols % G == 0;
  const unsigned grid = (unsigned)(rows < 256 * 64 ? rows : 256 * 64);
  const int64_t per_pass = 256 * (int64_t)G;
  const T* x = (const T*)src;
  T* y = (T*)dst;
  const int64_t groups = (cols + G - 1) / G;
  if (slices > 1) {
    const dim3 sgrid((unsigned)rows, (unsigned)slices);
    hipLaunchKernelGGL((softmax_split_stats_kernel<DT>), sgrid, dim3(256), 0, s, x, sld, cols, c, partial, vec);
    hipLaunchKernelGGL((softmax_split_write_kernel<DT>), sgrid, dim3(256), 0, s, x, sld, y, dld, cols, c, lse, (const float*)partial, vec);
    return hipGetLastError();
  }
  if (groups <= 256) {  // here a row that ends in a partial group still moves its whole groups 16 bytes at a time
    int lanes_log2 = 0;
    while (lanes_log2 < 6 && (int64_t(1) << lanes_log2) < groups) ++lanes_log2;
    const int64_t rows_per_group = 256 >> lanes_log2, blocks = (rows + rows_per_group - 1) / rows_per_group;
    const dim3 sgrid((unsigned)(blocks < (1 << 22) ? blocks : (1 << 22)));
    if (groups <= 64) hipLaunchKernelGGL((softmax_short_rows_kernel<DT, 1>), sgrid, dim3(256), 0, s, x, sld, y, dld, rows, cols, c, lse, rows_aligned, lanes_log2);
    else if (groups <= 128) hipLaunchKernelGGL((softmax_short_rows_kernel<DT, 2>), sgrid, dim3(256), 0, s, x, sld, y, dld, rows, cols, c, lse, rows_aligned, lanes_log2);
    else hipLaunchKernelGGL((softmax_short_rows_kernel<DT, 4>), sgrid, dim3(256), 0, s, x, sld, y, dld, rows, cols, c, lse, rows_aligned, lanes_log2);
    return hipGetLastError();
  }
  if (vec && cols <= 2 * per_pass) hipLaunchKernelGGL((softmax_rows_kernel<DT, 2>), dim3(grid), dim3(256), 0, s, x, sld, y, dld, rows, cols, c, lse, vec);
  else if (vec && cols <= 4 * per_pass) hipLaunchKernelGGL((softmax_rows_kernel<DT, 4>), dim3(grid), dim3(256), 0, s, x, sld, y, dld, rows, cols, c, lse, vec);
  else if (vec && cols <= 8 * per_pass) hipLaunchKernelGGL((softmax_rows_kernel<DT, 8>), dim3(grid), dim3(256), 0, s, x, sld, y, dld, rows, cols, c, lse, vec);
  else hipLaunchKernelGGL((softmax_rows_kernel<DT, 0>), dim3(grid), dim3(256), 0, s, x, sld, y, dld, rows, cols, c, lse, vec);
  return hipGetLastError();
}

}  // namespace

int softmax_slices(int dtype, int64_t rows, int64_t cols) {
  // Fewer than 1024 rows of at least 32 KiB: split each so that about 1024 work-groups exist, each with at least 16 KiB.
  const int64_t row_bytes = cols * (dtype == FRISK_F32 ? 4 : 2);
  int slices = 1;
  while (rows * slices < 1024 && row_bytes / (slices * 2) >= 16384 && slices < 256) slices *= 2;
  return slices;
}

// rows_aligned: pointers and leading dimensions put every row of both views on a 16-byte boundary
hipError_t launch_softmax_rows(int dtype, const void* src, int64_t sld, void* dst, int64_t dld, int64_t rows, int64_t cols, float scale_log2, float* lse,
                               int rows_aligned, float* partial, int slices, hipStream_t s) {
  switch (dtype) {
    case FRISK_F32: return launch_typed<FRISK_F32>(src, sld, dst, dld, rows, cols, scale_log2, lse, rows_aligned, partial, slices, s);
    case FRISK_F16: return launch_typed<FRISK_F16>(src, sld, dst, dld, rows, cols, scale_log2, lse, rows_aligned, partial, slices, s);
    default: return launch_typed<FRISK_BF16>(src, sld, dst, dld, rows, cols, scale_log2, lse, rows_aligned, partial, slices, s);
  }
}

}  // namespace frisk
