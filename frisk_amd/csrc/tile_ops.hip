// frisk.fill, frisk.copy and frisk.reduce on rank-2 views of device memory.  All three are bound by
// HBM traffic: a lane moves 16 bytes at a time wherever the view allows it (row start and row length
// multiples of 16 bytes), falls back to single elements otherwise, and a launch covers the view with
// many more work-groups than the 256 CUs.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "tile_ops.h"

namespace frisk {
namespace {

typedef unsigned v4u __attribute__((ext_vector_type(4)));

// streaming reads: every byte is read once, so the caches are told not to keep it; on stores the hint pays in copy
// between equally wide types (6.3 against 5.9 TB/s) and changes nothing in fill, so only copy uses it
__device__ __forceinline__ v4u load16(const void* p) { return __builtin_nontemporal_load((const v4u*)p); }
__device__ __forceinline__ void store16(void* p, v4u v) { *(v4u*)p = v; }
__device__ __forceinline__ void store16_stream(void* p, v4u v) { __builtin_nontemporal_store(v, (v4u*)p); }

template <int DT> struct Elem;
template <> struct Elem<FRISK_F32> { typedef float T; static __device__ float load(const T& x) { return x; } static __device__ T store(float x) { return x; } };
template <> struct Elem<FRISK_F16> { typedef _Float16 T; static __device__ float load(const T& x) { return (float)x; } static __device__ T store(float x) { return (_Float16)x; } };
template <> struct Elem<FRISK_BF16> { typedef __bf16 T; static __device__ float load(const T& x) { return (float)x; } static __device__ T store(float x) { return (__bf16)x; } };

// A rows x cols view is cut into groups of G columns (16 bytes of the narrower type) and walked without any division:
// 2^lanes_log2 lanes of a work-group lie along a row, the remaining 256 >> lanes_log2 across rows, work-groups step
// along the row in x and down the rows in y.  Every lane handles several groups per step, all loads issued before the
// first store: two neighbours along the row (4 KiB apart) where the row is long enough to give both of them work
// (ALONG; more than two measured slower), else the same columns of eight rows.
constexpr int kPerLaneAlong = 2, kPerLaneAcross = 8;

template <bool ALONG> struct Walk {
  static constexpr int PER = ALONG ? kPerLaneAlong : kPerLaneAcross;
  int64_t slabs, row_blocks, rows, groups_per_row;
  int lanes, lane_group, lane_row, row_step;
  __device__ Walk(int64_t rows_, int64_t groups_per_row_, int lanes_log2) : rows(rows_), groups_per_row(groups_per_row_) {
    lanes = 1 << lanes_log2;
    row_step = 256 >> lanes_log2;
    lane_group = threadIdx.x & (lanes - 1);
    lane_row = threadIdx.x >> lanes_log2;
    const int64_t per_x = (int64_t)lanes * (ALONG ? PER : 1), per_y = (int64_t)row_step * (ALONG ? 1 : PER);
    slabs = (groups_per_row + per_x - 1) / per_x;
    row_blocks = (rows + per_y - 1) / per_y;
  }
  // the u-th group of this lane in step (slab, rb); false when it lies outside the view
  __device__ bool at(int64_t slab, int64_t rb, int u, int64_t& row, int64_t& group) const {
    group = (ALONG ? slab * PER + u : slab) * lanes + lane_group;
    row = (ALONG ? rb : rb * PER + u) * row_step + lane_row;
    return group < groups_per_row && row < rows;
  }
};

template <int DT, bool ALONG> __global__ void __launch_bounds__(256)
fill_kernel(typename Elem<DT>::T* dst, int64_t rows, int64_t cols, int64_t ld, float value, int vec_ok, int lanes_log2) {
  typedef typename Elem<DT>::T T;
  constexpr int G = 16 / sizeof(T);
  const Walk<ALONG> w(rows, (cols + G - 1) / G, lanes_log2);
  constexpr int PER = Walk<ALONG>::PER;
  const T v = Elem<DT>::store(value);
  T tmp[G];
#pragma unroll
  for (int e = 0; e < G; ++e) tmp[e] = v;
  for (int64_t rb = blockIdx.y; rb < w.row_blocks; rb += gridDim.y)
    for (int64_t slab = blockIdx.x; slab < w.slabs; slab += gridDim.x) {
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        int64_t r, g;
        if (!w.at(slab, rb, u, r, g)) continue;
        const int64_t c0 = g * G;
        T* p = dst + r * ld + c0;
        if (vec_ok && c0 + G <= cols) store16(p, *(const v4u*)tmp);
        else for (int e = 0; e < G && c0 + e < cols; ++e) p[e] = v;
      }
    }
}

template <int SDT, int DDT, bool ALONG> __device__ __forceinline__ void
copy_window(const typename Elem<SDT>::T* src, int64_t sld, typename Elem<DDT>::T* dst, int64_t dld, int64_t rows, int64_t cols, int vec_ok, int lanes_log2) {
  typedef typename Elem<SDT>::T S;
  typedef typename Elem<DDT>::T D;
  constexpr int G = 16 / (sizeof(S) < sizeof(D) ? sizeof(S) : sizeof(D));  // 16 bytes of the narrower side, 32 of the wider
  const Walk<ALONG> w(rows, (cols + G - 1) / G, lanes_log2);
  constexpr int PER = Walk<ALONG>::PER;
  for (int64_t rb = blockIdx.y; rb < w.row_blocks; rb += gridDim.y)
    for (int64_t slab = blockIdx.x; slab < w.slabs; slab += gridDim.x) {
      S in[PER][G];
      bool whole[PER];
      // every load of the step is issued before the first store
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        int64_t r, g;
        whole[u] = w.at(slab, rb, u, r, g) && vec_ok && g * G + G <= cols;
        if (whole[u]) {
#pragma unroll
          for (int q = 0; q < (int)(G * sizeof(S) / 16); ++q) ((v4u*)in[u])[q] = load16((const v4u*)(src + r * sld + g * G) + q);
        }
      }
#pragma unroll
      for (int u = 0; u < PER; ++u) {
        int64_t r, g;
        if (!w.at(slab, rb, u, r, g)) continue;
        const int64_t c0 = g * G;
        const S* sp = src + r * sld + c0;
        D* dp = dst + r * dld + c0;
        if (whole[u]) {
          D out[G];
#pragma unroll
          for (int e = 0; e < G; ++e) {
            if constexpr (SDT == DDT) out[e] = in[u][e]; else out[e] = Elem<DDT>::store(Elem<SDT>::load(in[u][e]));
          }
#pragma unroll
          for (int q = 0; q < (int)(G * sizeof(D) / 16); ++q) {
            // a lane's two stores of a widening copy each cover half of its 32 bytes: the cache has to merge them
            if constexpr (sizeof(D) > sizeof(S)) store16((v4u*)dp + q, ((const v4u*)out)[q]); else store16_stream((v4u*)dp + q, ((const v4u*)out)[q]);
          }
        } else {
          for (int e = 0; e < G && c0 + e < cols; ++e) {
            if constexpr (SDT == DDT) dp[e] = sp[e]; else dp[e] = Elem<DDT>::store(Elem<SDT>::load(sp[e]));
          }
        }
      }
    }
}

template <int SDT, int DDT, bool ALONG> __global__ void __launch_bounds__(256)
copy_kernel(const typename Elem<SDT>::T* src, int64_t sld, typename Elem<DDT>::T* dst, int64_t dld, int64_t rows, int64_t cols, int vec_ok, int lanes_log2) {
  copy_window<SDT, DDT, ALONG>(src, sld, dst, dld, rows, cols, vec_ok, lanes_log2);
}

// the same window copied once per tile of a placement: z walks the n0 x n1 tiles, each displacing both sides by its steps
template <int SDT, int DDT, bool ALONG> __global__ void __launch_bounds__(256)
copy_tiles_kernel(const typename Elem<SDT>::T* src, int64_t sld, typename Elem<DDT>::T* dst, int64_t dld, int64_t rows, int64_t cols, TilePlacement t, int vec_ok,
                  int lanes_log2) {
  const int64_t tiles = t.n0 * t.n1;
  for (int64_t z = blockIdx.z; z < tiles; z += gridDim.z) {
    const int64_t a = z / t.n1, b = z - a * t.n1;
    copy_window<SDT, DDT, ALONG>(src + a * t.src_step0 + b * t.src_step1, sld, dst + a * t.dst_step0 + b * t.dst_step1, dld, rows, cols, vec_ok, lanes_log2);
  }
}

// ------------------------------------------------------------------ reduce
template <int KIND> struct Op;
template <> struct Op<FRISK_REDUCE_ADD> { static __device__ float id() { return 0.f; } static __device__ float f(float a, float b) { return a + b; } };
template <> struct Op<FRISK_REDUCE_MUL> { static __device__ float id() { return 1.f; } static __device__ float f(float a, float b) { return a * b; } };
template <> struct Op<FRISK_REDUCE_MIN> { static __device__ float id() { return __builtin_inff(); } static __device__ float f(float a, float b) { return __builtin_fminf(a, b); } };
template <> struct Op<FRISK_REDUCE_MAX> { static __device__ float id() { return -__builtin_inff(); } static __device__ float f(float a, float b) { return __builtin_fmaxf(a, b); } };

template <int KIND> __device__ __forceinline__ float wave_reduce(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v = Op<KIND>::f(v, __shfl_xor(v, off, 64));
  return v;
}

// along dim 1: work-group (x = row, y = column slice) reduces every gridDim.y-th run of 256 16-byte groups of one row, so that
// the slices of a row read neighbouring memory at any time.
// With gridDim.y == 1 the result goes to dst (combined with the old value unless clear), else to partial[y][row].
template <int DT, int KIND> __global__ void __launch_bounds__(256)
reduce_rows_kernel(const typename Elem<DT>::T* src, int64_t rows, int64_t cols, int64_t ld, int clear, typename Elem<DT>::T* dst, float* partial, int vec_ok) {
  typedef typename Elem<DT>::T T;
  constexpr int G = 16 / sizeof(T);
  const int64_t gpr = (cols + G - 1) / G;
  __shared__ float wsum[4];
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    float acc = Op<KIND>::id();
    const T* row = src + r * ld;
    for (int64_t g = (int64_t)blockIdx.y * 256 + threadIdx.x; g < gpr; g += (int64_t)gridDim.y * 256) {
      const int64_t c0 = g * G;
      if (vec_ok && c0 + G <= cols) {
        T in[G];
        *(v4u*)in = load16(row + c0);
#pragma unroll
        for (int e = 0; e < G; ++e) acc = Op<KIND>::f(acc, Elem<DT>::load(in[e]));
      } else {
        for (int e = 0; e < G && c0 + e < cols; ++e) acc = Op<KIND>::f(acc, Elem<DT>::load(row[c0 + e]));
      }
    }
    acc = wave_reduce<KIND>(acc);
    if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
      float v = Op<KIND>::f(Op<KIND>::f(wsum[0], wsum[1]), Op<KIND>::f(wsum[2], wsum[3]));
      if (gridDim.y > 1) partial[(int64_t)blockIdx.y * rows + r] = v;
      else dst[r] = Elem<DT>::store(clear ? v : Op<KIND>::f(Elem<DT>::load(dst[r]), v));
    }
    __syncthreads();
  }
}

// along dim 1, rows of at most 256 groups of 16 bytes: 2^lanes_log2 <= 64 lanes of one wave share a row, each taking up to
// NPT groups, and combine by shuffles; a work-group holds 256 >> lanes_log2 rows and takes 4 / NPT such sets of rows per
// step, so that every lane has four loads in flight before the first is used.
template <int DT, int KIND, int NPT> __global__ void __launch_bounds__(256)
reduce_short_rows_kernel(const typename Elem<DT>::T* src, int64_t rows, int64_t cols, int64_t ld, int clear, typename Elem<DT>::T* dst, int vec_ok, int lanes_log2) {
  typedef typename Elem<DT>::T T;
  constexpr int G = 16 / sizeof(T), SETS = 4 / NPT;
  const int lanes = 1 << lanes_log2, lane = threadIdx.x & (lanes - 1), rows_per_set = 256 >> lanes_log2;
  const int64_t blocks = (rows + rows_per_set * SETS - 1) / (rows_per_set * SETS);
  for (int64_t rb = blockIdx.x; rb < blocks; rb += gridDim.x) {
    T in[SETS][NPT][G];
    bool whole[SETS][NPT];
#pragma unroll
    for (int t = 0; t < SETS; ++t) {
      const int64_t r = (rb * SETS + t) * rows_per_set + (threadIdx.x >> lanes_log2);
#pragma unroll
      for (int q = 0; q < NPT; ++q) {
        const int64_t c0 = (int64_t)(q * lanes + lane) * G;
        whole[t][q] = r < rows && vec_ok && c0 + G <= cols;
        if (whole[t][q]) *(v4u*)in[t][q] = load16(src + r * ld + c0);
      }
    }
#pragma unroll
    for (int t = 0; t < SETS; ++t) {
      const int64_t r = (rb * SETS + t) * rows_per_set + (threadIdx.x >> lanes_log2);
      const bool live = r < rows;  // lanes of rows past the end still take part in the shuffles
      float acc = Op<KIND>::id();
#pragma unroll
      for (int q = 0; q < NPT; ++q) {
        const int64_t c0 = (int64_t)(q * lanes + lane) * G;
        if (whole[t][q]) {
#pragma unroll
          for (int e = 0; e < G; ++e) acc = Op<KIND>::f(acc, Elem<DT>::load(in[t][q][e]));
        } else if (live) {
          for (int e = 0; e < G && c0 + e < cols; ++e) acc = Op<KIND>::f(acc, Elem<DT>::load(src[r * ld + c0 + e]));
        }
      }
      for (int off = lanes >> 1; off >= 1; off >>= 1) acc = Op<KIND>::f(acc, __shfl_xor(acc, off, 64));
      if (live && lane == 0) dst[r] = Elem<DT>::store(clear ? acc : Op<KIND>::f(Elem<DT>::load(dst[r]), acc));
    }
  }
}

// along dim 0: a work-group owns a strip of 2^lanes_log2 x G columns and every gridDim.y-th chunk of rows; 2^lanes_log2 column
// lanes x (256 >> lanes_log2) row lanes, kStripFlight rows in flight per lane.  The strip is kStripLanes x 16 bytes of every
// row, or the power of two that covers a narrower view (of a dense one a wave then reads consecutive memory), or wider
// when the view has too few rows to give every row lane a full set of loads.  Four rows in flight (2 to 16 measure within
// 4 % of each other) when the view has many strips; a single strip gives one work-group per slice, 256 at most, and takes
// 16 (5.5 against 4.2 TB/s on a 1M x 128 f16 view).  The row lanes combine by halving in LDS.
constexpr int kStripLanes = 32;  // 16 and 64 lanes measured 9 % and 15 % slower on wide views

template <int DT, int KIND, int kStripFlight> __global__ void __launch_bounds__(256)
reduce_cols_kernel(const typename Elem<DT>::T* src, int64_t rows, int64_t cols, int64_t ld, int clear, typename Elem<DT>::T* dst, float* partial, int vec_ok,
                   int lanes_log2) {
  typedef typename Elem<DT>::T T;
  constexpr int G = 16 / sizeof(T);
  const int cl = threadIdx.x & ((1 << lanes_log2) - 1), rl = threadIdx.x >> lanes_log2, row_lanes = 256 >> lanes_log2;
  const int64_t c0 = (((int64_t)blockIdx.x << lanes_log2) + cl) * G;
  const int64_t chunk = (int64_t)kStripFlight * row_lanes;
  float acc[G];
#pragma unroll
  for (int e = 0; e < G; ++e) acc[e] = Op<KIND>::id();
  if (c0 < cols) {
    const bool whole = vec_ok && c0 + G <= cols;
    for (int64_t base = (int64_t)blockIdx.y * chunk; base < rows; base += (int64_t)gridDim.y * chunk) {
      if (whole && base + chunk <= rows) {
        T in[kStripFlight][G];
#pragma unroll
        for (int u = 0; u < kStripFlight; ++u) *(v4u*)in[u] = load16(src + (base + rl + (int64_t)row_lanes * u) * ld + c0);
#pragma unroll
        for (int u = 0; u < kStripFlight; ++u)
#pragma unroll
          for (int e = 0; e < G; ++e) acc[e] = Op<KIND>::f(acc[e], Elem<DT>::load(in[u][e]));
      } else {
        for (int64_t r = base + rl; r < rows && r < base + chunk; r += row_lanes) {
          const T* p = src + r * ld + c0;
          if (whole) {
            T in[G];
            *(v4u*)in = load16(p);
#pragma unroll
            for (int e = 0; e < G; ++e) acc[e] = Op<KIND>::f(acc[e], Elem<DT>::load(in[e]));
          } else {
            for (int e = 0; e < G && c0 + e < cols; ++e) acc[e] = Op<KIND>::f(acc[e], Elem<DT>::load(p[e]));
          }
        }
      }
    }
  }
  __shared__ float red[256][G + 1];  // [row lane * column lanes + column lane]
#pragma unroll
  for (int e = 0; e < G; ++e) red[threadIdx.x][e] = acc[e];
  __syncthreads();
  for (int half = row_lanes >> 1; half >= 1; half >>= 1) {
    if (rl < half) {
#pragma unroll
      for (int e = 0; e < G; ++e) red[threadIdx.x][e] = Op<KIND>::f(red[threadIdx.x][e], red[threadIdx.x + (half << lanes_log2)][e]);
    }
    __syncthreads();
  }
  if (rl == 0 && c0 < cols) {
    for (int e = 0; e < G && c0 + e < cols; ++e) {
      const float v = red[cl][e];
      if (gridDim.y > 1) partial[(int64_t)blockIdx.y * cols + c0 + e] = v;
      else dst[c0 + e] = Elem<DT>::store(clear ? v : Op<KIND>::f(Elem<DT>::load(dst[c0 + e]), v));
    }
  }
}

// second pass of a split reduction: out[i] = kind over s of partial[s][i] (combined with dst unless clear).  64 outputs x 4
// slice lanes per work-group: a lane combines every fourth slice with four loads in flight, so that 256 slices cost 16
// memory round trips instead of 256.
template <int DT, int KIND> __global__ void __launch_bounds__(256)
reduce_finish_kernel(const float* partial, int slices, int64_t n, int clear, typename Elem<DT>::T* dst) {
  const int ol = threadIdx.x & 63, sl = threadIdx.x >> 6;
  const int64_t i = (int64_t)blockIdx.x * 64 + ol;
  float v = Op<KIND>::id();
  if (i < n) {
    int s = sl;
    for (; s + 12 < slices; s += 16) {
      float t[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) t[u] = partial[(int64_t)(s + 4 * u) * n + i];
#pragma unroll
      for (int u = 0; u < 4; ++u) v = Op<KIND>::f(v, t[u]);
    }
    for (; s < slices; s += 4) v = Op<KIND>::f(v, partial[(int64_t)s * n + i]);
  }
  __shared__ float red[4][64];
  red[sl][ol] = v;
  __syncthreads();
  if (sl == 0 && i < n) {
    v = Op<KIND>::f(Op<KIND>::f(red[0][ol], red[1][ol]), Op<KIND>::f(red[2][ol], red[3][ol]));
    dst[i] = Elem<DT>::store(clear ? v : Op<KIND>::f(Elem<DT>::load(dst[i]), v));
  }
}

// grid and lane split of the division-free walk: lanes along a row = the power of two that covers the row's groups,
// at most 256; x steps along the row, y down the rows (65535 at most, work-groups loop beyond that)
struct WalkLaunch {
  dim3 grid;
  int lanes_log2, along;
  WalkLaunch(int64_t rows, int64_t groups_per_row) {
    lanes_log2 = 0;
    while (lanes_log2 < 8 && (int64_t(1) << lanes_log2) < groups_per_row) ++lanes_log2;
    along = groups_per_row >= 256 * kPerLaneAlong;
    const int kPerLane = along ? kPerLaneAlong : kPerLaneAcross;
    const int64_t per_x = (int64_t(1) << lanes_log2) * (along ? kPerLane : 1), per_y = (int64_t)(256 >> lanes_log2) * (along ? 1 : kPerLane);
    const int64_t slabs = (groups_per_row + per_x - 1) / per_x, row_blocks = (rows + per_y - 1) / per_y;
    grid = dim3((unsigned)(slabs < 1 ? 1 : (slabs > 0x7fffffff ? 0x7fffffff : slabs)), (unsigned)(row_blocks < 1 ? 1 : (row_blocks > 65535 ? 65535 : row_blocks)));
  }
};

template <int DT> hipError_t fill_t(void* dst, int64_t rows, int64_t cols, int64_t ld, double value, int vec_ok, hipStream_t s) {
  typedef typename Elem<DT>::T T;
  constexpr int G = 16 / sizeof(T);
  const WalkLaunch w(rows, (cols + G - 1) / G);
  if (w.along) hipLaunchKernelGGL((fill_kernel<DT, true>), w.grid, dim3(256), 0, s, (T*)dst, rows, cols, ld, (float)value, vec_ok, w.lanes_log2);
  else hipLaunchKernelGGL((fill_kernel<DT, false>), w.grid, dim3(256), 0, s, (T*)dst, rows, cols, ld, (float)value, vec_ok, w.lanes_log2);
  return hipGetLastError();
}

template <int SDT, int DDT> hipError_t copy_t(const void* src, int64_t sld, void* dst, int64_t dld, int64_t rows, int64_t cols, int vec_ok, hipStream_t s) {
  typedef typename Elem<SDT>::T S;
  typedef typename Elem<DDT>::T D;
  constexpr int G = 16 / (sizeof(S) < sizeof(D) ? sizeof(S) : sizeof(D));
  const WalkLaunch w(rows, (cols + G - 1) / G);
  if (w.along) hipLaunchKernelGGL((copy_kernel<SDT, DDT, true>), w.grid, dim3(256), 0, s, (const S*)src, sld, (D*)dst, dld, rows, cols, vec_ok, w.lanes_log2);
  else hipLaunchKernelGGL((copy_kernel<SDT, DDT, false>), w.grid, dim3(256), 0, s, (const S*)src, sld, (D*)dst, dld, rows, cols, vec_ok, w.lanes_log2);
  return hipGetLastError();
}

template <int SDT, int DDT> hipError_t copy_tiles_t(const void* src, int64_t sld, void* dst, int64_t dld, int64_t rows, int64_t cols, const TilePlacement& t, int vec_ok,
                                                    hipStream_t s) {
  typedef typename Elem<SDT>::T S;
  typedef typename Elem<DDT>::T D;
  constexpr int G = 16 / (sizeof(S) < sizeof(D) ? sizeof(S) : sizeof(D));
  WalkLaunch w(rows, (cols + G - 1) / G);
  const int64_t tiles = t.n0 * t.n1;
  w.grid.z = (unsigned)(tiles > 65535 ? 65535 : tiles);
  if (w.along) hipLaunchKernelGGL((copy_tiles_kernel<SDT, DDT, true>), w.grid, dim3(256), 0, s, (const S*)src, sld, (D*)dst, dld, rows, cols, t, vec_ok, w.lanes_log2);
  else hipLaunchKernelGGL((copy_tiles_kernel<SDT, DDT, false>), w.grid, dim3(256), 0, s, (const S*)src, sld, (D*)dst, dld, rows, cols, t, vec_ok, w.lanes_log2);
  return hipGetLastError();
}

// a launch may hold fewer than 2^32 lanes: grids are capped and work-groups loop
constexpr int64_t kMaxGrid = 1 << 22;

template <int DT, int KIND> hipError_t reduce_t(const void* src, int64_t rows, int64_t cols, int64_t ld, int dim, int clear, void* dst, float* partial,
                                                int slices, int vec_ok, hipStream_t s) {
  typedef typename Elem<DT>::T T;
  constexpr int G = 16 / sizeof(T);
  const int64_t gpr = (cols + G - 1) / G;
  if (dim == 1) {
    if (gpr <= 256 && slices == 1) {
      int lanes_log2 = 0;
      while (lanes_log2 < 6 && (int64_t(1) << lanes_log2) < gpr) ++lanes_log2;
      const int64_t rows_per_step = (256 >> lanes_log2) * (gpr <= 64 ? 4 : (gpr <= 128 ? 2 : 1)), blocks = (rows + rows_per_step - 1) / rows_per_step;
      const dim3 grid((unsigned)(blocks < kMaxGrid ? blocks : kMaxGrid));
      if (gpr <= 64) hipLaunchKernelGGL((reduce_short_rows_kernel<DT, KIND, 1>), grid, dim3(256), 0, s, (const T*)src, rows, cols, ld, clear, (T*)dst, vec_ok, lanes_log2);
      else if (gpr <= 128) hipLaunchKernelGGL((reduce_short_rows_kernel<DT, KIND, 2>), grid, dim3(256), 0, s, (const T*)src, rows, cols, ld, clear, (T*)dst, vec_ok, lanes_log2);
      else hipLaunchKernelGGL((reduce_short_rows_kernel<DT, KIND, 4>), grid, dim3(256), 0, s, (const T*)src, rows, cols, ld, clear, (T*)dst, vec_ok, lanes_log2);
    } else {
      hipLaunchKernelGGL((reduce_rows_kernel<DT, KIND>), dim3((unsigned)(rows < kMaxGrid ? rows : kMaxGrid), (unsigned)slices), dim3(256), 0, s, (const T*)src, rows, cols,
                         ld, clear, (T*)dst, partial, vec_ok);
    }
  } else {
    int lanes_log2 = 0;
    while ((1 << lanes_log2) < kStripLanes && (int64_t(1) << lanes_log2) < gpr) ++lanes_log2;
    while (lanes_log2 < 8 && (int64_t(1) << lanes_log2) < gpr && (256 >> lanes_log2) * 4 > rows) ++lanes_log2;  // few rows: wider strips
    const unsigned strips = (unsigned)((gpr + (1 << lanes_log2) - 1) >> lanes_log2);
    // a view of one strip gives at most one work-group per slice: its lanes keep more rows in flight instead
    if (strips == 1) hipLaunchKernelGGL((reduce_cols_kernel<DT, KIND, 16>), dim3(strips, (unsigned)slices), dim3(256), 0, s, (const T*)src, rows, cols, ld, clear, (T*)dst,
                                        partial, vec_ok, lanes_log2);
    else hipLaunchKernelGGL((reduce_cols_kernel<DT, KIND, 4>), dim3(strips, (unsigned)slices), dim3(256), 0, s, (const T*)src, rows, cols, ld, clear, (T*)dst, partial,
                            vec_ok, lanes_log2);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || slices == 1) return e;
  const int64_t n = dim == 1 ? rows : cols;
  hipLaunchKernelGGL((reduce_finish_kernel<DT, KIND>), dim3((unsigned)((n + 63) / 64)), dim3(256), 0, s, partial, slices, n, clear, (T*)dst);
  return hipGetLastError();
}

template <int DT> hipError_t reduce_k(int kind, const void* src, int64_t rows, int64_t cols, int64_t ld, int dim, int clear, void* dst, float* partial, int slices,
                                      int vec_ok, hipStream_t s) {
  switch (kind) {
    case FRISK_REDUCE_ADD: return reduce_t<DT, FRISK_REDUCE_ADD>(src, rows, cols, ld, dim, clear, dst, partial, slices, vec_ok, s);
    case FRISK_REDUCE_MUL: return reduce_t<DT, FRISK_REDUCE_MUL>(src, rows, cols, ld, dim, clear, dst, partial, slices, vec_ok, s);
    case FRISK_REDUCE_MIN: return reduce_t<DT, FRISK_REDUCE_MIN>(src, rows, cols, ld, dim, clear, dst, partial, slices, vec_ok, s);
    default: return reduce_t<DT, FRISK_REDUCE_MAX>(src, rows, cols, ld, dim, clear, dst, partial, slices, vec_ok, s);
  }
}

}  // namespace

int reduce_slices(int dtype, int64_t rows, int64_t cols, int dim) {
  // Split the reduced extent so that about 1024 work-groups exist, each still reducing at least 16 KiB.
  const int es = dtype == FRISK_F32 ? 4 : 2;
  const int G = 16 / es;
  const int64_t groups = dim == 1 ? rows : (cols + kStripLanes * G - 1) / (kStripLanes * G);
  const int64_t strip_bytes = cols * es < kStripLanes * 16 ? cols * es : kStripLanes * 16;
  const int64_t extent_bytes = dim == 1 ? cols * es : rows * strip_bytes;  // bytes one work-group would walk unsplit
  int slices = 1;
  while (groups * slices < 1024 && extent_bytes / (slices * 2) >= 16384 && slices < 256) slices *= 2;
  return slices;
}

hipError_t launch_fill(int dtype, void* dst, int64_t rows, int64_t cols, int64_t ld, double value, int vec_ok, hipStream_t s) {
  switch (dtype) {
    case FRISK_F32: return fill_t<FRISK_F32>(dst, rows, cols, ld, value, vec_ok, s);
    case FRISK_F16: return fill_t<FRISK_F16>(dst, rows, cols, ld, value, vec_ok, s);
    default: return fill_t<FRISK_BF16>(dst, rows, cols, ld, value, vec_ok, s);
  }
}

hipError_t launch_copy_tiles(int sdt, const void* src, int64_t sld, int ddt, void* dst, int64_t dld, int64_t rows, int64_t cols, const TilePlacement& t, int vec_ok,
                             hipStream_t s) {
#define FRISK_COPY_CASE(S, D) if (sdt == S && ddt == D) return copy_tiles_t<S, D>(src, sld, dst, dld, rows, cols, t, vec_ok, s);
  FRISK_COPY_CASE(FRISK_F32, FRISK_F32) FRISK_COPY_CASE(FRISK_F32, FRISK_F16) FRISK_COPY_CASE(FRISK_F32, FRISK_BF16)
  FRISK_COPY_CASE(FRISK_F16, FRISK_F32) FRISK_COPY_CASE(FRISK_F16, FRISK_F16) FRISK_COPY_CASE(FRISK_F16, FRISK_BF16)
  FRISK_COPY_CASE(FRISK_BF16, FRISK_F32) FRISK_COPY_CASE(FRISK_BF16, FRISK_F16) FRISK_COPY_CASE(FRISK_BF16, FRISK_BF16)
#undef FRISK_COPY_CASE
  return hipErrorInvalidValue;
}

hipError_t launch_copy(int sdt, const void* src, int64_t sld, int ddt, void* dst, int64_t dld, int64_t rows, int64_t cols, int vec_ok, hipStream_t s) {
#define FRISK_COPY_CASE(S, D) if (sdt == S && ddt == D) return copy_t<S, D>(src, sld, dst, dld, rows, cols, vec_ok, s);
  FRISK_COPY_CASE(FRISK_F32, FRISK_F32) FRISK_COPY_CASE(FRISK_F32, FRISK_F16) FRISK_COPY_CASE(FRISK_F32, FRISK_BF16)
  FRISK_COPY_CASE(FRISK_F16, FRISK_F32) FRISK_COPY_CASE(FRISK_F16, FRISK_F16) FRISK_COPY_CASE(FRISK_F16, FRISK_BF16)
  FRISK_COPY_CASE(FRISK_BF16, FRISK_F32) FRISK_COPY_CASE(FRISK_BF16, FRISK_F16) FRISK_COPY_CASE(FRISK_BF16, FRISK_BF16)
#undef FRISK_COPY_CASE
  return hipErrorInvalidValue;
}

hipError_t launch_reduce(int dtype, const void* src, int64_t rows, int64_t cols, int64_t ld, int dim, int kind, int clear, void* dst, float* partial, int slices,
                         int vec_ok, hipStream_t s) {
  switch (dtype) {
    case FRISK_F32: return reduce_k<FRISK_F32>(kind, src, rows, cols, ld, dim, clear, dst, partial, slices, vec_ok, s);
    case FRISK_F16: return reduce_k<FRISK_F16>(kind, src, rows, cols, ld, dim, clear, dst, partial, slices, vec_ok, s);
    default: return reduce_k<FRISK_BF16>(kind, src, rows, cols, ld, dim, clear, dst, partial, slices, vec_ok, s);
  }
}

}  // namespace frisk
