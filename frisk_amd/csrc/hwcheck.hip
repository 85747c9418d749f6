// libfrisk_hwcheck.so: device checks and a measurement that sit beside the product library, for the tests and the
// benchmark only.  Nothing in libfrisk_hip.so calls into this file.
//
//  1. frisk_hwcheck_mfma_atom: one MFMA instruction per atom of gfx950, operands packed by the lane convention the
//     GEMM kernels assume (the counterpart of the reference's NVIDIA fragment atoms makeFragment8x4/8x8/8x16,
//     lib/Dialect/Frisk/IR/FriskOps.cpp:233-287), so a host product can confirm the convention on the device.
//  2. frisk_hwcheck_fragment_path: the product's own LDS tile layout, fragment reader and MFMA wrapper
//     (TileLayout, FragReader, Mma of gemm_kernel.hip.inc) on one K tile of one wave, accumulators written out by the
//     accumulator convention of the epilogue.
//  3. frisk_hwcheck_tr_read: what each lane receives from ds_read_b64_tr_b16 / ds_read_b64_tr_b8 for given lane addresses.
//  4. frisk_hwcheck_mfma_loop: a loop of nothing but MFMAs, one wave per SIMD, accumulators of a 128 x 128 wave tile,
//     operands in registers (constant or pseudo-random per lane and register): the rate the matrix pipe sustains
//     when nothing else runs, i.e. an upper bound for any GEMM kernel on the part at its power limit.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#include "gemm_kernel.hip.inc"

using namespace frisk;

namespace frisk_hwcheck {

typedef float f4v __attribute__((ext_vector_type(4)));

// ------------------------------------------------------------------ 1. single atoms
// A is [M][K] and B is [K][N], floats holding small integers; D is [M][N].
// 32-row atoms: lane l holds row / column l % 32, K group l / 32; result register r of lane l is
// D[(r % 4) + 8 * (r / 4) + 4 * (l / 32)][l % 32].  16-row atoms: row / column l % 16, K group l / 16; register r is
// D[r + 4 * (l / 16)][l % 16].
template <int AT> __device__ int d_row(int l, int r) { return AT == 32 ? (r % 4) + 8 * (r / 4) + 4 * (l / 32) : r + 4 * (l / 16); }

__device__ unsigned char e4m3_of_small_int(float v) {  // exact codes of 0, +-1, +-2, +-3, +-4
  const float a = fabsf(v);
  const unsigned char c = a == 0 ? 0 : a == 1 ? 0x38 : a == 2 ? 0x40 : a == 3 ? 0x44 : a == 4 ? 0x48 : 0x7F;
  return c | (v < 0 ? 0x80 : 0);
}

template <int ID> __global__ void __launch_bounds__(64) atom_kernel(const float* A, const float* B, float* D) {
  const int l = threadIdx.x;
  if constexpr (ID == 0 || ID == 2) {  // f16 / bf16 32x32x16
    v8h ah, bh; v8b ab, bb;
    for (int e = 0; e < 8; ++e) {
      const int k = 8 * (l / 32) + e;
      ah[e] = (_Float16)A[(l % 32) * 16 + k]; bh[e] = (_Float16)B[k * 32 + (l % 32)];
      ab[e] = (__bf16)A[(l % 32) * 16 + k]; bb[e] = (__bf16)B[k * 32 + (l % 32)];
    }
    v16f c = {0};
    if (ID == 0) c = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh, c, 0, 0, 0); else c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ab, bb, c, 0, 0, 0);
    for (int r = 0; r < 16; ++r) D[d_row<32>(l, r) * 32 + (l % 32)] = c[r];
  } else if constexpr (ID == 1 || ID == 3) {  // f16 / bf16 16x16x32
    v8h ah, bh; v8b ab, bb;
    for (int e = 0; e < 8; ++e) {
      const int k = 8 * (l / 16) + e;
      ah[e] = (_Float16)A[(l % 16) * 32 + k]; bh[e] = (_Float16)B[k * 16 + (l % 16)];
      ab[e] = (__bf16)A[(l % 16) * 32 + k]; bb[e] = (__bf16)B[k * 16 + (l % 16)];
    }
    f4v c = {0};
    if (ID == 1) c = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, bh, c, 0, 0, 0); else c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ab, bb, c, 0, 0, 0);
    for (int r = 0; r < 4; ++r) D[d_row<16>(l, r) * 16 + (l % 16)] = c[r];
  } else if constexpr (ID == 4) {  // i8 32x32x32
    v4i a, b; signed char* pa = (signed char*)&a; signed char* pb = (signed char*)&b;
    for (int e = 0; e < 16; ++e) { const int k = 16 * (l / 32) + e; pa[e] = (signed char)A[(l % 32) * 32 + k]; pb[e] = (signed char)B[k * 32 + (l % 32)]; }
    v16i c = {0};
    c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
    for (int r = 0; r < 16; ++r) D[d_row<32>(l, r) * 32 + (l % 32)] = (float)c[r];
  } else if constexpr (ID == 5) {  // i8 16x16x64
    v4i a, b; signed char* pa = (signed char*)&a; signed char* pb = (signed char*)&b;
    for (int e = 0; e < 16; ++e) { const int k = 16 * (l / 16) + e; pa[e] = (signed char)A[(l % 16) * 64 + k]; pb[e] = (signed char)B[k * 16 + (l % 16)]; }
    v4i c = {0};
    c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
    for (int r = 0; r < 4; ++r) D[d_row<16>(l, r) * 16 + (l % 16)] = (float)c[r];
  } else if constexpr (ID == 6) {  // f8f6f4 (e4m3) 32x32x64
    v8i a, b; unsigned char* pa = (unsigned char*)&a; unsigned char* pb = (unsigned char*)&b;
    for (int e = 0; e < 32; ++e) { const int k = 32 * (l / 32) + e; pa[e] = e4m3_of_small_int(A[(l % 32) * 64 + k]); pb[e] = e4m3_of_small_int(B[k * 32 + (l % 32)]); }
    v16f c = {0};
    c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);  // zero scale operands: the instruction without block scales, as in the GEMM kernels
    for (int r = 0; r < 16; ++r) D[d_row<32>(l, r) * 32 + (l % 32)] = c[r];
  } else if constexpr (ID == 7) {  // f8f6f4 (e4m3) 16x16x128
    v8i a, b; unsigned char* pa = (unsigned char*)&a; unsigned char* pb = (unsigned char*)&b;
    for (int e = 0; e < 32; ++e) { const int k = 32 * (l / 16) + e; pa[e] = e4m3_of_small_int(A[(l % 16) * 128 + k]); pb[e] = e4m3_of_small_int(B[k * 16 + (l % 16)]); }
    f4v c = {0};
    c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
    for (int r = 0; r < 4; ++r) D[d_row<16>(l, r) * 16 + (l % 16)] = c[r];
  } else if constexpr (ID == 8) {  // fp8 16x16x32 (64-bit operands)
    long a, b; unsigned char* pa = (unsigned char*)&a; unsigned char* pb = (unsigned char*)&b;
    for (int e = 0; e < 8; ++e) { const int k = 8 * (l / 16) + e; pa[e] = e4m3_of_small_int(A[(l % 16) * 32 + k]); pb[e] = e4m3_of_small_int(B[k * 16 + (l % 16)]); }
    f4v c = {0};
    c = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a, b, c, 0, 0, 0);
    for (int r = 0; r < 4; ++r) D[d_row<16>(l, r) * 16 + (l % 16)] = c[r];
  } else if constexpr (ID == 9) {  // f32 32x32x2
    const int k = l / 32;
    v16f c = {0};
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(A[(l % 32) * 2 + k], B[k * 32 + (l % 32)], c, 0, 0, 0);
    for (int r = 0; r < 16; ++r) D[d_row<32>(l, r) * 32 + (l % 32)] = c[r];
  } else {  // f32 16x16x4
    const int k = l / 16;
    f4v c = {0};
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(A[(l % 16) * 4 + k], B[k * 16 + (l % 16)], c, 0, 0, 0);
    for (int r = 0; r < 4; ++r) D[d_row<16>(l, r) * 16 + (l % 16)] = c[r];
  }
}

// ------------------------------------------------------------------ 2. the product's fragment path
// One K tile of the default work-group tile: the stored tiles of A and B (dense, as they lie in memory) are placed in LDS
// chunk by chunk under the tile's swizzle, exactly where the direct-to-LDS stager puts them; wave blockIdx.x of the
// WM x WN grid then reads its fragments with FragReader and runs Mma::run as the main loop does (transposed atoms:
// MFMA "A" operand = fragment of B).  D receives the raw 32-bit accumulators of the whole BM x BN tile.
template <class C> __global__ void __launch_bounds__(64) fragment_path_kernel(const char* A, const char* B, int* D) {
  typedef typename C::M M;
  typedef typename C::LA LA;
  typedef typename C::LB LB;
  typedef FragReader<LA, M::FRAGB, C::AM, C::KSTEPS, 1, C::AT> RA;
  typedef FragReader<LB, M::FRAGB, C::AN, C::KSTEPS, 1, C::AT> RB;
  constexpr int FI = M::FRAGB / 4;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const unsigned smem_u = (unsigned)(uintptr_t)(FRISK_LDS char*)smem;
  const int lane = threadIdx.x;
  const int wm = blockIdx.x / C::WN, wn = blockIdx.x % C::WN;
  for (int ch = lane; ch < LA::BYTES / 16; ch += 64) {
    const int row = (ch * 16) / LA::ROWB, colbyte = (ch * 16) % LA::ROWB;
    *(v4i*)(smem + LA::offset(row, colbyte)) = *(const v4i*)(A + ch * 16);
  }
  for (int ch = lane; ch < LB::BYTES / 16; ch += 64) {
    const int row = (ch * 16) / LB::ROWB, colbyte = (ch * 16) % LB::ROWB;
    *(v4i*)(smem + LA::BYTES + LB::offset(row, colbyte)) = *(const v4i*)(B + ch * 16);
  }
  __syncthreads();
  unsigned ra[RA::NREG], rb[RB::NREG];
  RA::init(lane, wm * C::WTM, 0, ra);
  RB::init(lane, wn * C::WTN, 0, rb);
#pragma unroll
  for (int r = 0; r < RA::NREG; ++r) ra[r] += smem_u;
#pragma unroll
  for (int r = 0; r < RB::NREG; ++r) rb[r] += smem_u + LA::BYTES;
  typename M::Acc acc[C::AM][C::AN];
#pragma unroll
  for (int i = 0; i < C::AM; ++i)
#pragma unroll
    for (int j = 0; j < C::AN; ++j)
#pragma unroll
      for (int r = 0; r < M::NACC; ++r) acc[i][j][r] = 0;
#pragma unroll
  for (int i = 0; i < C::AM; ++i)
#pragma unroll
    for (int j = 0; j < C::AN; ++j) M::settle(acc[i][j]);
  M::drain();
#pragma unroll
  for (int ks = 0; ks < C::KSTEPS; ++ks) {
    int fa[C::AM][FI], fb[C::AN][FI];
#pragma unroll
    for (int i = 0; i < C::AM; ++i) RA::read(ra, i, ks, fa[i]);
#pragma unroll
    for (int j = 0; j < C::AN; ++j) RB::read(rb, j, ks, fb[j]);
#pragma unroll
    for (int i = 0; i < C::AM; ++i)
#pragma unroll
      for (int j = 0; j < C::AN; ++j) {
        typename M::Frag a, b;
        if constexpr (FI == 1) { a = fa[i][0]; b = fb[j][0]; }
        else {
#pragma unroll
          for (int q = 0; q < FI; ++q) { a[q] = fa[i][q]; b[q] = fb[j][q]; }
        }
        M::run(b, a, acc[i][j]);
      }
  }
  M::drain();
  // accumulator convention of the epilogue: register 4q + e of lane l in atom (i, j) is
  // C[i * AT + l % AT][j * AT + (AT == 32 ? 8q + 4 (l / 32) : 4 (l / 16)) + e]
#pragma unroll
  for (int i = 0; i < C::AM; ++i)
#pragma unroll
    for (int j = 0; j < C::AN; ++j)
#pragma unroll
      for (int r = 0; r < M::NACC; ++r) {
        const typename M::AccT t = acc[i][j][r];
        const int q = r / 4, e = r % 4;
        const int row = wm * C::WTM + i * C::AT + (lane & (C::AT - 1));
        const int col = wn * C::WTN + j * C::AT + (C::AT == 32 ? 8 * q + 4 * (lane >> 5) : 4 * (lane >> 4)) + e;
        D[row * C::BN + col] = __builtin_bit_cast(int, t);
      }
}

template <int DT, int AT, int BMN, int BK> struct PathCfg {
  template <bool TA, bool TB> using Cfg = GemmCfg<DT, TA, TB, BMN, BMN, BK, 2, 2, 2, false, false, 1, 2, AT>;
  template <bool TA, bool TB> static hipError_t launch1(const void* A, const void* B, void* D, hipStream_t s) {
    typedef Cfg<TA, TB> C;
    constexpr int LDS = C::LA::BYTES + C::LB::BYTES;
    if (hipError_t e = hipFuncSetAttribute((const void*)fragment_path_kernel<C>, hipFuncAttributeMaxDynamicSharedMemorySize, LDS); e != hipSuccess) return e;
    hipLaunchKernelGGL(fragment_path_kernel<C>, dim3(4), dim3(64), LDS, s, (const char*)A, (const char*)B, (int*)D);
    return hipGetLastError();
  }
  static hipError_t launch(int ta, int tb, const void* A, const void* B, void* D, hipStream_t s) {
    // the atom whose K is the whole K tile exists for K-contiguous operands only (A [M][K], B [N][K])
    if constexpr (DT == FRISK_E4M3 && AT == 16) return !ta && tb ? launch1<false, true>(A, B, D, s) : hipErrorInvalidValue;
    else {
    if (!ta && !tb) return launch1<false, false>(A, B, D, s);
    if (!ta && tb) return launch1<false, true>(A, B, D, s);
    if (ta && !tb) return launch1<true, false>(A, B, D, s);
    return launch1<true, true>(A, B, D, s);
    }
  }
};

// ------------------------------------------------------------------ 3. transpose reads
// LDS holds 16 KiB; element i of the 16-bit view holds i, byte i of the 8-bit view holds (i >> shift) & 255.
__global__ void __launch_bounds__(64) tr16_kernel(const int* lane_addr, unsigned short* out) {
  __shared__ unsigned short lds[8192];
  for (int i = threadIdx.x; i < 8192; i += 64) lds[i] = (unsigned short)i;
  __syncthreads();
  const int l = threadIdx.x;
  const v4s v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((FRISK_LDS v4s*)((FRISK_LDS char*)lds + lane_addr[l]));
  for (int e = 0; e < 4; ++e) out[l * 4 + e] = (unsigned short)v[e];
}
__global__ void __launch_bounds__(64) tr8_kernel(const int* lane_addr, unsigned char* out, int shift) {
  __shared__ unsigned char lds[16384];
  for (int i = threadIdx.x; i < 16384; i += 64) lds[i] = (unsigned char)((i >> shift) & 255);
  __syncthreads();
  const int l = threadIdx.x;
  const v2i v = __builtin_amdgcn_ds_read_tr8_b64_v2i32((FRISK_LDS v2i*)((FRISK_LDS char*)lds + lane_addr[l]));
  const unsigned char* p = (const unsigned char*)&v;
  for (int e = 0; e < 8; ++e) out[l * 8 + e] = p[e];
}

// ------------------------------------------------------------------ 4. MFMA-only loop
// KIND: 0 f16 32x32x16, 1 f16 16x16x32, 2 bf16 32x32x16, 3 bf16 16x16x32, 4 i8 32x32x32, 5 i8 16x16x64,
//       6 f8f6f4 (e4m3) 32x32x64, 7 f8f6f4 (e4m3) 16x16x128
// One wave holds the accumulators of a 128 x 128 tile (256 registers) and the operand fragments of KS K steps; an
// iteration issues every (K step, atom row, atom column) MFMA once.  Nothing else is in the loop.
__device__ float g_sink;

template <int KIND> struct LoopShape {
  static constexpr int AT = (KIND & 1) ? 16 : 32;
  static constexpr int NAT = 128 / AT;                       // atoms per side of the wave tile
  static constexpr int FRAG_INTS = KIND >= 6 ? 8 : 4;        // operand registers per lane and MFMA
  static constexpr int KS = 64 / (NAT * FRAG_INTS);        // K steps whose fragments fit in 64 registers per operand
  static constexpr int MFMAS_PER_ITER = KS * NAT * NAT;
  // flops (ops) of one MFMA: 2 * AT * AT * K of the atom
  static constexpr double K_ATOM = KIND < 4 ? (AT == 32 ? 16 : 32) : KIND < 6 ? (AT == 32 ? 32 : 64) : (AT == 32 ? 64 : 128);
  static constexpr double FLOPS_PER_MFMA = 2.0 * AT * AT * K_ATOM;
  // cycles one MFMA occupies the SIMD's matrix pipe at full rate
  static constexpr int CYCLES_PER_MFMA = AT == 32 ? (KIND >= 6 ? 64 : 32) : (KIND >= 6 ? 32 : 16);
};

// The operands of a data-fed loop: two row-major device arrays (the benchmark's own A and B); `rows` rows of at least 256 bytes; every lane takes its fragments from them exactly as a K-contiguous operand tile would deliver them
// (lane l of an atom: row l % AT, the l / AT-th group of consecutive bytes along the row).
struct LoopData {
  const char* a;
  const char* b;
  long long lda_bytes, ldb_bytes;
  int rows_a, rows_b;
};

template <int KIND, bool RANDOM> __global__ void __launch_bounds__(256) mfma_loop_kernel(int iters, LoopData data) {
#ifdef __HIP_DEVICE_COMPILE__  // the host pass only needs the launch stub; it cannot parse the 256-bit register operands
  typedef LoopShape<KIND> S;
  constexpr int NAT = S::NAT, KS = S::KS, FI = S::FRAG_INTS;
  typedef int frag_t __attribute__((ext_vector_type(FI)));
  typedef typename std::conditional<S::AT == 32, v16f, f4v>::type acc_f;
  typedef typename std::conditional<S::AT == 32, v16i, v4i>::type acc_i;
  typedef typename std::conditional<(KIND == 4 || KIND == 5), acc_i, acc_f>::type acc_t;
  acc_t acc[NAT * NAT];
#pragma unroll
  for (int g = 0; g < NAT * NAT; ++g)
#pragma unroll
    for (int r = 0; r < (S::AT == 32 ? 16 : 4); ++r) acc[g][r] = 0;
  frag_t a[KS][NAT], b[KS][NAT];
  // operand bits: a hash of (lane, register), kept finite for the floating types: f16 +-[0.5, 1), bf16 +-[0.5, 1),
  // e4m3 +-[1, 2); int8 takes the hash as it is.  Constant operands: the same value in every lane and register.
  unsigned h = (threadIdx.x + 1u) * 2246822519u + blockIdx.x * 3266489917u + 374761393u;
#pragma unroll
  for (int s = 0; s < KS; ++s)
#pragma unroll
    for (int i = 0; i < NAT; ++i)
#pragma unroll
      for (int e = 0; e < FI; ++e)
#pragma unroll
        for (int side = 0; side < 2; ++side) {
          h = h * 2654435761u + 40503u;
          unsigned x = h ^ (h >> 7);
          if (!RANDOM) x = 0;
          unsigned bits;
          if (KIND < 2) bits = 0x38003800u | (x & 0x83ff83ffu);
          else if (KIND < 4) bits = 0x3f003f00u | (x & 0x807f807fu);
          else if (KIND < 6) bits = RANDOM ? x : 0x11111111u;
          else bits = 0x38383838u | (x & 0x87878787u);
          if (side == 0) a[s][i][e] = (int)bits; else b[s][i][e] = (int)bits;
        }
  if (data.a) {
    // fragments of real operands: wave w of work-group g owns rows (4 g + w) * 128 ... + 127 of both arrays (modulo
    // their row counts); K step s, lane group l / AT reads FI * 4 consecutive bytes of its row
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row0 = (blockIdx.x * 4 + wave) * 128;
    const int kbyte = (lane / S::AT) * FI * 4;
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int i = 0; i < NAT; ++i) {
        const long long ko = (long long)s * (64 / S::AT) * FI * 4 + kbyte;
        const int ra = (row0 + i * S::AT + lane % S::AT) % data.rows_a, rb = (row0 + i * S::AT + lane % S::AT) % data.rows_b;
        a[s][i] = *(const frag_t*)(data.a + ra * data.lda_bytes + ko);
        b[s][i] = *(const frag_t*)(data.b + rb * data.ldb_bytes + ko);
      }
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int i = 0; i < NAT; ++i)
#pragma unroll
        for (int j = 0; j < NAT; ++j) {
          acc_t& c = acc[i * NAT + j];
          if constexpr (KIND == 0) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a[s][i]), "v"(b[s][j]));
          else if constexpr (KIND == 1) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a[s][i]), "v"(b[s][j]));
          else if constexpr (KIND == 2) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a[s][i]), "v"(b[s][j]));
          else if constexpr (KIND == 3) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a[s][i]), "v"(b[s][j]));
          else if constexpr (KIND == 4) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+a"(c) : "v"(a[s][i]), "v"(b[s][j]));
          else if constexpr (KIND == 5) asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+a"(c) : "v"(a[s][i]), "v"(b[s][j]));
          else if constexpr (KIND == 6) asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(a[s][i]), "v"(b[s][j]));
          else asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(c) : "v"(a[s][i]), "v"(b[s][j]));
        }
  }
  float r = 0;
#pragma unroll
  for (int g = 0; g < NAT * NAT; ++g) r += (float)acc[g][g % 4];
  if (r == 12345.678f) g_sink = r;  // never true for these operands; keeps the accumulators live
#endif
}

template <int KIND> hipError_t launch_loop(int iters, int random_operands, int workgroups, hipStream_t s, const LoopData& data = LoopData{}) {
  if (random_operands) hipLaunchKernelGGL((mfma_loop_kernel<KIND, true>), dim3(workgroups), dim3(256), 0, s, iters, data);
  else hipLaunchKernelGGL((mfma_loop_kernel<KIND, false>), dim3(workgroups), dim3(256), 0, s, iters, data);
  return hipGetLastError();
}

}  // namespace frisk_hwcheck

using namespace frisk_hwcheck;

extern "C" {

// atom ids: 0 f16 32x32x16, 1 f16 16x16x32, 2 bf16 32x32x16, 3 bf16 16x16x32, 4 i8 32x32x32, 5 i8 16x16x64,
// 6 f8f6f4 32x32x64, 7 f8f6f4 16x16x128, 8 fp8 16x16x32, 9 f32 32x32x2, 10 f32 16x16x4.  A [M][K], B [K][N], D [M][N]
// are device arrays of floats holding small integers (|v| <= 4 for the 8-bit floating atoms).  Returns a hipError_t.
int frisk_hwcheck_mfma_atom(int id, const float* A, const float* B, float* D, void* stream) {
  hipStream_t s = (hipStream_t)stream;
  switch (id) {
#define FRISK_ATOM_CASE(N) case N: hipLaunchKernelGGL(atom_kernel<N>, dim3(1), dim3(64), 0, s, A, B, D); break;
    FRISK_ATOM_CASE(0) FRISK_ATOM_CASE(1) FRISK_ATOM_CASE(2) FRISK_ATOM_CASE(3) FRISK_ATOM_CASE(4) FRISK_ATOM_CASE(5)
    FRISK_ATOM_CASE(6) FRISK_ATOM_CASE(7) FRISK_ATOM_CASE(8) FRISK_ATOM_CASE(9) FRISK_ATOM_CASE(10)
#undef FRISK_ATOM_CASE
    default: return -1;
  }
  return (int)hipGetLastError();
}

// One K tile through the product's LDS layout, fragment reader and MFMA wrapper.  dtype: frisk_dtype of A and B; atom 32 or
// 16 (16 only for F16 / BF16 / I8).  The tile is 256 x 256 x (64 | 128 for 8-bit), 128 x 128 x 32 for F32.  A and B are the
// stored tiles, dense: A [BM][BK] (transA: [BK][BM]), B [BK][BN] (transB: [BN][BK]).  D: BM x BN raw 32-bit accumulators.
// Returns a hipError_t, or -1 for a combination that is not compiled.
int frisk_hwcheck_fragment_path(int dtype, int atom, int transA, int transB, const void* A, const void* B, void* D, void* stream) {
  hipStream_t s = (hipStream_t)stream;
  if (dtype == FRISK_F16 && atom == 32) return (int)PathCfg<FRISK_F16, 32, 256, 64>::launch(transA, transB, A, B, D, s);
  if (dtype == FRISK_F16 && atom == 16) return (int)PathCfg<FRISK_F16, 16, 256, 64>::launch(transA, transB, A, B, D, s);
  if (dtype == FRISK_BF16 && atom == 32) return (int)PathCfg<FRISK_BF16, 32, 256, 64>::launch(transA, transB, A, B, D, s);
  if (dtype == FRISK_BF16 && atom == 16) return (int)PathCfg<FRISK_BF16, 16, 256, 64>::launch(transA, transB, A, B, D, s);
  if (dtype == FRISK_I8 && atom == 32) return (int)PathCfg<FRISK_I8, 32, 256, 128>::launch(transA, transB, A, B, D, s);
  if (dtype == FRISK_I8 && atom == 16) return (int)PathCfg<FRISK_I8, 16, 256, 128>::launch(transA, transB, A, B, D, s);
  if (dtype == FRISK_E4M3 && atom == 32) return (int)PathCfg<FRISK_E4M3, 32, 256, 128>::launch(transA, transB, A, B, D, s);
  if (dtype == FRISK_E4M3 && atom == 16) return (int)PathCfg<FRISK_E4M3, 16, 256, 128>::launch(transA, transB, A, B, D, s);
  if (dtype == FRISK_F32 && atom == 32) return (int)PathCfg<FRISK_F32, 32, 128, 32>::launch(transA, transB, A, B, D, s);
  return -1;
}

// bits 16: out receives 64 x 4 uint16 (LDS element i of the 16-bit view holds i); bits 8: 64 x 8 bytes (byte i holds
// (i >> shift) & 255).  lane_addr: 64 byte addresses below 16384 - 8, 8-byte aligned.  Returns a hipError_t.
int frisk_hwcheck_tr_read(int bits, const int* lane_addr, void* out, int shift, void* stream) {
  hipStream_t s = (hipStream_t)stream;
  if (bits == 16) hipLaunchKernelGGL(tr16_kernel, dim3(1), dim3(64), 0, s, lane_addr, (unsigned short*)out);
  else if (bits == 8) hipLaunchKernelGGL(tr8_kernel, dim3(1), dim3(64), 0, s, lane_addr, (unsigned char*)out, shift);
  else return -1;
  return (int)hipGetLastError();
}

// The MFMA-only loop: `workgroups` work-groups of 4 waves (one wave per SIMD when workgroups = number of CUs), `iters`
// iterations.  Returns a hipError_t, or -1 for an unknown kind.
int frisk_hwcheck_mfma_loop(int kind, int iters, int random_operands, int workgroups, void* stream) {
  hipStream_t s = (hipStream_t)stream;
  if (iters < 0 || workgroups <= 0) return -1;
  switch (kind) {
    case 0: return (int)launch_loop<0>(iters, random_operands, workgroups, s);
    case 1: return (int)launch_loop<1>(iters, random_operands, workgroups, s);
    case 2: return (int)launch_loop<2>(iters, random_operands, workgroups, s);
    case 3: return (int)launch_loop<3>(iters, random_operands, workgroups, s);
    case 4: return (int)launch_loop<4>(iters, random_operands, workgroups, s);
    case 5: return (int)launch_loop<5>(iters, random_operands, workgroups, s);
    case 6: return (int)launch_loop<6>(iters, random_operands, workgroups, s);
    case 7: return (int)launch_loop<7>(iters, random_operands, workgroups, s);
    default: return -1;
  }
}

// The same loop with its operand registers loaded once from two row-major device arrays (16-byte aligned rows of at least
// 256 bytes, leading dimensions in bytes): the bits the matrix pipe switches on are then those of the workload itself.
// Returns a hipError_t, -1 for an unknown kind, -2 for arrays that do not fit.
int frisk_hwcheck_mfma_loop_data(int kind, int iters, int workgroups, const void* A, long long lda_bytes, int rows_a, const void* B, long long ldb_bytes,
                                 int rows_b, void* stream) {
  hipStream_t s = (hipStream_t)stream;
  if (iters < 0 || workgroups <= 0) return -1;
  if (!A || !B || rows_a <= 0 || rows_b <= 0 || lda_bytes < 256 || ldb_bytes < 256 || ((uintptr_t)A | (uintptr_t)B | (uintptr_t)lda_bytes | (uintptr_t)ldb_bytes) & 31)
    return -2;
  const LoopData data{(const char*)A, (const char*)B, lda_bytes, ldb_bytes, rows_a, rows_b};
  switch (kind) {
    case 0: return (int)launch_loop<0>(iters, 1, workgroups, s, data);
    case 1: return (int)launch_loop<1>(iters, 1, workgroups, s, data);
    case 2: return (int)launch_loop<2>(iters, 1, workgroups, s, data);
    case 3: return (int)launch_loop<3>(iters, 1, workgroups, s, data);
    case 4: return (int)launch_loop<4>(iters, 1, workgroups, s, data);
    case 5: return (int)launch_loop<5>(iters, 1, workgroups, s, data);
    case 6: return (int)launch_loop<6>(iters, 1, workgroups, s, data);
    case 7: return (int)launch_loop<7>(iters, 1, workgroups, s, data);
    default: return -1;
  }
}

// flops (integer ops) one launch of the loop performs, and the matrix-pipe cycles one wave of it needs at full issue rate
double frisk_hwcheck_mfma_loop_flops(int kind, int iters, int workgroups) {
  double per_wave = 0;
  switch (kind) {
#define FRISK_LOOP_CASE(N) case N: per_wave = (double)LoopShape<N>::MFMAS_PER_ITER * LoopShape<N>::FLOPS_PER_MFMA; break;
    FRISK_LOOP_CASE(0) FRISK_LOOP_CASE(1) FRISK_LOOP_CASE(2) FRISK_LOOP_CASE(3) FRISK_LOOP_CASE(4) FRISK_LOOP_CASE(5) FRISK_LOOP_CASE(6) FRISK_LOOP_CASE(7)
#undef FRISK_LOOP_CASE
    default: return 0;
  }
  return per_wave * (double)iters * 4.0 * (double)workgroups;
}
double frisk_hwcheck_mfma_loop_cycles(int kind, int iters) {
  switch (kind) {
#define FRISK_LOOP_CASE(N) case N: return (double)LoopShape<N>::MFMAS_PER_ITER * LoopShape<N>::CYCLES_PER_MFMA * (double)iters;
    FRISK_LOOP_CASE(0) FRISK_LOOP_CASE(1) FRISK_LOOP_CASE(2) FRISK_LOOP_CASE(3) FRISK_LOOP_CASE(4) FRISK_LOOP_CASE(5) FRISK_LOOP_CASE(6) FRISK_LOOP_CASE(7)
#undef FRISK_LOOP_CASE
    default: return 0;
  }
}

// What the driver reports for the current device: compute units, shader clock and memory clock in kHz, memory bus width in
// bits.  The nominal peaks are priced at 256 CUs x 2.4 GHz and 8 TB/s; this is the figure to hold against them.  Returns a
// hipError_t.
int frisk_hwcheck_device_info(int* compute_units, int* clock_khz, int* memory_clock_khz, int* memory_bus_bits) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  struct { hipDeviceAttribute_t attr; int* out; } want[] = {{hipDeviceAttributeMultiprocessorCount, compute_units},
                                                            {hipDeviceAttributeClockRate, clock_khz},
                                                            {hipDeviceAttributeMemoryClockRate, memory_clock_khz},
                                                            {hipDeviceAttributeMemoryBusWidth, memory_bus_bits}};
  for (auto& w : want) {
    if (!w.out) continue;
    e = hipDeviceGetAttribute(w.out, w.attr, dev);
    if (e != hipSuccess) return (int)e;
  }
  return 0;
}

}  // extern "C"
