// Hardware probe for gfx950 (MI355X): the measurements the LDS cost model and the MFMA fragment
// maps of the GEMM kernels rest on.  Build: python -m frisk_amd.build --tools ; run: frisk_amd/lib/lds_probe
//  1. MFMA fragment maps: every atom is fed random integer matrices packed by the assumed lane layout and
//     compared with a host product.
//  2. ds_read_b64_tr_b16 / _tr_b8: which LDS elements each lane receives.
//  3. raw MFMA rate (all CUs, 4 independent accumulators per wave).
//  4. global_load_lds_dwordx4: where the bytes land in LDS, and its throughput against a register-staged copy.
//  5. LDS cycles per wave-wide instruction for the address patterns in tests/golden/lds_probe_gfx950.json
//     (16 waves of one work-group issue the same access in a loop; cycles = time / instructions at the clock
//     given by the all-lanes-one-bank case, 64 cycles).
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstdint>
#include <vector>
#include <cstring>
#include <cmath>

#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("HIP error %s at %s:%d\n", hipGetErrorString(e), __FILE__, __LINE__); fflush(stdout); exit(2);} } while (0)

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef int i4v __attribute__((ext_vector_type(4)));
typedef int i8v __attribute__((ext_vector_type(8)));
typedef int i16v __attribute__((ext_vector_type(16)));
typedef short s4v __attribute__((ext_vector_type(4)));
typedef int i2v __attribute__((ext_vector_type(2)));

// ---------------- 1. MFMA fragment hypothesis tests ----------------
// A given as [32 or 16][K] row-major float/int in global, B as [K][N]. Pack per hypothesis.
__global__ void k_f16_32x32x16(const float* A, const float* B, float* D) {
  int l = threadIdx.x; half8 a, b;
  for (int e = 0; e < 8; ++e) { int k = 8 * (l / 32) + e; a[e] = (_Float16)A[(l % 32) * 16 + k]; b[e] = (_Float16)B[k * 32 + (l % 32)]; }
  f16v c = {0}; c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  for (int r = 0; r < 16; ++r) { int i = (r % 4) + 8 * (r / 4) + 4 * (l / 32); D[i * 32 + (l % 32)] = c[r]; }
}
__global__ void k_f16_16x16x32(const float* A, const float* B, float* D) {
  int l = threadIdx.x; half8 a, b;
  for (int e = 0; e < 8; ++e) { int k = 8 * (l / 16) + e; a[e] = (_Float16)A[(l % 16) * 32 + k]; b[e] = (_Float16)B[k * 16 + (l % 16)]; }
  f4v c = {0}; c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  for (int r = 0; r < 4; ++r) { int i = r + 4 * (l / 16); D[i * 16 + (l % 16)] = c[r]; }
}
__global__ void k_bf16_32x32x16(const float* A, const float* B, float* D) {
  int l = threadIdx.x; bf8 a, b;
  for (int e = 0; e < 8; ++e) { int k = 8 * (l / 32) + e; a[e] = (__bf16)A[(l % 32) * 16 + k]; b[e] = (__bf16)B[k * 32 + (l % 32)]; }
  f16v c = {0}; c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  for (int r = 0; r < 16; ++r) { int i = (r % 4) + 8 * (r / 4) + 4 * (l / 32); D[i * 32 + (l % 32)] = c[r]; }
}
__global__ void k_i8_32x32x32(const float* A, const float* B, float* D) {
  int l = threadIdx.x; i4v a, b; signed char* pa = (signed char*)&a; signed char* pb = (signed char*)&b;
  for (int e = 0; e < 16; ++e) { int k = 16 * (l / 32) + e; pa[e] = (signed char)A[(l % 32) * 32 + k]; pb[e] = (signed char)B[k * 32 + (l % 32)]; }
  i16v c = {0}; c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
  for (int r = 0; r < 16; ++r) { int i = (r % 4) + 8 * (r / 4) + 4 * (l / 32); D[i * 32 + (l % 32)] = (float)c[r]; }
}
__global__ void k_i8_16x16x64(const float* A, const float* B, float* D) {
  int l = threadIdx.x; i4v a, b; signed char* pa = (signed char*)&a; signed char* pb = (signed char*)&b;
  for (int e = 0; e < 16; ++e) { int k = 16 * (l / 16) + e; pa[e] = (signed char)A[(l % 16) * 64 + k]; pb[e] = (signed char)B[k * 16 + (l % 16)]; }
  i4v c = {0}; c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
  for (int r = 0; r < 4; ++r) { int i = r + 4 * (l / 16); D[i * 16 + (l % 16)] = (float)c[r]; }
}
// fp8 e4m3 (OCP): small ints 0..3 -> codes: 0->0x00, 1->0x38, 2->0x40, 3->0x44, -1 -> 0xB8 ...
__device__ unsigned char f8code(float v) {
  int s = v < 0; float a = fabsf(v); unsigned char c = 0;
  if (a == 0) c = 0; else if (a == 1) c = 0x38; else if (a == 2) c = 0x40; else if (a == 3) c = 0x44; else if (a == 4) c = 0x48; else c = 0x7F;
  return c | (s ? 0x80 : 0);
}
__global__ void k_f8_32x32x64(const float* A, const float* B, float* D) {
  int l = threadIdx.x; i8v a, b; unsigned char* pa = (unsigned char*)&a; unsigned char* pb = (unsigned char*)&b;
  for (int e = 0; e < 32; ++e) { int k = 32 * (l / 32) + e; pa[e] = f8code(A[(l % 32) * 64 + k]); pb[e] = f8code(B[k * 32 + (l % 32)]); }
  f16v c = {0}; c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
  for (int r = 0; r < 16; ++r) { int i = (r % 4) + 8 * (r / 4) + 4 * (l / 32); D[i * 32 + (l % 32)] = c[r]; }
}
__global__ void k_f8_16x16x128(const float* A, const float* B, float* D) {
  int l = threadIdx.x; i8v a, b; unsigned char* pa = (unsigned char*)&a; unsigned char* pb = (unsigned char*)&b;
  for (int e = 0; e < 32; ++e) { int k = 32 * (l / 16) + e; pa[e] = f8code(A[(l % 16) * 128 + k]); pb[e] = f8code(B[k * 16 + (l % 16)]); }
  f4v c = {0}; c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
  for (int r = 0; r < 4; ++r) { int i = r + 4 * (l / 16); D[i * 16 + (l % 16)] = c[r]; }
}
__global__ void k_f8_16x16x32(const float* A, const float* B, float* D) {  // legacy fp8 mfma, i64 operands
  int l = threadIdx.x; long a, b; unsigned char* pa = (unsigned char*)&a; unsigned char* pb = (unsigned char*)&b;
  for (int e = 0; e < 8; ++e) { int k = 8 * (l / 16) + e; pa[e] = f8code(A[(l % 16) * 32 + k]); pb[e] = f8code(B[k * 16 + (l % 16)]); }
  f4v c = {0}; c = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(a, b, c, 0, 0, 0);
  for (int r = 0; r < 4; ++r) { int i = r + 4 * (l / 16); D[i * 16 + (l % 16)] = c[r]; }
}
__global__ void k_f32_32x32x2(const float* A, const float* B, float* D) {
  int l = threadIdx.x; int k = l / 32;
  float a = A[(l % 32) * 2 + k], b = B[k * 32 + (l % 32)];
  f16v c = {0}; c = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  for (int r = 0; r < 16; ++r) { int i = (r % 4) + 8 * (r / 4) + 4 * (l / 32); D[i * 32 + (l % 32)] = c[r]; }
}
__global__ void k_f32_16x16x4(const float* A, const float* B, float* D) {
  int l = threadIdx.x; int k = l / 16;
  float a = A[(l % 16) * 4 + k], b = B[k * 16 + (l % 16)];
  f4v c = {0}; c = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  for (int r = 0; r < 4; ++r) { int i = r + 4 * (l / 16); D[i * 16 + (l % 16)] = c[r]; }
}

typedef void (*mfma_kern)(const float*, const float*, float*);
static void test_mfma(const char* name, mfma_kern kern, int M, int N, int K, int maxv) {
  std::vector<float> A(M * K), B(K * N), D(M * N), R(M * N, 0.f);
  srand(123);
  for (auto& x : A) x = (float)(rand() % (2 * maxv + 1) - maxv);
  for (auto& x : B) x = (float)(rand() % (2 * maxv + 1) - maxv);
  for (int i = 0; i < M; ++i) for (int j = 0; j < N; ++j) { double s = 0; for (int k = 0; k < K; ++k) s += (double)A[i * K + k] * B[k * N + j]; R[i * N + j] = (float)s; }
  float *dA, *dB, *dD; CK(hipMalloc(&dA, A.size() * 4)); CK(hipMalloc(&dB, B.size() * 4)); CK(hipMalloc(&dD, D.size() * 4));
  CK(hipMemcpy(dA, A.data(), A.size() * 4, hipMemcpyHostToDevice)); CK(hipMemcpy(dB, B.data(), B.size() * 4, hipMemcpyHostToDevice));
  CK(hipMemset(dD, 0xff, D.size() * 4));
  hipLaunchKernelGGL(kern, dim3(1), dim3(64), 0, 0, dA, dB, dD); CK(hipDeviceSynchronize());
  CK(hipMemcpy(D.data(), dD, D.size() * 4, hipMemcpyDeviceToHost));
  int bad = 0; for (int i = 0; i < M * N; ++i) if (D[i] != R[i]) ++bad;
  printf("MFMA %-18s M=%d N=%d K=%d mismatches=%d  %s\n", name, M, N, K, bad, bad ? "FAIL" : "ok"); fflush(stdout);
  hipFree(dA); hipFree(dB); hipFree(dD);
}

// ---------------- 2. transpose reads ----------------
__global__ void k_tr16(unsigned short* out, int stride_bytes) {
  __shared__ unsigned short lds[4096];
  for (int i = threadIdx.x; i < 4096; i += 64) lds[i] = (unsigned short)i;
  __syncthreads();
  int l = threadIdx.x;
  typedef __attribute__((address_space(3))) s4v* lp;
  s4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lp)((__attribute__((address_space(3))) char*)lds + l * stride_bytes));
  for (int e = 0; e < 4; ++e) out[l * 4 + e] = (unsigned short)v[e];
}
__global__ void k_tr8(unsigned char* out, int stride_bytes) {
  __shared__ unsigned char lds[4096];
  for (int i = threadIdx.x; i < 4096; i += 64) lds[i] = (unsigned char)(i & 0xff);
  __syncthreads();
  int l = threadIdx.x;
  typedef __attribute__((address_space(3))) i2v* lp;
  i2v v = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lp)((__attribute__((address_space(3))) char*)lds + l * stride_bytes));
  unsigned char* p = (unsigned char*)&v;
  for (int e = 0; e < 8; ++e) out[l * 8 + e] = p[e];
}

// ---------------- 4. raw MFMA peak ----------------
template <int KIND>
__global__ void __launch_bounds__(256) k_peak(float* out, int iters) {
  f16v c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
  f4v d0 = {0}, d1 = {0}, d2 = {0}, d3 = {0};
  i16v e0 = {0}, e1 = {0}, e2 = {0}, e3 = {0};
  half8 a; i4v ai; i8v af;
  for (int e = 0; e < 8; ++e) { a[e] = (_Float16)(threadIdx.x * 0.001f); af[e] = threadIdx.x; }
  for (int e = 0; e < 4; ++e) ai[e] = threadIdx.x;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (KIND == 0) { c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, a, c0, 0, 0, 0); c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, a, c1, 0, 0, 0); c2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, a, c2, 0, 0, 0); c3 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, a, c3, 0, 0, 0); }
      if (KIND == 1) { d0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, a, d0, 0, 0, 0); d1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, a, d1, 0, 0, 0); d2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, a, d2, 0, 0, 0); d3 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, a, d3, 0, 0, 0); }
      if (KIND == 2) { e0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(ai, ai, e0, 0, 0, 0); e1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(ai, ai, e1, 0, 0, 0); e2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(ai, ai, e2, 0, 0, 0); e3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(ai, ai, e3, 0, 0, 0); }
      if (KIND == 3) { c0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af, af, c0, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F); c1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af, af, c1, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F); c2 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af, af, c2, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F); c3 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af, af, c3, 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F); }
    }
  }
  float s = 0;
  for (int r = 0; r < 16; ++r) s += c0[r] + c1[r] + c2[r] + c3[r] + (float)(e0[r] + e1[r] + e2[r] + e3[r]);
  for (int r = 0; r < 4; ++r) s += d0[r] + d1[r] + d2[r] + d3[r];
  if (s == 12345.678f) out[0] = s;
}
template <int KIND>
static void peak(const char* name, double flop_per_mfma, int wg_per_cu) {
  float* d; CK(hipMalloc(&d, 4));
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  int iters = 20000; int grid = 256 * wg_per_cu;
  hipLaunchKernelGGL(k_peak<KIND>, dim3(grid), dim3(256), 0, 0, d, 1000);
  for (int rep = 0; rep < 3; ++rep) {
    CK(hipEventRecord(e0, 0));
    hipLaunchKernelGGL(k_peak<KIND>, dim3(grid), dim3(256), 0, 0, d, iters);
    CK(hipEventRecord(e1, 0)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    double flops = (double)grid * 4 /*waves*/ * iters * 16.0 * flop_per_mfma;
    printf("PEAK %-16s wg/cu=%d: %.1f ms  %.1f TFLOP/s\n", name, wg_per_cu, ms, flops / (ms * 1e-3) / 1e12); fflush(stdout);
  }
  hipFree(d);
}

typedef int i4v_ __attribute__((ext_vector_type(4)));
#define LDSP(p) ((__attribute__((address_space(3))) void*)(p))
__global__ void k_dma_sem(const int* g, int* out, int lds_off_bytes, int imm_variant) {
  __shared__ int lds[4096];
  for (int i = threadIdx.x; i < 4096; i += blockDim.x) lds[i] = -1;
  __syncthreads();
  int l = threadIdx.x;
  // lane l loads 16 B from g + perm(l)*16 where perm(l) = l ^ 5
  const int* src = g + ((l ^ 5) * 4);
  if (imm_variant == 0) __builtin_amdgcn_global_load_lds(src, LDSP((char*)lds + lds_off_bytes), 16, 0, 0);
  else __builtin_amdgcn_global_load_lds(src, LDSP((char*)lds + lds_off_bytes), 16, 2048, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  for (int i = threadIdx.x; i < 4096; i += blockDim.x) out[i] = lds[i];
}

// throughput of direct-to-LDS loads: each wave loads `n` KiB-chunks per iteration from an L2-resident buffer
__global__ void __launch_bounds__(256) k_dma_tp(const char* g, int iters, int* sink) {
  __shared__ char lds[65536];
  int l = threadIdx.x & 63, w = threadIdx.x >> 6;
  const char* src = g + (size_t)(blockIdx.x % 256) * 65536 + w * 16384 + l * 16;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 16; ++u)
      __builtin_amdgcn_global_load_lds((const int*)(src + u * 1024), LDSP(lds + w * 16384 + u * 1024), 16, 0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __syncthreads();
  if (iters < 0) sink[0] = lds[threadIdx.x];
}
// same via registers: global_load_dwordx4 + ds_write_b128
__global__ void __launch_bounds__(256) k_reg_tp(const char* g, int iters, int* sink) {
  __shared__ char lds[65536];
  int l = threadIdx.x & 63, w = threadIdx.x >> 6;
  const char* src = g + (size_t)(blockIdx.x % 256) * 65536 + w * 16384 + l * 16;
  for (int it = 0; it < iters; ++it) {
    i4v v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) v[u] = __builtin_nontemporal_load((const i4v*)(src + u * 1024));
#pragma unroll
    for (int u = 0; u < 16; ++u) *(i4v*)(lds + w * 16384 + u * 1024 + l * 16) = v[u];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
  __syncthreads();
  if (iters < 0) sink[0] = lds[threadIdx.x];
}

template <int MODE>
__global__ void __launch_bounds__(1024) k_lds(const int* addr, int iters, int* sink) {
  __shared__ int lds[16384];
  for (int i = threadIdx.x; i < 16384; i += blockDim.x) lds[i] = i;
  __syncthreads();
  int a = addr[threadIdx.x & 63];
  unsigned base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) int*)lds + a;
  int acc = 0;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (MODE == 1) { i2v v; asm volatile("ds_read_b64 %0, %1" : "=v"(v) : "v"(base)); asm volatile("s_waitcnt lgkmcnt(4)" ::: "memory"); acc ^= v[0]; }
      if (MODE == 2) { i4v v; asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(base)); asm volatile("s_waitcnt lgkmcnt(4)" ::: "memory"); acc ^= v[0]; }
      if (MODE == 3) { i2v v; asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v) : "v"(base)); asm volatile("s_waitcnt lgkmcnt(4)" ::: "memory"); acc ^= v[0]; }
      if (MODE == 6) { i2v v; asm volatile("ds_read_b64_tr_b8 %0, %1" : "=v"(v) : "v"(base)); asm volatile("s_waitcnt lgkmcnt(4)" ::: "memory"); acc ^= v[0]; }
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  if (acc == 0x7fffffff) sink[0] = acc + lds[threadIdx.x];
}
static int* d_addr; static int* d_sink;
template <int MODE>
static float time_lds(const int* addr_host, int waves = 16) {
  CK(hipMemcpy(d_addr, addr_host, 64 * 4, hipMemcpyHostToDevice));
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  const int iters = 4000;
  hipLaunchKernelGGL(k_lds<MODE>, dim3(1), dim3(64 * waves), 0, 0, d_addr, 200, d_sink);
  CK(hipEventRecord(e0, 0));
  hipLaunchKernelGGL(k_lds<MODE>, dim3(1), dim3(64 * waves), 0, 0, d_addr, iters, d_sink);
  CK(hipEventRecord(e1, 0)); CK(hipEventSynchronize(e1));
  float ms; CK(hipEventElapsedTime(&ms, e0, e1));
  CK(hipEventDestroy(e0)); CK(hipEventDestroy(e1));
  return ms * 1e6f / (iters * 8.0f * waves) / 0.4156f;  // cycles per wave-instruction at 2.406 GHz
}

int main() {

  hipDeviceProp_t p; CK(hipGetDeviceProperties(&p, 0));
  printf("device %s arch %s CUs %d clock %d kHz memclk %d kHz L2 %d B lds/block %zu maxSharedPerMP %zu regs/block %d\n",
         p.name, p.gcnArchName, p.multiProcessorCount, p.clockRate, p.memoryClockRate, p.l2CacheSize, p.sharedMemPerBlock, p.maxSharedMemoryPerMultiProcessor, p.regsPerBlock);
  fflush(stdout);
  test_mfma("f16_32x32x16", k_f16_32x32x16, 32, 32, 16, 3);
  test_mfma("f16_16x16x32", k_f16_16x16x32, 16, 16, 32, 3);
  test_mfma("bf16_32x32x16", k_bf16_32x32x16, 32, 32, 16, 3);
  test_mfma("i8_32x32x32", k_i8_32x32x32, 32, 32, 32, 127);
  test_mfma("i8_16x16x64", k_i8_16x16x64, 16, 16, 64, 127);
  test_mfma("f8f6f4_32x32x64", k_f8_32x32x64, 32, 32, 64, 3);
  test_mfma("f8f6f4_16x16x128", k_f8_16x16x128, 16, 16, 128, 3);
  test_mfma("fp8_16x16x32", k_f8_16x16x32, 16, 16, 32, 3);
  test_mfma("f32_32x32x2", k_f32_32x32x2, 32, 32, 2, 100);
  test_mfma("f32_16x16x4", k_f32_16x16x4, 16, 16, 4, 100);

  {
    unsigned short* d; CK(hipMalloc(&d, 64 * 4 * 2)); std::vector<unsigned short> h(256);
    for (int stride : {8, 32, 64}) {
      hipLaunchKernelGGL(k_tr16, dim3(1), dim3(64), 0, 0, d, stride); CK(hipDeviceSynchronize());
      CK(hipMemcpy(h.data(), d, 512, hipMemcpyDeviceToHost));
      printf("TR16 lane-address stride %d bytes; per lane 4 values = u16 element index in LDS:\n", stride);
      for (int l = 0; l < 64; ++l) { printf("  l%02d: %4d %4d %4d %4d", l, h[l * 4], h[l * 4 + 1], h[l * 4 + 2], h[l * 4 + 3]); if (l % 4 == 3) printf("\n"); }
    }
    unsigned char* d8; CK(hipMalloc(&d8, 64 * 8)); std::vector<unsigned char> h8(512);
    for (int stride : {8, 16}) {
      hipLaunchKernelGGL(k_tr8, dim3(1), dim3(64), 0, 0, d8, stride); CK(hipDeviceSynchronize());
      CK(hipMemcpy(h8.data(), d8, 512, hipMemcpyDeviceToHost));
      printf("TR8 lane-address stride %d bytes; per lane 8 values = byte index (mod 256) in LDS:\n", stride);
      for (int l = 0; l < 64; ++l) { printf("  l%02d:", l); for (int e = 0; e < 8; ++e) printf(" %3d", h8[l * 8 + e]); if (l % 2 == 1) printf("\n"); }
    }
    fflush(stdout);
  }

  peak<0>("f16_32x32x16", 2.0 * 32 * 32 * 16, 1);
  peak<0>("f16_32x32x16", 2.0 * 32 * 32 * 16, 2);
  peak<1>("f16_16x16x32", 2.0 * 16 * 16 * 32, 2);
  peak<2>("i8_32x32x32", 2.0 * 32 * 32 * 32, 2);
  peak<3>("f8f6f4_32x32x64", 2.0 * 32 * 32 * 64, 2);


  // ---- DMA semantics
  {
    std::vector<int> h(4096); for (int i = 0; i < 4096; ++i) h[i] = i;
    int *g, *o; CK(hipMalloc(&g, 16384)); CK(hipMalloc(&o, 16384));
    CK(hipMemcpy(g, h.data(), 16384, hipMemcpyHostToDevice));
    for (int variant = 0; variant < 2; ++variant) {
      hipLaunchKernelGGL(k_dma_sem, dim3(1), dim3(64), 0, 0, g, o, 1024, variant); CK(hipDeviceSynchronize());
      std::vector<int> r(4096); CK(hipMemcpy(r.data(), o, 16384, hipMemcpyDeviceToHost));
      printf("DMA variant %d (lds base +1024 B, imm %d): nonneg entries (lds dword idx: value):\n", variant, variant ? 2048 : 0);
      int cnt = 0;
      for (int i = 0; i < 4096; ++i) if (r[i] != -1) { if (cnt < 24 || cnt % 64 == 0) printf("  [%d]=%d", i, r[i]); ++cnt; }
      printf("\n  total written dwords = %d\n", cnt);
    }
    fflush(stdout);
  }
  // ---- DMA throughput
  {
    char* g; CK(hipMalloc(&g, 256 * 65536)); CK(hipMemset(g, 1, 256 * 65536));
    int* sink; CK(hipMalloc(&sink, 64));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    for (int mode = 0; mode < 2; ++mode) for (int grid : {1, 32, 256, 512}) {
      int iters = 2000;
      if (mode == 0) hipLaunchKernelGGL(k_dma_tp, dim3(grid), dim3(256), 0, 0, g, 100, sink); else hipLaunchKernelGGL(k_reg_tp, dim3(grid), dim3(256), 0, 0, g, 100, sink);
      CK(hipEventRecord(e0, 0));
      if (mode == 0) hipLaunchKernelGGL(k_dma_tp, dim3(grid % 256 == 0 ? grid : grid), dim3(256), 0, 0, g, iters, sink); else hipLaunchKernelGGL(k_reg_tp, dim3(grid), dim3(256), 0, 0, g, iters, sink);
      CK(hipEventRecord(e1, 0)); CK(hipEventSynchronize(e1));
      float ms; CK(hipEventElapsedTime(&ms, e0, e1));
      double bytes_per_wg = (double)iters * 65536;
      int wg_per_cu = grid > 256 ? 2 : 1;
      printf("%s grid=%d: %.3f ms -> %.1f B/clk/CU (@2.4GHz), total %.2f TB/s\n", mode ? "REGSTAGE" : "DMA2LDS ", grid, ms,
             bytes_per_wg * wg_per_cu / (ms * 1e-3 * 2.4e9), bytes_per_wg * grid / (ms * 1e-3) / 1e12);
    }
    fflush(stdout);
  }
  CK(hipMalloc(&d_addr, 256)); CK(hipMalloc(&d_sink, 256));
  int addr[64];
  // ---- b128 grouping: lanes l and l^d conflict (same bank set, other rows) for a single d; everything else distinct banks in 16-lane consecutive groups
  // pattern: addr(l) = (l%16)*16 + (l/16)*256*? ... base linear pattern is l*16 (4 cycles). Variation: swap so that lanes l and l+D map to same 16B bank slot.
  for (int D : {1, 2, 4, 8, 16, 32}) {
    // slot(l) = bits of l with bit D removed -> 5 bits -> 32 slots; slot%16 is the bank group, rows differ
    for (int l = 0; l < 64; ++l) {
      int lo = l & (D - 1), hi = (l >> 1) & ~(D - 1);
      int slot = hi | lo;               // 0..31
      int bit = (l / D) & 1;
      addr[l] = (slot % 16) * 16 + (slot / 16) * 256 + bit * 512;   // lanes differing only in bit D: same banks, different row
    }
    printf("B128 pairD=%2d : %.2f cyc\n", D, time_lds<2>(addr));
  }
  // fragment-read patterns for K-contig tile with ROWB=128: row = l%32, chunk c = l/32, swizzles
  for (int sw = 0; sw < 4; ++sw) {
    for (int l = 0; l < 64; ++l) {
      int row = l % 32, c = l / 32;
      int f = sw == 0 ? 0 : sw == 1 ? (row & 7) : sw == 2 ? ((row >> 1) & 7) : ((row >> 2) & 7);
      addr[l] = row * 128 + ((c ^ f) * 16);
    }
    printf("B128 frag rowb128 swizzle%d : %.2f cyc\n", sw, time_lds<2>(addr));
  }
  // padded row 144
  for (int l = 0; l < 64; ++l) addr[l] = (l % 32) * 144 + (l / 32) * 16;
  printf("B128 frag rowb144 padded : %.2f cyc\n", time_lds<2>(addr));
  // tr16 B-operand patterns: MN-contig tile ROWB=512, block b=l/16, L=l%16: row = 8*(b/2) + L/4, byte col = 32*(b%2) + 8*(L%4)
  for (int sw = 0; sw < 5; ++sw) {
    for (int l = 0; l < 64; ++l) {
      int b = l / 16, L = l % 16;
      int row = 8 * (b / 2) + L / 4, colb = 32 * (b % 2) + 8 * (L % 4);
      int c = colb / 16, within = colb % 16;
      int x = sw == 0 ? 0 : sw == 1 ? ((row & 3) << 2) : sw == 2 ? ((row & 7) << 1) : sw == 3 ? ((row & 3) << 1) : (row & 7) << 2;
      addr[l] = row * 512 + ((c ^ x) * 16) + within;
    }
    printf("TR16 frag rowb512 swizzle%d : %.2f cyc\n", sw, time_lds<3>(addr));
  }
  // tr8 B-operand patterns: MN-contig tile ROWB=256, block b, L: row = 16*(b/2) + L/2, byte col = 16*(b%2) + 8*(L%2)
  for (int sw = 0; sw < 4; ++sw) {
    for (int l = 0; l < 64; ++l) {
      int b = l / 16, L = l % 16;
      int row = 16 * (b / 2) + L / 2, colb = 16 * (b % 2) + 8 * (L % 2);
      int c = colb / 16, within = colb % 16;
      int x = sw == 0 ? 0 : sw == 1 ? ((row & 7) << 1) : sw == 2 ? (row & 15) : ((row & 3) << 2);
      addr[l] = row * 256 + ((c ^ x) * 16) + within;
    }
    printf("TR8 frag rowb256 swizzle%d : %.2f cyc\n", sw, time_lds<6>(addr));
  }
  // issue-rate floor with fewer waves
  for (int l = 0; l < 64; ++l) addr[l] = l * 16;
  for (int w : {1, 2, 4, 8, 16}) printf("B128 linear waves=%d: %.2f cyc/inst\n", w, time_lds<2>(addr, w));
  for (int l = 0; l < 64; ++l) addr[l] = l * 8;
  for (int w : {4, 8, 16}) printf("B64 linear waves=%d: %.2f cyc/inst  TR16: %.2f\n", w, time_lds<1>(addr, w), time_lds<3>(addr, w));
    printf("DONE\n");
  return 0;
}
