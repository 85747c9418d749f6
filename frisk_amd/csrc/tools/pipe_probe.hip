// Hardware probe for gfx950: what the matrix pipe sustains on its own, and which vector instructions run beside it.
// The kernel designs of gemm_kernel.hip.inc and attention.hip rest on these measurements.
// Build: python -m frisk_amd.build --tools ; run: frisk_amd/lib/pipe_probe
//  1. MFMA-only ceiling: one wave per SIMD, the 16 accumulators of a 128 x 128 wave tile in AGPRs, 4 + 4 operand
//     fragments per K step, no memory traffic; operands constant or pseudo-random per lane and K step (the clock the
//     part holds depends on the values), and the same accumulator 1, 2 or 4 times in a row.
//  2. Vector work between the MFMAs of the same wave (two waves per SIMD): per 4 MFMAs, 16 instructions of one kind on
//     independent registers; time against the MFMAs alone.
//  3. v_permlane32_swap: what the two results hold when both operands are copies of one value.
#include <hip/hip_runtime.h>
#include <cstdio>
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

// ---------------------------------------------------------------- 1
template <int REP, bool RANDOM> __global__ void __launch_bounds__(256) mfma_only(float* out, int iters) {
  v16f acc[16];
  for (int i = 0; i < 16; ++i)
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  v8h a[4][4], b[4][4];  // [K step][atom]
  for (int s = 0; s < 4; ++s)
    for (int i = 0; i < 4; ++i)
      for (int e = 0; e < 8; ++e) {
        a[s][i][e] = RANDOM ? (_Float16)(__sinf(threadIdx.x * 0.37f + s * 1.3f + i * 0.7f + e) * 0.5f) : (_Float16)0.25f;
        b[s][i][e] = RANDOM ? (_Float16)(__cosf(threadIdx.x * 0.11f + s * 0.9f + i * 1.9f + e) * 0.5f) : (_Float16)0.5f;
      }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s0 = 0; s0 < 4; s0 += REP)
#pragma unroll
      for (int g = 0; g < 16; ++g)
#pragma unroll
        for (int s = s0; s < s0 + REP; ++s) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc[g]) : "v"(a[s][g / 4]), "v"(b[s][g % 4]));
  }
  float r = 0;
  for (int i = 0; i < 16; ++i) r += acc[i][i];
  if (r == 12345.678f) out[threadIdx.x] = r;  // keeps the loop alive
}

template <int REP, bool RANDOM> static void run_mfma_only(float* out) {
  const int iters = 4000;
  hipEvent_t e0, e1;
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  float ms = 0;
  for (int rep = 0; rep < 3; ++rep) {
    (void)hipEventRecord(e0);
    mfma_only<REP, RANDOM><<<256, 256>>>(out, iters);
    (void)hipEventRecord(e1);
    (void)hipEventSynchronize(e1);
    (void)hipEventElapsedTime(&ms, e0, e1);
  }
  const double mfmas_per_wave = (double)iters * 64, flop = mfmas_per_wave * 32768 * 1024;
  printf("  %-14s operands, same accumulator %d x in a row: %.3f ms  %.0f TFLOP/s  %.0f MHz at 32 cycles per MFMA\n", RANDOM ? "pseudo-random" : "constant", REP, ms,
         flop / (ms * 1e-3) * 1e-12, mfmas_per_wave * 32 / (ms * 1e3));
}

// ---------------------------------------------------------------- 2
enum { K_NONE, K_FMA, K_EXP, K_DOT2C, K_CVT_PK, K_MAX3, K_FMA_MIX };
template <int KIND> __global__ void __launch_bounds__(512) beside(float* out, int iters) {
  v16f a[4] = {};
  v8h x, y;
  for (int i = 0; i < 8; ++i) {
    x[i] = (_Float16)(threadIdx.x * 0.001f + i);
    y[i] = (_Float16)(i * 0.5f - threadIdx.x * 0.002f);
  }
  float v[32];
  for (int i = 0; i < 32; ++i) v[i] = threadIdx.x * 0.01f + i;
  const float m = 1.0001f;
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(a[q]) : "v"(x), "v"(y));
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int r = (q * 4 + j) % 32;
        float& d = v[r];
        const float s0 = v[(r + 7) % 32], s1 = v[(r + 13) % 32];
        if (KIND == K_FMA) asm volatile("v_fma_f32 %0, %1, %2, %3" : "=v"(d) : "v"(s0), "v"(m), "v"(s1));
        if (KIND == K_EXP) asm volatile("v_exp_f32 %0, %1" : "=v"(d) : "v"(s0));
        if (KIND == K_DOT2C) asm volatile("v_dot2c_f32_f16 %0, %1, %2" : "+v"(d) : "v"(s0), "v"(s1));
        if (KIND == K_CVT_PK) asm volatile("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(d) : "v"(s0), "v"(s1));
        if (KIND == K_MAX3) asm volatile("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(s0), "v"(m), "v"(s1));
        if (KIND == K_FMA_MIX) asm volatile("v_fma_mix_f32 %0, %1, %2, %0 op_sel_hi:[1,0,0]" : "+v"(d) : "v"(s0), "v"(m));
      }
    }
  }
  float r = 0;
  for (int q = 0; q < 4; ++q) r += a[q][q];
  for (int i = 0; i < 32; ++i) r += v[i];
  if (r == 12345.678f) out[threadIdx.x] = r;
}

template <int KIND> static float run_beside(float* out, const char* name, float base) {
  const int iters = 20000;
  hipEvent_t e0, e1;
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  float ms = 0;
  for (int rep = 0; rep < 2; ++rep) {
    (void)hipEventRecord(e0);
    beside<KIND><<<256, 512>>>(out, iters);
    (void)hipEventRecord(e1);
    (void)hipEventSynchronize(e1);
    (void)hipEventElapsedTime(&ms, e0, e1);
  }
  if (base > 0) printf("  4 MFMAs + 16 %-18s %.3f ms  (%+.0f %% against the MFMAs alone)\n", name, ms, (ms / base - 1) * 100);
  else printf("  4 MFMAs alone                  %.3f ms\n", ms);
  return ms;
}

// ---------------------------------------------------------------- 3
__global__ void swap_probe(int* out) {
  const int lane = threadIdx.x;
  const int c = 300 + lane;
  const auto s = __builtin_amdgcn_permlane32_swap(c, c, false, false);
  out[lane] = s[0];
  out[64 + lane] = s[1];
}

int main() {
  float* out;
  if (hipMalloc(&out, 4096) != hipSuccess) {
    printf("no device\n");
    return 1;
  }
  printf("1. MFMA-only loop, v_mfma_f32_32x32x16_f16 at 100 %% issue on every SIMD (nominal 2516.6 TFLOP/s at 2.4 GHz)\n");
  run_mfma_only<1, false>(out);
  run_mfma_only<1, true>(out);
  run_mfma_only<2, true>(out);
  run_mfma_only<4, true>(out);
  printf("2. vector instructions between the MFMAs of the same wave, two waves per SIMD\n");
  const float base = run_beside<K_NONE>(out, "", 0.f);
  run_beside<K_FMA>(out, "v_fma_f32", base);
  run_beside<K_EXP>(out, "v_exp_f32", base);
  run_beside<K_CVT_PK>(out, "v_cvt_pk_f16_f32", base);
  run_beside<K_MAX3>(out, "v_max3_f32", base);
  run_beside<K_FMA_MIX>(out, "v_fma_mix_f32", base);
  run_beside<K_DOT2C>(out, "v_dot2c_f32_f16", base);
  printf("3. v_permlane32_swap(c, c) with c = 300 + lane\n");
  int* d;
  (void)hipMalloc(&d, 512);
  swap_probe<<<1, 64>>>(d);
  int h[128];
  (void)hipMemcpy(h, d, 512, hipMemcpyDeviceToHost);
  printf("  result 0: lane 0 = %d, lane 31 = %d, lane 32 = %d, lane 63 = %d\n", h[0], h[31], h[32], h[63]);
  printf("  result 1: lane 0 = %d, lane 31 = %d, lane 32 = %d, lane 63 = %d\n", h[64], h[95], h[96], h[127]);
  return 0;
}
