/*
 * frisk_oracle.c -- CPU oracle for the tiled GEMM path.  TEST INFRASTRUCTURE ONLY.
 *
 * Nothing that ships (the HIP library, the builder module, the Python package)
 * may link, import or call this file; it is the checker used by tests, by the
 * smoke check and by the CPU-baseline leg of the benchmark.
 *
 * What it restates.  The reference (Xiebaokang/frisk) defines the GEMM only as
 * IR: `frisk.gemm` declares C (+)= op(A) . op(B) on rank-2 memrefs with the
 * attributes transA, transB, M, N, K, clear_accum
 * (include/Dialect/Frisk/IR/FriskOps.td:248-289, verifier
 * lib/Dialect/Frisk/IR/FriskOps.cpp:1264-1283, binding ffi/ir.cpp:322-366),
 * and the tiled program around it is sketched in tmp/ir.mlir:1-17
 * (fill 0 -> for k { copy A; copy B; gemm } -> copy C).  The reference holds no
 * arithmetic and no numerical test vectors for this path, so numerical parity
 * against the reference is UNPINNED; the functions below are pinned instead by
 * mathematics (see tests/test_oracle.py): exhaustive codec round trips against
 * numpy/torch, closed forms (identity, all-ones, rank-1 products), integer
 * exactness, and a naive triple loop on small shapes.
 *
 * Conventions shared with include/frisk_hip.h:
 *   - dtype codes: 0 f32, 1 f16, 2 bf16, 3 i8, 4 e4m3fn (OCP), 5 i32
 *   - transA = 0: A stored [M][K] (lda >= K);  transA = 1: A stored [K][M]
 *   - transB = 0: B stored [K][N] (ldb >= N);  transB = 1: B stored [N][K]
 *   - epilogue ROW_COL_SCALE: out = f16( (float(acc_i32) * sA[m]) * sB[n] )
 *   - epilogue TENSOR_SCALE : out = bf16( (acc_f32 * sA) * sB )
 *   all float->narrow conversions round to nearest even.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

enum { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2, DT_I8 = 3, DT_E4M3 = 4, DT_I32 = 5 };

/* ------------------------------------------------------------------ RNG --- */
/* Counter-based: value i of tensor t under seed s depends only on (s, t, i). */
static inline uint64_t splitmix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}
static inline uint64_t key_hash(uint64_t seed, uint64_t tensor, uint64_t idx) {
  return splitmix64(splitmix64(splitmix64(seed) ^ (tensor * 0xD6E8FEB86659FD93ull)) + idx);
}
static inline double u01(uint64_t h) { return (double)(h >> 11) * (1.0 / 9007199254740992.0); }

ORACLE_API uint64_t oracle_hash(uint64_t seed, uint64_t tensor, uint64_t idx) { return key_hash(seed, tensor, idx); }

ORACLE_API void oracle_fill_uniform_f32(float* out, int64_t n, uint64_t seed, uint64_t tensor, float lo, float hi) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) out[i] = (float)((double)lo + ((double)hi - (double)lo) * u01(key_hash(seed, tensor, (uint64_t)i)));
}

ORACLE_API void oracle_fill_normal_f32(float* out, int64_t n, uint64_t seed, uint64_t tensor, float scale) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    double u1 = 1.0 - u01(key_hash(seed, tensor, 2 * (uint64_t)i)); /* (0,1] */
    double u2 = u01(key_hash(seed, tensor, 2 * (uint64_t)i + 1));
    out[i] = (float)((double)scale * sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2));
  }
}

ORACLE_API void oracle_fill_int8(int8_t* out, int64_t n, uint64_t seed, uint64_t tensor, int lo, int hi) {
  uint64_t span = (uint64_t)(hi - lo + 1);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) out[i] = (int8_t)(lo + (int)(key_hash(seed, tensor, (uint64_t)i) % span));
}

/* --------------------------------------------------------------- codecs --- */
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* IEEE binary16, round to nearest even, overflow -> inf, NaN kept quiet. */
ORACLE_API uint16_t oracle_f32_to_f16(float f) {
  uint32_t x = f32_bits(f), sign = (x >> 16) & 0x8000u, ax = x & 0x7FFFFFFFu;
  if (ax >= 0x7F800000u) return (uint16_t)(sign | (ax > 0x7F800000u ? 0x7E00u : 0x7C00u));
  if (ax >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);           /* >= 65520 rounds to inf */
  if (ax >= 0x38800000u) {                                            /* normal half */
    uint32_t m = ax - 0x38000000u;                                    /* rebias 127 -> 15 */
    uint32_t r = m >> 13, rem = m & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) ++r;
    return (uint16_t)(sign | r);
  }
  if (ax < 0x33000000u) return (uint16_t)sign;                        /* < 2^-25 -> 0 (tie at 2^-25 -> even 0) */
  /* subnormal half: value = mant * 2^-24 */
  int e = (int)(ax >> 23);                                            /* biased exp, 102..112 */
  uint32_t mant = (ax & 0x7FFFFFu) | 0x800000u;                       /* 24-bit */
  int shift = 126 - e;                                                /* 14..24 */
  uint32_t r = mant >> shift, rem = mant & ((1u << shift) - 1u), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (r & 1u))) ++r;
  return (uint16_t)(sign | r);
}
ORACLE_API float oracle_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16, e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
  if (e == 0x1F) return bits_f32(sign | 0x7F800000u | (m << 13));
  if (e) return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
  float v = (float)m * (1.0f / 16777216.0f);                           /* m * 2^-24, exact */
  return sign ? -v : v;
}

ORACLE_API uint16_t oracle_f32_to_bf16(float f) {
  uint32_t x = f32_bits(f);
  if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x0040u);
  uint32_t lsb = (x >> 16) & 1u;
  return (uint16_t)((x + 0x7FFFu + lsb) >> 16);
}
ORACLE_API float oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* OCP FP8 E4M3FN: bias 7, no inf, S.1111.111 = NaN, max finite 448. */
ORACLE_API float oracle_e4m3_to_f32(uint8_t c) {
  uint32_t e = (c >> 3) & 0xFu, m = c & 7u;
  float v;
  if (e == 0xF && m == 7) return bits_f32(0x7FC00000u | ((uint32_t)(c & 0x80u) << 24));
  if (e == 0) v = (float)m * (1.0f / 512.0f);                          /* subnormal: m * 2^-9 */
  else v = ldexpf((float)(8u + m), (int)e - 10);                       /* (1+m/8) * 2^(e-7) */
  return (c & 0x80u) ? -v : v;
}
/* round to nearest even; finite values beyond 448 saturate to +-448; NaN -> 0x7F|sign. */
ORACLE_API uint8_t oracle_f32_to_e4m3(float f) {
  uint32_t x = f32_bits(f);
  uint8_t sign = (uint8_t)((x >> 24) & 0x80u);
  uint32_t ax = x & 0x7FFFFFFFu;
  if (ax > 0x7F800000u) return (uint8_t)(sign | 0x7Fu);
  float a = bits_f32(ax);
  if (a >= 448.0f) return (uint8_t)(sign | 0x7Eu);
  if (a < 0.015625f) {                                                 /* below 2^-6: subnormal grid 2^-9 */
    float q = a * 512.0f;                                              /* exact scaling */
    uint32_t r = (uint32_t)q; float rem = q - (float)r;
    if (rem > 0.5f || (rem == 0.5f && (r & 1u))) ++r;
    return (uint8_t)(sign | r);                                        /* r == 8 encodes 2^-6 correctly */
  }
  int e = (int)(ax >> 23) - 127;                                       /* -6..8 */
  uint32_t mant = ax & 0x7FFFFFu;
  uint32_t r = mant >> 20, rem = mant & 0xFFFFFu;
  if (rem > 0x80000u || (rem == 0x80000u && (r & 1u))) ++r;
  uint32_t code = ((uint32_t)(e + 7) << 3) + r;                        /* mantissa carry bumps exponent */
  if (code > 0x7Eu) code = 0x7Eu;
  return (uint8_t)(sign | code);
}

ORACLE_API void oracle_encode(int dtype, const float* in, void* out, int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    switch (dtype) {
      case DT_F32: ((float*)out)[i] = in[i]; break;
      case DT_F16: ((uint16_t*)out)[i] = oracle_f32_to_f16(in[i]); break;
      case DT_BF16: ((uint16_t*)out)[i] = oracle_f32_to_bf16(in[i]); break;
      case DT_E4M3: ((uint8_t*)out)[i] = oracle_f32_to_e4m3(in[i]); break;
      case DT_I8: ((int8_t*)out)[i] = (int8_t)in[i]; break;
      default: break;
    }
  }
}
static inline float decode_one(int dtype, const void* p, int64_t i) {
  switch (dtype) {
    case DT_F32: return ((const float*)p)[i];
    case DT_F16: return oracle_f16_to_f32(((const uint16_t*)p)[i]);
    case DT_BF16: return oracle_bf16_to_f32(((const uint16_t*)p)[i]);
    case DT_E4M3: return oracle_e4m3_to_f32(((const uint8_t*)p)[i]);
    case DT_I8: return (float)((const int8_t*)p)[i];
    case DT_I32: return (float)((const int32_t*)p)[i];
    default: return 0.0f;
  }
}
ORACLE_API void oracle_decode(int dtype, const void* in, float* out, int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) out[i] = decode_one(dtype, in, i);
}

/* ----------------------------------------------------------- naive GEMM --- */
/* Textbook triple loop, double accumulation, no blocking: the definition that
 * the blocked routines below are checked against on small shapes. */
ORACLE_API int oracle_gemm_naive(int dtype, int transA, int transB, int64_t M, int64_t N, int64_t K,
                                 const void* A, int64_t lda, const void* B, int64_t ldb, double* C) {
  if (!A || !B || !C || M < 0 || N < 0 || K < 0) return 1;
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
      double s = 0.0;
      for (int64_t k = 0; k < K; ++k) {
        double a = decode_one(dtype, A, transA ? k * lda + i : i * lda + k);
        double b = decode_one(dtype, B, transB ? j * ldb + k : k * ldb + j);
        s += a * b;
      }
      C[i * N + j] = s;
    }
  return 0;
}

/* --------------------------------------------------------- blocked GEMM --- */
/* Goto-style: pack a KC x NC panel of op(B) and MC x KC blocks of op(A) into
 * contiguous micro-panels, then an MR x NR register-blocked micro-kernel
 * (GCC vector extensions, 256-bit).
 * Three instantiations: (float in, double acc) for parity, (float in, float
 * acc) for the timed CPU baseline, (int32 in, int32 acc) for exact int8. */
#define MR 4
#define KC 256
#define MC 128
#define NC 2048

typedef float vf8 __attribute__((vector_size(32)));
typedef double vd4 __attribute__((vector_size(32)));
typedef int32_t vi8 __attribute__((vector_size(32)));

/* micro-kernels: C[mr x nr] += Apanel[kc x MR] . Bpanel[kc x NR], accumulators in registers */
#define NR_f64 8
static void micro_f64(int64_t kc, const double* restrict ap, const double* restrict bp, double* restrict c, int64_t ldc,
                      int mr, int nr) {
  vd4 acc[MR][2];
  for (int r = 0; r < MR; ++r) acc[r][0] = acc[r][1] = (vd4){0, 0, 0, 0};
  for (int64_t k = 0; k < kc; ++k) {
    vd4 b0, b1;
    memcpy(&b0, bp + k * 8, 32);
    memcpy(&b1, bp + k * 8 + 4, 32);
    for (int r = 0; r < MR; ++r) {
      double a = ap[k * MR + r];
      vd4 av = {a, a, a, a};
      acc[r][0] += av * b0;
      acc[r][1] += av * b1;
    }
  }
  for (int r = 0; r < mr; ++r)
    for (int q = 0; q < nr; ++q) c[r * ldc + q] += acc[r][q / 4][q % 4];
}
#define NR_f32 16
static void micro_f32(int64_t kc, const float* restrict ap, const float* restrict bp, float* restrict c, int64_t ldc,
                      int mr, int nr) {
  vf8 acc[MR][2];
  for (int r = 0; r < MR; ++r) acc[r][0] = acc[r][1] = (vf8){0, 0, 0, 0, 0, 0, 0, 0};
  for (int64_t k = 0; k < kc; ++k) {
    vf8 b0, b1;
    memcpy(&b0, bp + k * 16, 32);
    memcpy(&b1, bp + k * 16 + 8, 32);
    for (int r = 0; r < MR; ++r) {
      float a = ap[k * MR + r];
      vf8 av = {a, a, a, a, a, a, a, a};
      acc[r][0] += av * b0;
      acc[r][1] += av * b1;
    }
  }
  for (int r = 0; r < mr; ++r)
    for (int q = 0; q < nr; ++q) c[r * ldc + q] += acc[r][q / 8][q % 8];
}
#define NR_i32 16
static void micro_i32(int64_t kc, const int32_t* restrict ap, const int32_t* restrict bp, int32_t* restrict c,
                      int64_t ldc, int mr, int nr) {
  vi8 acc[MR][2];
  for (int r = 0; r < MR; ++r) acc[r][0] = acc[r][1] = (vi8){0, 0, 0, 0, 0, 0, 0, 0};
  for (int64_t k = 0; k < kc; ++k) {
    vi8 b0, b1;
    memcpy(&b0, bp + k * 16, 32);
    memcpy(&b1, bp + k * 16 + 8, 32);
    for (int r = 0; r < MR; ++r) {
      int32_t a = ap[k * MR + r];
      vi8 av = {a, a, a, a, a, a, a, a};
      acc[r][0] += av * b0;
      acc[r][1] += av * b1;
    }
  }
  for (int r = 0; r < mr; ++r)
    for (int q = 0; q < nr; ++q) c[r * ldc + q] += acc[r][q / 8][q % 8];
}

#define DEFINE_BLOCKED(NAME, TIN, TACC, LOAD_A, LOAD_B)                                                       \
  static int blocked_##NAME(int dtype, int transA, int transB, int64_t M, int64_t N, int64_t K,              \
                            const void* A, int64_t lda, const void* B, int64_t ldb, int64_t row0,            \
                            int64_t nrows, TACC* C) {                                                        \
    enum { NR = NR_##NAME };                                                                                 \
    (void)dtype;                                                                                             \
    if (!A || !B || !C || M < 0 || N < 0 || K < 0 || row0 < 0 || nrows < 0 || row0 + nrows > M) return 1;    \
    for (int64_t i = 0; i < nrows * N; ++i) C[i] = 0;                                                        \
    if (nrows == 0 || N == 0 || K == 0) return 0;                                                            \
    TIN* bpack = (TIN*)aligned_alloc(64, sizeof(TIN) * KC * (NC + NR));                                      \
    if (!bpack) return 2;                                                                                    \
    int status = 0;                                                                                          \
    for (int64_t jc = 0; jc < N; jc += NC) {                                                                 \
      int64_t nc = N - jc < NC ? N - jc : NC;                                                                \
      int64_t npan = (nc + NR - 1) / NR;                                                                     \
      for (int64_t pc = 0; pc < K; pc += KC) {                                                               \
        int64_t kc = K - pc < KC ? K - pc : KC;                                                              \
        _Pragma("omp parallel for schedule(static)") for (int64_t p = 0; p < npan; ++p) {                    \
          TIN* dst = bpack + p * kc * NR;                                                                    \
          for (int64_t k = 0; k < kc; ++k)                                                                   \
            for (int q = 0; q < NR; ++q) {                                                                   \
              int64_t j = jc + p * NR + q, kk = pc + k;                                                      \
              dst[k * NR + q] = j < N ? (TIN)LOAD_B(transB ? j * ldb + kk : kk * ldb + j) : (TIN)0;          \
            }                                                                                                \
        }                                                                                                    \
        _Pragma("omp parallel") {                                                                            \
          TIN* apack = (TIN*)aligned_alloc(64, sizeof(TIN) * KC * (MC + MR));                                \
          if (!apack) {                                                                                      \
            _Pragma("omp atomic write") status = 2;                                                          \
          } else {                                                                                           \
            _Pragma("omp for schedule(dynamic, 1)") for (int64_t ic = 0; ic < nrows; ic += MC) {             \
              int64_t mc = nrows - ic < MC ? nrows - ic : MC;                                                \
              int64_t mpan = (mc + MR - 1) / MR;                                                             \
              for (int64_t p = 0; p < mpan; ++p)                                                             \
                for (int64_t k = 0; k < kc; ++k)                                                             \
                  for (int r = 0; r < MR; ++r) {                                                             \
                    int64_t il = ic + p * MR + r, i = row0 + il, kk = pc + k;                                \
                    apack[(p * kc + k) * MR + r] =                                                           \
                        il < nrows ? (TIN)LOAD_A(transA ? kk * lda + i : i * lda + kk) : (TIN)0;             \
                  }                                                                                          \
              for (int64_t pn = 0; pn < npan; ++pn)                                                          \
                for (int64_t pm = 0; pm < mpan; ++pm) {                                                      \
                  int64_t il = ic + pm * MR, j = jc + pn * NR;                                               \
                  int mr = (int)(nrows - il < MR ? nrows - il : MR), nr = (int)(N - j < NR ? N - j : NR);    \
                  micro_##NAME(kc, apack + pm * kc * MR, bpack + pn * kc * NR, C + il * N + j, N, mr, nr);   \
                }                                                                                            \
            }                                                                                                \
            free(apack);                                                                                     \
          }                                                                                                  \
        }                                                                                                    \
      }                                                                                                      \
    }                                                                                                        \
    free(bpack);                                                                                             \
    return status;                                                                                           \
  }

#define LD_A_F(idx) decode_one(dtype, A, (idx))
#define LD_B_F(idx) decode_one(dtype, B, (idx))
#define LD_A_I(idx) ((const int8_t*)A)[(idx)]
#define LD_B_I(idx) ((const int8_t*)B)[(idx)]

DEFINE_BLOCKED(f64, double, double, LD_A_F, LD_B_F)
DEFINE_BLOCKED(f32, float, float, LD_A_F, LD_B_F)
DEFINE_BLOCKED(i32, int32_t, int32_t, LD_A_I, LD_B_I)

/* rows [row0, row0+nrows) of C = op(A).op(B); C is nrows x N, dense. */
ORACLE_API int oracle_gemm_f64(int dtype, int transA, int transB, int64_t M, int64_t N, int64_t K, const void* A,
                               int64_t lda, const void* B, int64_t ldb, int64_t row0, int64_t nrows, double* C) {
  if (dtype == DT_I32) return 1;
  return blocked_f64(dtype, transA, transB, M, N, K, A, lda, B, ldb, row0, nrows, C);
}
ORACLE_API int oracle_gemm_f32(int dtype, int transA, int transB, int64_t M, int64_t N, int64_t K, const void* A,
                               int64_t lda, const void* B, int64_t ldb, int64_t row0, int64_t nrows, float* C) {
  if (dtype == DT_I32) return 1;
  return blocked_f32(dtype, transA, transB, M, N, K, A, lda, B, ldb, row0, nrows, C);
}
ORACLE_API int oracle_gemm_i32(int transA, int transB, int64_t M, int64_t N, int64_t K, const int8_t* A, int64_t lda,
                               const int8_t* B, int64_t ldb, int64_t row0, int64_t nrows, int32_t* C) {
  int dtype = DT_I8;
  return blocked_i32(dtype, transA, transB, M, N, K, A, lda, B, ldb, row0, nrows, C);
}

/* ------------------------------------------------------------ epilogues --- */
/* out[m][n] = f16( (float(acc[m][n]) * sA[m]) * sB[n] ); two separately rounded fp32 multiplies. */
ORACLE_API void oracle_epilogue_rowcol_f16(const int32_t* acc, int64_t rows, int64_t N, const float* sA,
                                           const float* sB, uint16_t* out) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < rows; ++i)
    for (int64_t j = 0; j < N; ++j) {
      volatile float t = (float)acc[i * N + j] * sA[i];
      volatile float u = t * sB[j];
      out[i * N + j] = oracle_f32_to_f16(u);
    }
}
/* float view of the same epilogue without the final narrowing (for tolerance checks) */
ORACLE_API void oracle_epilogue_rowcol_f32(const int32_t* acc, int64_t rows, int64_t N, const float* sA,
                                           const float* sB, float* out) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < rows; ++i)
    for (int64_t j = 0; j < N; ++j) {
      volatile float t = (float)acc[i * N + j] * sA[i];
      out[i * N + j] = t * sB[j];
    }
}
/* out = (acc * sA) * sB in double (reference value before narrowing) */
ORACLE_API void oracle_epilogue_tensor_f64(double* acc, int64_t n, float sA, float sB) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) acc[i] = (acc[i] * (double)sA) * (double)sB;
}

/* ---------------------------------------------------------- error norms --- */
/* got is in the output dtype; ref is the double reference.  Returns through
 * res[0] = max over elements of |d-r| / max(|r|, rms(ref)); res[1] = ||D-R||_F / ||R||_F;
 * res[2] = rms(ref); res[3] = count of non-finite outputs. */
ORACLE_API void oracle_compare(int dtype_out, const void* got, const double* ref, int64_t n, double* res) {
  double ss = 0.0;
#pragma omp parallel for schedule(static) reduction(+ : ss)
  for (int64_t i = 0; i < n; ++i) ss += ref[i] * ref[i];
  double rms = n ? sqrt(ss / (double)n) : 0.0;
  double worst = 0.0, dd = 0.0, bad = 0.0;
#pragma omp parallel for schedule(static) reduction(max : worst) reduction(+ : dd, bad)
  for (int64_t i = 0; i < n; ++i) {
    double d = (double)decode_one(dtype_out, got, i);
    if (!isfinite(d)) { bad += 1.0; continue; }
    double e = fabs(d - ref[i]);
    double den = fabs(ref[i]) > rms ? fabs(ref[i]) : rms;
    double rel = den > 0.0 ? e / den : (e > 0.0 ? INFINITY : 0.0);
    if (rel > worst) worst = rel;
    dd += e * e;
  }
  res[0] = worst;
  res[1] = ss > 0.0 ? sqrt(dd / ss) : (dd > 0.0 ? INFINITY : 0.0);
  res[2] = rms;
  res[3] = bad;
}

ORACLE_API int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
