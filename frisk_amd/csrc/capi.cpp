// C ABI of libfrisk_hip.so: descriptor validation, the planner (tile / wave
// grid / LDS layout choice) and kernel dispatch.  Host code only.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "frisk_hip.h"
#include "gemm_internal.h"
#include "lds_model.h"
#include "tile_ops.h"
#include "attention.h"

// Scratch memory of frisk_hip_gemm_static_ws: the split-K / tail-split partial sums of callers that cannot allocate.
// Every GPU the library runs on holds its own copy of this array, at its own address, until the process ends.  In host
// code the name below is only a handle for hipGetSymbolAddress; kernels and copies get the device address it returns.
static __device__ __align__(256) unsigned char scratch[FRISK_HIP_STATIC_WS_BYTES];

namespace frisk {

static thread_local std::string g_last_error;

// device address of `scratch` on each device, resolved once per device with that device current
static constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

static hipError_t scratch_of_current_device(void** out) {
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)); e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // racing threads resolve the same address
  }
  *out = p;
  return hipSuccess;
}

static int fail(int status, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return status;
}

static const std::vector<const KernelEntry*>& kernels() {
  static const std::vector<const KernelEntry*> all = [] {
    std::vector<const KernelEntry*> v;
    for (int i = 0; i < kNumKernelsF16; ++i) v.push_back(&kKernelsF16[i]);
    for (int i = 0; i < kNumKernelsF16_2; ++i) v.push_back(&kKernelsF16_2[i]);
    for (int i = 0; i < kNumKernelsBF16; ++i) v.push_back(&kKernelsBF16[i]);
    for (int i = 0; i < kNumKernelsBF16_2; ++i) v.push_back(&kKernelsBF16_2[i]);
    for (int i = 0; i < kNumKernelsI8; ++i) v.push_back(&kKernelsI8[i]);
    for (int i = 0; i < kNumKernelsI8_2; ++i) v.push_back(&kKernelsI8_2[i]);
    for (int i = 0; i < kNumKernelsE4M3; ++i) v.push_back(&kKernelsE4M3[i]);
    for (int i = 0; i < kNumKernelsE4M3_2; ++i) v.push_back(&kKernelsE4M3_2[i]);
    for (int i = 0; i < kNumKernelsF32; ++i) v.push_back(&kKernelsF32[i]);
    for (int i = 0; i < kNumKernelsF32_2; ++i) v.push_back(&kKernelsF32_2[i]);
    return v;
  }();
  return all;
}

static int elem_size(int dt) {
  switch (dt) {
    case FRISK_F32: case FRISK_I32: return 4;
    case FRISK_F16: case FRISK_BF16: return 2;
    case FRISK_I8: case FRISK_E4M3: return 1;
    default: return 0;
  }
}
static int frag_bytes(int dt) { return dt == FRISK_E4M3 ? 32 : 16; }
static int mfma_k(int dt) { return dt == FRISK_F32 ? 2 : (2 * frag_bytes(dt)) / elem_size(dt); }

// Wave partition of a block tile: the reference's computeWarpPartition
// (lib/Dialect/Frisk/IR/FriskOps.cpp:825-888) with waves of 64 lanes and
// per-wave granularity kM x kN (32 x 32 for the MFMA atoms used here).
static void wave_partition(int policy, int64_t M, int64_t N, int num_waves, int kM, int kN, int* wm, int* wn) {
  int64_t m_w = 1, n_w = num_waves;
  if (M == 0 || N == 0 || num_waves == 0) { *wm = 1; *wn = 1; return; }
  if (policy == FRISK_POLICY_FULL_ROW) {
    m_w = num_waves;
    if (M % (m_w * kM) != 0) {
      int64_t max_m = std::max<int64_t>(1, M / kM);
      m_w = std::max<int64_t>(1, std::min<int64_t>(num_waves, max_m));
    }
    n_w = std::max<int64_t>(1, num_waves / m_w);
  } else if (policy == FRISK_POLICY_FULL_COL) {
    n_w = num_waves;
    if (N % (n_w * kN) != 0) {
      int64_t max_n = std::max<int64_t>(1, N / kN);
      n_w = std::max<int64_t>(1, std::min<int64_t>(num_waves, max_n));
    }
    m_w = std::max<int64_t>(1, num_waves / n_w);
  } else {
    float ideal = (float)M / (float)N;
    float best = INFINITY;
    for (int64_t m = 1; m <= num_waves; ++m) {
      if (num_waves % m) continue;
      int64_t n = num_waves / m;
      float mp = (float)M / (float)(m * kM), np = (float)N / (float)(n * kN);
      if (mp < 1 || np < 1) continue;
      float score = std::fabs(mp / np - ideal);
      if (score < best) { best = score; m_w = m; n_w = n; }
    }
  }
  *wm = (int)std::max<int64_t>(1, m_w);
  *wn = (int)std::max<int64_t>(1, n_w);
}

static int validate(const frisk_gemm_desc* d) {
  if (!d) return fail(FRISK_ERR_NULL, "descriptor is null");
  if (d->abi_version != FRISK_HIP_ABI_VERSION)
    return fail(FRISK_ERR_ABI, "descriptor abi_version %d, library %d", d->abi_version, FRISK_HIP_ABI_VERSION);
  const int ab = d->dtype_ab, acc = d->dtype_acc, out = d->dtype_out;
  bool ok = false;
  switch (ab) {
    case FRISK_F32: ok = acc == FRISK_F32 && out == FRISK_F32; break;
    case FRISK_F16: ok = acc == FRISK_F32 && (out == FRISK_F16 || out == FRISK_F32); break;
    case FRISK_BF16: ok = acc == FRISK_F32 && (out == FRISK_BF16 || out == FRISK_F32); break;
    case FRISK_I8: ok = acc == FRISK_I32 && (out == FRISK_I32 || out == FRISK_F16 || out == FRISK_F32); break;
    case FRISK_E4M3: ok = acc == FRISK_F32 && (out == FRISK_BF16 || out == FRISK_F16 || out == FRISK_F32); break;
    default: ok = false;
  }
  if (!ok) return fail(FRISK_ERR_DTYPE, "unsupported element types: ab=%d acc=%d out=%d", ab, acc, out);
  if (d->epilogue < FRISK_EPI_NONE || d->epilogue > FRISK_EPI_TENSOR_SCALE)
    return fail(FRISK_ERR_EPILOGUE, "unknown epilogue %d", d->epilogue);
  if (out == FRISK_I32 && d->epilogue != FRISK_EPI_NONE)
    return fail(FRISK_ERR_EPILOGUE, "int32 output carries the raw accumulators; scales need a floating output type");
  if (d->policy < FRISK_POLICY_SQUARE || d->policy > FRISK_POLICY_FULL_COL)
    return fail(FRISK_ERR_TILE, "unknown wave policy %d", d->policy);
  if (d->atom != 0 && d->atom != 16 && d->atom != 32) return fail(FRISK_ERR_TILE, "MFMA atoms have 32 or 16 rows, not %d", d->atom);
  if (d->M < 0 || d->N < 0 || d->K < 0) return fail(FRISK_ERR_SHAPE, "negative extent M=%lld N=%lld K=%lld", (long long)d->M, (long long)d->N, (long long)d->K);
  if (d->M > INT32_MAX || d->N > INT32_MAX || d->K > INT32_MAX) return fail(FRISK_ERR_SHAPE, "extent exceeds 2^31-1");
  const int64_t a_cols = d->transA ? d->M : d->K, b_cols = d->transB ? d->K : d->N;
  if (d->lda < std::max<int64_t>(1, a_cols)) return fail(FRISK_ERR_SHAPE, "lda=%lld smaller than the stored row length %lld", (long long)d->lda, (long long)a_cols);
  if (d->ldb < std::max<int64_t>(1, b_cols)) return fail(FRISK_ERR_SHAPE, "ldb=%lld smaller than the stored row length %lld", (long long)d->ldb, (long long)b_cols);
  if (d->ldc < std::max<int64_t>(1, d->N)) return fail(FRISK_ERR_SHAPE, "ldc=%lld smaller than N=%lld", (long long)d->ldc, (long long)d->N);
  return FRISK_OK;
}

static void fill_layout(frisk_lds_layout* L, bool kcontig, int es, int fragb, int mn, int bk, int nw, bool with_model, int atom) {
  TileShape t{kcontig ? mn : bk, (kcontig ? bk : mn) * es, kcontig, es, fragb, mn, bk, atom};
  Swizzle s = default_swizzle(kcontig, es, t.rowb, atom);
  L->rows = t.rows;
  L->row_bytes = t.rowb;
  L->k_contiguous = kcontig;
  L->row_shift = s.sh;
  L->row_mask = s.mk;
  L->chunk_shift = s.cs;
  L->row_shift2 = s.sh2;
  L->row_mask2 = s.mk2;
  L->chunk_shift2 = s.cs2;
  L->read_instr = kcontig ? 0 : (es == 4 ? 3 : (es == 2 ? 1 : 2));
  int atoms = mn / atom < 4 ? mn / atom : 4;
  int n_access = atoms * ((bk * es) / frag_kstep_bytes(fragb, atom)) * frag_instr_count(kcontig, es, fragb);
  // evaluating the bank model costs ~0.1 ms of host time: only when the caller asks for the plan
  L->read_cycles = (with_model && n_access) ? (float)swizzle_read_cycles(t, s) / (float)n_access : 0.f;
  // the direct-to-LDS transfer writes 64 consecutive 16-byte slots: no conflicts by construction
  L->write_cycles = 16.f;
  (void)nw;
}

// Tail split: a grid of a little more than a whole number of rounds of 256 tiles leaves most CUs idle in its last round.
// With a kernel that has the split-K store path, the last tiles % 256 tiles (at most half a round) are computed by 2, 4 or
// 8 work-groups each, every one taking an equal share of the K tiles (at least 4).  Returns that count, 1 for no split.
static int tail_split_of(const KernelEntry* k, int64_t tiles, int64_t kt, bool whole_k_tiles) {
  if (!k->splitk || k->bm < 128 || k->wk > 1 || !whole_k_tiles || tiles <= 256) return 1;
  const int64_t rest = tiles % 256;
  if (rest == 0 || rest > 128) return 1;
  // shallower slices do not repay the second launch (measured); the 8-bit kernels run a K tile of twice the depth in the same
  // time, so the summing pass weighs twice as much against their slices (fp8 5120x4096x4096: 64 tiles in 4 slices of 8 K tiles
  // 92.4 us, unsplit 84, 256x128 tiles 81.4)
  const int min_slice = elem_size(k->dtype) == 1 ? 16 : 8;
  for (int s = 8; s >= 2; s /= 2)
    if (rest * s <= 256 && kt % s == 0 && kt / s >= min_slice) return s;
  return 1;
}

// Relative time of a problem on a kernel variant, used only to rank the variants.  One wave of work-groups = one per CU
// (256); a K tile of a 256x256 tile costs 1.5 units when every CU runs one, and less when the chip is partly idle
// (less contention in the L2 and a higher clock): factor 0.6 + 0.4 * fill.  The constants are measured on fp16 problems
// between 1024^3 and 8192^3 and carry over to the 8-bit types, whose K tiles hold the same number of bytes.
// the split the planner gives a grid below one round of a variant with the split-K store path: up to one work-group per CU,
// at least 4 K tiles per slice
static int sub_round_split(const KernelEntry* k, int64_t tiles, int64_t kt) {
  int split = 1;
  for (int c = 2; c <= 64; c *= 2)
    if (kt % c == 0 && kt / c >= std::max(4, k->min_k_tiles) && tiles * c <= 256) split = c;
  return split;
}

static double estimated_cost(const KernelEntry* k, const frisk_gemm_desc* d, bool may_split = false) {
  const int64_t tiles = ((d->M + k->bm - 1) / k->bm) * ((d->N + k->bn - 1) / k->bn);
  const double kt = (double)((d->K + k->bk - 1) / k->bk);
  double c;  // cost of one K tile with the chip full
  const int64_t area = (int64_t)k->bm * k->bn;
  if (k->dtype == FRISK_F32) {
    // Measured with 16-byte fragments (K-contiguous tiles read by ds_read_b128), us, NN: 1024^3 64x64x32 18.8, x64 19.4, x128 on 8 waves
    // 19.5; 1536^3 69.4 / 73.8 / 78.6; 2048^3 128x128x32 120.8, x16 in a ring of 4 124.1, 64x64x32 123.3; 4096^3 928 / 941 / 962.
    const double c128 = k->bk <= 16 ? ((!k->transA && k->transB) ? 1.0 : 0.91) : 1.74;
    // 64x64x32 per round and K tile of 32: 0.497 us over 9, 25 and 43 rounds (3072^3 429, 5120^3 1987, 4096x11008x4096 2779 us) against
    // 1.81 us for a round of 128x128x32 (4096^3 926, 4096x11008x4096 2549): a quarter of the tile at 0.27 of the cost
    c = area >= 128 * 128 ? c128 : (k->wk > 1 ? (tiles <= 256 ? 1.8 : 2.3) : (k->bk >= 64 ? 1.0 : (tiles <= 256 ? 0.44 : 0.465)));
  } else if (k->bm == 32) {
    // 32x32 with a 4x deeper K tile; 32x128 (8-bit: 60.1 us for 256 tiles x 64 K tiles, the rate of the 32x32 kernel per K tile)
    c = k->wk > 1 ? 0.8 : (elem_size(k->dtype) == 1 ? 0.85 : 0.25);
  } else if (area >= 256 * 256) {
    c = k->wm * k->wn > 4 ? 1.56 : (k->stages_b > k->stages ? 1.5 : 1.55);  // 2 + 3 ring < 2 + 2 < 8 waves
    // 16x16 atoms: the same cycles at a higher clock when most CUs are busy (fp16 4096^3 NT 100 against 112 us); with an operand
    // read by transpose reads (twice the LDS instructions) less of it is left (NN 104 against 108).  How full the round is decides:
    // 192 or 196 tiles, NN 78 against 82 us (3584^3) and 164 against 172 (4096x3072x8192), TN 79 against 85 and 169 against 182;
    // 144 tiles (3072^3): NN 61 against 59 and TN even while the loop held several LDS reads per MFMA slot, NN 51.3 against 53.7
    // (fp16), 50.4 against 51.3 (bf16), 30.6 against 31.2 (int8) since it holds one
    // 8-bit floats on the 16x16x128 atom (NT only), us against the 32x32x64 atoms: 8192^3 331 / 351, 4096^3 45.1 / 48.8, 4096x4096x512
    // 11.8 / 12.9, 4096x11008x4096 128 / 133, 6144^3 176 / 183; 3072^3 (144 tiles) 29.6 / 28.6
    if (k->atom == 16) c *= k->dtype == FRISK_E4M3 ? (tiles >= 176 ? 0.94 : 1.04) : (!k->transA && k->transB) ? 0.93 : (tiles >= 176 ? 0.96 : 0.98);
  } else if (area >= 256 * 128) {
    c = 0.93;
  } else {
    // 3 + 3 tiles when the grid is one wave, 2 + 2 (two work-groups per CU) beyond
    c = k->stages >= 3 ? (tiles <= 256 ? 0.46 : 0.55) : (tiles <= 256 ? 0.55 : 0.52);
  }
  if (k->guard) c *= 3.0;
  if (k->bm == 32 && k->wk > 1) {
    // The 32x32 kernel streams B.  With a ring of 4 tiles one work-group fills a CU: whole rounds of 256, each paying its
    // own start (measured 14.8 us for 256 tiles, 35.8 for 512).  With a ring of 2 two work-groups share a CU: slower alone
    // (17.5 us for 256 tiles), but beyond 256 tiles the rounds overlap (29.3 us for 512, 46.6 for 896).
    if (k->stages >= 3) return (double)((tiles + 255) / 256) * kt * c * (tiles > 256 ? 1.2 : 1.0) / (tiles < 256 ? std::max((double)tiles / 256.0, 0.25) : 1.0);
    return tiles <= 256 ? kt * c * 1.19 / std::max((double)tiles / 256.0, 0.25) : (double)tiles / 256.0 * kt * c;
  }
  const int64_t full = tiles / 256, rest = tiles % 256;
  const double rest_fill = (double)rest / 256.0;
  if (may_split && k->splitk && k->bm >= 128 && tiles < 256 && d->K % k->bk == 0) {
    // below one round with a deep K the planner splits K over the idle CUs (2048x4096x16384 fp16: 128 tiles of 256x256 in 2
    // slices 209.5 us, 256 tiles of 256x128 unsplit 243.6): the slices' K tiles at the fill they reach, plus the summing pass
    const int cs = sub_round_split(k, tiles, (int64_t)kt);
    // (measured: the slices' loops 8 % above the per-K-tile rate of a long loop, the pass at 256 KiB per tile and slice in 0.07 us;
    // 1024x8192x8192 comes out even with 256x128 tiles unsplit, 123.7 against 123.9 us, and stays unsplit)
    if (cs > 1) return kt / cs * c * (0.6 + 0.4 * rest_fill * cs) * 1.08 + 5.0 + 0.07 * (double)(tiles * cs);
  }
  double cost = (double)full * kt * c;
  if (const int ts = tail_split_of(k, tiles, (int64_t)kt, d->K % k->bk == 0); ts > 1) {
    // the last `rest` tiles as ts work-groups each, a ts-th of the K tiles apiece, plus the pass that sums them
    // (a dependent launch, and rest * ts tiles of 32-bit partial sums to read)
    return cost + kt / ts * c * (0.6 + 0.4 * rest_fill * ts) + 5.0 + 0.04 * (double)(rest * ts);
  }
  if (rest) {
    if (k->bm == 32)  // the skinny kernels are bound by streaming B and need the parallelism: idle CUs are lost bandwidth
      cost += full ? kt * c : kt * c / std::max(rest_fill, 0.25);
    else
      cost += kt * c * (0.6 + 0.4 * rest_fill);
  }
  return cost;
}

// Grids of at most 256 tiles of 128 x 128 (a few hundred rows, or a small square): no variant fills the chip with one
// work-group per tile, so the choice is a (variant, split of K) pair.  Measured per element type over 81 skinny shapes (M 32 ..
// 2048, N and K 1024 .. 28672) and 90 squarish ones (sides 768 .. 2048, K 1024 .. 8192), both layouts of B, every variant at
// every split 1 .. 32, B taken in turn from as many copies as fill 400 MiB so that it streams from HBM as the weights of a model
// do (with one B of at most 128 MiB the last-level cache serves it: 26.5 instead of 38 us at fp16 64x8192x8192).  A variant's splits are the powers of two that keep tiles x split within `w` work-groups and `kmin` K
// tiles per slice; variants and splits are compared by a time model fitted to the sweep, in microseconds:
//   launch + whole rounds x (K tiles x tk + ps) + a last round at K tiles x tk x (a + (1 - a) x fill) + the summing pass
//   (r0 + r1 x megabytes of partial sums) when split;
// variants of which a CU holds two work-groups (`cap` 512) pay tk2 per K tile more once any CU holds its second one:
// K tiles x tk2 x (a2 + (1 - a2) x fill of the second half).  The pair chosen this way is 2 % slower on average than the
// best pair of the sweep (more than 1.2x in 24 of 966 cases); the one-size rule used before lost 35-40 % on
// average on the skinny shapes.
struct SmallGridModel { int cap, w, kmin; float launch, tk, a, r0, r1, ps, tk2, a2; };
static const SmallGridModel kSmallGrid[3][14] = {
    {  // 16-bit
        {512, 0, 0, 0.57f, 0.783f, 0.77f, 5.00f, 0.200f, 1.00f, 0.300f, 0.50f},  // 128x128 s2
        {256, 256, 16, 2.32f, 0.551f, 0.73f, 5.64f, 0.300f, 4.27f, 0.000f, 0.00f},  // 128x128 s3
        {256, 0, 0, 3.66f, 0.879f, 0.76f, 5.00f, 0.200f, 1.00f, 0.000f, 0.00f},  // 128x256 s3
        {256, 0, 0, 4.17f, 0.833f, 0.74f, 5.00f, 0.200f, 1.00f, 0.000f, 0.00f},  // 256x128 s3
        {256, 256, 16, 9.37f, 1.496f, 0.52f, 0.00f, 0.300f, 8.37f, 0.000f, 0.00f},  // 256x256 s2
        {256, 256, 16, 5.82f, 1.307f, 0.66f, 2.98f, 0.300f, 8.84f, 0.000f, 0.00f},  // 256x256 s2 a16
        {256, 0, 0, 0.83f, 2.046f, 0.53f, 5.00f, 0.200f, 1.00f, 0.000f, 0.00f},  // 256x256 s2 w8
        {512, 128, 16, 0.36f, 0.456f, 0.74f, 6.46f, 0.300f, 0.00f, 0.211f, 0.88f},  // 32x128 s3 n
        {512, 128, 16, 0.12f, 0.465f, 0.76f, 6.43f, 0.300f, 0.00f, 0.170f, 1.00f},  // 32x128 s3 t
        {512, 256, 16, 2.40f, 0.744f, 0.68f, 7.68f, 0.000f, 0.00f, 0.222f, 0.72f},  // 32x32 s2 t
        {256, 128, 16, 2.88f, 0.580f, 0.65f, 6.64f, 0.000f, 0.03f, 0.000f, 0.00f},  // 32x32 s4 t
        {512, 256, 16, 1.56f, 0.436f, 0.69f, 7.25f, 0.300f, 2.21f, 0.315f, 0.41f},  // 64x128 s3
        {256, 256, 16, 3.28f, 0.638f, 0.82f, 6.76f, 0.000f, 1.01f, 0.000f, 0.00f},  // 64x32 s3
        {256, 256, 16, 2.59f, 0.851f, 0.83f, 5.42f, 0.065f, 0.79f, 0.000f, 0.00f},  // 128x64 s3
    },
    {  // int8
        {512, 0, 0, 2.56f, 0.726f, 0.76f, 5.00f, 0.200f, 1.00f, 0.300f, 0.50f},  // 128x128 s2
        {256, 256, 16, 3.38f, 0.558f, 0.65f, 5.70f, 0.300f, 4.52f, 0.000f, 0.00f},  // 128x128 s3
        {256, 0, 0, 4.88f, 0.908f, 0.71f, 5.00f, 0.200f, 1.00f, 0.000f, 0.00f},  // 128x256 s3
        {256, 0, 0, 4.92f, 0.827f, 0.76f, 5.00f, 0.200f, 1.00f, 0.000f, 0.00f},  // 256x128 s3
        {256, 256, 16, 8.27f, 1.618f, 0.56f, 0.00f, 0.300f, 7.84f, 0.000f, 0.00f},  // 256x256 s2
        {256, 256, 16, 6.65f, 1.471f, 0.60f, 2.63f, 0.300f, 5.73f, 0.000f, 0.00f},  // 256x256 s2 a16
        {256, 0, 0, 4.80f, 1.741f, 0.61f, 5.00f, 0.200f, 1.00f, 0.000f, 0.00f},  // 256x256 s2 w8
        {512, 128, 16, 2.00f, 0.461f, 0.65f, 4.98f, 0.300f, 0.00f, 0.222f, 0.70f},  // 32x128 s3 n
        {512, 128, 16, 1.96f, 0.436f, 0.69f, 5.27f, 0.300f, 0.00f, 0.188f, 0.88f},  // 32x128 s3 t
        {512, 256, 16, 3.09f, 0.678f, 0.71f, 4.29f, 0.300f, 0.59f, 0.199f, 1.00f},  // 32x32 s2 t
        {256, 128, 16, 3.29f, 0.532f, 0.66f, 4.15f, 0.000f, 0.53f, 0.000f, 0.00f},  // 32x32 s4 t
        {512, 256, 16, 2.72f, 0.443f, 0.65f, 6.47f, 0.300f, 1.56f, 0.377f, 0.36f},  // 64x128 s3
        {256, 256, 16, 3.47f, 0.646f, 0.87f, 4.48f, 0.300f, 1.19f, 0.000f, 0.00f},  // 64x32 s3
        {256, 256, 16, 3.04f, 0.844f, 0.83f, 4.14f, 0.300f, 0.89f, 0.000f, 0.00f},  // 128x64 s3
    },
    {  // 8-bit float
        {512, 0, 0, 2.63f, 0.708f, 0.74f, 5.00f, 0.200f, 1.00f, 0.300f, 0.50f},  // 128x128 s2
        {256, 256, 16, 3.32f, 0.485f, 0.67f, 4.85f, 0.300f, 2.07f, 0.000f, 0.00f},  // 128x128 s3
        {256, 0, 0, 4.85f, 0.854f, 0.62f, 5.00f, 0.200f, 1.00f, 0.000f, 0.00f},  // 128x256 s3
        {256, 0, 0, 4.62f, 0.802f, 0.67f, 5.00f, 0.200f, 1.00f, 0.000f, 0.00f},  // 256x128 s3
        {256, 256, 16, 7.47f, 1.283f, 0.68f, 0.41f, 0.300f, 7.22f, 0.000f, 0.00f},  // 256x256 s2
        {256, 256, 16, 6.48f, 1.195f, 0.74f, 1.99f, 0.300f, 6.48f, 0.000f, 0.00f},  // 256x256 s2 a16
        {256, 0, 0, 4.17f, 1.217f, 1.00f, 5.00f, 0.200f, 1.00f, 0.000f, 0.00f},  // 256x256 s2 w8
        {512, 128, 16, 1.98f, 0.421f, 0.67f, 5.23f, 0.300f, 0.00f, 0.148f, 1.00f},  // 32x128 s3 n
        {512, 128, 16, 1.98f, 0.421f, 0.67f, 5.23f, 0.300f, 0.00f, 0.148f, 1.00f},  // 32x128 s3 t
        {512, 256, 16, 2.79f, 0.698f, 0.71f, 4.93f, 0.000f, 0.57f, 0.225f, 1.00f},  // 32x32 s2 t
        {256, 128, 16, 2.98f, 0.514f, 0.73f, 4.23f, 0.000f, 0.67f, 0.000f, 0.00f},  // 32x32 s4 t
        {512, 256, 16, 2.79f, 0.386f, 0.74f, 5.38f, 0.300f, 0.88f, 0.302f, 0.44f},  // 64x128 s3
        {256, 256, 16, 3.53f, 0.630f, 0.89f, 4.81f, 0.291f, 1.23f, 0.000f, 0.00f},  // 64x32 s3
        {256, 256, 16, 3.26f, 0.649f, 0.80f, 5.42f, 0.095f, 1.14f, 0.000f, 0.00f},  // 128x64 s3
    },
};
// fp32: one 64x64 work-group of four waves already keeps a CU's matrix pipe busy (a 32x32x2 MFMA is 64 cycles), so time follows
// the work of the busiest CU and idle CUs are lost outright: 256x256x8192 runs 127 us on its 16 tiles and 23 us with K split 16
// ways.  Fitted to 70 skinny and 50 squarish shapes, both layouts of B, B from HBM.
static const SmallGridModel kSmallGridF32[11] = {
    {512, 0, 0, 4.84f, 1.832f, 0.94f, 0.00f, 0.000f, 1.00f, 0.300f, 0.50f},  // 128x128x32 s2
    {512, 0, 0, 4.95f, 0.944f, 0.91f, 0.00f, 0.000f, 1.00f, 0.300f, 0.50f},  // 128x128x16 s4
    {512, 0, 0, 2.36f, 0.612f, 0.73f, 0.00f, 0.000f, 0.00f, 0.398f, 0.87f},  // 64x64x32 s2
    {512, 4096, 8, 3.95f, 0.536f, 0.72f, 5.54f, 0.071f, 1.66f, 0.443f, 0.83f},  // 64x64x32 s3
    {512, 0, 0, 2.38f, 1.208f, 0.82f, 0.00f, 0.000f, 0.00f, 0.905f, 0.87f},  // 64x64x64 s2
    {256, 0, 0, 4.18f, 2.138f, 0.87f, 0.00f, 0.000f, 1.27f, 0.000f, 0.00f},  // 64x64x128 s2, 8 waves
    {512, 512, 8, 3.12f, 0.630f, 0.76f, 4.56f, 0.817f, 0.00f, 0.635f, 0.48f},  // 32x128x32 s3 n
    {512, 512, 8, 2.58f, 0.639f, 0.72f, 5.36f, 0.534f, 0.36f, 0.594f, 0.53f},  // 32x128x32 s3 t
    {512, 512, 4, 2.35f, 0.857f, 0.78f, 4.01f, 0.947f, 0.00f, 0.573f, 0.50f},  // 32x32x128 s2 t
    {256, 256, 4, 3.06f, 0.735f, 0.89f, 3.36f, 1.485f, 1.05f, 0.000f, 0.00f},  // 32x32x128 s4 t
    {256, 256, 4, 3.32f, 1.127f, 0.98f, 4.25f, 0.048f, 2.24f, 0.000f, 0.00f},  // 64x32x128 s3 t
};
static int small_grid_class_f32(const KernelEntry* k) {
  if (k->bm == 32) return k->bn == 32 ? (k->stages >= 3 ? 9 : 8) : (k->transB ? 7 : 6);
  if (k->bn == 32) return 10;
  if (k->bm == 128) return k->bk <= 16 ? 1 : 0;
  if (k->bk >= 128) return 5;
  if (k->bk >= 64) return 4;
  return k->stages >= 3 ? 3 : 2;
}
static int small_grid_class(const KernelEntry* k) {
  if (k->bm == 32) return k->bn == 32 ? (k->stages >= 3 ? 10 : 9) : (k->transB ? 8 : 7);
  if (k->bm == 64) return k->wk > 1 ? 12 : 11;
  if (k->bm == 128 && k->bn == 64) return 13;
  if ((int64_t)k->bm * k->bn >= 256 * 256) return k->wm * k->wn > 4 ? 6 : (k->atom == 16 ? 5 : 4);
  if (k->bm == 256) return 3;
  if (k->bn == 256) return 2;
  return k->stages >= 3 ? 1 : 0;
}
static bool small_grid(const frisk_gemm_desc* d) {
  return d->split_k <= 1 && ((d->M + 127) / 128) * ((d->N + 127) / 128) <= 256;
}
static const SmallGridModel& small_grid_model(const KernelEntry* k) {
  if (k->dtype == FRISK_F32) return kSmallGridF32[small_grid_class_f32(k)];
  return kSmallGrid[k->dtype == FRISK_I8 ? 1 : (k->dtype == FRISK_E4M3 ? 2 : 0)][small_grid_class(k)];
}
static double small_grid_time(const SmallGridModel& m, const KernelEntry* k, const frisk_gemm_desc* d, int split) {
  const int64_t tiles = ((d->M + k->bm - 1) / k->bm) * ((d->N + k->bn - 1) / k->bn);
  const double kt = (double)((d->K + k->bk - 1) / k->bk) / split;
  const int64_t wgs = tiles * split, full = wgs / m.cap, rest = wgs % m.cap;
  double t = m.launch, whole = kt * m.tk + m.ps, last = 0.0;
  if (m.cap == 512) {  // two work-groups per CU: the second one of any CU sets the pace of the round
    whole += kt * m.tk2;
    const double f1 = (double)std::min<int64_t>(rest, 256) / 256.0, f2 = (double)std::max<int64_t>(rest - 256, 0) / 256.0;
    last = kt * (m.tk * (m.a + (1.0 - m.a) * f1) + (rest > 256 ? m.tk2 * (m.a2 + (1.0 - m.a2) * f2) : 0.0));
  } else {
    last = kt * m.tk * (m.a + (1.0 - m.a) * (double)rest / m.cap);
  }
  t += (double)full * whole + (rest ? last : 0.0);
  if (split > 1) t += m.r0 + m.r1 * ((double)d->M * (double)d->N * split * 4.0 / 1e6);
  return k->guard ? 3.0 * t : t;
}
// the split of a variant: among the powers of two the rule admits, the one the model makes fastest; *cost receives its time
static int small_grid_split(const KernelEntry* k, const frisk_gemm_desc* d, bool no_split, double* cost = nullptr) {
  const SmallGridModel& m = small_grid_model(k);
  int best = 1;
  double best_t = small_grid_time(m, k, d, 1);
  if (k->splitk && !no_split && d->split_k != 1 && m.w != 0 && d->K % k->bk == 0) {
    const int64_t tiles = ((d->M + k->bm - 1) / k->bm) * ((d->N + k->bn - 1) / k->bn), kt = d->K / k->bk;
    for (int c = 2; c <= (k->dtype == FRISK_F32 ? 32 : 64); c *= 2)  // the sweeps behind the tables: fp32 up to 32 slices
      if (tiles * c <= m.w && kt % c == 0 && kt / c >= std::max(m.kmin, k->min_k_tiles)) {
        const double t = small_grid_time(m, k, d, c);
        if (t < best_t) { best = c; best_t = t; }
      }
  }
  if (cost) *cost = best_t;
  return best;
}
static double small_grid_cost(const KernelEntry* k, const frisk_gemm_desc* d, bool no_split) {
  double t = 0.0;
  small_grid_split(k, d, no_split, &t);
  return t;
}

static int make_plan(const frisk_gemm_desc* d, frisk_gemm_plan* plan, bool with_model, bool force_guard = false, bool no_split = false) {
  int st = validate(d);
  if (st != FRISK_OK) return st;
  if (!plan) return fail(FRISK_ERR_NULL, "plan is null");
  std::memset(plan, 0, sizeof *plan);
  plan->kernel_id = -1;
  const int es = elem_size(d->dtype_ab), os = elem_size(d->dtype_out);
  plan->flops = 2.0 * (double)d->M * (double)d->N * (double)d->K;
  plan->bytes = (double)d->M * d->K * es + (double)d->K * d->N * es + (double)d->M * d->N * os;
  if (d->epilogue == FRISK_EPI_ROW_COL_SCALE) plan->bytes += 4.0 * ((double)d->M + (double)d->N);
  if (d->epilogue == FRISK_EPI_TENSOR_SCALE) plan->bytes += 8.0;
  plan->split_k = 1;

  const bool rows_aligned = (d->lda * es) % 16 == 0 && (d->ldb * es) % 16 == 0 && (d->ldc * os) % 16 == 0;
  const auto& ks = kernels();
  int best = -1;
  double best_cost = 0.0;
  bool policy_excluded = false;
  bool any_layout = false, tile_requested = d->tile_m || d->tile_n || d->tile_k || d->waves_m || d->waves_n || d->stages || d->atom;
  const bool small = small_grid(d);
  auto search = [&](bool want_split) {
    for (size_t i = 0; i < ks.size(); ++i) {
      const KernelEntry* k = ks[i];
      if (k->dtype != d->dtype_ab || k->transA != (d->transA != 0) || k->transB != (d->transB != 0)) continue;
      any_layout = true;
      if (d->tile_m && d->tile_m != k->bm) continue;
      if (d->tile_n && d->tile_n != k->bn) continue;
      if (d->tile_k && d->tile_k != k->bk) continue;
      if (d->waves_m && d->waves_m != k->wm) continue;
      if (d->waves_n && d->waves_n != k->wn) continue;
      if (d->stages && d->stages != k->stages_b) continue;  // the deeper ring names the variant
      if (d->atom && d->atom != k->atom) continue;
      // frisk.gemm's wave policy (FriskOps.td:248-289) decides the wave grid unless the descriptor names one: only variants
      // whose compiled grid is what computeWarpPartition gives for their tile and wave count under that policy qualify
      if (!d->waves_m && !d->waves_n) {
        int pm = 0, pn = 0;
        wave_partition(d->policy, k->bm, k->bn, k->wm * k->wn, k->atom, k->atom, &pm, &pn);
        if (pm != k->wm || pn != k->wn) { policy_excluded = true; continue; }
      }
      if (want_split && !k->splitk) continue;
      // a kernel whose loop needs a minimum of K tiles: per slice when the descriptor asks for a split
      if (k->min_k_tiles > 1 && (d->K + k->bk - 1) / k->bk / (want_split && d->split_k > 1 ? d->split_k : 1) < k->min_k_tiles) continue;
      // the fast kernels need whole tiles and rows that start on 16-byte boundaries; their edge variants take any M and N (and
      // are left out where the plain twin fits); the guarded ones take anything
      const bool whole_mn = d->M % k->bm == 0 && d->N % k->bn == 0;
      if (!k->guard && (force_guard || !rows_aligned || d->K % k->bk || (k->edge ? whole_mn : !whole_mn))) continue;
      // the guarded kernels that move whole 16-byte chunks: aligned rows and pointers, K a whole number of chunks
      if (k->guard && k->edge && (force_guard || !rows_aligned || d->K % (16 / es))) continue;
      // ... and address a tile's chunks by 32-bit lane offsets from its first row: the stored rows of one tile must span
      // less than 4 GiB
      const double span_a = (double)d->lda * es * (d->transA ? k->bk : k->bm), span_b = (double)d->ldb * es * (d->transB ? k->bn : k->bk);
      if (!k->guard && (span_a >= 4294967296.0 || span_b >= 4294967296.0)) continue;
      if (k->guard && best >= 0 && !ks[best]->guard) continue;  // never a guarded kernel when a fast one fits
      double cost = small && !want_split ? small_grid_cost(k, d, no_split) : estimated_cost(k, d, !want_split && !no_split && d->split_k == 0);
      // (a 32-row edge tile above 64 rows streams B once per 32 rows where the 64-row tile wastes at most as much: 130x11008x4096
      // NT 64.5 against 53.5 us)
      if (k->edge && k->bm == 32 && d->M > 64 && !d->tile_m) continue;
      if (k->edge && !k->guard) {
        // the models see whole tiles; rows and columns beyond M and N are work all the same (a 64-row tile on 32 rows is no
        // better than the 32-row tile that fits): the square root of the covered area over M x N, as a penalty
        const double covered = (double)((d->M + k->bm - 1) / k->bm * k->bm) * (double)((d->N + k->bn - 1) / k->bn * k->bn);
        cost *= std::sqrt(covered / ((double)d->M * (double)d->N));
      }
      // ties: the first listed variant is the tuned default
      if (best < 0 || (ks[best]->guard && !k->guard) || cost < best_cost) { best = (int)i; best_cost = cost; }
    }
  };
  // an explicit split_k looks among the variants with the split-K store path first; if none of them fits, the choice among
  // all variants reports below that it cannot split
  const bool explicit_split = d->split_k > 1 && !no_split;
  search(explicit_split);
  if (best < 0 && explicit_split) search(false);
  if (d->M == 0 || d->N == 0) {  // nothing to compute
    plan->grid_x = plan->grid_y = 0;
    return FRISK_OK;
  }
  if (best < 0) {
    if (!any_layout) return fail(FRISK_ERR_DTYPE, "no kernel compiled for dtype %d transA=%d transB=%d", d->dtype_ab, d->transA, d->transB);
    if (policy_excluded && d->policy != FRISK_POLICY_SQUARE)
      return fail(FRISK_ERR_TILE, "wave policy %s: no compiled kernel for M=%lld N=%lld K=%lld has the wave grid that policy gives (compiled grids: 2x2, 1x4, 2x4, 1x1)",
                  d->policy == FRISK_POLICY_FULL_ROW ? "FullRow" : "FullCol", (long long)d->M, (long long)d->N, (long long)d->K);
    if (tile_requested)
      return fail(FRISK_ERR_TILE, "no compiled kernel with tile %dx%dx%d waves %dx%d atom %d divides M=%lld N=%lld K=%lld", d->tile_m, d->tile_n,
                  d->tile_k, d->waves_m, d->waves_n, d->atom, (long long)d->M, (long long)d->N, (long long)d->K);
    return fail(FRISK_ERR_SHAPE, "M=%lld N=%lld K=%lld is not a multiple of any compiled tile", (long long)d->M, (long long)d->N, (long long)d->K);
  }
  const KernelEntry* k = ks[best];
  if (k->lds_bytes > 160 * 1024) return fail(FRISK_ERR_LDS, "tile needs %d bytes of LDS", k->lds_bytes);
  plan->kernel_id = best;
  plan->tile_m = k->bm; plan->tile_n = k->bn; plan->tile_k = k->bk;
  plan->waves_m = k->wm; plan->waves_n = k->wn; plan->waves_k = k->wk; plan->threads = k->wm * k->wn * k->wk * 64;
  plan->mfma_m = k->atom; plan->mfma_n = k->atom; plan->mfma_k = mfma_k(d->dtype_ab) * (32 / k->atom);
  plan->lds_bytes = k->lds_bytes;
  plan->stages = k->stages;
  plan->stages_b = k->stages_b;
  plan->grid_x = (int)((d->N + k->bn - 1) / k->bn);
  plan->grid_y = (int)((d->M + k->bm - 1) / k->bm);
  plan->guarded = k->guard;
  plan->xcd_remap = ((int64_t)plan->grid_x * plan->grid_y) % 8 == 0;
  fill_layout(&plan->lds_a, !d->transA, es, frag_bytes(d->dtype_ab), k->bm, k->bk, k->wm * k->wn * k->wk, with_model, k->atom);
  fill_layout(&plan->lds_b, d->transB != 0, es, frag_bytes(d->dtype_ab), k->bn, k->bk, k->wm * k->wn * k->wk, with_model, k->atom);
  plan->workspace_bytes = 0;
  // Split K over the grid's y dimension when the tile grid alone leaves most CUs idle (skinny problems are
  // bound by streaming the large operand, which needs many work-groups in flight).  Slices hold whole K tiles.
  const int64_t kt = d->K / k->bk, tiles = (int64_t)plan->grid_x * plan->grid_y;
  int split = 1;
  if (k->splitk && !no_split && d->K % k->bk == 0) {
    if (d->split_k > 1) {
      if (kt % d->split_k) return fail(FRISK_ERR_TILE, "split_k=%d does not divide the %lld K tiles", d->split_k, (long long)kt);
      if (kt / d->split_k < k->min_k_tiles)
        return fail(FRISK_ERR_TILE, "split_k=%d leaves %lld K tiles per slice, the chosen kernel %s needs %d", d->split_k, (long long)(kt / d->split_k), k->name, k->min_k_tiles);
      split = d->split_k;
    } else if (small) {
      split = small_grid_split(k, d, no_split);
    } else if (d->split_k == 0 && tiles < 256) {
      split = sub_round_split(k, tiles, kt);
    } else if (d->split_k == 0) {
      const int ts = tail_split_of(k, tiles, kt, true);
      if (ts > 1) {
        plan->tail_split = ts;
        plan->tail_tiles = (int)(tiles % 256);
        plan->workspace_bytes = (size_t)ts * (size_t)plan->tail_tiles * (size_t)k->bm * (size_t)k->bn * 4;
      }
    }
  } else if (d->split_k > 1 && !no_split) {
    return fail(FRISK_ERR_TILE, "split_k=%d: the chosen kernel %s has no split-K path", d->split_k, k->name);
  }
  plan->split_k = split;
  if (split > 1) plan->workspace_bytes = (size_t)split * (size_t)d->M * (size_t)d->N * 4;
  if (plan->tail_split <= 1) { plan->tail_split = 1; plan->tail_tiles = 0; }
  return FRISK_OK;
}

// rows of tiles walked together so that the work-groups resident on one XCD form a compact block
static int group_rows(int tiles_m, int tiles_n) {
  int64_t total = (int64_t)tiles_m * tiles_n;
  int64_t per_xcd = std::max<int64_t>(1, std::min<int64_t>(total / 8, 32));
  int g = 1;
  while ((int64_t)(2 * g) * (2 * g) <= per_xcd) g *= 2;
  return std::max(1, std::min(g, tiles_m));
}

static int device_ok() {
  static std::atomic<int> cached{-1};  // the answer for the process's GPU; racing threads compute the same value
  int c = cached.load(std::memory_order_relaxed);
  if (c >= 0) return c;
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
  c = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 0;
  cached.store(c, std::memory_order_relaxed);
  return c;
}

// a rank-2 view handed to the tile ops: element type, extents, leading dimension, pointer
static int check_view(const char* what, int dtype, const void* p, int64_t rows, int64_t cols, int64_t ld) {
  if (dtype != FRISK_F32 && dtype != FRISK_F16 && dtype != FRISK_BF16) return fail(FRISK_ERR_DTYPE, "%s: element type %d is not f32, f16 or bf16", what, dtype);
  if (rows < 0 || cols < 0) return fail(FRISK_ERR_SHAPE, "%s: negative extent %lld x %lld", what, (long long)rows, (long long)cols);
  if (rows > INT32_MAX || cols > INT32_MAX) return fail(FRISK_ERR_SHAPE, "%s: extent exceeds 2^31-1", what);
  if (ld < cols) return fail(FRISK_ERR_SHAPE, "%s: leading dimension %lld smaller than the row length %lld", what, (long long)ld, (long long)cols);
  if (rows * cols > 0 && !p) return fail(FRISK_ERR_NULL, "%s: pointer is null", what);
  if ((uintptr_t)p & (uintptr_t)(elem_size(dtype) - 1)) return fail(FRISK_ERR_ALIGNMENT, "%s: pointer is not aligned to its element size", what);
  return FRISK_OK;
}

static bool rows_on_16_bytes(int dtype, const void* p, int64_t ld) { return ((uintptr_t)p & 15) == 0 && (ld * elem_size(dtype)) % 16 == 0; }

}  // namespace frisk

using namespace frisk;

extern "C" {

int frisk_hip_abi_version(void) { return FRISK_HIP_ABI_VERSION; }

const char* frisk_hip_last_error(void) { return g_last_error.c_str(); }

int frisk_hip_init(void) {
  if (!device_ok()) return fail(FRISK_ERR_DEVICE, "no gfx950 device is current");
  for (const KernelEntry* k : kernels())
    if (hipError_t e = k->prepare(); e != hipSuccess) return fail(FRISK_ERR_DEVICE, "preparing %s failed: %s", k->name, hipGetErrorString(e));
  if (hipError_t e = prepare_attention(); e != hipSuccess) return fail(FRISK_ERR_DEVICE, "preparing the attention kernels failed: %s", hipGetErrorString(e));
  void* ws = nullptr;
  if (hipError_t e = scratch_of_current_device(&ws); e != hipSuccess) return fail(FRISK_ERR_DEVICE, "resolving the static workspace failed: %s", hipGetErrorString(e));
  return FRISK_OK;
}

int frisk_hip_plan(const frisk_gemm_desc* desc, frisk_gemm_plan* plan) { return make_plan(desc, plan, true); }

size_t frisk_hip_workspace_bytes(const frisk_gemm_desc* desc) {
  frisk_gemm_plan plan;
  if (make_plan(desc, &plan, false) != FRISK_OK) return 0;
  return plan.workspace_bytes;
}

int frisk_hip_gemm(const frisk_gemm_desc* desc, const void* A, const void* B, void* C, const float* scaleA,
                   const float* scaleB, void* workspace, size_t workspace_bytes, void* stream) {
  frisk_gemm_plan plan;
  int st = make_plan(desc, &plan, false);
  if (st != FRISK_OK) return st;
  if (desc->M == 0 || desc->N == 0) return FRISK_OK;
  if (!A || !B || !C) return fail(FRISK_ERR_NULL, "A, B and C must be device pointers");
  if (desc->epilogue != FRISK_EPI_NONE && (!scaleA || !scaleB)) return fail(FRISK_ERR_EPILOGUE, "epilogue %d needs scaleA and scaleB", desc->epilogue);
  const uintptr_t es = (uintptr_t)elem_size(desc->dtype_ab), os = (uintptr_t)elem_size(desc->dtype_out);
  if (((uintptr_t)A | (uintptr_t)B) & (es - 1) || (uintptr_t)C & (os - 1) || (((uintptr_t)scaleA | (uintptr_t)scaleB) & 3))
    return fail(FRISK_ERR_ALIGNMENT, "pointers must be aligned to their element size");
  const bool ptrs16 = ((((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15) == 0) &&
                      !(desc->epilogue == FRISK_EPI_ROW_COL_SCALE && ((uintptr_t)scaleB & 15));
  if (!ptrs16 && !plan.guarded) {  // the fast kernels move 16-byte chunks: fall back to the guarded kernel
    st = make_plan(desc, &plan, false, true);
    if (st != FRISK_OK) return st;
  }
  if (plan.workspace_bytes > 0 && (!workspace || workspace_bytes < plan.workspace_bytes)) {
    // an explicit split_k needs its workspace; the planner's own choice degrades to a single pass without one
    if (desc->split_k > 1) return fail(FRISK_ERR_WORKSPACE, "split_k=%d needs %zu bytes of workspace", desc->split_k, plan.workspace_bytes);
    st = make_plan(desc, &plan, false, plan.guarded != 0, true);
    if (st != FRISK_OK) return st;
  }
  if ((plan.split_k > 1 || plan.tail_split > 1) && ((uintptr_t)workspace & 15)) return fail(FRISK_ERR_ALIGNMENT, "workspace must be 16-byte aligned");
  if (!device_ok()) return fail(FRISK_ERR_DEVICE, "no gfx950 device is current");

  GemmParams p;
  p.A = A; p.B = B; p.C = C; p.scaleA = scaleA; p.scaleB = scaleB;
  p.lda = desc->lda; p.ldb = desc->ldb; p.ldc = desc->ldc;
  p.M = (int)desc->M; p.N = (int)desc->N; p.K = (int)desc->K;
  p.tiles_m = plan.grid_y; p.tiles_n = plan.grid_x;
  p.group_m = group_rows(p.tiles_m, p.tiles_n);
  p.xcd_remap = plan.xcd_remap;
  p.epilogue = desc->epilogue; p.dtype_out = desc->dtype_out; p.accumulate = desc->clear_accum ? 0 : 1;
  const KernelEntry* k = kernels()[plan.kernel_id];
  p.split_k = plan.split_k;
  p.kt_per_slice = (int)((desc->K + k->bk - 1) / k->bk) / plan.split_k;
  p.partial = plan.split_k > 1 || plan.tail_split > 1 ? workspace : nullptr;
  p.tail_split = plan.tail_split;
  p.tail_tiles = plan.tail_tiles;
  p.tail_from = p.tiles_m * p.tiles_n - plan.tail_tiles;
  p.tail_kt = plan.tail_split > 1 ? p.kt_per_slice / plan.tail_split : 0;
  p.tile_m = k->bm; p.tile_n = k->bn;
  p.k_rotate = 1;
  hipError_t e = k->launch(p, (hipStream_t)stream);
  if (e != hipSuccess) return fail(FRISK_ERR_DEVICE, "launch of %s failed: %s", k->name, hipGetErrorString(e));
  if (plan.split_k > 1) {
    e = launch_splitk_reduce(p, desc->dtype_acc == FRISK_I32, (hipStream_t)stream);
    if (e != hipSuccess) return fail(FRISK_ERR_DEVICE, "launch of the split-K reduction failed: %s", hipGetErrorString(e));
  }
  if (plan.tail_split > 1) {
    e = launch_tail_reduce(p, desc->dtype_acc == FRISK_I32, (hipStream_t)stream);
    if (e != hipSuccess) return fail(FRISK_ERR_DEVICE, "launch of the tail reduction failed: %s", hipGetErrorString(e));
  }
  return FRISK_OK;
}

size_t frisk_hip_static_workspace_bytes(void) { return (size_t)FRISK_HIP_STATIC_WS_BYTES; }

int frisk_hip_gemm_static_ws(const frisk_gemm_desc* desc, const void* A, const void* B, void* C, const float* scaleA, const float* scaleB,
                             void* stream) {
  frisk_gemm_plan plan;
  int st = make_plan(desc, &plan, false);
  if (st != FRISK_OK) return st;
  // What does not fit the array: an explicit split_k is refused (the caller asked for exactly that split); a split the
  // planner chose by itself (tail splits of large grids reach 64 MiB) is dropped, and the launch runs as one pass, which
  // is what frisk_hip_gemm does for the same descriptor without a workspace.
  if (plan.workspace_bytes > (size_t)FRISK_HIP_STATIC_WS_BYTES) {
    if (desc->split_k > 1)
      return fail(FRISK_ERR_WORKSPACE, "split_k=%d needs %zu bytes of partial sums, the static workspace holds %zu: pass a smaller split_k, or use frisk_hip_gemm with a workspace",
                  desc->split_k, plan.workspace_bytes, (size_t)FRISK_HIP_STATIC_WS_BYTES);
    return frisk_hip_gemm(desc, A, B, C, scaleA, scaleB, nullptr, 0, stream);
  }
  void* ws = nullptr;
  if (plan.workspace_bytes > 0) {
    if (!device_ok()) return fail(FRISK_ERR_DEVICE, "no gfx950 device is current");
    if (hipError_t e = scratch_of_current_device(&ws); e != hipSuccess) return fail(FRISK_ERR_DEVICE, "resolving the static workspace failed: %s", hipGetErrorString(e));
  }
  // every slice of a split stores its whole share of the partial sums before the reduction reads it: nothing to clear
  return frisk_hip_gemm(desc, A, B, C, scaleA, scaleB, ws, ws ? (size_t)FRISK_HIP_STATIC_WS_BYTES : 0, stream);
}

float frisk_hip_lds_access_cycles(int instr, const int32_t* lane_byte_addr) {
  if (!lane_byte_addr) return -1.f;
  int addr[64];
  for (int i = 0; i < 64; ++i) addr[i] = lane_byte_addr[i];
  return (float)lds_access_cycles(instr == 2 ? 1 : instr, addr);
}

int frisk_hip_lds_search(const frisk_lds_layout* shape, int elem_bytes, int frag_bytes, int tile_mn, int tile_k, int waves,
                         frisk_lds_layout* best, float* unswizzled_cycles) {
  return frisk_hip_lds_search_atom(shape, elem_bytes, frag_bytes, tile_mn, tile_k, waves, 32, best, unswizzled_cycles);
}

int frisk_hip_lds_search_atom(const frisk_lds_layout* shape, int elem_bytes, int frag_bytes, int tile_mn, int tile_k, int waves, int atom,
                              frisk_lds_layout* best, float* unswizzled_cycles) {
  if (atom != 32 && atom != 16) return fail(FRISK_ERR_TILE, "MFMA atoms have 32 or 16 rows, not %d", atom);
  if (atom == 16 && elem_bytes == 4) return fail(FRISK_ERR_TILE, "the 32-bit operands have no 16-row atom here");
  if (!shape || !best) return fail(FRISK_ERR_NULL, "shape and best must be given");
  if (shape->rows <= 0 || shape->row_bytes < 16 || shape->row_bytes % 16 || shape->row_bytes > 1024 || 1024 % shape->row_bytes)
    return fail(FRISK_ERR_TILE, "tile rows must be 16..1024 bytes and divide 1024");
  if ((elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4) || frag_bytes < elem_bytes || waves <= 0 || tile_mn < 32 || tile_k <= 0)
    return fail(FRISK_ERR_TILE, "unsupported operand description");
  const bool kc = shape->k_contiguous != 0;
  TileShape t{shape->rows, shape->row_bytes, kc, elem_bytes, frag_bytes, tile_mn, tile_k, atom};
  const Swizzle s = choose_swizzle(t, waves);
  const int atoms = tile_mn / atom < 4 ? tile_mn / atom : 4;
  const int n_access = atoms * ((tile_k * elem_bytes) / frag_kstep_bytes(frag_bytes, atom)) * frag_instr_count(kc, elem_bytes, frag_bytes);
  if (n_access <= 0) return fail(FRISK_ERR_TILE, "tile holds no whole MFMA step");
  *best = *shape;
  best->row_shift = s.sh; best->row_mask = s.mk; best->chunk_shift = s.cs;
  best->row_shift2 = s.sh2; best->row_mask2 = s.mk2; best->chunk_shift2 = s.cs2;
  best->read_instr = elem_bytes == 4 ? (kc && frag_bytes >= 16 ? 0 : 3) : (kc ? 0 : (elem_bytes == 2 ? 1 : 2));
  best->read_cycles = (float)swizzle_read_cycles(t, s) / (float)n_access;
  best->write_cycles = 16.f;
  if (unswizzled_cycles) *unswizzled_cycles = (float)swizzle_read_cycles(t, Swizzle{0, 0, 0}) / (float)n_access;
  return FRISK_OK;
}

int32_t frisk_hip_lds_offset(const frisk_lds_layout* L, int32_t row, int32_t col_byte) {
  if (!L) return -1;
  return lds_offset(L->row_bytes, Swizzle{L->row_shift, L->row_mask, L->chunk_shift, L->row_shift2, L->row_mask2, L->chunk_shift2}, row, col_byte);
}

int frisk_hip_wave_partition(int policy, int tile_m, int tile_n, int num_waves, int* waves_m, int* waves_n) {
  if (!waves_m || !waves_n) return fail(FRISK_ERR_NULL, "output pointers are null");
  if (policy < FRISK_POLICY_SQUARE || policy > FRISK_POLICY_FULL_COL) return fail(FRISK_ERR_TILE, "unknown wave policy %d", policy);
  wave_partition(policy, tile_m, tile_n, num_waves, 32, 32, waves_m, waves_n);
  return FRISK_OK;
}

int frisk_hip_fill(int dtype, void* dst, int64_t rows, int64_t cols, int64_t ld, double value, void* stream) {
  if (int st = check_view("fill destination", dtype, dst, rows, cols, ld)) return st;
  if (rows == 0 || cols == 0) return FRISK_OK;
  if (!device_ok()) return fail(FRISK_ERR_DEVICE, "no gfx950 device is current");
  if (ld == cols) { cols *= rows; rows = 1; ld = cols; }  // a dense view is one long row
  hipError_t e = launch_fill(dtype, dst, rows, cols, ld, value, rows_on_16_bytes(dtype, dst, ld), (hipStream_t)stream);
  if (e != hipSuccess) return fail(FRISK_ERR_DEVICE, "fill launch failed: %s", hipGetErrorString(e));
  return FRISK_OK;
}

int frisk_hip_copy(int src_dtype, const void* src, int64_t src_ld, int dst_dtype, void* dst, int64_t dst_ld, int64_t rows, int64_t cols,
                   void* stream) {
  if (int st = check_view("copy source", src_dtype, src, rows, cols, src_ld)) return st;
  if (int st = check_view("copy destination", dst_dtype, dst, rows, cols, dst_ld)) return st;
  if (rows == 0 || cols == 0) return FRISK_OK;
  if (!device_ok()) return fail(FRISK_ERR_DEVICE, "no gfx950 device is current");
  if (src_ld == cols && dst_ld == cols) { cols *= rows; rows = 1; src_ld = dst_ld = cols; }
  const int vec = rows_on_16_bytes(src_dtype, src, src_ld) && rows_on_16_bytes(dst_dtype, dst, dst_ld);
  hipError_t e = launch_copy(src_dtype, src, src_ld, dst_dtype, dst, dst_ld, rows, cols, vec, (hipStream_t)stream);
  if (e != hipSuccess) return fail(FRISK_ERR_DEVICE, "copy launch failed: %s", hipGetErrorString(e));
  return FRISK_OK;
}

int frisk_hip_copy_tiles(int src_dtype, const void* src, int64_t src_ld, int dst_dtype, void* dst, int64_t dst_ld, int64_t tile_rows, int64_t tile_cols,
                         int64_t n0, int64_t src_step0, int64_t dst_step0, int64_t n1, int64_t src_step1, int64_t dst_step1, void* stream) {
  const int64_t view_rows = (n0 == 0 || n1 == 0) ? 0 : tile_rows;  // no tile: no pointer is looked at
  if (int st = check_view("tiled copy source", src_dtype, src, view_rows, tile_cols, src_ld)) return st;
  if (int st = check_view("tiled copy destination", dst_dtype, dst, view_rows, tile_cols, dst_ld)) return st;
  if (n0 < 0 || n1 < 0 || src_step0 < 0 || src_step1 < 0 || dst_step0 < 0 || dst_step1 < 0) return fail(FRISK_ERR_SHAPE, "tiled copy: negative tile count or step");
  if (n0 > INT32_MAX || n1 > INT32_MAX || n0 * n1 > INT32_MAX) return fail(FRISK_ERR_SHAPE, "tiled copy: more than 2^31-1 tiles");
  if (tile_rows == 0 || tile_cols == 0 || n0 == 0 || n1 == 0) return FRISK_OK;
  if (!device_ok()) return fail(FRISK_ERR_DEVICE, "no gfx950 device is current");
  const int ss = elem_size(src_dtype), ds = elem_size(dst_dtype);
  const bool steps16 = (src_step0 * ss) % 16 == 0 && (src_step1 * ss) % 16 == 0 && (dst_step0 * ds) % 16 == 0 && (dst_step1 * ds) % 16 == 0;
  const int vec = steps16 && rows_on_16_bytes(src_dtype, src, src_ld) && rows_on_16_bytes(dst_dtype, dst, dst_ld);
  TilePlacement t;
  t.n0 = n0; t.n1 = n1; t.src_step0 = src_step0; t.src_step1 = src_step1; t.dst_step0 = dst_step0; t.dst_step1 = dst_step1;
  hipError_t e = launch_copy_tiles(src_dtype, src, src_ld, dst_dtype, dst, dst_ld, tile_rows, tile_cols, t, vec, (hipStream_t)stream);
  if (e != hipSuccess) return fail(FRISK_ERR_DEVICE, "tiled copy launch failed: %s", hipGetErrorString(e));
  return FRISK_OK;
}

int frisk_hip_elementwise(const frisk_elementwise_desc* d, const void* const* inputs, void* out, void* stream) {
  if (!d) return fail(FRISK_ERR_NULL, "elementwise descriptor is null");
  if (d->abi_version != FRISK_HIP_ABI_VERSION) return fail(FRISK_ERR_ABI, "descriptor abi_version %d, library %d", d->abi_version, FRISK_HIP_ABI_VERSION);
  if (d->n_inputs < 0 || d->n_inputs > FRISK_EW_MAX_INPUTS) return fail(FRISK_ERR_ARGUMENT, "elementwise: %d operands, at most %d", d->n_inputs, FRISK_EW_MAX_INPUTS);
  if (d->n_ops < 1 || d->n_ops > FRISK_EW_MAX_OPS) return fail(FRISK_ERR_ARGUMENT, "elementwise: a program of %d steps, 1 to %d allowed", d->n_ops, FRISK_EW_MAX_OPS);
  if (int st = check_view("elementwise output", d->out_dtype, out, d->rows, d->cols, d->out_ld)) return st;
  if (d->n_inputs > 0 && !inputs) return fail(FRISK_ERR_NULL, "elementwise: the operand pointer array is null");
  // the program on a counting stack: never empty when it pops, never deeper than the interpreter's registers, one value left
  int depth = 0;
  for (int i = 0; i < d->n_ops; ++i) {
    const int op = d->op[i];
    if (op < FRISK_EW_INPUT || op > FRISK_EW_LOG2) return fail(FRISK_ERR_ARGUMENT, "elementwise: unknown opcode %d at step %d", op, i);
    if (op == FRISK_EW_INPUT && (d->arg[i] < 0 || d->arg[i] >= d->n_inputs)) return fail(FRISK_ERR_ARGUMENT, "elementwise: step %d reads operand %d of %d", i, d->arg[i], d->n_inputs);
    const int pops = op <= FRISK_EW_CONST ? 0 : (op >= FRISK_EW_NEG ? 1 : 2);
    if (depth < pops) return fail(FRISK_ERR_ARGUMENT, "elementwise: step %d pops an empty stack", i);
    depth += 1 - pops;
    if (depth > FRISK_EW_MAX_STACK) return fail(FRISK_ERR_ARGUMENT, "elementwise: the program needs a stack deeper than %d", FRISK_EW_MAX_STACK);
  }
  if (depth != 1) return fail(FRISK_ERR_ARGUMENT, "elementwise: the program leaves %d values, not one", depth);
  if (d->rows == 0 || d->cols == 0) return FRISK_OK;
  EwParams p{};
  // a dense problem (every operand walked, every row following the one before) is one long row
  bool dense = d->out_ld == d->cols;
  for (int k = 0; k < d->n_inputs; ++k) dense = dense && d->in_col_stride[k] == 1 && d->in_row_stride[k] == d->cols;
  p.rows = dense ? 1 : d->rows;
  p.cols = dense ? d->rows * d->cols : d->cols;
  bool vec = p.cols % 8 == 0 && rows_on_16_bytes(d->out_dtype, out, dense ? 0 : d->out_ld);
  for (int k = 0; k < d->n_inputs; ++k) {
    const int dt = d->in_dtype[k];
    if (dt != FRISK_F32 && dt != FRISK_F16 && dt != FRISK_BF16) return fail(FRISK_ERR_DTYPE, "elementwise operand %d: element type %d is not f32, f16 or bf16", k, dt);
    if (d->in_col_stride[k] != 0 && d->in_col_stride[k] != 1) return fail(FRISK_ERR_SHAPE, "elementwise operand %d: column stride %d is not 0 or 1", k, d->in_col_stride[k]);
    if (d->in_row_stride[k] < 0) return fail(FRISK_ERR_SHAPE, "elementwise operand %d: negative row stride", k);
    if (!inputs[k]) return fail(FRISK_ERR_NULL, "elementwise operand %d: pointer is null", k);
    if ((uintptr_t)inputs[k] & (uintptr_t)(elem_size(dt) - 1)) return fail(FRISK_ERR_ALIGNMENT, "elementwise operand %d: pointer is not aligned to its element size", k);
    if (d->in_col_stride[k] == 1) vec = vec && rows_on_16_bytes(dt, inputs[k], dense ? 0 : d->in_row_stride[k]);
    p.in[k] = inputs[k]; p.in_row_stride[k] = d->in_row_stride[k]; p.in_dtype[k] = dt; p.in_col_stride[k] = d->in_col_stride[k];
  }
  if (!device_ok()) return fail(FRISK_ERR_DEVICE, "no gfx950 device is current");
  p.out = out; p.out_ld = d->out_ld; p.out_dtype = d->out_dtype; p.n_ops = d->n_ops;
  for (int i = 0; i < d->n_ops; ++i) { p.op[i] = d->op[i]; p.arg[i] = d->arg[i]; p.imm[i] = d->imm[i]; }
  hipError_t e = launch_elementwise(p, vec ? 1 : 0, (hipStream_t)stream);
  if (e != hipSuccess) return fail(FRISK_ERR_DEVICE, "elementwise launch failed: %s", hipGetErrorString(e));
  return FRISK_OK;
}

size_t frisk_hip_reduce_workspace_bytes(int dtype, int64_t rows, int64_t cols, int dim) {
  if ((dtype != FRISK_F32 && dtype != FRISK_F16 && dtype != FRISK_BF16) || rows <= 0 || cols <= 0 || (dim != 0 && dim != 1)) return 0;
  const int slices = reduce_slices(dtype, rows, cols, dim);
  return slices > 1 ? (size_t)slices * (size_t)(dim == 1 ? rows : cols) * 4 : 0;
}

int frisk_hip_reduce(int dtype, const void* src, int64_t rows, int64_t cols, int64_t ld, int dim, int kind, int clear, void* dst, void* workspace,
                     size_t workspace_bytes, void* stream) {
  if (int st = check_view("reduce source", dtype, src, rows, cols, ld)) return st;
  if (dim != 0 && dim != 1) return fail(FRISK_ERR_ARGUMENT, "reduce dim %d is out of range for a source of rank 2", dim);
  if (kind < FRISK_REDUCE_ADD || kind > FRISK_REDUCE_MAX) return fail(FRISK_ERR_ARGUMENT, "unsupported reduce kind %d (add, mul, min, max)", kind);
  const int64_t kept = dim == 1 ? rows : cols;
  if (kept == 0) return FRISK_OK;
  if (!dst) return fail(FRISK_ERR_NULL, "reduce destination: pointer is null");
  if ((uintptr_t)dst & (uintptr_t)(elem_size(dtype) - 1)) return fail(FRISK_ERR_ALIGNMENT, "reduce destination: pointer is not aligned to its element size");
  if (!device_ok()) return fail(FRISK_ERR_DEVICE, "no gfx950 device is current");
  int slices = (rows > 0 && cols > 0) ? reduce_slices(dtype, rows, cols, dim) : 1;
  // without a (large enough, 4-byte aligned) workspace the reduction runs unsplit: same result, fewer work-groups
  if (slices > 1 && (!workspace || workspace_bytes < (size_t)slices * (size_t)kept * 4 || ((uintptr_t)workspace & 3))) slices = 1;
  hipError_t e = launch_reduce(dtype, src, rows, cols, ld, dim, kind, clear ? 1 : 0, dst, (float*)workspace, slices, rows_on_16_bytes(dtype, src, ld),
                               (hipStream_t)stream);
  if (e != hipSuccess) return fail(FRISK_ERR_DEVICE, "reduce launch failed: %s", hipGetErrorString(e));
  return FRISK_OK;
}

size_t frisk_hip_softmax_workspace_bytes(int dtype, int64_t rows, int64_t cols) {
  if ((dtype != FRISK_F32 && dtype != FRISK_F16 && dtype != FRISK_BF16) || rows <= 0 || cols <= 0) return 0;
  const int slices = softmax_slices(dtype, rows, cols);
  return slices > 1 ? (size_t)rows * (size_t)slices * 8 : 0;
}

int frisk_hip_softmax(int dtype, const void* src, int64_t src_ld, void* dst, int64_t dst_ld, int64_t rows, int64_t cols, float scale_log2, float* lse,
                      void* workspace, size_t workspace_bytes, void* stream) {
  if (int st = check_view("softmax source", dtype, src, rows, cols, src_ld)) return st;
  if (int st = check_view("softmax destination", dtype, dst, rows, cols, dst_ld)) return st;
  if (!std::isfinite(scale_log2)) return fail(FRISK_ERR_ARGUMENT, "softmax scale %g is not finite", (double)scale_log2);
  if ((uintptr_t)lse & 3) return fail(FRISK_ERR_ALIGNMENT, "lse must be 4-byte aligned");
  if (rows == 0 || cols == 0) return FRISK_OK;
  if (!device_ok()) return fail(FRISK_ERR_DEVICE, "no gfx950 device is current");
  const int rows_aligned = rows_on_16_bytes(dtype, src, src_ld) && rows_on_16_bytes(dtype, dst, dst_ld);
  int slices = softmax_slices(dtype, rows, cols);
  // without a (large enough, 4-byte aligned) workspace the rows are not split: same result, fewer work-groups
  if (slices > 1 && (!workspace || workspace_bytes < (size_t)rows * (size_t)slices * 8 || ((uintptr_t)workspace & 3))) slices = 1;
  hipError_t e = launch_softmax_rows(dtype, src, src_ld, dst, dst_ld, rows, cols, scale_log2, lse, rows_aligned, (float*)workspace, slices, (hipStream_t)stream);
  if (e != hipSuccess) return fail(FRISK_ERR_DEVICE, "softmax launch failed: %s", hipGetErrorString(e));
  return FRISK_OK;
}

int frisk_hip_attention(const frisk_attention_desc* d, const void* Q, const void* K, const void* V, void* O, float* lse, void* stream) {
  if (!d) return fail(FRISK_ERR_NULL, "attention descriptor is null");
  if (d->abi_version != FRISK_HIP_ABI_VERSION) return fail(FRISK_ERR_ABI, "descriptor abi_version %d, library %d", d->abi_version, FRISK_HIP_ABI_VERSION);
  if (d->dtype != FRISK_F16 && d->dtype != FRISK_BF16) return fail(FRISK_ERR_DTYPE, "attention element type %d is not f16 or bf16", d->dtype);
  if (d->batch < 0 || d->heads < 0 || d->seq_q < 0 || d->seq_k < 0) return fail(FRISK_ERR_SHAPE, "negative extent");
  if (d->head_dim != kAttnHeadDim) return fail(FRISK_ERR_SHAPE, "head_dim %lld: the attention kernel is built for %d", (long long)d->head_dim, kAttnHeadDim);
  if (d->seq_q % kAttnQueriesPerGroup) return fail(FRISK_ERR_SHAPE, "seq_q %lld is not a multiple of %d", (long long)d->seq_q, kAttnQueriesPerGroup);
  if (d->seq_k % kAttnKeysPerTile || d->seq_k == 0) return fail(FRISK_ERR_SHAPE, "seq_k %lld is not a positive multiple of %d", (long long)d->seq_k, kAttnKeysPerTile);
  if (!(d->scale > 0.f) || !std::isfinite(d->scale)) return fail(FRISK_ERR_ARGUMENT, "softmax scale %g is not a positive finite number", (double)d->scale);
  const int64_t bh = d->batch * d->heads, groups = bh * (d->seq_q / kAttnQueriesPerGroup);
  if (d->seq_q > INT32_MAX || d->seq_k > INT32_MAX || bh > INT32_MAX || groups > INT32_MAX) return fail(FRISK_ERR_SHAPE, "extent exceeds 2^31-1");
  if (groups == 0) return FRISK_OK;
  if (!Q || !K || !V || !O) return fail(FRISK_ERR_NULL, "attention operand pointer is null");
  if (((uintptr_t)Q | (uintptr_t)K | (uintptr_t)V | (uintptr_t)O) & 15) return fail(FRISK_ERR_ALIGNMENT, "attention operands must be 16-byte aligned");
  if ((uintptr_t)lse & 3) return fail(FRISK_ERR_ALIGNMENT, "lse must be 4-byte aligned");
  if (!device_ok()) return fail(FRISK_ERR_DEVICE, "no gfx950 device is current");
  AttentionParams p;
  p.Q = Q; p.K = K; p.V = V; p.O = O; p.lse = lse;
  p.batch_heads = (int32_t)bh; p.seq_q = (int32_t)d->seq_q; p.seq_k = (int32_t)d->seq_k;
  p.q_blocks = (int32_t)(d->seq_q / kAttnQueriesPerGroup);
  p.xcd_remap = groups % 8 == 0 ? 1 : 0;
  p.scale_log2 = d->scale * 1.4426950408889634f;
  hipError_t e = launch_attention(d->dtype, d->k_transposed ? 1 : 0, p, (hipStream_t)stream);
  if (e != hipSuccess) return fail(FRISK_ERR_DEVICE, "attention launch failed: %s", hipGetErrorString(e));
  return FRISK_OK;
}

int frisk_hip_kernel_count(void) { return (int)kernels().size(); }
const char* frisk_hip_kernel_name(int id) {
  if (id < 0 || id >= (int)kernels().size()) return nullptr;
  return kernels()[id]->name;
}

}  // extern "C"
