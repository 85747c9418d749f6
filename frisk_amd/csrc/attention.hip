// Fused attention forward for gfx950: O = softmax(scale * Q K^T) V, one pass over the keys with a running
// maximum and denominator, the program of the reference's sketch tmp/ir.mlir:87-157 (copy Q; for each key tile:
// copy K, gemm, reduce max, exp2, reduce sum, rescale, copy V, gemm; copy O) executed as one kernel.
//
// A work-group of 8 waves owns 256 queries of one (batch, head); a wave owns 32 of them for the whole kernel, two
// waves share a SIMD.  Key / value tiles of 64 keys stream HBM/L2 -> LDS with global_load_lds_dwordx4 through rings
// of three (K) and four (V) tiles.  The two waves of a SIMD alternate between an MFMA phase and a softmax (VALU)
// phase in opposite order, so the matrix pipe and the vector pipe of the SIMD are busy at the same time.
// Both products are computed transposed so that a lane owns one query:
//   S^T[key][q] = sum_d K[key][d] Q[q][d]     MFMA A = K fragment (LDS), B = Q fragment (registers, loaded once)
//   O^T[d][q]   = sum_key V[key][d] P[q][key] MFMA A = V fragment (LDS, transpose read), B = P fragment
// In the 32x32 result layout lane l holds column l % 32 (a query) and rows 4*(l/32) + (r%4) + 8*(r/4): the maximum
// and the sum over keys are 16 in-register operations per atom plus one exchange with lane l ^ 32, and the
// probabilities of S^T are already the B operand of the second product if its K slots are read in the same
// permuted key order (slot 8g+e of a 16-key step is key 4g + e%4 + 8*(e/4)) -- the transpose reads of V fetch
// their 4-row groups in that order, so P never goes through LDS.
#include "gemm_kernel.hip.inc"
#include "attention.h"

namespace frisk {

template <int DT_, bool KT_> struct AttnCfg {
  static constexpr int DT = DT_;
  static constexpr bool KT = KT_;  // K stored [head_dim][seq_k]
  static constexpr int D = kAttnHeadDim, QB = kAttnQueriesPerGroup, KB = kAttnKeysPerTile;
  static constexpr int NW = 8, QW = QB / NW, KA = KB / 32, DA = D / 32;
  static constexpr int NSK = 3, NSV = 4;  // LDS ring depths: K is consumed one tile ahead of V
  typedef Mma<DT> M;
  typedef TileLayout<2, !KT, KB, D> LK;    // first product contracts over head_dim
  typedef TileLayout<2, false, D, KB> LV;  // second product contracts over keys; head_dim runs along the row
  static constexpr int RING_BYTES = NSK * LK::BYTES + NSV * LV::BYTES;
  static constexpr int OUT_BYTES_PER_WAVE = 32 * (64 * 2 + 16);  // output staging: 32 queries x 64 columns, rows padded by 16 B
  static constexpr int LDS_BYTES = RING_BYTES + NW * OUT_BYTES_PER_WAVE;
  static_assert(QW == 32, "one 32-query atom per wave");
  static_assert(M::ES == 2 && M::KA == 16, "16-bit operands");
  static_assert(LV::SH == 0 && LV::MK <= 3, "the V swizzle may only depend on the key row modulo 4");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");
};

// Address of the transpose read that serves head_dim atom `da` (32 columns of V) with K slots in the permuted key
// order: the lane's register holds key row 4g + (l%16)/4 of the tile, instruction q of step t adds 16t + 8q rows.
template <class LV> struct PermutedKeyReader {
  FRISK_DEV unsigned lane_reg(int lane, int da) {
    const int blk = lane >> 4, l16 = lane & 15, g = blk >> 1;
    return (unsigned)LV::offset(4 * g + (l16 >> 2), (32 * da + 16 * (blk & 1) + 4 * (l16 & 3)) * 2);
  }
  static constexpr int delta(int t, int q) { return (16 * t + 8 * q) * LV::ROWB; }
  FRISK_DEV void read(unsigned reg, int t, int* out) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      FRISK_LDS const char* p = (FRISK_LDS const char*)(uintptr_t)reg + delta(t, q);
      v2i w = __builtin_bit_cast(v2i, __builtin_amdgcn_ds_read_tr16_b64_v4i16((FRISK_LDS v4s*)p));
      out[2 * q] = w[0];
      out[2 * q + 1] = w[1];
    }
  }
};

// two fp32 -> one packed 16-bit pair, and sum of a packed pair added to an fp32 (one v_dot2 with a pair of ones)
template <int DT> struct Pack16;
template <> struct Pack16<FRISK_F16> {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  FRISK_DEV int two(float a, float b) {
    h2 v = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(int, v);
  }
  FRISK_DEV float add_pair(int pair, float acc) { return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, pair), h2{(_Float16)1, (_Float16)1}, acc, false); }
};
template <> struct Pack16<FRISK_BF16> {
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  FRISK_DEV int two(float a, float b) {
    b2 v = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(int, v);
  }
  FRISK_DEV float add_pair(int pair, float acc) { return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, pair), b2{(__bf16)1.f, (__bf16)1.f}, acc, false); }
};

// The exponent reference of a query row is only raised when the row maximum has grown by more than this many powers
// of two since it was last set: the accumulators are then rescaled (rarely), and probabilities stay below 2^8.
// The final division by the denominator makes the result independent of the reference.
constexpr float kAttnRescaleSlack = 8.f;

constexpr int kAttnPrefetch = 4;  // MFMA units between a fragment's LDS read and its use

template <class C>
__global__ void __launch_bounds__(C::NW * 64) attention_kernel(AttentionParams p) {
  typedef typename C::M M;
  typedef typename C::LK LK;
  typedef typename C::LV LV;
  typedef TileStager<LK, C::NW> SK;
  typedef TileStager<LV, C::NW> SV;
  typedef FragReader<LK, 16, C::KA, C::D / 16> RK;
  typedef PermutedKeyReader<LV> RV;
  typedef Pack16<C::DT> PK;
  constexpr int D = C::D, KB = C::KB, KA = C::KA, DA = C::DA, DSTEPS = D / 16, KSTEPS = KB / 16;
  constexpr int N1 = DSTEPS * KA;   // MFMAs of the first product per tile
  constexpr int N2 = KSTEPS * DA;   // MFMAs of the second product per tile
  constexpr int NE = KA * 16;       // scores per lane per tile
  static_assert(N1 == 16 && N2 == 16 && NE == 32, "the interleaving below is written for 64 keys x 128 head_dim");

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const unsigned smem_u = (unsigned)(uintptr_t)(FRISK_LDS char*)smem;
  const unsigned k_ring = smem_u, v_ring = smem_u + C::NSK * LK::BYTES;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lq = lane & 31, lh = lane >> 5;

  // consecutive work-group ids go to the 8 XCDs round-robin: give each XCD whole heads
  int cid = blockIdx.x;
  if (p.xcd_remap) {
    const int per = gridDim.x >> 3;
    if (cid < per * 8) cid = (cid & 7) * per + (cid >> 3);
  }
  const int bh = cid / p.q_blocks, qb = cid % p.q_blocks;
  const int64_t q0 = (int64_t)qb * C::QB + wave * C::QW;

  // Q fragments for the whole kernel: lane (q, g) holds Q[q][16 ks + 8 g .. + 7]
  v4i qf[DSTEPS];
  {
    const char* qbase = (const char*)p.Q + (((int64_t)bh * p.seq_q + q0 + lq) * D + 8 * lh) * 2;
#pragma unroll
    for (int ks = 0; ks < DSTEPS; ++ks) qf[ks] = *(const v4i*)(qbase + 32 * ks);
  }

  // staging: wave-uniform tile pointers plus one lane offset per operand
  const int64_t k_ld = C::KT ? (int64_t)p.seq_k * 2 : (int64_t)D * 2;
  const int64_t k_step = C::KT ? (int64_t)KB * 2 : (int64_t)KB * D * 2;
  const char* srcK = (const char*)p.K + (int64_t)bh * p.seq_k * D * 2 + SK::wave_src_offset(wave, k_ld);
  const char* srcV = (const char*)p.V + (int64_t)bh * p.seq_k * D * 2 + SV::wave_src_offset(wave, D * 2);
  unsigned voffK[SK::PER_WAVE], voffV[SV::PER_WAVE];
#pragma unroll
  for (int i = 0; i < SK::PER_WAVE; ++i) voffK[i] = SK::transfer_src_offset(i, lane, wave, k_ld);
#pragma unroll
  for (int i = 0; i < SV::PER_WAVE; ++i) voffV[i] = SV::transfer_src_offset(i, lane, wave, D * 2);
  constexpr int PER_TILE = SK::PER_WAVE + SV::PER_WAVE;
  int k_slot_issue = 0, v_slot_issue = 0;
  auto stage_tile = [&]() {
    const unsigned kdst = k_ring + k_slot_issue * LK::BYTES + (unsigned)wave * 1024u, vdst = v_ring + v_slot_issue * LV::BYTES + (unsigned)wave * 1024u;
#pragma unroll
    for (int i = 0; i < SK::PER_WAVE; ++i) SK::issue_one(i, srcK, voffK, kdst);
#pragma unroll
    for (int i = 0; i < SV::PER_WAVE; ++i) SV::issue_one(i, srcV, voffV, vdst);
    srcK += k_step;
    srcV += (int64_t)KB * D * 2;
    k_slot_issue = k_slot_issue == C::NSK - 1 ? 0 : k_slot_issue + 1;
    v_slot_issue = v_slot_issue == C::NSV - 1 ? 0 : v_slot_issue + 1;
  };

  unsigned rk[RK::NREG], rv[DA];
  RK::init(lane, 0, 0, rk);
#pragma unroll
  for (int da = 0; da < DA; ++da) rv[da] = RV::lane_reg(lane, da);

  v16f o[DA];
#pragma unroll
  for (int da = 0; da < DA; ++da)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[da][r] = 0.f;
  float l_run = 0.f;  // this lane's share of the denominator (its 32 keys of every tile)

  const int nkt = p.seq_k / KB;
  const float c = p.scale_log2;
  // One tile of work is an M phase (32 MFMAs: second product of tile j, then scores of tile j+1) and a V phase
  // (probabilities of a tile: maximum, exp2, rounding, denominator).  The two waves that share a SIMD run them in
  // opposite order -- waves 0-3 do V then M between two barriers, waves 4-7 M then V, half a tile behind -- so one
  // wave's MFMAs always run beside the other wave's VALU work.
  v16f s[KA];
  v4i pf[KSTEPS];
  float m_run = -INFINITY;  // exponent reference of this lane's query
  auto k_read = [&](const unsigned* ck, int u, int* f) { RK::read(ck, u % KA, u / KA, f); };
  auto v_read = [&](unsigned vbase, int u, int* f) { RV::read(rv[u % DA] + vbase, u / DA, f); };
  // M phase of tile j: o += V_j^T P_j^T (unit u: key step u / DA, head_dim atom u % DA), then, if `scores`,
  // s = K_{j+1} Q^T (unit u: head_dim step u / KA, key atom u % KA).  Fragments are read two units ahead.
  auto m_phase = [&](unsigned vbase, unsigned kbase, bool scores) {
    unsigned ck[RK::NREG];
#pragma unroll
    for (int r = 0; r < RK::NREG; ++r) ck[r] = rk[r] + kbase;
    // fragment of unit x (0 .. N2-1: V, N2 .. N2+N1-1: K) goes to f[x % NB], read PF units ahead of its MFMA
    constexpr int PF = kAttnPrefetch, NB = PF + 1;
    int f[NB][4];
    const int last = scores ? N2 + N1 : N2;
    auto fetch = [&](int x) {
      if (x < N2) v_read(vbase, x, f[x % NB]);
      else if (x < last) k_read(ck, x - N2, f[x % NB]);
    };
#pragma unroll
    for (int x = 0; x < PF; ++x) fetch(x);
#pragma unroll
    for (int u = 0; u < N2; ++u) {
      const v4i vfrag = {f[u % NB][0], f[u % NB][1], f[u % NB][2], f[u % NB][3]};
      M::run(vfrag, pf[u / DA], o[u % DA]);
      fetch(u + PF);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (scores) {
#pragma unroll
      for (int u = 0; u < N1; ++u) {
        const int x = u + N2;
        const v4i kfrag = {f[x % NB][0], f[x % NB][1], f[x % NB][2], f[x % NB][3]};
        if (u < KA) s[u % KA] = v16f{};  // folds into the MFMA's C operand: no registers are cleared
        M::run(kfrag, qf[u / KA], s[u % KA]);
        fetch(x + PF);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  // V phase: probabilities of the tile whose scores are in s.  Score e of the lane, e = 16 ka + r, belongs to
  // 16-key step e / 8.
  auto v_phase = [&]() {
    float mx = s[0][0];
#pragma unroll
    for (int ka = 0; ka < KA; ++ka)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[ka][r]);
    {
      // lanes l and l ^ 32 hold the two halves of a query's keys.  One v_permlane32_swap of two copies of the value leaves
      // the lower half's maximum in every lane of one result and the upper half's in the other; unlike a shuffle it
      // does not go through the LDS queue (291 against 300 us at 32 x 4096 x 4096)
      const int mine = __builtin_bit_cast(int, mx);
      const auto both = __builtin_amdgcn_permlane32_swap(mine, mine, false, false);
      mx = fmaxf(__builtin_bit_cast(float, (int)both[0]), __builtin_bit_cast(float, (int)both[1])) * c;
    }
    if (__builtin_amdgcn_ballot_w64(mx > m_run + kAttnRescaleSlack) != 0) {
      const float m_new = fmaxf(m_run, mx);
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int da = 0; da < DA; ++da)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[da][r] *= alpha;
    }
    float l_part[4] = {l_run, 0.f, 0.f, 0.f};  // four chains instead of one of 16 dependent additions
#pragma unroll
    for (int e = 0; e < NE; e += 2) {
      const float x0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[e / 16][e % 16], c, -m_run));
      const float x1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[e / 16][e % 16 + 1], c, -m_run));
      const int pair = PK::two(x0, x1);
      pf[e / 8][(e % 8) / 2] = pair;
      l_part[(e / 2) % 4] = PK::add_pair(pair, l_part[(e / 2) % 4]);
      if (e % 8 == 6) __builtin_amdgcn_sched_barrier(0);  // keeps the scheduler from holding all 32 exponentials in flight
    }
    // The probabilities are only used by the MFMAs of the M phase, two barriers away: left alone, the compiler sinks
    // the whole computation there.  Pin the values to this phase.
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(pf[t][j]));
    l_run = (l_part[0] + l_part[1]) + (l_part[2] + l_part[3]);
    asm volatile("" : "+v"(l_run));
  };

  // prologue: tiles 0..2 in flight, scores of tile 0
  stage_tile();
  if (nkt > 1) stage_tile();
  if (nkt > 2) stage_tile();
  if (nkt > 2) wait_vmcnt<2 * PER_TILE>(); else if (nkt > 1) wait_vmcnt<PER_TILE>(); else wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  {
    unsigned ck[RK::NREG];
#pragma unroll
    for (int r = 0; r < RK::NREG; ++r) ck[r] = rk[r] + k_ring;
#pragma unroll
    for (int ka = 0; ka < KA; ++ka)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[ka][r] = 0.f;
#pragma unroll
    for (int u = 0; u < N1; ++u) {
      int f[4];
      k_read(ck, u, f);
      const v4i kfrag = {f[0], f[1], f[2], f[3]};
      M::run(kfrag, qf[u / KA], s[u % KA]);
    }
  }

  // Every wave runs the same loop -- barrier, V(kt), barrier, M(kt) -- but waves 4-7 pass one extra barrier first,
  // which puts them half an iteration behind waves 0-3 for the whole kernel (waves 0-3 pass the matching barrier at
  // the end).  Before either barrier of iteration kt a wave's share of tile kt+1 has landed (at most tile kt+2 is
  // outstanding), so tile kt+1 is complete in LDS before any wave's M(kt); when a wave stages tile kt+3, every wave
  // has passed the barrier that follows its M(kt-1), the last reader of K tile kt and V tile kt-1.
  const bool trails = wave >= C::NW / 2;
  if (trails) __builtin_amdgcn_s_barrier();
  int k_slot = 1, v_slot = 0;  // ring slots M(kt) reads: K tile kt+1 and V tile kt
  for (int kt = 0; kt < nkt; ++kt) {
    if (kt + 2 < nkt) wait_vmcnt<PER_TILE>(); else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);  // the phases are register-only work: without these the compiler moves it across the barriers
    v_phase();
    __builtin_amdgcn_sched_barrier(0);
    if (kt + 2 < nkt) wait_vmcnt<PER_TILE>(); else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if (kt + 3 < nkt) stage_tile();
    m_phase(v_ring + v_slot * LV::BYTES, k_ring + k_slot * LK::BYTES, kt + 1 < nkt);
    __builtin_amdgcn_sched_barrier(0);
    k_slot = k_slot == C::NSK - 1 ? 0 : k_slot + 1;
    v_slot = v_slot == C::NSV - 1 ? 0 : v_slot + 1;
  }
  if (!trails) __builtin_amdgcn_s_barrier();

  // O = O^T / l.  Lane (q, h) holds head_dim columns 32 da + 8 (r/4) + 4 h + r%4 of its query: 8-byte pieces.  They
  // go through a wave-private LDS region (64 columns at a time, rows padded by 16 B) and come back as 16-byte
  // pieces, 8 lanes per row, so that every global store covers whole 128-byte lines of O.  LDS operations of one
  // wave execute in order and the region lies behind the rings, which other waves may still be reading.
  {
    const float l = l_run + __shfl_xor(l_run, 32);
    const float inv = 1.f / l;
    const int64_t row = (int64_t)bh * p.seq_q + q0 + lq;
    constexpr int OROW = 64 * 2 + 16;
    const unsigned region = smem_u + C::RING_BYTES + wave * C::OUT_BYTES_PER_WAVE;
    char* obase = (char*)p.O + ((int64_t)bh * p.seq_q + q0) * D * 2;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
      for (int d2 = 0; d2 < 2; ++d2)
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          const int da = 2 * half + d2;
          v2i w;
          w[0] = PK::two(o[da][4 * r4] * inv, o[da][4 * r4 + 1] * inv);
          w[1] = PK::two(o[da][4 * r4 + 2] * inv, o[da][4 * r4 + 3] * inv);
          *(FRISK_LDS v2i*)(uintptr_t)(region + lq * OROW + (32 * d2 + 8 * r4 + 4 * lh) * 2) = w;
        }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int orow = (lane >> 3) + 8 * j, chunk = lane & 7;
        const v4i w = *(const FRISK_LDS v4i*)(uintptr_t)(region + orow * OROW + chunk * 16);
        FRISK_STORE_C((v4i*)(obase + (int64_t)orow * D * 2 + (64 * half + 8 * chunk) * 2), w);
      }
    }
    if (p.lse && lh == 0) p.lse[row] = (m_run + __builtin_amdgcn_logf(l)) * 0.6931471805599453f;
  }
}

template <class C> static hipError_t prepare_one() {
  return hipFuncSetAttribute((const void*)attention_kernel<C>, hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
}

// Raising the dynamic-LDS cap is not a stream operation and must precede a captured launch; done once per process.
hipError_t prepare_attention() {
  static std::atomic<bool> done{false};
  if (done.load(std::memory_order_acquire)) return hipSuccess;
  if (hipError_t e = prepare_one<AttnCfg<FRISK_F16, false>>(); e != hipSuccess) return e;
  if (hipError_t e = prepare_one<AttnCfg<FRISK_F16, true>>(); e != hipSuccess) return e;
  if (hipError_t e = prepare_one<AttnCfg<FRISK_BF16, false>>(); e != hipSuccess) return e;
  if (hipError_t e = prepare_one<AttnCfg<FRISK_BF16, true>>(); e != hipSuccess) return e;
  done.store(true, std::memory_order_release);
  return hipSuccess;
}

template <class C> static hipError_t launch_one(const AttentionParams& p, hipStream_t stream) {
  hipLaunchKernelGGL(attention_kernel<C>, dim3(p.batch_heads * p.q_blocks), dim3(C::NW * 64), C::LDS_BYTES, stream, p);
  return hipGetLastError();
}

hipError_t launch_attention(int dtype, int k_transposed, const AttentionParams& p, hipStream_t stream) {
  if (hipError_t e = prepare_attention(); e != hipSuccess) return e;
  if (dtype == FRISK_F16) return k_transposed ? launch_one<AttnCfg<FRISK_F16, true>>(p, stream) : launch_one<AttnCfg<FRISK_F16, false>>(p, stream);
  return k_transposed ? launch_one<AttnCfg<FRISK_BF16, true>>(p, stream) : launch_one<AttnCfg<FRISK_BF16, false>>(p, stream);
}

}  // namespace frisk
