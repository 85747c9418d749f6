// Fused attention forward for gfx950: O = softmax(scale * Q K^T) V, one pass over the keys with a running
// maximum and denominator, the program of the reference's sketch tmp/ir.mlir:87-157 (copy Q; for each key tile:
// copy K, gemm, reduce max, exp2, reduce sum, rescale, copy V, gemm; copy O) executed as one kernel.
//
// A work-group of 4 waves owns 256 queries of one (batch, head); a wave owns 64 of them for the whole kernel.
// Key / value tiles of 64 keys stream HBM/L2 -> LDS with global_load_lds_dwordx4 through a ring of three stages.
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
  static constexpr int NW = 4, QW = QB / NW, QA = QW / 32, KA = KB / 32, DA = D / 32;
  static constexpr int NS = 3;  // LDS ring depth
  typedef Mma<DT> M;
  typedef TileLayout<2, !KT, KB, D> LK;    // first product contracts over head_dim
  typedef TileLayout<2, false, D, KB> LV;  // second product contracts over keys; head_dim runs along the row
  static constexpr int STAGE_BYTES = LK::BYTES + LV::BYTES;
  static constexpr int LDS_BYTES = NS * STAGE_BYTES;
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

template <int DT> struct Pack16;
template <> struct Pack16<FRISK_F16> {
  typedef _Float16 T;
  FRISK_DEV int two(float a, float b) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 v = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(int, v);
  }
};
template <> struct Pack16<FRISK_BF16> {
  typedef __bf16 T;
  FRISK_DEV int two(float a, float b) {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    b2 v = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(int, v);
  }
};

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
  constexpr int D = C::D, KB = C::KB, QA = C::QA, KA = C::KA, DA = C::DA, DSTEPS = D / 16, KSTEPS = KB / 16;
  static_assert(SK::NVOFF == 1 && SV::NVOFF == 1, "one lane offset per operand");

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const unsigned smem_u = (unsigned)(uintptr_t)(FRISK_LDS char*)smem;
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
  v4i qf[QA][DSTEPS];
  {
    const char* qbase = (const char*)p.Q + (((int64_t)bh * p.seq_q + q0 + lq) * D + 8 * lh) * 2;
#pragma unroll
    for (int b = 0; b < QA; ++b)
#pragma unroll
      for (int ks = 0; ks < DSTEPS; ++ks) qf[b][ks] = *(const v4i*)(qbase + ((int64_t)b * 32 * D + 16 * ks) * 2);
  }

  // staging: wave-uniform tile pointers plus one lane offset per operand
  const int64_t k_ld = C::KT ? (int64_t)p.seq_k * 2 : (int64_t)D * 2;
  const int64_t k_step = C::KT ? (int64_t)KB * 2 : (int64_t)KB * D * 2;
  const char* srcK = (const char*)p.K + (int64_t)bh * p.seq_k * D * 2 + SK::wave_src_offset(wave, k_ld);
  const char* srcV = (const char*)p.V + (int64_t)bh * p.seq_k * D * 2 + SV::wave_src_offset(wave, D * 2);
  const unsigned voffK[1] = {SK::lane_src_offset(lane, wave, k_ld)};
  const unsigned voffV[1] = {SV::lane_src_offset(lane, wave, D * 2)};
  constexpr int PER_TILE = SK::PER_WAVE + SV::PER_WAVE;
  auto stage_tile = [&](int slot) {
    const unsigned kdst = smem_u + slot * C::STAGE_BYTES, vdst = kdst + LK::BYTES;
#pragma unroll
    for (int i = 0; i < SK::PER_WAVE; ++i) SK::issue_one(i, srcK, voffK, k_ld, kdst, wave);
#pragma unroll
    for (int i = 0; i < SV::PER_WAVE; ++i) SV::issue_one(i, srcV, voffV, D * 2, vdst, wave);
    srcK += k_step;
    srcV += (int64_t)KB * D * 2;
  };

  unsigned rk[RK::NREG], rv[DA];
  RK::init(lane, 0, 0, rk);
#pragma unroll
  for (int da = 0; da < DA; ++da) rv[da] = RV::lane_reg(lane, da);

  v16f o[QA][DA];
  float m_run[QA], l_run[QA];
#pragma unroll
  for (int b = 0; b < QA; ++b) {
    m_run[b] = -INFINITY;
    l_run[b] = 0.f;
#pragma unroll
    for (int da = 0; da < DA; ++da)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[b][da][r] = 0.f;
  }

  const int nkt = p.seq_k / KB;
  const float c = p.scale_log2;
  stage_tile(0);
  if (nkt > 1) stage_tile(1);
  int slot = 0, slot_issue = 2;
  for (int kt = 0; kt < nkt; ++kt) {
    // tile kt has landed when at most the transfers of tile kt+1 are outstanding; the barrier also tells that every
    // wave is done reading tile kt-1, whose slot the transfers of tile kt+2 reuse
    if (kt + 1 < nkt) wait_vmcnt<PER_TILE>(); else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    if (kt + 2 < nkt) stage_tile(slot_issue);
    slot_issue = slot_issue == C::NS - 1 ? 0 : slot_issue + 1;
    const unsigned kbase = smem_u + slot * C::STAGE_BYTES, vbase = kbase + LK::BYTES;
    slot = slot == C::NS - 1 ? 0 : slot + 1;
    unsigned ck[RK::NREG];
#pragma unroll
    for (int r = 0; r < RK::NREG; ++r) ck[r] = rk[r] + kbase;

    // S^T = K Q^T
    v16f s[QA][KA];
#pragma unroll
    for (int b = 0; b < QA; ++b)
#pragma unroll
      for (int ka = 0; ka < KA; ++ka)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[b][ka][r] = 0.f;
#pragma unroll
    for (int ks = 0; ks < DSTEPS; ++ks) {
#pragma unroll
      for (int ka = 0; ka < KA; ++ka) {
        int kf[4];
        RK::read(ck, ka, ks, kf);
        const v4i kfrag = {kf[0], kf[1], kf[2], kf[3]};
#pragma unroll
        for (int b = 0; b < QA; ++b) M::run(kfrag, qf[b][ks], s[b][ka]);
      }
    }

    // running softmax, one query per lane
    v4i pf[QA][KSTEPS];
#pragma unroll
    for (int b = 0; b < QA; ++b) {
      float mx = s[b][0][0];
#pragma unroll
      for (int ka = 0; ka < KA; ++ka)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[b][ka][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float m_new = fmaxf(m_run[b], mx * c);
      const float alpha = __builtin_amdgcn_exp2f(m_run[b] - m_new);
      m_run[b] = m_new;
      float sum = 0.f;
#pragma unroll
      for (int ka = 0; ka < KA; ++ka)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[b][ka][r], c, -m_new));
          s[b][ka][r] = e;
          sum += e;
        }
      l_run[b] = l_run[b] * alpha + sum;
#pragma unroll
      for (int da = 0; da < DA; ++da)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[b][da][r] *= alpha;
#pragma unroll
      for (int t = 0; t < KSTEPS; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) pf[b][t][e] = PK::two(s[b][t / 2][8 * (t % 2) + 2 * e], s[b][t / 2][8 * (t % 2) + 2 * e + 1]);
    }

    // O^T += V^T P^T
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t) {
#pragma unroll
      for (int da = 0; da < DA; ++da) {
        int vf[4];
        RV::read(rv[da] + vbase, t, vf);
        const v4i vfrag = {vf[0], vf[1], vf[2], vf[3]};
#pragma unroll
        for (int b = 0; b < QA; ++b) M::run(vfrag, pf[b][t], o[b][da]);
      }
    }
  }

  // O = O^T / l; lane (q, h) holds head_dim columns 32 da + 8 (r/4) + 4 h + r%4
#pragma unroll
  for (int b = 0; b < QA; ++b) {
    const float l = l_run[b] + __shfl_xor(l_run[b], 32);
    const float inv = 1.f / l;
    const int64_t row = (int64_t)bh * p.seq_q + q0 + 32 * b + lq;
    char* orow = (char*)p.O + row * D * 2;
#pragma unroll
    for (int da = 0; da < DA; ++da)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        v2i w;
        w[0] = PK::two(o[b][da][4 * r4] * inv, o[b][da][4 * r4 + 1] * inv);
        w[1] = PK::two(o[b][da][4 * r4 + 2] * inv, o[b][da][4 * r4 + 3] * inv);
        FRISK_STORE_C((v2i*)(orow + (32 * da + 8 * r4 + 4 * lh) * 2), w);
      }
    if (p.lse && lh == 0) p.lse[row] = (m_run[b] + __builtin_amdgcn_logf(l)) * 0.6931471805599453f;
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
