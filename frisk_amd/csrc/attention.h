// Launch helper of attention.hip, called by the C ABI after argument validation.
#pragma once
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include "frisk_hip.h"

namespace frisk {

// queries per work-group, keys per LDS tile and the head dimension the kernel is built for
constexpr int kAttnQueriesPerGroup = 256;
constexpr int kAttnKeysPerTile = 64;
constexpr int kAttnHeadDim = 128;

struct AttentionParams {
  const void* Q;   // [batch*heads][seq_q][128]
  const void* K;   // [batch*heads][seq_k][128], or [batch*heads][128][seq_k] when k_transposed
  const void* V;   // [batch*heads][seq_k][128]
  void* O;         // [batch*heads][seq_q][128]
  float* lse;      // optional [batch*heads][seq_q]: natural log of the softmax denominator, scale included
  int32_t batch_heads, seq_q, seq_k;
  int32_t q_blocks;     // seq_q / 256
  int32_t xcd_remap;    // 1: work-groups of one head run on one XCD (one L2)
  float scale_log2;     // softmax scale times log2(e): probabilities are exp2(scale_log2 * (s - max))
};

hipError_t prepare_attention();
hipError_t launch_attention(int dtype, int k_transposed, const AttentionParams& p, hipStream_t stream);

}  // namespace frisk
