// Pieces of the fused linear-LogP reduction contract shared by its forward and
// backward kernels: the vocabulary tiling and the pinned exponential.
#pragma once

#include "det_gemm_tile.h"

namespace rlk {

constexpr int kLogpTileCols = 256;
constexpr int kLogpStreams = 16;
constexpr int kLogpSplitTiles = 4;
constexpr int kLogpSplitCols = kLogpTileCols * kLogpSplitTiles;
constexpr float kNegInf = -__builtin_huge_valf();

// e(x) of the contract: v_exp_f32 of an unfused fp32 product.
__device__ __forceinline__ float pinned_exp(float x) {
  return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f);
}

// The scaled logit y of the contract for accumulator value z at column `col`:
// bias added, padded lanes -inf, then the temperature scaling.
__device__ __forceinline__ float scaled_logit(float z, bool has_bias, float bias, int col, int vocab_limit,
                                              bool has_temp, float inv_t) {
  if (has_bias) z = z + bias;
  z = (col < vocab_limit) ? z : kNegInf;
  if (has_temp) z = z * inv_t;
  return z;
}

}  // namespace rlk
