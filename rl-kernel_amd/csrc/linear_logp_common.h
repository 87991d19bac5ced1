// Pieces of the fused linear-LogP reduction contract shared by its forward and
// backward kernels (the vocabulary tiling and the pinned exponential), and the SwiGLU
// arithmetic built on the same exponential.
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

// SwiGLU arithmetic shared by the elementwise kernels and the fused projections: s = rcp(1 + e(-g))
// (v_rcp_f32), y = (g * s) * u, on the bf16-rounded gate and up values.
__device__ __forceinline__ float bf16_to_f32(uint32_t bits) { return __uint_as_float(bits << 16); }
__device__ __forceinline__ float round_through_bf16(float v) { return bf16_to_f32(pack_bf16x2(v, 0.f) & 0xffffu); }
__device__ __forceinline__ float sigmoid_f32(float x) { return __builtin_amdgcn_rcpf(1.0f + pinned_exp(-x)); }
__device__ __forceinline__ float swiglu_f32(float g, float u) { return (g * sigmoid_f32(g)) * u; }

// The logit of the contract before the temperature: accumulator value z at column `col` with the bias
// added and padded lanes set to -inf. This is the value a caller who asks for the logits receives.
__device__ __forceinline__ float biased_logit(float z, bool has_bias, float bias, int col, int vocab_limit) {
  if (has_bias) z = z + bias;
  return (col < vocab_limit) ? z : kNegInf;
}

// The scaled logit y of the contract: the biased logit, then the temperature scaling.
__device__ __forceinline__ float scaled_logit(float z, bool has_bias, float bias, int col, int vocab_limit,
                                              bool has_temp, float inv_t) {
  z = biased_logit(z, has_bias, bias, col, vocab_limit);
  if (has_temp) z = z * inv_t;
  return z;
}

// A lane's run of 16 consecutive biased logits of one token -> row[col0 .. col0 + 16) of the fp32 logits,
// cut at V: four 16-byte stores when the run is whole and aligned, element stores otherwise.
__device__ __forceinline__ void store_logit_run(float* __restrict__ row, int col0, int V, const float (&u)[16]) {
  float* dst = row + col0;
  if (col0 + 16 <= V && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
      *reinterpret_cast<f32x4_t*>(dst + 4 * q) = f32x4_t{u[4 * q], u[4 * q + 1], u[4 * q + 2], u[4 * q + 3]};
  } else {
#pragma unroll
    for (int c = 0; c < 16; ++c)
      if (col0 + c < V) dst[c] = u[c];
  }
}

// The same store for the four lanes of one token together (lanes l, l + 16, l + 32, l + 48 of a wave hold the four
// adjacent 16-column runs of the token's 64-column span that starts at span0): the 4 x 4 grid of 16-byte chunks is
// transposed between the lanes (two butterfly stages of lane swaps over distances 32 and 16: the chunk that lane
// g held at position c ends at lane c, position g), so that store q of lane g writes bytes [64 q + 16 g, + 16) of
// the span and one instruction covers whole 64-byte sectors instead of a quarter of each. Every lane of the wave
// must call it (the swaps read the other lanes whatever their `live`); needs span0 + 64 <= V and 16-byte aligned
// rows, both uniform over the wave. The values stored are the ones store_logit_run stores.
__device__ __forceinline__ void store_logit_span(float* __restrict__ row, int span0, int grp, bool live,
                                                 const float (&u)[16]) {
  uint32_t w[4][4];  // [chunk][word]
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int e = 0; e < 4; ++e) w[c][e] = __float_as_uint(u[4 * c + e]);
#pragma unroll
  for (int c = 0; c < 2; ++c)  // lane bit 5 <-> chunk bit 1
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const auto r = __builtin_amdgcn_permlane32_swap(w[c][e], w[c + 2][e], false, false);
      w[c][e] = r[0];
      w[c + 2][e] = r[1];
    }
#pragma unroll
  for (int c = 0; c < 4; c += 2)  // lane bit 4 <-> chunk bit 0
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const auto r = __builtin_amdgcn_permlane16_swap(w[c][e], w[c + 1][e], false, false);
      w[c][e] = r[0];
      w[c + 1][e] = r[1];
    }
  if (live) {
    float* dst = row + span0 + 4 * grp;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      *reinterpret_cast<u32x4_t*>(dst + 16 * q) = u32x4_t{w[q][0], w[q][1], w[q][2], w[q][3]};
  }
}

// One step of a stream's online chain: the 16 scaled logits y of the stream's run in one
// tile are folded into the running (max, sum), exponentials added in ascending column order;
// `tl` is the target's position inside the run (outside [0, 16): not in this run). A run that
// is all -inf (a fully padded tile) leaves the state unchanged.
__device__ __forceinline__ void logp_fold_run(const float (&y)[16], int tl, float& run_m, float& run_s,
                                              float& run_zt) {
  float tmax = kNegInf;
#pragma unroll
  for (int c = 0; c < 16; ++c) tmax = fmaxf(tmax, y[c]);
  if (tl >= 0 && tl < 16) {
    float sel = y[0];
#pragma unroll
    for (int c = 1; c < 16; ++c) sel = (tl == c) ? y[c] : sel;
    run_zt = sel;
  }
  const float old_m = run_m;
  const float new_m = fmaxf(old_m, tmax);
  float sum = pinned_exp(y[0] - new_m);
#pragma unroll
  for (int c = 1; c < 16; ++c) sum = sum + pinned_exp(y[c] - new_m);
  const float scaled = run_s * pinned_exp(old_m - new_m);
  run_s = (new_m > kNegInf) ? (scaled + sum) : run_s;
  run_m = new_m;
}

// The 16 stream states of a (split, token), merged in ascending stream order. pm / ps / pz
// point at stream 0; consecutive streams are `stride` floats apart.
__device__ __forceinline__ void logp_merge_streams(const float* pm, const float* ps, const float* pz, int64_t stride,
                                                   float& big, float& sum, float& zt) {
  big = kNegInf;
#pragma unroll
  for (int j = 0; j < kLogpStreams; ++j) big = fmaxf(big, pm[j * stride]);
  sum = 0.f;
  zt = 0.f;
#pragma unroll
  for (int j = 0; j < kLogpStreams; ++j) {
    const float m = pm[j * stride];
    const float term = ps[j * stride] * pinned_exp(m - big);
    sum = sum + ((m > kNegInf) ? term : 0.f);
    zt = zt + pz[j * stride];
  }
}

}  // namespace rlk
