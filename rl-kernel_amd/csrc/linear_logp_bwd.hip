// Backward of the fused linear-LogP for gfx950.
//
// Stands in for _DetTritonLinearLogpAutograd.backward + _det_reference_dlogits
// (reference rl_engine/backends/shared/triton/logprob/linear_logp.py:522-570, 600-628)
// and for the bf16 branch of chunked_linear_logp_backward
// (rl_engine/reference/logprob/linear_logp.py:642-715): the logits are recomputed,
// d(logits) is rounded to bf16 once and feeds two GEMMs.
//
// Three steps, all in fixed order:
//   1. dlogits kernel. The same MFMA chain as the forward gives z; with y the scaled
//      logit of the forward contract and lse the forward's saved value,
//          p  = e(y - lse)                          (0 on padded lanes)
//          dz = p * (g_lse - g_logp)                (+ g_logp at the target column)
//          dz = dz * (1 / temperature)              when a temperature is given
//      rounded once to bf16 and written to dz[T, ld] (the only [T, V]-sized buffer;
//      2 bytes per logit).
//   2. grad_hidden[T, D] = dz[T, V] @ W[V, D]: det_gemm over the vocabulary, ascending,
//      with W read as a K-major operand. A row depends on that token's dz row only, so
//      it is batch invariant like the forward.
//   3. grad_weight[V, D] = dz^T[V, T] @ H[T, D]: det_gemm over tokens, ascending, both
//      operands read K-major (no transposed copies).
//      grad_bias[V] = column sums of the UNROUNDED fp32 dz (the reference sums dz before it is cast,
//      rl_engine/reference/logprob/linear_logp.py:704-705), accumulated by the dlogits kernel itself in a
//      fixed tree over the token index that no tile configuration changes: inside a block of 256 tokens,
//      token t = 16 g + l; first the 16 tokens of a group g are added in an xor butterfly over l (steps
//      1, 2, 4, 8), then the 16 groups in a balanced binary tree over g (adjacent pairs first); tokens past T
//      and groups past the last tile enter as +0, so every configuration performs the same additions; the
//      256-token block sums are added ascending.
#include "linear_logp_common.h"
#include "rlk_host.h"

namespace rlk {

struct LogpBwdArgs {
  MatView W;  // [V, D] lm_head weight
  MatView H;  // [T, D] hidden states
  const int64_t* target;
  const float* bias;         // [V] or null
  const float* temperature;  // [T] or null
  const float* lse;          // [T] forward result
  const float* grad_logp;    // [T] or null (= 0)
  const float* grad_lse;     // [T] or null (= 0)
  bf16_bits* dz;             // [T, ld_dz]
  int64_t ld_dz;
  float* bias_part;          // [tiles_m, V] per-token-tile column sums of the fp32 dz (BIAS_GRAD kernels)
  int T, V, D;
  int vocab_limit;
  int64_t vocab_start;
  int tiles_m, tiles_v, group_m;
};

// Sum over the 16 lanes of a lane group (lanes that share lane >> 4), identical in all of them: xor butterfly.
__device__ __forceinline__ float group16_sum(float v) {
  v = v + __shfl_xor(v, 1);
  v = v + __shfl_xor(v, 2);
  v = v + __shfl_xor(v, 4);
  v = v + __shfl_xor(v, 8);
  return v;
}

// LOOP: 0 generic element loader, 1 register-staged 16-byte loads, 2 direct-to-LDS ping-pong.
// BIAS_GRAD: also write the tile's column sums of the fp32 dz to a.bias_part (see the header for the order).
template <class S, int LOOP, bool BIAS_GRAD>
__global__ __launch_bounds__(S::kThreads) void linear_logp_dlogits_kernel(LogpBwdArgs a) {
  static_assert(S::BN == kLogpTileCols && S::kRun == 16 && S::WN == 4, "a lane owns 16 consecutive columns");
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int total = a.tiles_m * a.tiles_v;
  const int id = xcd_compact_id(blockIdx.x, total);
  const int per_group = a.group_m * a.tiles_v;
  const int group = id / per_group;
  const int first_m = group * a.group_m;
  const int width = (a.tiles_m - first_m) < a.group_m ? (a.tiles_m - first_m) : a.group_m;
  const int within = id - group * per_group;
  const int tile_m = first_m + within % width;
  const int tile_v = within / width;
  const int m0 = tile_m * S::BM;
  const int v0 = tile_v * kLogpTileCols;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wave_n = wave % S::WN;
  const int wave_m = wave / S::WN;
  const int l16 = lane & 15;
  const int grp = lane >> 4;
  const int tok_local = wave_m * 16 * S::TM + l16;
  const int col0 = v0 + (wave_n * 4 + grp) * 16;  // first column of this lane's run

  f32x4_t acc[S::TN][S::TM];
  if constexpr (LOOP == 2) {
    tile_mainloop_pingpong<S>(a.W, a.H, v0, m0, a.D, lds, acc);
  } else {
    tile_mainloop_staged<S, LOOP == 1>(a.W, a.H, v0, m0, a.D, lds, acc);
  }

  float bias_run[16];
#pragma unroll
  for (int c = 0; c < 16; ++c) bias_run[c] = 0.f;
  if (a.bias) {
#pragma unroll
    for (int c = 0; c < 16; ++c) bias_run[c] = (col0 + c < a.V) ? a.bias[col0 + c] : 0.f;
  }

  // Tree slots of the bias gradient: level[L] holds the finished sum of 2^L consecutive 16-token groups.
  constexpr int kLevels = S::TM >= 8 ? 4 : S::TM >= 4 ? 3 : S::TM >= 2 ? 2 : 1;
  static_assert((S::TM & (S::TM - 1)) == 0 && S::TM <= 8, "token groups per lane: a power of two");
  float level[BIAS_GRAD ? kLevels : 1][16];

#pragma unroll
  for (int jm = 0; jm < S::TM; ++jm) {
    const int m = m0 + tok_local + jm * 16;
    const bool live = m < a.T;
    if (!BIAS_GRAD && !live) continue;
    const int mr = live ? m : a.T - 1;  // a dead row reads a valid row's scalars and contributes +0
    const int64_t local = a.target[mr] - a.vocab_start;
    const int tl = (local >= 0 && local < a.vocab_limit) ? (int)local - col0 : -1;
    const float inv_t = a.temperature ? 1.0f / a.temperature[mr] : 1.0f;
    const float row_lse = a.lse[mr];
    const float g_logp = a.grad_logp ? a.grad_logp[mr] : 0.f;
    const float g_lse = a.grad_lse ? a.grad_lse[mr] : 0.f;
    const float coeff = g_lse - g_logp;
    uint32_t packed[8];
    float cur[16];
#pragma unroll
    for (int c = 0; c < 16; c += 2) {
      float d[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int cc = c + e;
        const float y = scaled_logit(acc[cc >> 2][jm][cc & 3], a.bias != nullptr, bias_run[cc], col0 + cc,
                                     a.vocab_limit, a.temperature != nullptr, inv_t);
        float v = pinned_exp(y - row_lse) * coeff;
        if (tl == cc) v = v + g_logp;
        if (a.temperature) v = v * inv_t;
        d[e] = v;
        if constexpr (BIAS_GRAD) cur[cc] = group16_sum(live ? v : 0.f);
      }
      packed[c >> 1] = pack_bf16x2(d[0], d[1]);
    }
    if constexpr (BIAS_GRAD) {
      // binary-counter merge: group jm closes every tree node whose last group it is
#pragma unroll
      for (int L = 0; L < kLevels; ++L) {
        if (((jm >> L) & 1) == 0) {
#pragma unroll
          for (int c = 0; c < 16; ++c) level[L][c] = cur[c];
          break;
        }
#pragma unroll
        for (int c = 0; c < 16; ++c) cur[c] = level[L][c] + cur[c];
      }
    }
    if (!live) continue;
    bf16_bits* dst = a.dz + (int64_t)m * a.ld_dz + col0;
    if (col0 + 16 <= a.V) {
      *reinterpret_cast<u32x4_t*>(dst) = u32x4_t{packed[0], packed[1], packed[2], packed[3]};
      *reinterpret_cast<u32x4_t*>(dst + 8) = u32x4_t{packed[4], packed[5], packed[6], packed[7]};
    } else {
#pragma unroll
      for (int c = 0; c < 16; ++c)
        if (col0 + c < a.V) dst[c] = (bf16_bits)((packed[c >> 1] >> ((c & 1) * 16)) & 0xffffu);
    }
  }

  if constexpr (BIAS_GRAD) {
    // A lane's node covers its wave's S::TM groups and sits in the slot of that size; the waves along the
    // token axis hold consecutive nodes and are added in pairs through LDS (the main loop ended on a
    // barrier, so the staging memory is free).
    constexpr int kTop = S::TM >= 8 ? 3 : S::TM >= 4 ? 2 : S::TM >= 2 ? 1 : 0;
    static_assert(S::WM == 1 || S::WM == 2, "one or two waves along the token axis");
    float* sums = reinterpret_cast<float*>(lds);  // [WM][256 columns]
    if (l16 == 0) {
#pragma unroll
      for (int c = 0; c < 16; ++c) sums[wave_m * kLogpTileCols + (wave_n * 4 + grp) * 16 + c] = level[kTop][c];
    }
    __syncthreads();
    for (int col = threadIdx.x; col < kLogpTileCols; col += S::kThreads) {
      float total = sums[col];
      if constexpr (S::WM == 2) total = total + sums[kLogpTileCols + col];
      if (v0 + col < a.V) a.bias_part[(int64_t)tile_m * a.V + v0 + col] = total;
    }
  }
}

// grad_bias from the per-tile column sums: the `per_block` tiles of a 256-token block are added in the
// balanced tree that continues the in-kernel one (adjacent pairs first, a tile past the last one is +0),
// then the block sums ascending.
constexpr int kBiasBlockTokens = 256;

__global__ void logp_bias_merge_kernel(const float* __restrict__ part, float* __restrict__ grad_bias, int tiles,
                                       int per_block, int V) {
  const int col = blockIdx.x * blockDim.x + threadIdx.x;
  if (col >= V) return;
  float s = 0.f;
  for (int t0 = 0; t0 < tiles; t0 += per_block) {
    float node[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) node[i] = (i < per_block && t0 + i < tiles) ? part[(int64_t)(t0 + i) * V + col] : 0.f;
#pragma unroll
    for (int w = 1; w < 16; w *= 2) {
      if (w < per_block) {
#pragma unroll
        for (int i = 0; i < 16; i += 2 * w) node[i] = node[i] + node[i + w];
      }
    }
    s = s + node[0];
  }
  grad_bias[col] = s;
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------

using LogpShape256 = TileShape<256, 256, 4, 2>;
using LogpShape128 = TileShape<256, 128, 4, 2>;
using LogpShape64 = TileShape<256, 64, 4, 2>;
using LogpShape16 = TileShape<256, 16, 4, 1>;

int64_t linear_logp_dz_row_stride(int V) { return ((int64_t)V + 63) / 64 * 64; }

static size_t dz_bytes(int T, int V) {
  // 256-byte multiple so the fp32 block sums behind it stay aligned
  const size_t raw = (size_t)(T > 0 ? T : 0) * (size_t)linear_logp_dz_row_stride(V) * sizeof(bf16_bits);
  return (raw + 255) / 256 * 256;
}

// Token tiles the bias gradient may be collected over: 16-token tiles up to 1024 tokens, else 64-token ones.
constexpr int kBiasSmallTileMaxTokens = 1024;

static int bias_part_rows(int T) { return T <= kBiasSmallTileMaxTokens ? (T + 15) / 16 : (T + 63) / 64; }

size_t linear_logp_bwd_workspace_bytes(int T, int V, bool with_bias) {
  size_t bytes = dz_bytes(T, V);
  if (with_bias && T > 0) bytes += (size_t)bias_part_rows(T) * (size_t)V * sizeof(float);
  return bytes;
}

template <class S, int LOOP, bool BIAS_GRAD>
static hipError_t launch_dlogits_as(LogpBwdArgs a, hipStream_t stream) {
  auto kernel = linear_logp_dlogits_kernel<S, LOOP, BIAS_GRAD>;
  constexpr int kSumBytes = 2 * kLogpTileCols * (int)sizeof(float);
  static_assert(S::kLdsBytes >= kSumBytes, "the column sums reuse the staging memory");
  static PerDeviceOnce once;
  hipError_t err = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), S::kLdsBytes, once);
  if (err != hipSuccess) return err;
  a.tiles_m = (a.T + S::BM - 1) / S::BM;
  a.tiles_v = (a.V + kLogpTileCols - 1) / kLogpTileCols;
  a.group_m = a.tiles_m < 8 ? a.tiles_m : 8;
  hipLaunchKernelGGL(kernel, dim3(a.tiles_m * a.tiles_v), dim3(S::kThreads), S::kLdsBytes, stream, a);
  return hipGetLastError();
}

template <class S, int LOOP>
static hipError_t launch_dlogits(LogpBwdArgs a, hipStream_t stream) {
  return a.bias_part ? launch_dlogits_as<S, LOOP, true>(a, stream) : launch_dlogits_as<S, LOOP, false>(a, stream);
}

// bf16 in[rows, cols] (row stride ld_in) -> out[cols, rows], contiguous. rows % 8 == 0, cols % 8 == 0, 16-byte
// aligned rows on both sides. A workgroup moves a 64 x 64 tile through LDS (rows of 33 dwords).
constexpr int kTransposeTile = 64;
constexpr int kTransposePitch = 33;  // dwords
__global__ __launch_bounds__(256) void transpose_bf16_kernel(const bf16_bits* __restrict__ in, int64_t ld_in,
                                                             bf16_bits* __restrict__ out, int rows, int cols) {
  __shared__ uint32_t tile[kTransposeTile * kTransposePitch];
  const int tid = threadIdx.x;
  const int r0 = blockIdx.y * kTransposeTile;
  const int c0 = blockIdx.x * kTransposeTile;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int ci = tid + i * 256;
    const int r = ci >> 3;
    const int ch = ci & 7;
    u32x4_t v = {0u, 0u, 0u, 0u};
    if (r0 + r < rows && c0 + ch * kChunkElems < cols)
      v = *reinterpret_cast<const u32x4_t*>(in + (int64_t)(r0 + r) * ld_in + c0 + ch * kChunkElems);
#pragma unroll
    for (int e = 0; e < 4; ++e) tile[r * kTransposePitch + ch * 4 + e] = v[e];
  }
  __syncthreads();
  const bf16_bits* halves = reinterpret_cast<const bf16_bits*>(tile);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int ci = tid + i * 256;
    const int c = ci >> 3;   // column of the input tile = row of the output
    const int ch = ci & 7;   // 8 consecutive input rows
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t lo = halves[(ch * 8 + 2 * e) * (2 * kTransposePitch) + c];
      const uint32_t hi = halves[(ch * 8 + 2 * e + 1) * (2 * kTransposePitch) + c];
      w[e] = lo | (hi << 16);
    }
    if (c0 + c < cols && r0 + ch * kChunkElems < rows)
      *reinterpret_cast<u32x4_t*>(out + (int64_t)(c0 + c) * rows + r0 + ch * kChunkElems) =
          u32x4_t{w[0], w[1], w[2], w[3]};
  }
}

hipError_t linear_logp_bwd_launch(const MatView& H, const MatView& W, const int64_t* target, const float* bias,
                                  const float* temperature, const float* lse, const float* grad_logp,
                                  const float* grad_lse, void* grad_hidden, int64_t gh_row_stride, void* grad_weight,
                                  int64_t gw_row_stride, float* grad_bias, void* workspace, int T, int D, int V,
                                  int64_t vocab_start, int vocab_limit, int config, hipStream_t stream) {
  LogpBwdArgs a;
  a.W = W;
  a.H = H;
  a.target = target;
  a.bias = bias;
  a.temperature = temperature;
  a.lse = lse;
  a.grad_logp = grad_logp;
  a.grad_lse = grad_lse;
  a.dz = reinterpret_cast<bf16_bits*>(workspace);
  a.ld_dz = linear_logp_dz_row_stride(V);
  a.T = T;
  a.V = V;
  a.D = D;
  a.vocab_limit = vocab_limit;
  a.vocab_start = vocab_start;
  a.tiles_m = a.tiles_v = 0;
  a.group_m = 1;
  a.bias_part = grad_bias ? reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + dz_bytes(T, V)) : nullptr;

  const bool vec = W.k_stride == 1 && H.k_stride == 1 && (W.row_stride % kChunkElems) == 0 &&
                   (H.row_stride % kChunkElems) == 0 && (reinterpret_cast<uintptr_t>(W.ptr) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(H.ptr) & 15) == 0 && (D % kChunkElems) == 0 &&
                   pitch_fits_lane_offsets(W.row_stride) && pitch_fits_lane_offsets(H.row_stride);
  const bool force_staged = (config & RLK_LOGP_CFG_FORCE_STAGED) != 0;
  config &= ~RLK_LOGP_CFG_FORCE_STAGED;
  if (config == RLK_LOGP_CFG_AUTO) config = pick_linear_logp_config(T, V);
  // the stream-group configurations are forward-only work splits
  if (config == RLK_LOGP_CFG_64_STREAMS) config = RLK_LOGP_CFG_64;
  if (config == RLK_LOGP_CFG_128_STREAMS) config = RLK_LOGP_CFG_128;
  if (config == RLK_LOGP_CFG_256_STREAMS) config = RLK_LOGP_CFG_256;
  if (!vec && config == RLK_LOGP_CFG_256) config = RLK_LOGP_CFG_128;
  // the bias-gradient partials of 16-token tiles only fit the workspace up to kBiasSmallTileMaxTokens
  if (grad_bias && config == RLK_LOGP_CFG_16 && T > kBiasSmallTileMaxTokens) config = RLK_LOGP_CFG_64;
  const int tile_tokens = config == RLK_LOGP_CFG_256 ? 256 : config == RLK_LOGP_CFG_128 ? 128 : config == RLK_LOGP_CFG_64 ? 64 : 16;
  const int loop = !vec ? 0 : (D % kTileK == 0 && !force_staged) ? 2 : 1;
  hipError_t err;
  switch (config) {
    case RLK_LOGP_CFG_256:
      err = loop == 2 ? launch_dlogits<LogpShape256, 2>(a, stream) : launch_dlogits<LogpShape256, 1>(a, stream);
      break;
    case RLK_LOGP_CFG_128:
      err = loop == 2   ? launch_dlogits<LogpShape128, 2>(a, stream)
            : loop == 1 ? launch_dlogits<LogpShape128, 1>(a, stream)
                        : launch_dlogits<LogpShape128, 0>(a, stream);
      break;
    case RLK_LOGP_CFG_64:
      err = loop == 2   ? launch_dlogits<LogpShape64, 2>(a, stream)
            : loop == 1 ? launch_dlogits<LogpShape64, 1>(a, stream)
                        : launch_dlogits<LogpShape64, 0>(a, stream);
      break;
    case RLK_LOGP_CFG_16:
      err = loop >= 1 ? launch_dlogits<LogpShape16, 1>(a, stream) : launch_dlogits<LogpShape16, 0>(a, stream);
      break;
    default:
      return hipErrorInvalidValue;
  }
  if (err != hipSuccess) return err;

  const int gemm_config = force_staged ? (RLK_GEMM_CFG_AUTO | RLK_GEMM_CFG_FORCE_STAGED) : RLK_GEMM_CFG_AUTO;
  if (grad_weight) {
    // grad_weight[v, d] = sum over t ascending of dz[t, v] * H[t, d]
    const MatView dz_by_column{a.dz, 1, a.ld_dz, V};  // rows = v, reduction index = t
    // Both operands are K-major as they lie. From 512 tokens on the hidden states are transposed first (into the
    // grad_hidden buffer, which has exactly their size and is written only afterwards), so that the feature operand
    // runs the plain ping-pong loads: lm_head at 8192 tokens 8.32 -> 7.79 ms plus 0.04 ms for the transposition.
    // Up to 256 tokens the streaming kernel takes the K-major operand as it is.
    const bool via_transposed_hidden =
        grad_hidden != nullptr && gh_row_stride == D && !force_staged && T >= 512 && T % kChunkElems == 0 && vec &&
        (reinterpret_cast<uintptr_t>(grad_hidden) & 15) == 0;
    if (via_transposed_hidden) {
      bf16_bits* hidden_t = reinterpret_cast<bf16_bits*>(grad_hidden);
      hipLaunchKernelGGL(transpose_bf16_kernel, dim3((D + kTransposeTile - 1) / kTransposeTile, (T + kTransposeTile - 1) / kTransposeTile),
                         dim3(256), 0, stream, H.ptr, H.row_stride, hidden_t, T, D);
      err = hipGetLastError();
      if (err != hipSuccess) return err;
      const MatView h_rows{hidden_t, T, 1, D};  // rows = d, reduction index = t contiguous
      err = det_gemm_launch(h_rows, dz_by_column, grad_weight, gw_row_stride, V, D, T, false, gemm_config, stream);
    } else {
      const MatView h_by_feature{H.ptr, 1, H.row_stride, D};  // rows = d, reduction index = t
      err = det_gemm_launch(h_by_feature, dz_by_column, grad_weight, gw_row_stride, V, D, T, false, gemm_config, stream);
    }
    if (err != hipSuccess) return err;
  }
  if (grad_hidden) {
    // grad_hidden[t, d] = sum over v ascending of dz[t, v] * W[v, d]
    const MatView w_by_feature{W.ptr, 1, W.row_stride, D};  // rows = d, reduction index = v
    const MatView dz_by_token{a.dz, a.ld_dz, 1, T};
    err = det_gemm_launch(w_by_feature, dz_by_token, grad_hidden, gh_row_stride, T, D, V, false, gemm_config, stream);
    if (err != hipSuccess) return err;
  }
  if (grad_bias) {
    const int tiles = (T + tile_tokens - 1) / tile_tokens;
    hipLaunchKernelGGL(logp_bias_merge_kernel, dim3((V + 255) / 256), dim3(256), 0, stream, a.bias_part, grad_bias,
                       tiles, kBiasBlockTokens / tile_tokens, V);
    err = hipGetLastError();
  }
  return err;
}

}  // namespace rlk
