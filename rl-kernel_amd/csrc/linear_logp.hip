// Fused linear-LogP for gfx950: lm_head GEMM -> online log-sum-exp over the
// vocabulary in a fixed order -> target-token gather. The [tokens, vocab] logits
// never leave registers.
//
// Stands in for rl_engine._C.fused_linear_logp_sm90 (reference
// csrc/cuda/logprob/fused_linear_logp_sm90.cu:104-325, 488-513, 2040-2176), for
// triton_deterministic_linear_logp (rl_engine/backends/shared/triton/logprob/
// linear_logp.py:277-418, 631-700) and for the unfused ROCm route
// DetGemmOp().linear + hip_deterministic_logp_tile_stats
// (rl_engine/integrations/common/linear_logp.py:1083-1102).
//
// Reduction contract (everything that decides the bits of logp / lse; all of it
// is a function of the vocabulary axis only, never of the token count, the
// position of a token in the batch or the launch geometry):
//   z_v   = fp32 MFMA chain of det_gemm over the hidden dimension, + bias_v
//   y_v   = z_v                      (v < real vocabulary bound)
//         = -inf                     (padded lane)
//         then y_v * (1 / temperature) when a temperature is given
//   tile  = 256 consecutive vocabulary columns; stream j (0..15) of a tile is
//           its columns [16 j, 16 j + 16)
//   split = 4 consecutive tiles (1024 columns); n_split = ceil(V / 1024)
//   stream chain (per split, per j), tiles ascending, state (m, s) = (-inf, 0):
//           t = max of the 16 y;  n = max(m, t);
//           if n > -inf:  s = s * e(m - n) + (((e(y0 - n) + e(y1 - n)) + ...) + e(y15 - n));  m = n
//   split merge:  M = max_j m_j;  S = sum over j ascending of s_j * e(m_j - M)  (terms with m_j = -inf skipped)
//   final merge over splits ascending with the same formula;
//   lse = M + log(S);  zt = y_target;  logp = min(zt - lse, 0)
//   e(x) = v_exp_f32(x * log2(e)) with an unfused fp32 multiply.
#include "linear_logp_common.h"
#include "rlk_host.h"

namespace rlk {

struct LogpArgs {
  MatView W;  // [V, D] lm_head weight, rows = vocabulary
  MatView H;  // [T, D] hidden states, rows = tokens
  const int64_t* target;     // [T] global vocabulary ids
  const float* bias;         // [V] or null
  const float* temperature;  // [T] or null
  float* part;               // [3][n_split][T]: max, sum, target logit
  float* logits;             // [T, logits_ld] fp32 biased logits (no temperature), or null: not wanted
  int64_t logits_ld;
  int T, V, D;
  int vocab_limit;  // local column bound of the real vocabulary (<= V)
  int64_t vocab_start;
  int tiles_m, n_split, group_m;
};

// LOOP: 0 generic element loader, 1 register-staged 16-byte loads, 2 direct-to-LDS ping-pong.
template <class S, int LOOP>
__global__ __launch_bounds__(S::kThreads) void linear_logp_partial_kernel(LogpArgs a) {
  static_assert(S::BN == kLogpTileCols && S::kRun == 16 && S::WN == 4, "stream layout is pinned");
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int total = a.tiles_m * a.n_split;
  const int id = xcd_compact_id(blockIdx.x, total);
  const int per_group = a.group_m * a.n_split;
  const int group = id / per_group;
  const int first_m = group * a.group_m;
  const int width = (a.tiles_m - first_m) < a.group_m ? (a.tiles_m - first_m) : a.group_m;
  const int within = id - group * per_group;
  const int tile_m = first_m + within % width;
  const int split = within / width;
  const int m0 = tile_m * S::BM;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wave_n = wave % S::WN;
  const int wave_m = wave / S::WN;
  const int l16 = lane & 15;
  const int grp = lane >> 4;
  const int stream = wave_n * 4 + grp;
  const int tok_local = wave_m * 16 * S::TM + l16;

  float run_m[S::TM], run_s[S::TM], run_zt[S::TM], inv_t[S::TM];
  int tgt[S::TM];
#pragma unroll
  for (int jm = 0; jm < S::TM; ++jm) {
    const int m = m0 + tok_local + jm * 16;
    run_m[jm] = kNegInf;
    run_s[jm] = 0.f;
    run_zt[jm] = 0.f;
    inv_t[jm] = 1.0f;
    tgt[jm] = -1;
    if (m < a.T) {
      const int64_t local = a.target[m] - a.vocab_start;
      tgt[jm] = (local >= 0 && local < a.vocab_limit) ? (int)local : -1;
      if (a.temperature) inv_t[jm] = 1.0f / a.temperature[m];
    }
  }

  for (int t = 0; t < kLogpSplitTiles; ++t) {
    const int v0 = split * kLogpSplitCols + t * kLogpTileCols;
    if (v0 >= a.V) break;
    f32x4_t acc[S::TN][S::TM];
    if constexpr (LOOP == 2) {
      tile_mainloop_pingpong<S>(a.W, a.H, v0, m0, a.D, lds, acc);
    } else {
      tile_mainloop_staged<S, LOOP == 1>(a.W, a.H, v0, m0, a.D, lds, acc);
    }

    const int col0 = v0 + stream * 16;  // first column of this lane's run
    const int span0 = v0 + wave_n * 64;  // first column of the wave's four runs
    // whole spans into 16-byte aligned rows are stored by the four lanes of a token together (wave uniform)
    const bool span_stores = a.logits != nullptr && span0 + 64 <= a.V && (a.logits_ld & 3) == 0 &&
                             (reinterpret_cast<uintptr_t>(a.logits) & 15) == 0;
    float bias_run[16];
#pragma unroll
    for (int c = 0; c < 16; ++c) bias_run[c] = 0.f;
    if (a.bias) {
#pragma unroll
      for (int c = 0; c < 16; ++c) bias_run[c] = (col0 + c < a.V) ? a.bias[col0 + c] : 0.f;
    }
#pragma unroll
    for (int jm = 0; jm < S::TM; ++jm) {
      float y[16];
#pragma unroll
      for (int c = 0; c < 16; ++c) y[c] = biased_logit(acc[c >> 2][jm][c & 3], a.bias != nullptr, bias_run[c], col0 + c, a.vocab_limit);
      if (a.logits) {  // the same accumulators the reduction sees, stored before the temperature
        const int m = m0 + tok_local + jm * 16;
        float* row = a.logits + (int64_t)(m < a.T ? m : 0) * a.logits_ld;
        if (span_stores) store_logit_span(row, span0, grp, m < a.T, y);
        else if (m < a.T) store_logit_run(row, col0, a.V, y);
      }
      if (a.temperature) {
#pragma unroll
        for (int c = 0; c < 16; ++c) y[c] = y[c] * inv_t[jm];
      }
      logp_fold_run(y, tgt[jm] - col0, run_m[jm], run_s[jm], run_zt[jm]);
    }
  }

  // Fold the 16 streams of every token in ascending stream order. The main loop
  // ended on a barrier, so the staging LDS is free.
  float* xm = reinterpret_cast<float*>(lds);
  float* xs = xm + kLogpStreams * S::BM;
  float* xz = xs + kLogpStreams * S::BM;
#pragma unroll
  for (int jm = 0; jm < S::TM; ++jm) {
    const int slot = stream * S::BM + tok_local + jm * 16;
    xm[slot] = run_m[jm];
    xs[slot] = run_s[jm];
    xz[slot] = run_zt[jm];
  }
  __syncthreads();
  for (int tok = threadIdx.x; tok < S::BM; tok += S::kThreads) {
    const int m = m0 + tok;
    if (m >= a.T) continue;
    float big, sum, zt;
    logp_merge_streams(xm + tok, xs + tok, xz + tok, S::BM, big, sum, zt);
    const int64_t plane = (int64_t)a.n_split * a.T;
    const int64_t at = (int64_t)split * a.T + m;
    a.part[at] = big;
    a.part[plane + at] = sum;
    a.part[2 * plane + at] = zt;
  }
}

// Few token tiles: a split of 1024 columns gives the chip only tiles_m * ceil(V / 1024)
// workgroups of four K loops each. Streams are independent until the stream merge, so here a
// workgroup takes four of the sixteen streams of a split, i.e. the 64-column slice
// [64 g, 64 g + 64) of each of the split's four tiles, as ONE 256-row GEMM tile (wave column t
// holds tile t's slice): four times the workgroups, one K loop each. The online chain of a
// (token, stream) still visits the tiles in ascending order: wave column t folds its sixteen
// columns into the state that column t - 1 left in LDS. Per-(split, stream) states go to
// linear_logp_stream_merge_kernel, which repeats the in-kernel stream merge above. Same bits
// as every other configuration.
template <class S, int NS>
__global__ __launch_bounds__(S::kThreads) void linear_logp_streamgroup_kernel(LogpArgs a, float* __restrict__ spart,
                                                                              int split_first, int split_count) {
  static_assert(S::BN == kLogpTileCols && S::kRun == 16 && S::WN == 4, "wave column = tile of the split");
  constexpr int kGroups = kLogpStreams / 4;  // stream groups per split
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int total = a.tiles_m * split_count * kGroups;  // this launch covers splits [split_first, + split_count)
  const int id = xcd_compact_id(blockIdx.x, total);
  const int tile_m = id % a.tiles_m;
  const int unit = id / a.tiles_m;
  const int split = split_first + unit / kGroups;
  const int sg = unit % kGroups;
  const int m0 = tile_m * S::BM;
  const int n0 = split * kLogpSplitCols + sg * 64;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int tile = wave % S::WN;
  const int wave_m = wave / S::WN;
  const int l16 = lane & 15;
  const int grp = lane >> 4;  // stream inside the group
  const int tok_local = wave_m * 16 * S::TM + l16;

  f32x4_t acc[S::TN][S::TM];
  tile_mainloop_pingpong<S, false, false, StridedColumnRowMap<S, kLogpTileCols>, 1, NS>(a.W, a.H, n0, m0, a.D, lds, acc);

  const int v0 = split * kLogpSplitCols + tile * kLogpTileCols;
  const int col0 = v0 + (sg * 4 + grp) * 16;  // first column of this lane's run
  float bias_run[16];
#pragma unroll
  for (int c = 0; c < 16; ++c) bias_run[c] = (a.bias && col0 + c < a.V) ? a.bias[col0 + c] : 0.f;

  // The main loop ended on a barrier, so the staging LDS is free: states [3][4 streams][BM].
  float* sm = reinterpret_cast<float*>(lds);
  float* ss = sm + 4 * S::BM;
  float* sz = ss + 4 * S::BM;
#pragma unroll 1
  for (int t = 0; t < kLogpSplitTiles; ++t) {
    if (tile == t && v0 < a.V) {  // a tile past the vocabulary leaves the states alone
#pragma unroll
      for (int jm = 0; jm < S::TM; ++jm) {
        const int slot = grp * S::BM + tok_local + jm * 16;
        const int m = m0 + tok_local + jm * 16;
        int tgt = -1;
        float inv_t = 1.0f;
        if (m < a.T) {
          const int64_t local = a.target[m] - a.vocab_start;
          tgt = (local >= 0 && local < a.vocab_limit) ? (int)local : -1;
          if (a.temperature) inv_t = 1.0f / a.temperature[m];
        }
        float run_m = kNegInf, run_s = 0.f, run_zt = 0.f;
        if (t > 0) {
          run_m = sm[slot];
          run_s = ss[slot];
          run_zt = sz[slot];
        }
        float y[16];
#pragma unroll
        for (int c = 0; c < 16; ++c) y[c] = biased_logit(acc[c >> 2][jm][c & 3], a.bias != nullptr, bias_run[c], col0 + c, a.vocab_limit);
        if (a.logits && m < a.T) store_logit_run(a.logits + (int64_t)m * a.logits_ld, col0, a.V, y);
        if (a.temperature) {
#pragma unroll
          for (int c = 0; c < 16; ++c) y[c] = y[c] * inv_t;
        }
        logp_fold_run(y, tgt - col0, run_m, run_s, run_zt);
        sm[slot] = run_m;
        ss[slot] = run_s;
        sz[slot] = run_zt;
      }
    }
    __syncthreads();
  }

  const int64_t plane = (int64_t)a.n_split * kLogpStreams * a.T;
  for (int idx = threadIdx.x; idx < 4 * S::BM; idx += S::kThreads) {
    const int sl = idx / S::BM;
    const int m = m0 + idx % S::BM;
    if (m >= a.T) continue;
    const int64_t at = ((int64_t)split * kLogpStreams + sg * 4 + sl) * a.T + m;
    spart[at] = sm[idx];
    spart[plane + at] = ss[idx];
    spart[2 * plane + at] = sz[idx];
  }
}

// Per-(split, stream) states [3][n_split * 16][T] -> per-split partials [3][n_split][T], streams
// ascending: the arithmetic of the stream merge at the end of linear_logp_partial_kernel.
__global__ __launch_bounds__(256) void linear_logp_stream_merge_kernel(const float* __restrict__ spart,
                                                                      float* __restrict__ part, int T, int n_split) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= T * n_split) return;
  const int m = idx % T;
  const int split = idx / T;
  const int64_t splane = (int64_t)n_split * kLogpStreams * T;
  const float* xm = spart + (int64_t)split * kLogpStreams * T + m;
  float big, sum, zt;
  logp_merge_streams(xm, xm + splane, xm + 2 * splane, T, big, sum, zt);
  const int64_t plane = (int64_t)n_split * T;
  const int64_t at = (int64_t)split * T + m;
  part[at] = big;
  part[plane + at] = sum;
  part[2 * plane + at] = zt;
}

// Final merge over splits. 16 tokens per workgroup, 16 threads per token: the maximum and
// the rescaled terms s_p * e(m_p - M) are computed by all threads (neither depends on an
// order), then one thread per token adds the terms of a chunk in ascending split order,
// chunk after chunk. The target logit has a single non-zero contribution, so its sum is
// exact in any order.
constexpr int kMergeTokens = 16;
constexpr int kMergeLanes = 16;                           // threads per token
constexpr int kMergeChunk = 8 * kMergeLanes;              // splits staged per round
constexpr int kMergeThreads = kMergeTokens * kMergeLanes;  // 256

__global__ __launch_bounds__(kMergeThreads) void linear_logp_merge_kernel(const float* __restrict__ part,
                                                                          float* __restrict__ logp,
                                                                          float* __restrict__ lse,
                                                                          float* __restrict__ target_logit, int T,
                                                                          int n_split, bool clamp,
                                                                          const int64_t* __restrict__ target,
                                                                          int64_t target_lo, int64_t target_hi,
                                                                          const float* __restrict__ temperature) {
  __shared__ float red[kMergeLanes][kMergeTokens];
  __shared__ float terms[kMergeChunk][kMergeTokens];
  const int tk = threadIdx.x % kMergeTokens;
  const int sp = threadIdx.x / kMergeTokens;
  const int m = blockIdx.x * kMergeTokens + tk;
  const bool live = m < T;
  const int64_t plane = (int64_t)n_split * T;

  float big = kNegInf, zt = 0.f;
  if (live) {
    for (int p = sp; p < n_split; p += kMergeLanes) {
      big = fmaxf(big, part[(int64_t)p * T + m]);
      zt = zt + part[2 * plane + (int64_t)p * T + m];
    }
  }
  red[sp][tk] = big;
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kMergeLanes; ++j) big = fmaxf(big, red[j][tk]);
  __syncthreads();
  red[sp][tk] = zt;
  __syncthreads();
  if (sp == 0) {
    zt = 0.f;
#pragma unroll
    for (int j = 0; j < kMergeLanes; ++j) zt = zt + red[j][tk];
  }

  float sum = 0.f;
  for (int c0 = 0; c0 < n_split; c0 += kMergeChunk) {
#pragma unroll
    for (int i = 0; i < kMergeChunk / kMergeLanes; ++i) {
      const int local = i * kMergeLanes + sp;
      const int p = c0 + local;
      float term = 0.f;
      if (live && p < n_split) {
        const float pm = part[(int64_t)p * T + m];
        const float scaled = part[plane + (int64_t)p * T + m] * pinned_exp(pm - big);
        term = (pm > kNegInf) ? scaled : 0.f;
      }
      terms[local][tk] = term;
    }
    __syncthreads();
    if (sp == 0) {
      const int count = (n_split - c0) < kMergeChunk ? (n_split - c0) : kMergeChunk;
      for (int j = 0; j < count; ++j) sum = sum + terms[j][tk];
    }
    __syncthreads();
  }
  if (sp == 0 && live) {
    float l = big + logf(sum);
    // A temperature that is not a positive number scales nothing meaningful: both results of the row are NaN.
    const bool bad_temperature = temperature != nullptr && !(temperature[m] > 0.f);
    // A target id outside [target_lo, target_hi) names no column this call reduces over: the row's log-prob is
    // NaN instead of a number made of a zero target logit (lse is that of the row all the same).
    const bool bad_target = target != nullptr && (target[m] < target_lo || target[m] >= target_hi);
    if (bad_temperature) l = __builtin_nanf("");
    if (lse) lse[m] = l;
    if (logp) {
      float value = clamp ? fminf(zt - l, 0.f) : zt - l;
      if (bad_temperature || bad_target) value = __builtin_nanf("");  // fminf would drop a NaN operand
      logp[m] = value;
    }
    if (target_logit) target_logit[m] = zt;
  }
}

hipError_t linear_logp_merge_launch(const float* part, float* logp, float* lse, float* target_logit, int T,
                                    int n_split, bool clamp, hipStream_t stream, const int64_t* target,
                                    int64_t target_lo, int64_t target_hi, const float* temperature) {
  hipLaunchKernelGGL(linear_logp_merge_kernel, dim3((T + kMergeTokens - 1) / kMergeTokens), dim3(kMergeThreads), 0,
                     stream, part, logp, lse, target_logit, T, n_split, clamp, target, target_lo, target_hi,
                     temperature);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------

using LogpShape256 = TileShape<256, 256, 4, 2>;
using LogpShape128 = TileShape<256, 128, 4, 2>;
using LogpShape64 = TileShape<256, 64, 4, 2>;
using LogpShape16 = TileShape<256, 16, 4, 1>;

int linear_logp_split_count(int V) { return (V + kLogpSplitCols - 1) / kLogpSplitCols; }

constexpr int kStreamGroupMaxTokens = 1024;  // token counts the stream-group kernels serve

size_t linear_logp_workspace_bytes(int T, int V) {
  if (T <= 0) return 0;
  // per-split partials, plus per-(split, stream) states where the stream-group kernel may run
  const size_t per_split = (size_t)3 * linear_logp_split_count(V) * (size_t)T * sizeof(float);
  return T <= kStreamGroupMaxTokens ? per_split * (1 + kLogpStreams) : per_split;
}

template <class S, int LOOP>
static hipError_t launch_logp(LogpArgs a, hipStream_t stream) {
  auto kernel = linear_logp_partial_kernel<S, LOOP>;
  constexpr int kMergeBytes = 3 * kLogpStreams * S::BM * (int)sizeof(float);
  constexpr int kLds = S::kLdsBytes > kMergeBytes ? S::kLdsBytes : kMergeBytes;
  static PerDeviceOnce once;
  hipError_t err = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLds, once);
  if (err != hipSuccess) return err;
  a.tiles_m = (a.T + S::BM - 1) / S::BM;
  a.group_m = a.tiles_m < 8 ? a.tiles_m : 8;
  hipLaunchKernelGGL(kernel, dim3(a.tiles_m * a.n_split), dim3(S::kThreads), kLds, stream, a);
  return hipGetLastError();
}

// Up to 128 tokens every weight tile is used by one workgroup only: three stages for the
// 64- and 128-token tiles (120 / 144 KiB); the 256-token tile has room for two.
template <class S>
static hipError_t launch_streamgroup_range(LogpArgs a, float* spart, int split_first, int split_count,
                                           hipStream_t stream) {
  constexpr int kStages = S::BM <= 128 ? 3 : 2;
  auto kernel = linear_logp_streamgroup_kernel<S, kStages>;
  constexpr int kLdsBytes = kStages * S::kStageBytes;
  static PerDeviceOnce once;
  hipError_t err = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLdsBytes, once);
  if (err != hipSuccess) return err;
  a.tiles_m = (a.T + S::BM - 1) / S::BM;
  hipLaunchKernelGGL(kernel, dim3(a.tiles_m * split_count * (kLogpStreams / 4)), dim3(S::kThreads), kLdsBytes, stream,
                     a, spart, split_first, split_count);
  return hipGetLastError();
}

// `balance`: with the 256-token tile, a last round that would fill at most half of the chip
// runs as 128-token tiles instead (twice the workgroups, each about 0.57 of the time): for
// 256 tokens and V = 151936, 596 workgroups are 2.33 rounds of 256; 512 of them plus 168
// half-height ones are two rounds and a short one (350 -> 290 us). Same bits: the tile height
// is not part of the contract.
template <class S>
static hipError_t launch_streamgroup(LogpArgs a, bool balance, hipStream_t stream) {
  const int kCus = device_cu_count();
  float* spart = a.part + (size_t)3 * a.n_split * a.T;  // behind the per-split partials
  const int tiles_m = (a.T + S::BM - 1) / S::BM;
  const int per_split = tiles_m * (kLogpStreams / 4);
  int main_splits = a.n_split;
  if (balance && S::BM == 256 && per_split <= kCus && kCus % per_split == 0) {
    const int per_round = kCus / per_split;
    const int tail = a.n_split % per_round;
    if (tail * per_split * 2 <= kCus && a.n_split > tail) main_splits = a.n_split - tail;
  }
  hipError_t err = launch_streamgroup_range<S>(a, spart, 0, main_splits, stream);
  if (err != hipSuccess) return err;
  if (main_splits < a.n_split) {
    err = launch_streamgroup_range<LogpShape128>(a, spart, main_splits, a.n_split - main_splits, stream);
    if (err != hipSuccess) return err;
  }
  const int threads = a.T * a.n_split;
  hipLaunchKernelGGL(linear_logp_stream_merge_kernel, dim3((threads + 255) / 256), dim3(256), 0, stream, spart,
                     a.part, a.T, a.n_split);
  return hipGetLastError();
}

int pick_linear_logp_config(int T, int V) {
  (void)V;
  // Measured at V = 151936, D = 4096: the 64-token tile (two workgroups per CU, direct-to-LDS
  // loop) is the fastest from decode sizes up to 64 tokens, the 256-token tile from 256 tokens on
  // even where it leaves the last round of workgroups part empty.
  if (T <= 64) return RLK_LOGP_CFG_64_STREAMS;
  if (T <= 128) return RLK_LOGP_CFG_128_STREAMS;
  // 257 ... 384 tokens are three 128-token tiles or two 256-token ones, a third of them padding (544 against 582 us
  // at 384 tokens); wherever 128-token tiles save no padded tile the 256-token tile wins (798 against 966 us at 768).
  if (T > 256 && T <= 384) return RLK_LOGP_CFG_128_STREAMS;
  if (T <= 1024) return RLK_LOGP_CFG_256_STREAMS;
  return RLK_LOGP_CFG_256;
}

hipError_t linear_logp_launch(const MatView& H, const MatView& W, const int64_t* target, const float* bias,
                              const float* temperature, float* logp, float* lse, float* target_logit,
                              float* logits, int64_t logits_ld, float* workspace, int T, int D, int V,
                              int64_t vocab_start, int vocab_limit, int config, hipStream_t stream) {
  LogpArgs a;
  a.logits = logits;
  a.logits_ld = logits_ld;
  a.W = W;
  a.H = H;
  a.target = target;
  a.bias = bias;
  a.temperature = temperature;
  a.part = workspace;
  a.T = T;
  a.V = V;
  a.D = D;
  a.vocab_limit = vocab_limit;
  a.vocab_start = vocab_start;
  a.n_split = linear_logp_split_count(V);
  a.tiles_m = 0;
  a.group_m = 1;
  const bool vec = W.k_stride == 1 && H.k_stride == 1 && (W.row_stride % kChunkElems) == 0 &&
                   (H.row_stride % kChunkElems) == 0 && (reinterpret_cast<uintptr_t>(W.ptr) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(H.ptr) & 15) == 0 && (D % kChunkElems) == 0 &&
                   pitch_fits_lane_offsets(W.row_stride) && pitch_fits_lane_offsets(H.row_stride);
  const bool force_staged = (config & RLK_LOGP_CFG_FORCE_STAGED) != 0;
  config &= ~RLK_LOGP_CFG_FORCE_STAGED;
  const int requested = config;
  if (config == RLK_LOGP_CFG_AUTO) config = pick_linear_logp_config(T, V);
  if (!vec && config == RLK_LOGP_CFG_256) config = RLK_LOGP_CFG_128;
  const int loop = !vec ? 0 : (D % kTileK == 0 && !force_staged) ? 2 : 1;
  // The stream-group kernels have the direct-to-LDS loop only and a bounded workspace.
  if (loop != 2 || T > kStreamGroupMaxTokens) {
    if (config == RLK_LOGP_CFG_64_STREAMS) config = RLK_LOGP_CFG_64;
    if (config == RLK_LOGP_CFG_128_STREAMS) config = RLK_LOGP_CFG_128;
    if (config == RLK_LOGP_CFG_256_STREAMS) config = RLK_LOGP_CFG_256;
  }
  hipError_t err;
  switch (config) {
    case RLK_LOGP_CFG_64_STREAMS:
      err = launch_streamgroup<LogpShape64>(a, false, stream);
      break;
    case RLK_LOGP_CFG_128_STREAMS:
      err = launch_streamgroup<LogpShape128>(a, false, stream);
      break;
    case RLK_LOGP_CFG_256_STREAMS:
      err = launch_streamgroup<LogpShape256>(a, requested == RLK_LOGP_CFG_AUTO, stream);
      break;
    case RLK_LOGP_CFG_256:
      err = loop == 2 ? launch_logp<LogpShape256, 2>(a, stream) : launch_logp<LogpShape256, 1>(a, stream);
      break;
    case RLK_LOGP_CFG_128:
      err = loop == 2   ? launch_logp<LogpShape128, 2>(a, stream)
            : loop == 1 ? launch_logp<LogpShape128, 1>(a, stream)
                        : launch_logp<LogpShape128, 0>(a, stream);
      break;
    case RLK_LOGP_CFG_64:
      err = loop == 2   ? launch_logp<LogpShape64, 2>(a, stream)
            : loop == 1 ? launch_logp<LogpShape64, 1>(a, stream)
                        : launch_logp<LogpShape64, 0>(a, stream);
      break;
    case RLK_LOGP_CFG_16:
      err = loop >= 1 ? launch_logp<LogpShape16, 1>(a, stream) : launch_logp<LogpShape16, 0>(a, stream);
      break;
    default:
      return hipErrorInvalidValue;
  }
  if (err != hipSuccess) return err;
  // The whole-vocabulary entries (those that write logp) mark rows whose target lies outside the real vocabulary;
  // a shard's target logit is legitimately 0 for a target another shard owns.
  return linear_logp_merge_launch(workspace, logp, lse, target_logit, T, a.n_split, true, stream,
                                  logp != nullptr ? target : nullptr, vocab_start, vocab_start + vocab_limit,
                                  temperature);
}

}  // namespace rlk
