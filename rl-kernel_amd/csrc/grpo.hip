// GRPO ratio / k3-KL / clipped-surrogate epilogue on per-token log-probs.
//
// Restates compute_policy_ratio, compute_reference_kl and masked_mean
// (reference rl_engine/reference/definitions.py:50-106) and the surrogate of
// NativeGRPOLossOp.apply (rl_engine/reference/loss/grpo_loss.py:114-125, 162-168)
// with the fixed summation order the reference names SEQUENCE_MAJOR_FIXED
// (rl_engine/contracts/operators/loss.py:7-12): tokens are summed per sequence
// over the fixed padded length, then sequences are combined in ascending index.
//
// Per-sequence order: thread i of a 256-thread workgroup adds tokens
// i, i+256, i+512, ... ascending; the 256 partials are combined by a balanced
// binary tree over adjacent lanes (xor 1, 2, 4, ... 32), then the four waves in
// ascending order. Sequence partials are added ascending by one thread.
#include "rlk_host.h"

namespace rlk {

constexpr int kGrpoThreads = 256;

struct GrpoArgs {
  const float* logp;
  const float* old_logp;
  const float* ref_logp;
  const float* advantages;  // [rollouts]
  const uint8_t* mask;      // [rollouts * tokens] or null (all active)
  float* ratio;             // [rollouts * tokens] or null
  float* k3;                // [rollouts * tokens] or null
  float* seq_part;          // [3][rollouts]: policy sum, kl sum, active count
  int rollouts;
  int tokens;
  float clip_lo, clip_hi;
};

__device__ __forceinline__ float wave_tree_sum(float v) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) v = v + __shfl_xor(v, off, 64);
  return v;
}

__global__ __launch_bounds__(kGrpoThreads) void grpo_sequence_kernel(GrpoArgs a) {
  const int seq = blockIdx.x;
  const float adv = a.advantages[seq];
  const int64_t base = (int64_t)seq * a.tokens;
  float pol = 0.f, kl = 0.f, cnt = 0.f;
  for (int t = threadIdx.x; t < a.tokens; t += kGrpoThreads) {
    const bool active = a.mask ? (a.mask[base + t] != 0) : true;
    const float lp = a.logp[base + t];
    float r = expf(lp - a.old_logp[base + t]);
    const float d = a.ref_logp[base + t] - lp;
    float k = expf(d) - d - 1.0f;
    r = active ? r : 0.f;
    k = active ? k : 0.f;
    const float adv_t = active ? adv : 0.f;
    const float unclipped = r * adv_t;
    const float clipped = fminf(fmaxf(r, a.clip_lo), a.clip_hi) * adv_t;
    float term = -fminf(unclipped, clipped);
    term = active ? term : 0.f;
    if (a.ratio) a.ratio[base + t] = r;
    if (a.k3) a.k3[base + t] = k;
    pol = pol + term;
    kl = kl + k;
    cnt = cnt + (active ? 1.f : 0.f);
  }
  pol = wave_tree_sum(pol);
  kl = wave_tree_sum(kl);
  cnt = wave_tree_sum(cnt);
  __shared__ float sh[3][kGrpoThreads / 64];
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    sh[0][wave] = pol;
    sh[1][wave] = kl;
    sh[2][wave] = cnt;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float p = sh[0][0], k = sh[1][0], c = sh[2][0];
    for (int w = 1; w < kGrpoThreads / 64; ++w) {
      p = p + sh[0][w];
      k = k + sh[1][w];
      c = c + sh[2][w];
    }
    a.seq_part[seq] = p;
    a.seq_part[a.rollouts + seq] = k;
    a.seq_part[2 * a.rollouts + seq] = c;
  }
}

__global__ void grpo_finish_kernel(const float* __restrict__ seq_part, int rollouts, float beta,
                                   float* __restrict__ out3) {
  if (blockIdx.x != 0 || threadIdx.x != 0) return;
  float p = 0.f, k = 0.f, c = 0.f;
  for (int s = 0; s < rollouts; ++s) {
    p = p + seq_part[s];
    k = k + seq_part[rollouts + s];
    c = c + seq_part[2 * rollouts + s];
  }
  const float denom = fmaxf(c, 1e-8f);
  const float policy = p / denom;
  const float klm = k / denom;
  out3[0] = policy + beta * klm;
  out3[1] = policy;
  out3[2] = klm;
}

hipError_t grpo_launch(const float* logp, const float* old_logp, const float* ref_logp, const float* advantages,
                       const uint8_t* mask, int rollouts, int tokens, float clip_eps, float beta, float* ratio,
                       float* k3, float* out3, float* workspace, hipStream_t stream) {
  GrpoArgs a;
  a.logp = logp;
  a.old_logp = old_logp;
  a.ref_logp = ref_logp;
  a.advantages = advantages;
  a.mask = mask;
  a.ratio = ratio;
  a.k3 = k3;
  a.seq_part = workspace;
  a.rollouts = rollouts;
  a.tokens = tokens;
  a.clip_lo = 1.0f - clip_eps;
  a.clip_hi = 1.0f + clip_eps;
  if (rollouts > 0) {
    hipLaunchKernelGGL(grpo_sequence_kernel, dim3(rollouts), dim3(kGrpoThreads), 0, stream, a);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return err;
  }
  hipLaunchKernelGGL(grpo_finish_kernel, dim3(1), dim3(64), 0, stream, workspace, rollouts, beta, out3);
  return hipGetLastError();
}

}  // namespace rlk
