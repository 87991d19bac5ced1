// Host-side declarations shared by the translation units of librlk_gfx950.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/rlk.h"
#include "det_gemm_tile.h"

namespace rlk {

constexpr int kMaxDevices = 64;

// Raises a kernel's dynamic-LDS limit once per device (the attribute is per device and
// sticky). Safe to call from several host threads: the flag is only ever set after the
// attribute call has succeeded, and setting the attribute twice is harmless.
struct PerDeviceOnce {
  std::atomic<bool> done[kMaxDevices];
};

inline hipError_t allow_dynamic_lds(const void* kernel, int bytes, PerDeviceOnce& once) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  const bool tracked = dev >= 0 && dev < kMaxDevices;
  if (tracked && once.done[dev].load(std::memory_order_acquire)) return hipSuccess;
  err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (err == hipSuccess && tracked) once.done[dev].store(true, std::memory_order_release);
  return err;
}

// The direct-to-LDS loaders keep a lane's offset inside its block of rows (up to 64 rows of a tile) as a 32-bit
// element count; a row (or K-row) pitch below 2^24 elements keeps that exact. Larger pitches take the element loaders,
// which index in 64 bits.
inline bool pitch_fits_lane_offsets(int64_t ld) { return ld >= 0 && ld < (int64_t(1) << 24); }

// Compute units of the current device (hipDeviceProp_t::multiProcessorCount, read once per device; 256 on an
// MI355X, which is also the answer when no device can be asked).
int device_cu_count();

// What a launch of `tiles` equal workgroups costs in rounds of one workgroup per compute unit: the whole rounds plus
// a last, partly filled one priced at max(0.9, its share) - the chip is power limited and a round that keeps fewer
// compute units busy runs at a higher clock, so its cost is little more than its share, but never free.
inline double rounds_of_workgroups(int64_t tiles, int cus) {
  const int64_t full = tiles / cus;
  const double part = (double)(tiles - full * cus) / cus;
  return (double)full + (part > 0.0 ? (part > 0.9 ? part : 0.9) : 0.0);
}

int pick_det_gemm_config(int M, int N, int K);

// W[N,K] is the operand whose rows are output features, X[M,K] the one whose
// rows are tokens; C[m*ldc + n].
hipError_t det_gemm_launch(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                           bool out_f32, int config, hipStream_t stream);

// The k-tree contract (fp32 leaves of at most 32 K values, bf16 midpoint tree). A[M, K]; B holds
// one row per output column (B.rows == N); any strides. K <= det_gemm_tree_max_k().
int det_gemm_tree_max_k();
// leaf_space: the midpoint split counts fixed 32-wide leaves instead of elements (its own contract id).
hipError_t det_gemm_tree_launch(const MatView& A, const MatView& B, void* C, int64_t ldc, int M, int N, int K,
                                int config, hipStream_t stream, bool leaf_space = false);

// The strictly sequential fp32 chain (one fused multiply-add per k, ascending, no rounding below fp32).
// An operand is bf16 or fp32, addressed as ptr[row * row_stride + k * k_stride] in elements; B holds one
// row per output column. C is fp32 [M, ldc], or bf16 when out_bf16. K >= 1.
struct SeqOperand {
  const void* ptr;
  int64_t row_stride;
  int64_t k_stride;
};
hipError_t det_gemm_seq_launch(const SeqOperand& A, bool a_f32, const SeqOperand& B, bool b_f32, void* C, int64_t ldc,
                               int M, int N, int K, bool out_bf16, hipStream_t stream);

// Up to 64 tokens, unit K stride, 16-byte aligned rows, K % 64 == 0. `shallow`: M <= 16 with
// two workgroups per CU.
hipError_t det_gemm_stream_launch(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                                  bool out_f32, bool shallow, hipStream_t stream);
// The same kernel on a packed gate/up weight [2 I, K] with the SwiGLU epilogue, M <= 16: Y[M, I].
hipError_t det_gemm_stream_gated_launch(const MatView& W, const MatView& X, void* Y, int64_t ldy, int M, int I, int K,
                                        hipStream_t stream);

// A reduction of 64 ... 256 values (K % 64 == 0) against a K-major token operand (x[k * ld + m], 16-byte aligned
// K rows, M % 8 == 0): the feature operand (any strides) stays in registers, the tokens stream through LDS.
bool det_gemm_shortk_supported(const MatView& W, const MatView& X, int M, int N, int K);
bool det_gemm_shortk_pays(int M, int N);  // enough token tiles per workgroup to amortise its start
hipError_t det_gemm_shortk_launch(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                                  bool out_f32, hipStream_t stream);

hipError_t fill_zero_launch(void* dst, int64_t rows, int64_t cols, int64_t ld, int elem_bytes,
                            hipStream_t stream);

int pick_linear_logp_config(int T, int V);
int linear_logp_split_count(int V);
size_t linear_logp_workspace_bytes(int T, int V);

// H[T,D] hidden states, W[V,D] lm_head weight; workspace holds
// linear_logp_workspace_bytes(T, V) bytes of fp32 partials. logp, lse and target_logit
// (the unclamped scaled logit of a target this weight owns, else 0) may each be null, and so may
// logits ([T, logits_ld] fp32: the accumulators with the bias added and padded lanes -inf, before
// the temperature, stored by the same pass).
hipError_t linear_logp_launch(const MatView& H, const MatView& W, const int64_t* target, const float* bias,
                              const float* temperature, float* logp, float* lse, float* target_logit,
                              float* logits, int64_t logits_ld, float* workspace, int T, int D, int V,
                              int64_t vocab_start, int vocab_limit, int config, hipStream_t stream);

// Ascending merge of (max, sum, target logit) partials laid out [3][n_split][T] into
// lse = M + log(S), logp = target - lse (clamped at 0 when `clamp`) and the merged target
// logit itself (0 for a target no partial owns); each output may be null. With `target` given, a row whose
// target id lies outside [target_lo, target_hi) gets logp = NaN; with `temperature` given, a row whose
// temperature is not a positive number gets logp = lse = NaN.
hipError_t linear_logp_merge_launch(const float* part, float* logp, float* lse, float* target_logit, int T,
                                    int n_split, bool clamp, hipStream_t stream, const int64_t* target = nullptr,
                                    int64_t target_lo = 0, int64_t target_hi = 0, const float* temperature = nullptr);

// Per-row, per-tile (max, sum of exp relative to it[, target logit]) of materialised logits
// of element type `dtype` (rlk_dtype); element (row, tile) of each output sits at
// out[row * out_row_stride + tile * out_tile_stride]. V % num_tiles == 0.
hipError_t logits_tile_stats_launch(const void* logits, int dtype, int64_t row_stride, const int64_t* target,
                                    const float* temperature, int T, int64_t V, int64_t vocab_start,
                                    int64_t real_vocab, int num_tiles, float* out_max, float* out_sum,
                                    float* out_target, int64_t out_row_stride, int64_t out_tile_stride,
                                    hipStream_t stream);

// d(logits) of logp / lse computed from materialised logits, in the dtype of the logits.
hipError_t logits_backward_launch(const void* logits, int dtype, int64_t row_stride, const float* lse,
                                  const float* coef_logp, const float* coef_lse, const int64_t* target_local,
                                  const float* temperature, void* grad, int64_t grad_row_stride, int T, int64_t V,
                                  int64_t vocab_start, int64_t real_vocab, hipStream_t stream);

// Backward of the fused linear-LogP. workspace holds linear_logp_bwd_workspace_bytes() bytes
// (the bf16 d(logits) with row stride linear_logp_dz_row_stride(V), then the bias block sums).
// grad_hidden / grad_weight / grad_bias may each be null.
int64_t linear_logp_dz_row_stride(int V);
size_t linear_logp_bwd_workspace_bytes(int T, int V, bool with_bias);
hipError_t linear_logp_bwd_launch(const MatView& H, const MatView& W, const int64_t* target, const float* bias,
                                  const float* temperature, const float* lse, const float* grad_logp,
                                  const float* grad_lse, void* grad_hidden, int64_t gh_row_stride, void* grad_weight,
                                  int64_t gw_row_stride, float* grad_bias, void* workspace, int T, int D, int V,
                                  int64_t vocab_start, int vocab_limit, int config, hipStream_t stream);

// SwiGLU on rows of `dtype` (rlk_dtype; strides in elements): forward writes y = out; backward
// writes d_gate = out, d_up = out2.
hipError_t swiglu_launch(const void* gate, int64_t ld_g, const void* up, int64_t ld_u, const void* dy, int64_t ld_dy,
                         void* out, int64_t ld_out, void* out2, int64_t ld_out2, int rows, int cols, bool backward,
                         int dtype, hipStream_t stream);

// Packed gate/up projection W[2 I, K] with the SwiGLU epilogue; workspace ([M, 2 I] bf16) is
// only touched when det_gemm_swiglu_fused_supported() is false.
bool det_gemm_swiglu_fused_supported(const MatView& W, const MatView& X, int M, int K);
hipError_t det_gemm_swiglu_launch(const MatView& W, const MatView& X, void* Y, int64_t ldy, void* workspace, int M,
                                  int I, int K, hipStream_t stream);

// workspace: 3 * rollouts floats.
hipError_t grpo_launch(const float* logp, const float* old_logp, const float* ref_logp, const float* advantages,
                       const uint8_t* mask, int rollouts, int tokens, float clip_eps, float beta, float* ratio,
                       float* k3, float* out3, float* workspace, hipStream_t stream);

void set_last_error(const char* fmt, ...);

}  // namespace rlk
