// extern "C" surface of librlk_gfx950.so: argument checking and dispatch only.
#include <stdarg.h>
#include <stdio.h>

#include "rlk_host.h"

namespace rlk {

static thread_local char g_last_error[512] = "";

void set_last_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
}

__global__ void fill_zero_kernel(char* dst, int64_t rows, int64_t row_bytes, int64_t ld_bytes) {
  const int64_t total = rows * row_bytes;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    dst[(i / row_bytes) * ld_bytes + (i % row_bytes)] = 0;
  }
}

hipError_t fill_zero_launch(void* dst, int64_t rows, int64_t cols, int64_t ld, int elem_bytes,
                            hipStream_t stream) {
  const int64_t total = rows * cols * elem_bytes;
  if (total == 0) return hipSuccess;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (char*)dst, rows,
                     cols * elem_bytes, ld * elem_bytes);
  return hipGetLastError();
}

static int device_error(const char* what, hipError_t err) {
  set_last_error("%s: %s", what, hipGetErrorString(err));
  return RLK_ERR_DEVICE;
}

// Scratch of rlk_linear_logp_fwd_noalloc: device memory that belongs to the loaded code object, one copy
// per GPU, held until the process ends. In host code the array's name is only a handle for
// hipGetSymbolAddress; kernels and fills get the per-device address looked up below.
static __device__ __align__(256) unsigned char scratch[RLK_NOALLOC_SCRATCH_BYTES];

static std::atomic<void*> g_scratch_ptr[kMaxDevices];

// The current device's copy of `scratch` (looked up once per device; no allocation).
static hipError_t scratch_for_current_device(void** out) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return err;
    if (ptr == nullptr) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // several threads may store the same address
  }
  *out = ptr;
  return hipSuccess;
}

}  // namespace rlk

using namespace rlk;

extern "C" {

const char* rlk_contract_id(void) { return "rlkernel.det_gemm.hip_mfma16x16x32_gfx950.v1"; }

const char* rlk_version(void) { return "0.1.0"; }

const char* rlk_last_error(void) { return g_last_error; }

int rlk_det_gemm_pick_config(int M, int N, int K) { return pick_det_gemm_config(M, N, K); }

int rlk_det_gemm_bf16(const void* a, int64_t a_row_stride, int64_t a_k_stride, const void* b,
                      int64_t b_k_stride, int64_t b_n_stride, void* c, int64_t ldc, int M, int N, int K,
                      int out_fp32, int config, void* stream) {
  if (M < 0 || N < 0 || K < 0) {
    set_last_error("rlk_det_gemm_bf16: negative size M=%d N=%d K=%d", M, N, K);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (a_row_stride < 0 || a_k_stride < 0 || b_k_stride < 0 || b_n_stride < 0) {
    set_last_error("rlk_det_gemm_bf16: operands must not use negative strides");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (config < 0 || (config & ~RLK_GEMM_CFG_FORCE_STAGED) >= RLK_GEMM_CFG_COUNT) {
    set_last_error("rlk_det_gemm_bf16: unknown config %d", config);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (M == 0 || N == 0) return RLK_OK;
  if (c == nullptr || ldc < N) {
    set_last_error("rlk_det_gemm_bf16: output needs a non-null pointer and ldc >= N (ldc=%lld N=%d)",
                   (long long)ldc, N);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (K == 0) {
    hipError_t err = fill_zero_launch(c, M, N, ldc, out_fp32 ? 4 : 2, s);
    return err == hipSuccess ? RLK_OK : device_error("rlk_det_gemm_bf16(fill)", err);
  }
  if (a == nullptr || b == nullptr) {
    set_last_error("rlk_det_gemm_bf16: null operand");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  MatView X{reinterpret_cast<const bf16_bits*>(a), a_row_stride, a_k_stride, M};
  MatView W{reinterpret_cast<const bf16_bits*>(b), b_n_stride, b_k_stride, N};
  hipError_t err = det_gemm_launch(W, X, c, ldc, M, N, K, out_fp32 != 0, config, s);
  return err == hipSuccess ? RLK_OK : device_error("rlk_det_gemm_bf16", err);
}

const char* rlk_det_gemm_tree_contract_id(void) { return "rlkernel.det_gemm.hip_ktree32_gfx950.v1"; }
const char* rlk_det_gemm_tree_leaf_space_contract_id(void) { return "rlkernel.det_gemm.hip_ktree32_leafspace_gfx950.v1"; }

int rlk_det_gemm_tree_bf16(const void* a, int64_t a_row_stride, int64_t a_k_stride, const void* b,
                           int64_t b_k_stride, int64_t b_n_stride, void* c, int64_t ldc, int M, int N, int K,
                           void* stream) {
  return rlk_det_gemm_tree_bf16_config(a, a_row_stride, a_k_stride, b, b_k_stride, b_n_stride, c, ldc, M, N, K,
                                       RLK_TREE_CFG_AUTO, stream);
}

int rlk_det_gemm_tree_bf16_config(const void* a, int64_t a_row_stride, int64_t a_k_stride, const void* b,
                                  int64_t b_k_stride, int64_t b_n_stride, void* c, int64_t ldc, int M, int N,
                                  int K, int config, void* stream) {
  const bool leaf_space = config >= 0 && (config & RLK_TREE_CFG_LEAF_SPACE) != 0;
  if (leaf_space) config &= ~RLK_TREE_CFG_LEAF_SPACE;
  if (config < 0 || config >= RLK_TREE_CFG_COUNT) {
    set_last_error("rlk_det_gemm_tree_bf16: unknown configuration %d", config);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (leaf_space && config != RLK_TREE_CFG_AUTO && config != RLK_TREE_CFG_MFMA_F32) {
    set_last_error("rlk_det_gemm_tree_bf16: RLK_TREE_CFG_LEAF_SPACE goes with RLK_TREE_CFG_AUTO or RLK_TREE_CFG_MFMA_F32");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (M < 0 || N < 0 || K < 0) {
    set_last_error("rlk_det_gemm_tree_bf16: negative size M=%d N=%d K=%d", M, N, K);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (K > det_gemm_tree_max_k()) {
    set_last_error("rlk_det_gemm_tree_bf16: K=%d exceeds the supported %d", K, det_gemm_tree_max_k());
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (a_row_stride < 0 || a_k_stride < 0 || b_k_stride < 0 || b_n_stride < 0) {
    set_last_error("rlk_det_gemm_tree_bf16: operands must not use negative strides");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (M == 0 || N == 0) return RLK_OK;
  if (c == nullptr || ldc < N) {
    set_last_error("rlk_det_gemm_tree_bf16: output needs a non-null pointer and ldc >= N (ldc=%lld N=%d)",
                   (long long)ldc, N);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (K == 0) {
    hipError_t err = fill_zero_launch(c, M, N, ldc, 2, s);
    return err == hipSuccess ? RLK_OK : device_error("rlk_det_gemm_tree_bf16(fill)", err);
  }
  if (a == nullptr || b == nullptr) {
    set_last_error("rlk_det_gemm_tree_bf16: null operand");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  MatView A{reinterpret_cast<const bf16_bits*>(a), a_row_stride, a_k_stride, M};
  MatView B{reinterpret_cast<const bf16_bits*>(b), b_n_stride, b_k_stride, N};
  hipError_t err = det_gemm_tree_launch(A, B, c, ldc, M, N, K, config, s, leaf_space);
  if (err == hipErrorInvalidValue && (config == RLK_TREE_CFG_SKINNY || config == RLK_TREE_CFG_NODES)) {
    set_last_error(
        "rlk_det_gemm_tree_bf16: RLK_TREE_CFG_SKINNY needs M <= 16, K-contiguous 16-byte aligned operands and a tree "
        "of 4 to 12 levels whose leaves are equally long and a multiple of 8; RLK_TREE_CFG_NODES the same with any M "
        "and 4 to 10 levels (M=%d K=%d)", M, K);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  return err == hipSuccess ? RLK_OK : device_error("rlk_det_gemm_tree_bf16", err);
}

const char* rlk_det_gemm_seq_contract_id(void) { return "rlkernel.det_gemm.hip_seqfma32_gfx950.v1"; }

int rlk_det_gemm_seq(const void* a, int a_dtype, int64_t a_row_stride, int64_t a_k_stride, const void* b, int b_dtype,
                     int64_t b_k_stride, int64_t b_n_stride, void* c, int c_dtype, int64_t ldc, int M, int N, int K,
                     void* stream) {
  if (M < 0 || N < 0 || K < 0) {
    set_last_error("rlk_det_gemm_seq: negative size M=%d N=%d K=%d", M, N, K);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  auto operand_ok = [](int dtype) { return dtype == RLK_DTYPE_BF16 || dtype == RLK_DTYPE_FP32; };
  if (!operand_ok(a_dtype) || !operand_ok(b_dtype) || !operand_ok(c_dtype)) {
    set_last_error("rlk_det_gemm_seq: operands and output must be bf16 or fp32 (a=%d b=%d c=%d)", a_dtype, b_dtype,
                   c_dtype);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (a_row_stride < 0 || a_k_stride < 0 || b_k_stride < 0 || b_n_stride < 0) {
    set_last_error("rlk_det_gemm_seq: operands must not use negative strides");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (M == 0 || N == 0) return RLK_OK;
  if (c == nullptr || ldc < N) {
    set_last_error("rlk_det_gemm_seq: output needs a non-null pointer and ldc >= N (ldc=%lld N=%d)", (long long)ldc, N);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bool out_bf16 = c_dtype == RLK_DTYPE_BF16;
  if (K == 0) {
    hipError_t err = fill_zero_launch(c, M, N, ldc, out_bf16 ? 2 : 4, s);
    return err == hipSuccess ? RLK_OK : device_error("rlk_det_gemm_seq(fill)", err);
  }
  if (a == nullptr || b == nullptr) {
    set_last_error("rlk_det_gemm_seq: null operand");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  SeqOperand A{a, a_row_stride, a_k_stride};
  SeqOperand B{b, b_n_stride, b_k_stride};
  hipError_t err = det_gemm_seq_launch(A, a_dtype == RLK_DTYPE_FP32, B, b_dtype == RLK_DTYPE_FP32, c, ldc, M, N, K,
                                       out_bf16, s);
  return err == hipSuccess ? RLK_OK : device_error("rlk_det_gemm_seq", err);
}

const char* rlk_linear_logp_contract_id(void) { return "rlkernel.linear_logp.hip_streams16x256_split1024_gfx950.v1"; }

int rlk_linear_logp_split_count(int V) { return V > 0 ? linear_logp_split_count(V) : 0; }

size_t rlk_linear_logp_workspace_bytes(int T, int V) {
  if (T <= 0 || V <= 0) return 0;
  return linear_logp_workspace_bytes(T, V);
}

static int linear_logp_fwd_checked(const char* who, const void* hidden, int64_t h_row_stride, const void* weight,
                                   int64_t w_row_stride, const int64_t* target, const float* bias,
                                   const float* temperature, float* logp, float* lse, float* target_logit,
                                   void* workspace, size_t workspace_bytes, int T, int D, int V, int64_t vocab_start,
                                   int real_vocab_end, int config, void* stream, float* logits = nullptr,
                                   int64_t logits_row_stride = 0) {
  if (T < 0 || D <= 0 || V <= 0) {
    set_last_error("%s: bad sizes T=%d D=%d V=%d", who, T, D, V);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (real_vocab_end <= 0 || real_vocab_end > V) {
    set_last_error("%s: real_vocab_end must be in [1, %d], got %d", who, V, real_vocab_end);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (config < 0 || (config & ~RLK_LOGP_CFG_FORCE_STAGED) >= RLK_LOGP_CFG_COUNT) {
    set_last_error("%s: unknown config %d", who, config);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (T == 0) return RLK_OK;
  if (hidden == nullptr || weight == nullptr || target == nullptr) {
    set_last_error("%s: null hidden / weight / target", who);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (h_row_stride < D || w_row_stride < D) {
    set_last_error("%s: row strides must be >= D", who);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (logits != nullptr && logits_row_stride < V) {
    set_last_error("%s: logits row stride must be >= V", who);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  const size_t need = linear_logp_workspace_bytes(T, V);
  if (workspace == nullptr || workspace_bytes < need) {
    set_last_error("%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  MatView H{reinterpret_cast<const bf16_bits*>(hidden), h_row_stride, 1, T};
  MatView W{reinterpret_cast<const bf16_bits*>(weight), w_row_stride, 1, V};
  hipError_t err = linear_logp_launch(H, W, target, bias, temperature, logp, lse, target_logit, logits,
                                      logits_row_stride, reinterpret_cast<float*>(workspace), T, D, V, vocab_start,
                                      real_vocab_end, config, reinterpret_cast<hipStream_t>(stream));
  return err == hipSuccess ? RLK_OK : device_error(who, err);
}

int rlk_linear_logp_fwd(const void* hidden, int64_t h_row_stride, const void* weight, int64_t w_row_stride,
                        const int64_t* target, const float* bias, const float* temperature, float* logp,
                        float* lse, void* workspace, size_t workspace_bytes, int T, int D, int V,
                        int64_t vocab_start, int real_vocab_end, int config, void* stream) {
  return linear_logp_fwd_checked("rlk_linear_logp_fwd", hidden, h_row_stride, weight, w_row_stride, target, bias,
                                 temperature, logp, lse, nullptr, workspace, workspace_bytes, T, D, V, vocab_start,
                                 real_vocab_end, config, stream);
}

int rlk_linear_logp_fwd_logits(const void* hidden, int64_t h_row_stride, const void* weight, int64_t w_row_stride,
                               const int64_t* target, const float* bias, const float* temperature, float* logp,
                               float* lse, float* logits, int64_t logits_row_stride, void* workspace,
                               size_t workspace_bytes, int T, int D, int V, int64_t vocab_start, int real_vocab_end,
                               int config, void* stream) {
  if (logits == nullptr && T > 0) {
    set_last_error("rlk_linear_logp_fwd_logits: null logits (use rlk_linear_logp_fwd when they are not wanted)");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  return linear_logp_fwd_checked("rlk_linear_logp_fwd_logits", hidden, h_row_stride, weight, w_row_stride, target,
                                 bias, temperature, logp, lse, nullptr, workspace, workspace_bytes, T, D, V,
                                 vocab_start, real_vocab_end, config, stream, logits, logits_row_stride);
}

int rlk_linear_logp_fwd_shard(const void* hidden, int64_t h_row_stride, const void* weight, int64_t w_row_stride,
                              const int64_t* target, const float* bias, const float* temperature,
                              float* target_logit, float* lse, void* workspace, size_t workspace_bytes, int T,
                              int D, int V, int64_t vocab_start, int real_vocab_end, int config, void* stream) {
  return linear_logp_fwd_checked("rlk_linear_logp_fwd_shard", hidden, h_row_stride, weight, w_row_stride, target,
                                 bias, temperature, nullptr, lse, target_logit, workspace, workspace_bytes, T, D, V,
                                 vocab_start, real_vocab_end, config, stream);
}

int rlk_linear_logp_fwd_noalloc(const void* hidden, int64_t h_row_stride, const void* weight, int64_t w_row_stride,
                                const int64_t* target, const float* bias, const float* temperature, float* logp,
                                float* lse, int T, int D, int V, int64_t vocab_start, int real_vocab_end, int config,
                                void* stream) {
  const size_t need = (T > 0 && V > 0) ? linear_logp_workspace_bytes(T, V) : 0;
  if (need > (size_t)RLK_NOALLOC_SCRATCH_BYTES) {
    set_last_error(
        "rlk_linear_logp_fwd_noalloc: T=%d tokens x V=%d vocabulary rows need %zu bytes of partials, the built-in "
        "scratch holds %zu; use rlk_linear_logp_fwd with a workspace",
        T, V, need, (size_t)RLK_NOALLOC_SCRATCH_BYTES);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  void* ptr = nullptr;
  hipError_t err = scratch_for_current_device(&ptr);
  if (err != hipSuccess) return device_error("rlk_linear_logp_fwd_noalloc(scratch lookup)", err);
  // Every partial a call reads was written by that call's own kernels first, so nothing left in the
  // scratch by an earlier (larger) call needs clearing.
  return linear_logp_fwd_checked("rlk_linear_logp_fwd_noalloc", hidden, h_row_stride, weight, w_row_stride, target,
                                 bias, temperature, logp, lse, nullptr, ptr, (size_t)RLK_NOALLOC_SCRATCH_BYTES, T, D,
                                 V, vocab_start, real_vocab_end, config, stream);
}

size_t rlk_linear_logp_bwd_workspace_bytes(int T, int V, int with_bias) {
  if (T <= 0 || V <= 0) return 0;
  return linear_logp_bwd_workspace_bytes(T, V, with_bias != 0);
}

int rlk_linear_logp_bwd(const void* hidden, int64_t h_row_stride, const void* weight, int64_t w_row_stride,
                        const int64_t* target, const float* bias, const float* temperature, const float* lse,
                        const float* grad_logp, const float* grad_lse, void* grad_hidden, int64_t gh_row_stride,
                        void* grad_weight, int64_t gw_row_stride, float* grad_bias, void* workspace,
                        size_t workspace_bytes, int T, int D, int V, int64_t vocab_start, int real_vocab_end,
                        int config, void* stream) {
  if (T < 0 || D <= 0 || V <= 0) {
    set_last_error("rlk_linear_logp_bwd: bad sizes T=%d D=%d V=%d", T, D, V);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (real_vocab_end <= 0 || real_vocab_end > V) {
    set_last_error("rlk_linear_logp_bwd: real_vocab_end must be in [1, %d], got %d", V, real_vocab_end);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (config < 0 || (config & ~RLK_LOGP_CFG_FORCE_STAGED) >= RLK_LOGP_CFG_COUNT) {
    set_last_error("rlk_linear_logp_bwd: unknown config %d", config);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if ((grad_hidden && gh_row_stride < D) || (grad_weight && gw_row_stride < D)) {
    set_last_error("rlk_linear_logp_bwd: gradient row strides must be >= D");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (T > 0) {
    if (hidden == nullptr || weight == nullptr || target == nullptr || lse == nullptr) {
      set_last_error("rlk_linear_logp_bwd: null hidden / weight / target / lse");
      return RLK_ERR_INVALID_ARGUMENT;
    }
    if (h_row_stride < D || w_row_stride < D) {
      set_last_error("rlk_linear_logp_bwd: row strides must be >= D");
      return RLK_ERR_INVALID_ARGUMENT;
    }
  }
  if (T == 0) {
    // No tokens: the token-summed gradients are zero.
    hipError_t err = hipSuccess;
    if (grad_weight) err = fill_zero_launch(grad_weight, V, D, gw_row_stride, 2, s);
    if (err == hipSuccess && grad_bias) err = fill_zero_launch(grad_bias, 1, V, V, 4, s);
    return err == hipSuccess ? RLK_OK : device_error("rlk_linear_logp_bwd", err);
  }
  const size_t need = linear_logp_bwd_workspace_bytes(T, V, grad_bias != nullptr);
  if (workspace == nullptr || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0) {
    set_last_error("rlk_linear_logp_bwd: 256-byte aligned workspace of %zu bytes needed, %zu given", need,
                   workspace_bytes);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  MatView H{reinterpret_cast<const bf16_bits*>(hidden), h_row_stride, 1, T};
  MatView W{reinterpret_cast<const bf16_bits*>(weight), w_row_stride, 1, V};
  hipError_t err = linear_logp_bwd_launch(H, W, target, bias, temperature, lse, grad_logp, grad_lse, grad_hidden,
                                          gh_row_stride, grad_weight, gw_row_stride, grad_bias, workspace, T, D, V,
                                          vocab_start, real_vocab_end, config, s);
  return err == hipSuccess ? RLK_OK : device_error("rlk_linear_logp_bwd", err);
}

static int check_logits_args(const char* what, const void* logits, int dtype, int64_t row_stride, int T, int64_t V,
                             int64_t vocab_start, int64_t real_vocab) {
  if (T < 0 || V <= 0 || V > 0x7fffffff) {
    set_last_error("%s: bad sizes T=%d V=%lld", what, T, (long long)V);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (dtype != RLK_DTYPE_BF16 && dtype != RLK_DTYPE_FP16 && dtype != RLK_DTYPE_FP32) {
    set_last_error("%s: logits must be float16, bfloat16, or float32", what);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (vocab_start < 0 || real_vocab <= 0) {
    set_last_error("%s: invalid vocabulary metadata", what);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (T > 0 && (logits == nullptr || row_stride < V)) {
    set_last_error("%s: null logits or row stride < V", what);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  return RLK_OK;
}

int rlk_logits_tile_stats(const void* logits, int dtype, int64_t row_stride, const float* temperature, int T,
                          int64_t V, int64_t vocab_start, int64_t real_vocab, int num_tiles, float* tile_max,
                          float* tile_sum, void* stream) {
  int rc = check_logits_args("rlk_logits_tile_stats", logits, dtype, row_stride, T, V, vocab_start, real_vocab);
  if (rc != RLK_OK) return rc;
  if (num_tiles <= 0 || num_tiles > 65535 || V % num_tiles != 0) {
    set_last_error("rlk_logits_tile_stats: local_vocab must be divisible by num_tiles (1..65535)");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (T == 0) return RLK_OK;
  if (tile_max == nullptr || tile_sum == nullptr) {
    set_last_error("rlk_logits_tile_stats: null output");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  hipError_t err = logits_tile_stats_launch(logits, dtype, row_stride, nullptr, temperature, T, V, vocab_start,
                                            real_vocab, num_tiles, tile_max, tile_sum, nullptr, num_tiles, 1,
                                            reinterpret_cast<hipStream_t>(stream));
  return err == hipSuccess ? RLK_OK : device_error("rlk_logits_tile_stats", err);
}

const char* rlk_logits_logp_contract_id(void) { return "rlkernel.logits_logp.hip_tiles_x16lanes_gfx950.v2"; }

size_t rlk_logp_from_logits_workspace_bytes(int T, int num_tiles) {
  if (T <= 0 || num_tiles <= 0) return 0;
  return (size_t)3 * (size_t)num_tiles * (size_t)T * sizeof(float);
}

int rlk_logp_from_logits(const void* logits, int dtype, int64_t row_stride, const int64_t* target,
                         const float* temperature, int T, int64_t V, int64_t vocab_start, int64_t real_vocab,
                         int num_tiles, float* logp, float* lse, void* workspace, size_t workspace_bytes,
                         void* stream) {
  int rc = check_logits_args("rlk_logp_from_logits", logits, dtype, row_stride, T, V, vocab_start, real_vocab);
  if (rc != RLK_OK) return rc;
  if (num_tiles <= 0 || num_tiles > 65535 || V % num_tiles != 0) {
    set_last_error("rlk_logp_from_logits: local_vocab must be divisible by num_tiles (1..65535)");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (T == 0) return RLK_OK;
  if (target == nullptr) {
    set_last_error("rlk_logp_from_logits: null target");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  const size_t need = rlk_logp_from_logits_workspace_bytes(T, num_tiles);
  if (workspace == nullptr || workspace_bytes < need) {
    set_last_error("rlk_logp_from_logits: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  float* part = reinterpret_cast<float*>(workspace);
  const int64_t plane = (int64_t)num_tiles * T;
  hipError_t err = logits_tile_stats_launch(logits, dtype, row_stride, target, temperature, T, V, vocab_start,
                                            real_vocab, num_tiles, part, part + plane, part + 2 * plane, 1, T, s);
  if (err == hipSuccess) err = linear_logp_merge_launch(part, logp, lse, nullptr, T, num_tiles, false, s);
  return err == hipSuccess ? RLK_OK : device_error("rlk_logp_from_logits", err);
}

int rlk_logits_logp_backward(const void* logits, int dtype, int64_t row_stride, const float* lse,
                             const float* coef_logp, const float* coef_lse, const int64_t* target_local,
                             const float* temperature, void* grad, int64_t grad_row_stride, int T, int64_t V,
                             int64_t vocab_start, int64_t real_vocab, void* stream) {
  int rc = check_logits_args("rlk_logits_logp_backward", logits, dtype, row_stride, T, V, vocab_start, real_vocab);
  if (rc != RLK_OK) return rc;
  if (T == 0) return RLK_OK;
  if (lse == nullptr || coef_logp == nullptr || target_local == nullptr || grad == nullptr || grad_row_stride < V) {
    set_last_error("rlk_logits_logp_backward: null lse / coef_logp / target_local / grad, or grad row stride < V");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  hipError_t err = logits_backward_launch(logits, dtype, row_stride, lse, coef_logp, coef_lse, target_local,
                                          temperature, grad, grad_row_stride, T, V, vocab_start, real_vocab,
                                          reinterpret_cast<hipStream_t>(stream));
  return err == hipSuccess ? RLK_OK : device_error("rlk_logits_logp_backward", err);
}

static bool activation_dtype_ok(int dtype) {
  return dtype == RLK_DTYPE_BF16 || dtype == RLK_DTYPE_FP16 || dtype == RLK_DTYPE_FP32;
}

int rlk_swiglu_fwd(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, void* y, int64_t ld_y, int rows,
                   int cols, int dtype, void* stream) {
  if (rows < 0 || cols < 0) {
    set_last_error("rlk_swiglu_fwd: negative sizes");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (!activation_dtype_ok(dtype)) {
    set_last_error("rlk_swiglu_fwd: unknown dtype %d", dtype);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (rows == 0 || cols == 0) return RLK_OK;
  if (gate == nullptr || up == nullptr || y == nullptr || ld_gate < cols || ld_up < cols || ld_y < cols) {
    set_last_error("rlk_swiglu_fwd: null operand or row stride < cols");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  hipError_t err = swiglu_launch(gate, ld_gate, up, ld_up, nullptr, 0, y, ld_y, nullptr, 0, rows, cols, false, dtype,
                                 reinterpret_cast<hipStream_t>(stream));
  return err == hipSuccess ? RLK_OK : device_error("rlk_swiglu_fwd", err);
}

int rlk_swiglu_bwd(const void* dy, int64_t ld_dy, const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                   void* d_gate, int64_t ld_d_gate, void* d_up, int64_t ld_d_up, int rows, int cols, int dtype,
                   void* stream) {
  if (rows < 0 || cols < 0) {
    set_last_error("rlk_swiglu_bwd: negative sizes");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (!activation_dtype_ok(dtype)) {
    set_last_error("rlk_swiglu_bwd: unknown dtype %d", dtype);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (rows == 0 || cols == 0) return RLK_OK;
  if (dy == nullptr || gate == nullptr || up == nullptr || d_gate == nullptr || d_up == nullptr || ld_dy < cols ||
      ld_gate < cols || ld_up < cols || ld_d_gate < cols || ld_d_up < cols) {
    set_last_error("rlk_swiglu_bwd: null operand or row stride < cols");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  hipError_t err = swiglu_launch(gate, ld_gate, up, ld_up, dy, ld_dy, d_gate, ld_d_gate, d_up, ld_d_up, rows, cols,
                                 true, dtype, reinterpret_cast<hipStream_t>(stream));
  return err == hipSuccess ? RLK_OK : device_error("rlk_swiglu_bwd", err);
}

size_t rlk_det_gemm_swiglu_workspace_bytes(const void* a, int64_t a_row_stride, const void* w_packed,
                                           int64_t w_row_stride, int M, int I, int K) {
  if (M <= 0 || I <= 0 || K <= 0) return 0;
  MatView X{reinterpret_cast<const bf16_bits*>(a), a_row_stride, 1, M};
  MatView W{reinterpret_cast<const bf16_bits*>(w_packed), w_row_stride, 1, 2 * I};
  return det_gemm_swiglu_fused_supported(W, X, M, K) ? 0 : (size_t)M * 2 * (size_t)I * sizeof(bf16_bits);
}

int rlk_det_gemm_swiglu_bf16(const void* a, int64_t a_row_stride, const void* w_packed, int64_t w_row_stride,
                             void* y, int64_t ldy, void* workspace, size_t workspace_bytes, int M, int I, int K,
                             void* stream) {
  if (M < 0 || I < 0 || K < 0 || I > 0x3fffffff) {
    set_last_error("rlk_det_gemm_swiglu_bf16: bad sizes M=%d I=%d K=%d", M, I, K);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (M == 0 || I == 0) return RLK_OK;
  if (y == nullptr || ldy < I) {
    set_last_error("rlk_det_gemm_swiglu_bf16: null output or ldy < I");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (K == 0) {  // both projections are zero and swiglu(0, 0) = 0
    hipError_t err = fill_zero_launch(y, M, I, ldy, 2, s);
    return err == hipSuccess ? RLK_OK : device_error("rlk_det_gemm_swiglu_bf16(fill)", err);
  }
  if (a == nullptr || w_packed == nullptr || a_row_stride < K || w_row_stride < K) {
    set_last_error("rlk_det_gemm_swiglu_bf16: null operand or row stride < K");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  const size_t need = rlk_det_gemm_swiglu_workspace_bytes(a, a_row_stride, w_packed, w_row_stride, M, I, K);
  if (need > 0 && (workspace == nullptr || workspace_bytes < need)) {
    set_last_error("rlk_det_gemm_swiglu_bf16: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  MatView X{reinterpret_cast<const bf16_bits*>(a), a_row_stride, 1, M};
  MatView W{reinterpret_cast<const bf16_bits*>(w_packed), w_row_stride, 1, 2 * I};
  hipError_t err = det_gemm_swiglu_launch(W, X, y, ldy, workspace, M, I, K, s);
  return err == hipSuccess ? RLK_OK : device_error("rlk_det_gemm_swiglu_bf16", err);
}

size_t rlk_grpo_workspace_bytes(int rollouts) { return rollouts > 0 ? (size_t)3 * rollouts * sizeof(float) : 0; }

int rlk_grpo_ratio_kl_loss(const float* logp, const float* old_logp, const float* ref_logp,
                           const float* advantages, const uint8_t* mask, int rollouts, int tokens_per_rollout,
                           float clip_eps, float beta, float* ratio, float* k3, float* out3, void* workspace,
                           size_t workspace_bytes, void* stream) {
  if (rollouts < 0 || tokens_per_rollout < 0) {
    set_last_error("rlk_grpo_ratio_kl_loss: negative sizes");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (out3 == nullptr) {
    set_last_error("rlk_grpo_ratio_kl_loss: out3 is required");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (rollouts > 0 && (logp == nullptr || old_logp == nullptr || ref_logp == nullptr || advantages == nullptr)) {
    set_last_error("rlk_grpo_ratio_kl_loss: null input");
    return RLK_ERR_INVALID_ARGUMENT;
  }
  if (rollouts > 0 && (workspace == nullptr || workspace_bytes < rlk_grpo_workspace_bytes(rollouts))) {
    set_last_error("rlk_grpo_ratio_kl_loss: workspace of %zu bytes needed, %zu given",
                   rlk_grpo_workspace_bytes(rollouts), workspace_bytes);
    return RLK_ERR_INVALID_ARGUMENT;
  }
  hipError_t err = grpo_launch(logp, old_logp, ref_logp, advantages, mask, rollouts, tokens_per_rollout, clip_eps,
                               beta, ratio, k3, out3, reinterpret_cast<float*>(workspace),
                               reinterpret_cast<hipStream_t>(stream));
  return err == hipSuccess ? RLK_OK : device_error("rlk_grpo_ratio_kl_loss", err);
}

}  // extern "C"
