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
  if (config < 0 || config >= RLK_GEMM_CFG_COUNT) {
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

}  // extern "C"
