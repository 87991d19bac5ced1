/*
 * rlk.h - C ABI of librlk_gfx950.so, the MI355X (gfx950) implementation of
 * RL-Kernel's batch-invariant dense path: deterministic bf16 GEMM, fused
 * linear-LogP and the GRPO ratio / k3-KL epilogue.
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer on the current HIP device unless the
 *     parameter name starts with "host_". The library never allocates, frees
 *     or synchronises: the caller owns every buffer, including workspaces.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *     All work is enqueued on it; the calls are HIP-graph capturable.
 *   - Return value: RLK_OK (0) or a negative rlk_status. After a failure
 *     rlk_last_error() returns a message for the calling thread.
 *   - bf16 values are raw 16-bit patterns (uint16_t), strides are in elements.
 *
 * Citations name the interface of the reference (ryankert01/RL-Kernel) that
 * each entry point stands in for.
 */
#ifndef RLK_H_
#define RLK_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum rlk_status {
  RLK_OK = 0,
  RLK_ERR_INVALID_ARGUMENT = -1, /* shape / stride / pointer contract violated */
  RLK_ERR_DEVICE = -2,           /* a HIP runtime call failed                  */
  RLK_ERR_UNSUPPORTED = -3       /* valid request this build does not serve    */
} rlk_status;

/* Tile configurations of the GEMM main loop. The choice never changes a result
 * bit; RLK_GEMM_CFG_AUTO picks by shape. Exposed so tests can prove that. */
typedef enum rlk_gemm_config {
  RLK_GEMM_CFG_AUTO = 0,
  RLK_GEMM_CFG_256x256 = 1,
  RLK_GEMM_CFG_256x128 = 2,
  RLK_GEMM_CFG_128x128 = 3,
  RLK_GEMM_CFG_128x64 = 4,
  RLK_GEMM_CFG_64x64 = 5,
  RLK_GEMM_CFG_64x16 = 6,
  RLK_GEMM_CFG_16x16 = 7,
  RLK_GEMM_CFG_COUNT = 8
} rlk_gemm_config;

/* Arithmetic contract identifier (provenance string).
 * Stands in for det_gemm_backend_id(), rl_engine/backends/rocm/gemm/det_gemm.py:101-105. */
const char* rlk_contract_id(void);

/* Library version string. */
const char* rlk_version(void);

/* Message of the last failure on the calling thread ("" if none). */
const char* rlk_last_error(void);

/*
 * C[M,N] = A[M,K] @ B[K,N], bf16 in, fp32 accumulate in fixed K order, one
 * rounding to bf16 (or fp32 output when out_fp32 != 0).
 *
 * A is addressed as a[m*a_row_stride + k*a_k_stride], B as
 * b[k*b_k_stride + n*b_n_stride], C as c[m*ldc + n]. Any non-negative strides
 * are accepted; the fast path needs a_k_stride == 1 and b_k_stride == 1 (the
 * native [N,K] linear weight), 16-byte aligned bases, K % 8 == 0 and row
 * strides % 8 == 0. Other layouts run a slower loader with identical results.
 * C must not alias A or B.
 *
 * One entry point serves rl_engine._C.det_gemm_fwd, det_gemm_fwd_rhs_transposed,
 * det_gemm_da, det_gemm_db and det_gemm_db_transposed
 * (csrc/bindings/ops.cpp:240-245, 706-719; csrc/cuda/gemm/det_gemm_kernel.cu:519-602)
 * and mfma_gemm (rl_engine/backends/rocm/gemm/mfma_gemm.py:293-373): the
 * variants differ only in which strides the caller passes.
 */
int rlk_det_gemm_bf16(const void* a, int64_t a_row_stride, int64_t a_k_stride, const void* b,
                      int64_t b_k_stride, int64_t b_n_stride, void* c, int64_t ldc, int M, int N, int K,
                      int out_fp32, int config, void* stream);

/* The configuration RLK_GEMM_CFG_AUTO resolves to for a shape (host only, no GPU call).
 * Stands in for select_config, rl_engine/backends/rocm/gemm/mfma_gemm.py:76-92. */
int rlk_det_gemm_pick_config(int M, int N, int K);

#ifdef __cplusplus
}
#endif

#endif /* RLK_H_ */
