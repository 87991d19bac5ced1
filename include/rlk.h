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
  RLK_GEMM_CFG_STREAM16_DEEP = 8, /* M <= 16: 16-feature panel per workgroup streamed through a 128 KiB LDS ring */
  RLK_GEMM_CFG_STREAM16 = 9,      /* M <= 16: same with a 64 KiB ring, two workgroups per CU */
  RLK_GEMM_CFG_256x64 = 10,
  RLK_GEMM_CFG_64x64_DEEP = 11,   /* 64x64 tile, 256 K values per barrier pair (few, long tiles) */
  RLK_GEMM_CFG_128x64_DEEP = 12,  /* 128x64 tile, 128 K values per barrier pair */
  RLK_GEMM_CFG_128x128_DEEP = 13, /* 128x128 tile, 128 K values per barrier pair */
  RLK_GEMM_CFG_STREAM64 = 14,     /* M <= 64: 16-feature panels streamed through an LDS ring, one consumer wave per 16 tokens */
  RLK_GEMM_CFG_256x256_SOLO = 15, /* 256 x 256 tile on four waves (one per SIMD, 128 x 128 each) */
  RLK_GEMM_CFG_192x256 = 16,      /* 192 features x 256 tokens (N / 192 tiles where N / 256 leaves a round half empty) */
  RLK_GEMM_CFG_SHORTK = 17,       /* K <= 256, K-major token operand: features stationary in registers, tokens streamed */
  RLK_GEMM_CFG_192x128 = 18,      /* 192 features x 128 tokens, three stages (N / 192 x M / 128 tiles that fill one round) */
  RLK_GEMM_CFG_COUNT = 19,
  /* OR-ed into a configuration: use the register-staged main loop even where the
   * direct-to-LDS ping-pong loop applies. Bit-neutral; exists so tests can
   * compare the two loops. */
  RLK_GEMM_CFG_FORCE_STAGED = 0x100
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
 * are accepted. Fast paths, per operand: reduction axis contiguous (a_k_stride == 1;
 * b_k_stride == 1, the native [N,K] linear weight) with K % 8 == 0 and row strides
 * % 8 == 0; or, when K % 64 == 0, the other axis contiguous (a_row_stride == 1 with
 * M % 8 == 0, the transposed operand of a weight gradient; b_n_stride == 1 with
 * N % 8 == 0, a plain B[K,N]) with k strides % 8 == 0. Bases 16-byte aligned. Other
 * layouts run a slower element loader with identical results.
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

/*
 * C[M,N] = A[M,K] @ B[K,N] under the k-tree contract (rlk_det_gemm_tree_contract_id):
 *   T(lo,hi) = bf16(sum of a_k*b_k, k = lo..hi-1, fp32 from +0, k ascending, fused multiply-add)
 *              when hi - lo <= 32, else bf16(float(T(lo,mid)) + float(T(mid,hi))) with
 *              mid = lo + (hi - lo) / 2;  C = T(0, K).
 * Rounding points depend on K only: rows are batch invariant, and a K range that is a subtree
 * (the contiguous half, quarter, ... of a K-sharded rank) evaluates to exactly that node.
 * Strides as in rlk_det_gemm_bf16; any non-negative strides are accepted (no fast layout:
 * a leaf is a chain of single fp32 multiply-adds, which runs on the fp32 matrix pipe one k at a
 * time or on the vector ALU, about ten times slower than the bf16 MFMA contract). bf16 output only.
 *
 * Stands in for the reference's "triton_tree" backend: _triton_tree_gemm and its tree plan
 * (rl_engine/backends/shared/triton/gemm/det_gemm.py:218-258, 355-417, 514-546), the CUDA
 * k_tree_naive kernel (csrc/cuda/gemm/det_gemm_kernel.cu:74-85) and the specification the
 * reference's tests evaluate (tests/ops/gemm/test_det_gemm.py:156-168).
 */
int rlk_det_gemm_tree_bf16(const void* a, int64_t a_row_stride, int64_t a_k_stride, const void* b,
                           int64_t b_k_stride, int64_t b_n_stride, void* c, int64_t ldc, int M, int N, int K,
                           void* stream);

/* Leaf loops of the k-tree kernel. Both compute every bit of the contract; exposed so tests can
 * prove that. No counterpart in the reference. */
typedef enum rlk_tree_config {
  RLK_TREE_CFG_AUTO = 0,
  RLK_TREE_CFG_VALU = 1,     /* one v_fma_f32 per term */
  RLK_TREE_CFG_MFMA_F32 = 2, /* one v_mfma_f32_16x16x1_4b_f32 per k (reduction length one: a single fused step) */
  RLK_TREE_CFG_SKINNY = 3,   /* up to 16 rows: the 16 tree nodes at depth 4 on 16 waves, folded in tree order;
                                needs K-contiguous aligned operands and equal leaves, else invalid argument */
  RLK_TREE_CFG_NODES = 4,    /* any row count: 16 rows x 64 columns per workgroup, the 8 depth-3 nodes on 8 waves
                                (fp32 MFMA, each wave streams its own leaves through LDS); same eligibility as
                                SKINNY but trees of 4 to 10 levels and row strides below 2^24 elements. What
                                RLK_TREE_CFG_AUTO picks whenever it is eligible */
  RLK_TREE_CFG_COUNT = 5,
  /* OR-ed into RLK_TREE_CFG_AUTO or RLK_TREE_CFG_MFMA_F32: the leaf-space split, a different contract
   * (rlk_det_gemm_tree_leaf_space_contract_id). */
  RLK_TREE_CFG_LEAF_SPACE = 0x100
} rlk_tree_config;

/*
 * Contract id of the k-tree with the midpoint split in LEAF space (RLK_TREE_CFG_LEAF_SPACE): the leaves are the
 * fixed K tiles [32 i, min(32 i + 32, K)), each summed as above, and a node over leaves [lo, hi) is
 * bf16(float(T(lo,mid)) + float(T(mid,hi))) with mid = lo + (hi - lo) / 2 counted in leaves. Same bits as the
 * element-space contract whenever K / 32 is a power of two (K = 1024, 4096); a different tree otherwise
 * (K = 12288: 384 leaves of 32 here, 512 leaves of 24 there).
 *
 * Stands in for the split of DetGemmTreeReferenceOp (rl_engine/reference/gemm/det_gemm.py:29-60) and of the SM90
 * kernel (csrc/cuda/gemm/det_gemm_kernel.cu:221-234, 351-379); a leaf here is the same chain of single fused
 * multiply-adds as in the element-space contract.
 */
const char* rlk_det_gemm_tree_leaf_space_contract_id(void);

/* rlk_det_gemm_tree_bf16 with an explicit leaf loop (rlk_tree_config). */
int rlk_det_gemm_tree_bf16_config(const void* a, int64_t a_row_stride, int64_t a_k_stride, const void* b,
                                  int64_t b_k_stride, int64_t b_n_stride, void* c, int64_t ldc, int M, int N,
                                  int K, int config, void* stream);

/* Contract id of rlk_det_gemm_tree_bf16 (the reference reports
 * "rlkernel.det_gemm.triton_tree_rocm.v1", rl_engine/backends/rocm/gemm/det_gemm.py:101-104). */
const char* rlk_det_gemm_tree_contract_id(void);

/* The configuration RLK_GEMM_CFG_AUTO resolves to for a shape (host only, no GPU call).
 * Stands in for select_config, rl_engine/backends/rocm/gemm/mfma_gemm.py:76-92. */
int rlk_det_gemm_pick_config(int M, int N, int K);

/* Token-tile configurations of the fused linear-LogP kernel (bit-neutral). */
typedef enum rlk_logp_config {
  RLK_LOGP_CFG_AUTO = 0,
  RLK_LOGP_CFG_256 = 1, /* 256 tokens per workgroup */
  RLK_LOGP_CFG_128 = 2,
  RLK_LOGP_CFG_64 = 3,
  RLK_LOGP_CFG_16 = 4,
  /* up to 1024 tokens: four workgroups per vocabulary split, four streams each (64 / 128 / 256-token tiles) */
  RLK_LOGP_CFG_64_STREAMS = 5,
  RLK_LOGP_CFG_128_STREAMS = 6,
  RLK_LOGP_CFG_256_STREAMS = 7,
  RLK_LOGP_CFG_COUNT = 8,
  /* OR-ed into a configuration: register-staged main loop instead of the
   * direct-to-LDS ping-pong loop (bit-neutral; for tests). */
  RLK_LOGP_CFG_FORCE_STAGED = 0x100
} rlk_logp_config;

/* Reduction contract identifier of the fused linear-LogP.
 * Stands in for TRITON_LINEAR_LOGP_CONTRACT_VERSION,
 * rl_engine/backends/shared/triton/logprob/linear_logp.py:273. */
const char* rlk_linear_logp_contract_id(void);

/* Number of fixed vocabulary splits for a local vocabulary of V rows: ceil(V / 1024),
 * a function of V only. Stands in for TRITON_N_SPLIT_CONTRACT / N_SPLIT_CONTRACT
 * (linear_logp.py:274; csrc/cuda/logprob/fused_linear_logp_sm90.cu:50, 2120-2124). */
int rlk_linear_logp_split_count(int V);

/* Bytes of fp32 partials rlk_linear_logp_fwd needs for T tokens and V vocabulary rows
 * (3 * splits * T floats; 17 times that for T <= 1024, where per-stream states are staged). */
size_t rlk_linear_logp_workspace_bytes(int T, int V);

/*
 * Fused lm_head GEMM -> fixed-order online log-sum-exp -> target gather.
 *   hidden  [T, D] bf16, row stride h_row_stride, unit stride along D
 *   weight  [V, D] bf16, row stride w_row_stride, unit stride along D (native lm_head layout)
 *   target  [T] int64 GLOBAL vocabulary ids; the local column is target - vocab_start
 *   bias    [V] fp32 or NULL;  temperature [T] fp32 (> 0) or NULL
 *   logp    [T] fp32 out (may be NULL): min(y_target - lse, 0)
 *   lse     [T] fp32 out (may be NULL)
 *   real_vocab_end: local column bound of the real vocabulary (columns >= it are
 *                   padding and contribute -inf / 0); pass V for "no padding".
 * A target outside [vocab_start, vocab_start + real_vocab_end) names no column of this
 * call: that row's logp is NaN (its lse is unaffected), so a caller that does not check
 * the range on the host beforehand (the reference's Python layer does, with a device
 * read-back, linear_logp.py:664-672) still sees the mistake in the result; likewise a
 * temperature that is not a positive number makes the row's logp and lse NaN.
 * rlk_linear_logp_fwd_shard, whose targets may belong to another shard, writes a target
 * logit of 0 for them instead. The full [T, V] logits are never written.
 *
 * Stands in for rl_engine._C.fused_linear_logp_sm90 (csrc/bindings/ops.cpp:514-526;
 * csrc/cuda/logprob/fused_linear_logp_sm90.cu:2040-2176), for
 * triton_deterministic_linear_logp (linear_logp.py:631-700) and for the ROCm route
 * DetGemmOp().linear + _C.hip_deterministic_logp_tile_stats
 * (rl_engine/integrations/common/linear_logp.py:1083-1102; csrc/bindings/ops.cpp:122-126).
 */
int rlk_linear_logp_fwd(const void* hidden, int64_t h_row_stride, const void* weight, int64_t w_row_stride,
                        const int64_t* target, const float* bias, const float* temperature, float* logp,
                        float* lse, void* workspace, size_t workspace_bytes, int T, int D, int V,
                        int64_t vocab_start, int real_vocab_end, int config, void* stream);

/*
 * rlk_linear_logp_fwd that also stores the logits, from the same pass (no second GEMM):
 *   logits [T, logits_row_stride >= V] fp32 out: the fp32 accumulators of the lm_head GEMM with the
 *          bias added and padded lanes (columns >= real_vocab_end) set to -inf, NOT scaled by the
 *          temperature. Bit for bit what rlk_det_gemm_bf16 with out_fp32 writes for hidden @ weight^T,
 *          plus the bias. logp and lse have the bits rlk_linear_logp_fwd gives.
 * Everything else as in rlk_linear_logp_fwd. HBM-bound on the T * V * 4 bytes it writes.
 *
 * Stands in for return_logits=True of rl_engine._C.fused_linear_logp_sm90 (csrc/bindings/ops.cpp:514-520;
 * csrc/cuda/logprob/fused_linear_logp_sm90.cu:2040-2176) and of triton_deterministic_linear_logp
 * (store_logits, rl_engine/backends/shared/triton/logprob/linear_logp.py:366-380, 693).
 */
int rlk_linear_logp_fwd_logits(const void* hidden, int64_t h_row_stride, const void* weight, int64_t w_row_stride,
                               const int64_t* target, const float* bias, const float* temperature, float* logp,
                               float* lse, float* logits, int64_t logits_row_stride, void* workspace,
                               size_t workspace_bytes, int T, int D, int V, int64_t vocab_start, int real_vocab_end,
                               int config, void* stream);

/*
 * The same pass for one shard of a vocabulary split over ranks: `weight` holds rows
 * [vocab_start, vocab_start + V) of the lm_head, `target` stays in global ids, and the
 * outputs are the two terms a caller merges across shards,
 *   target_logit [T] fp32 out (may be NULL): the scaled logit y_target (bias and
 *                temperature applied, not clamped) when this shard owns the target, else 0
 *   lse          [T] fp32 out (may be NULL): log-sum-exp over this shard's real columns
 * so that logp = sum_shards(target_logit) - log(sum_shards(exp(lse))). With one shard,
 * min(target_logit - lse, 0) is bit-for-bit rlk_linear_logp_fwd's logp. Workspace, configs,
 * order of summation and errors are those of rlk_linear_logp_fwd.
 *
 * Stands in for rl_engine._C.fused_linear_logp_sm90_global_target
 * (csrc/bindings/ops.cpp:522-526; csrc/cuda/logprob/fused_linear_logp_sm90.cu:2169-2176),
 * whose caller merges the pair in _merge_tp_local_logp
 * (rl_engine/backends/cuda/logprob/linear_logp.py:711-740).
 */
int rlk_linear_logp_fwd_shard(const void* hidden, int64_t h_row_stride, const void* weight, int64_t w_row_stride,
                              const int64_t* target, const float* bias, const float* temperature,
                              float* target_logit, float* lse, void* workspace, size_t workspace_bytes, int T,
                              int D, int V, int64_t vocab_start, int real_vocab_end, int config, void* stream);

/* Size of the scratch array built into the library for rlk_linear_logp_fwd_noalloc (32 MiB per GPU). */
#define RLK_NOALLOC_SCRATCH_BYTES (32u << 20)

/*
 * rlk_linear_logp_fwd for callers that cannot allocate device memory or pass a workspace: code
 * under HIP-graph capture, tight serving loops, harnesses that forbid hipMalloc. Same inputs,
 * outputs, checks, kernels and result bits as rlk_linear_logp_fwd; the fp32 partials go into a
 * scratch array that is part of the loaded library (RLK_NOALLOC_SCRATCH_BYTES of device memory per
 * GPU, held until the process ends) instead of a caller workspace. The call allocates and frees
 * nothing and calls no allocating routine. It serves every (T, V) with
 * rlk_linear_logp_workspace_bytes(T, V) <= RLK_NOALLOC_SCRATCH_BYTES (V = 151936: up to 1024
 * tokens, and 1025 ... 18765 tokens, whose partials are 17 times smaller per token) and returns
 * RLK_ERR_INVALID_ARGUMENT beyond that. All calls on one GPU share that GPU's array: calls that
 * may overlap on one GPU (different streams, different host threads) race on it and must be
 * ordered by the caller. The first call on a device looks the array's address up once
 * (hipGetSymbolAddress), so make that call outside graph capture.
 *
 * No counterpart in the reference: it exists for the callers named above.
 */
int rlk_linear_logp_fwd_noalloc(const void* hidden, int64_t h_row_stride, const void* weight, int64_t w_row_stride,
                                const int64_t* target, const float* bias, const float* temperature, float* logp,
                                float* lse, int T, int D, int V, int64_t vocab_start, int real_vocab_end, int config,
                                void* stream);

/* Bytes of workspace rlk_linear_logp_bwd needs: the bf16 d(logits) [T, V rounded up to 64]
 * plus, when a bias gradient is wanted, fp32 column sums per token tile
 * ([ceil(T / 16), V] up to 1024 tokens, [ceil(T / 64), V] above). */
size_t rlk_linear_logp_bwd_workspace_bytes(int T, int V, int with_bias);

/*
 * Backward of rlk_linear_logp_fwd. Inputs as in the forward, plus
 *   lse        [T] fp32: the forward's result for the same inputs
 *   grad_logp  [T] fp32 or NULL (zero);  grad_lse [T] fp32 or NULL (zero)
 * Outputs (each may be NULL when not wanted):
 *   grad_hidden [T, D] bf16, row stride gh_row_stride
 *   grad_weight [V, D] bf16, row stride gw_row_stride
 *   grad_bias   [V] fp32
 * With p = exp(y - lse) on the forward's scaled logits y (0 on padded lanes),
 *   d(logits) = (p * (grad_lse - grad_logp) + [column == target] * grad_logp) / temperature,
 * rounded once to bf16; grad_hidden = d(logits) @ weight over the vocabulary ascending,
 * grad_weight = d(logits)^T @ hidden over tokens ascending (both under the det_gemm
 * contract), grad_bias = column sums of the fp32 d(logits) BEFORE that rounding (as the
 * reference's chunked backward sums them), in a fixed tree over the token index inside
 * 256-token blocks, blocks added ascending. The clamp
 * logp = min(., 0) of the forward is not differentiated (gradient 1), as in the reference.
 * workspace must be 256-byte aligned.
 * grad_hidden is also scratch during the call: from 512 tokens on (T % 8 == 0, gh_row_stride == D,
 * 16-byte aligned) it first holds the transposed hidden states that the weight-gradient GEMM reads,
 * and receives its result last. It must not alias hidden, weight, or any other argument.
 *
 * Stands in for _DetTritonLinearLogpAutograd.backward and _det_reference_dlogits
 * (rl_engine/backends/shared/triton/logprob/linear_logp.py:522-570, 600-628) and for
 * chunked_linear_logp_backward (rl_engine/reference/logprob/linear_logp.py:642-715).
 */
int rlk_linear_logp_bwd(const void* hidden, int64_t h_row_stride, const void* weight, int64_t w_row_stride,
                        const int64_t* target, const float* bias, const float* temperature, const float* lse,
                        const float* grad_logp, const float* grad_lse, void* grad_hidden, int64_t gh_row_stride,
                        void* grad_weight, int64_t gw_row_stride, float* grad_bias, void* workspace,
                        size_t workspace_bytes, int T, int D, int V, int64_t vocab_start, int real_vocab_end,
                        int config, void* stream);

/* Element types of materialised logits. */
typedef enum rlk_dtype { RLK_DTYPE_BF16 = 0, RLK_DTYPE_FP16 = 1, RLK_DTYPE_FP32 = 2 } rlk_dtype;

/*
 * C[M,N] = A[M,K] @ B[K,N] with a strictly sequential fp32 chain (rlk_det_gemm_seq_contract_id):
 *   C[i,j] = fma(a[i,K-1], b[K-1,j], ... fma(a[i,1], b[1,j], fma(a[i,0], b[0,j], +0)) ...),
 * one fp32 fused multiply-add per k, k ascending, one accumulator per element, nothing rounded below fp32.
 * a_dtype / b_dtype / c_dtype are RLK_DTYPE_BF16 or RLK_DTYPE_FP32 (bf16 operands are widened exactly; a
 * bf16 output is the fp32 result rounded once). Strides in elements as in rlk_det_gemm_bf16, any
 * non-negative values. Rows are batch invariant. Runs on the fp32 matrix pipe, one reduction-length-one
 * MFMA per k (that instruction is a fused multiply-add on fp32 operands as well), at 120-135 TFLOP/s: the
 * fp32-result path of the strict GEMM, not a replacement for rlk_det_gemm_bf16.
 *
 * Stands in for _triton_gemm_fp32 / _det_gemm_fp32_kernel
 * (rl_engine/backends/shared/triton/gemm/det_gemm.py:680-749), i.e. DetGemmOp.forward_fp32 and
 * forward_accum_fp32 with bf16 or fp32 operands (rl_engine/backends/rocm/gemm/det_gemm.py:545-555), and for
 * rl_engine._C.det_gemm_fwd_fp32 / det_gemm_accum_fwd_fp32 (rl_engine/_C.pyi:244-248; csrc/musa/det_gemm.mu:25-48).
 */
int rlk_det_gemm_seq(const void* a, int a_dtype, int64_t a_row_stride, int64_t a_k_stride, const void* b, int b_dtype,
                     int64_t b_k_stride, int64_t b_n_stride, void* c, int c_dtype, int64_t ldc, int M, int N, int K,
                     void* stream);

/* Contract id of rlk_det_gemm_seq. */
const char* rlk_det_gemm_seq_contract_id(void);

/*
 * Per-row, per-tile statistics of materialised logits [T, V] (row stride in elements):
 * tile t covers columns [t * V / num_tiles, (t + 1) * V / num_tiles), cut at the real
 * vocabulary (global column vocab_start + c counts only while it is < real_vocab).
 *   tile_max [T, num_tiles] fp32: max of the tile (-inf for an all-padding tile)
 *   tile_sum [T, num_tiles] fp32: sum of exp(z - tile_max) (0 when tile_max is not finite)
 * temperature [T] fp32 or NULL scales the logits by 1 / temperature in registers first
 * (the scaling of rlk_linear_logp_fwd). V % num_tiles == 0.
 * A row's result depends on that row only.
 *
 * Stands in for rl_engine._C.hip_deterministic_logp_tile_stats
 * (csrc/bindings/ops.cpp:122-126; csrc/rocm/logprob/hip_deterministic_logp_kernel.hip:389-467, 550-588).
 */
int rlk_logits_tile_stats(const void* logits, int dtype, int64_t row_stride, const float* temperature, int T,
                          int64_t V, int64_t vocab_start, int64_t real_vocab, int num_tiles, float* tile_max,
                          float* tile_sum, void* stream);

/* Reduction contract identifier of rlk_logits_tile_stats / rlk_logp_from_logits (which lanes fold which
 * columns of a tile, and in which order the partial results merge). No counterpart in the reference, whose
 * tile-stats kernel documents no order beyond its tile boundaries
 * (csrc/rocm/logprob/hip_deterministic_logp_kernel.hip:389-467). */
const char* rlk_logits_logp_contract_id(void);

/* Bytes of workspace rlk_logp_from_logits needs. */
size_t rlk_logp_from_logits_workspace_bytes(int T, int num_tiles);

/*
 * Selected-token log-probabilities from materialised logits, without another GEMM:
 * tile statistics as above, tiles merged ascending (M = max_t m_t,
 * S = sum_t s_t * exp(m_t - M), lse = M + log S), target logit gathered in fp32,
 * logp = target * (1 / temperature) - lse. target holds GLOBAL ids; one outside
 * [vocab_start, vocab_start + V) or in the padding contributes a target logit of 0.
 *
 * Stands in for the ROCm branch of LinearLogpWrapper.from_local_logits
 * (rl_engine/integrations/common/linear_logp.py:750-815, 817-923), i.e.
 * _RocmVocabParallelLogprobFunction.forward + _merge_tile_partials
 * (rl_engine/backends/rocm/logprob/vocab_parallel_logp.py:308-352;
 * rl_engine/reference/logprob/vocab_parallel_logp.py:355-363) on one GPU.
 */
int rlk_logp_from_logits(const void* logits, int dtype, int64_t row_stride, const int64_t* target,
                         const float* temperature, int T, int64_t V, int64_t vocab_start, int64_t real_vocab,
                         int num_tiles, float* logp, float* lse, void* workspace, size_t workspace_bytes,
                         void* stream);

/*
 * d(logits) for logp / lse computed from materialised logits, in the dtype of the logits:
 *   grad[c] = coef_logp * ([c == target_local] - p_c) + coef_lse * p_c,  p_c = exp(y_c - lse)
 * with y = z * (1 / temperature) (and the result scaled by it once more), 0 on
 * padded columns, p = 0 on a row whose lse is not finite. coef_lse and temperature may be
 * NULL; target_local is the LOCAL column or -1.
 *
 * Stands in for rl_engine._C.hip_deterministic_logp_backward
 * (csrc/bindings/ops.cpp:127-135; hip_deterministic_logp_kernel.hip:472-540, 590-640).
 */
int rlk_logits_logp_backward(const void* logits, int dtype, int64_t row_stride, const float* lse,
                             const float* coef_logp, const float* coef_lse, const int64_t* target_local,
                             const float* temperature, void* grad, int64_t grad_row_stride, int T, int64_t V,
                             int64_t vocab_start, int64_t real_vocab, void* stream);

/*
 * SwiGLU on rows of element type `dtype` (rlk_dtype: bf16, fp16 or fp32; every tensor of a
 * call has it; strides in elements): y[m, c] = round((g * sigmoid(g)) * u) with
 * g = gate[m * ld_gate + c], u = up[m * ld_up + c] widened to fp32 and
 * sigmoid(g) = 1 / (1 + exp(-g)) (hardware reciprocal and exponential, each within 1 ulp);
 * one rounding to the element type. A packed [rows, 2 * cols] projection is the case
 * up = gate + cols, ld_gate = ld_up = 2 * cols.
 *
 * Stands in for rl_engine._C.swiglu_forward / swiglu_packed_forward
 * (csrc/bindings/ops.cpp:400-413; csrc/cuda/activation/activation.cu:62-75, 97-112).
 */
int rlk_swiglu_fwd(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up, void* y, int64_t ld_y, int rows,
                   int cols, int dtype, void* stream);

/*
 * Backward of rlk_swiglu_fwd: d_up = round(dy * silu(g)), d_gate = round(dy * u * silu'(g)),
 * silu'(g) = s * (1 + g * (1 - s)), s = sigmoid(g).
 *
 * Stands in for rl_engine._C.swiglu_backward / swiglu_packed_backward
 * (csrc/bindings/ops.cpp:404-419; activation.cu:77-95, 114-135).
 */
int rlk_swiglu_bwd(const void* dy, int64_t ld_dy, const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                   void* d_gate, int64_t ld_d_gate, void* d_up, int64_t ld_d_up, int rows, int cols, int dtype,
                   void* stream);

/* Bytes of workspace rlk_det_gemm_swiglu_bf16 needs for these operands: 0 when the fused
 * kernels apply (unit K strides, 16-byte aligned rows, K % 64 == 0, and M > 128 or M <= 16 with
 * K >= 1024), else the bf16 [M, 2 I] projection. */
size_t rlk_det_gemm_swiglu_workspace_bytes(const void* a, int64_t a_row_stride, const void* w_packed,
                                           int64_t w_row_stride, int M, int I, int K);

/*
 * y[M, I] = swiglu(a @ w_packed[0:I]^T, a @ w_packed[I:2I]^T): the packed gate/up projection
 * of a gated FFN (weight rows [0, I) gate, [I, 2 I) up, unit stride along K) under the
 * det_gemm contract, each projection rounded to bf16 before the activation, so the result
 * equals rlk_det_gemm_bf16 followed by rlk_swiglu_fwd bit for bit. When the fused kernel
 * applies the [M, 2 I] projection is never written.
 *
 * Stands in for rl_engine/backends/rocm/gemm/swiglu_gemm.py:36-86 (forward) and for
 * _packed_gate_up_inference (rl_engine/backends/rocm/ffn/ffn.py:69-83).
 */
int rlk_det_gemm_swiglu_bf16(const void* a, int64_t a_row_stride, const void* w_packed, int64_t w_row_stride,
                             void* y, int64_t ldy, void* workspace, size_t workspace_bytes, int M, int I, int K,
                             void* stream);

/* Bytes of workspace rlk_grpo_ratio_kl_loss needs. */
size_t rlk_grpo_workspace_bytes(int rollouts);

/*
 * GRPO epilogue on per-token log-probs (all fp32):
 *   ratio = exp(logp - old_logp);  d = ref_logp - logp;  k3 = exp(d) - d - 1
 *   term  = -min(ratio * A, clamp(ratio, 1 - clip_eps, 1 + clip_eps) * A)
 *   policy_loss = sum(term) / max(active, 1e-8);  kl = sum(k3) / max(active, 1e-8)
 *   loss = policy_loss + beta * kl          out3 = {loss, policy_loss, kl}
 * with masked entries (mask byte == 0) set to zero and excluded from the count.
 * logp/old/ref/ratio/k3 are [rollouts * tokens_per_rollout] sequence-major,
 * advantages is [rollouts]; mask, ratio and k3 may be NULL. Sums run per sequence
 * in a fixed tree, then over sequences ascending.
 *
 * Stands in for compute_policy_ratio / compute_reference_kl / masked_mean
 * (rl_engine/reference/definitions.py:50-106) and NativeGRPOLossOp.apply
 * (rl_engine/reference/loss/grpo_loss.py:96-125, 162-168).
 */
int rlk_grpo_ratio_kl_loss(const float* logp, const float* old_logp, const float* ref_logp,
                           const float* advantages, const uint8_t* mask, int rollouts, int tokens_per_rollout,
                           float clip_eps, float beta, float* ratio, float* k3, float* out3, void* workspace,
                           size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* RLK_H_ */
