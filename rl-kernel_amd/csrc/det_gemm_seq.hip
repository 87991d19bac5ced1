// det_gemm with a strictly sequential fp32 chain, for gfx950:
//
//   C[i, j] = fma(a[i, K-1], b[K-1, j], ... fma(a[i, 1], b[1, j], fma(a[i, 0], b[0, j], +0)) ...)
//
// one fp32 fused multiply-add per k, k ascending, a single accumulator per output element and no
// rounding below fp32. Operands are bf16 or fp32 (widened exactly), the result is stored as fp32 or
// rounded once to bf16. This is the chain a k-tree leaf is made of, run over the whole of K.
//
// Stands in for the reference's fp32-output strict GEMM, _triton_gemm_fp32 / _det_gemm_fp32_kernel
// (rl_engine/backends/shared/triton/gemm/det_gemm.py:680-749: inputs promoted to fp32, one output tile per
// program walking K in a fixed order, no split-K), which serves DetGemmOp.forward_fp32 /
// forward_accum_fp32 (rl_engine/backends/rocm/gemm/det_gemm.py:545-555), and for its native twin
// det_gemm_fwd_fp32 / det_gemm_accum_fwd_fp32 (csrc/musa/det_gemm.mu:25-48: float acc = 0, k ascending).
// With bf16 operands every product is exact in fp32, so the fused step equals multiply-then-add there.
//
// Vector ALU kernel: a workgroup owns a 64 x 128 output tile, a thread 4 rows x 8 columns (32 independent
// chains); K is walked in chunks of 32 staged in LDS as fp32 [k][row], the next chunk fetched while the
// current one is summed. Any non-negative strides. The row of a result depends on that row of A only.
#include "rlk_device.h"
#include "rlk_host.h"

namespace rlk {

constexpr int kSeqChunk = 32;
constexpr int kSeqBM = 64;
constexpr int kSeqBN = 128;
constexpr int kSeqThreads = 256;
constexpr int kSeqAStride = kSeqBM + 4;  // floats per k row (keeps 16-byte alignment, spreads banks)
constexpr int kSeqBStride = kSeqBN + 4;
constexpr int kSeqStageFloats = kSeqChunk * (kSeqAStride + kSeqBStride);
constexpr int kSeqALoads = kSeqBM * kSeqChunk / kSeqThreads;  // 8 elements per thread per chunk
constexpr int kSeqBLoads = kSeqBN * kSeqChunk / kSeqThreads;  // 16

template <bool F32>
__device__ __forceinline__ float seq_load(const void* base, int64_t index) {
  if constexpr (F32) {
    return reinterpret_cast<const float*>(base)[index];
  } else {
    return bf16_bits_to_float(reinterpret_cast<const bf16_bits*>(base)[index]);
  }
}

template <bool A_F32, bool B_F32, bool OUT_BF16>
__global__ __launch_bounds__(kSeqThreads, 2) void det_gemm_seq_kernel(SeqOperand A, SeqOperand B, void* __restrict__ C,
                                                                      int64_t ldc, int M, int N, int K, int tiles_m) {
  __shared__ __attribute__((aligned(16))) float stage[2][kSeqStageFloats];

  const int tid = threadIdx.x;
  const int tile_m = blockIdx.x % tiles_m;
  const int tile_n = blockIdx.x / tiles_m;
  const int m0 = tile_m * kSeqBM;
  const int n0 = tile_n * kSeqBN;
  const int tx = tid & 15;  // columns 4 tx .. 4 tx + 3 and 64 + 4 tx .. 64 + 4 tx + 3
  const int ty = tid >> 4;  // rows 4 ty .. 4 ty + 3

  // Loader role: element (row, k) with k = tid % 32, rows tid / 32 + 8 j. Rows past the edge are clamped to
  // the last valid row (their results are never stored); k past K reads index K - 1 and deposits zero.
  const int load_k = tid & 31;
  const int load_row = tid >> 5;
  const int a_last = M - 1 - m0, b_last = N - 1 - n0;
  float a_reg[kSeqALoads], b_reg[kSeqBLoads];
  auto fetch = [&](int k0) {
    const bool live = k0 + load_k < K;
    const int k = live ? k0 + load_k : K - 1;
#pragma unroll
    for (int j = 0; j < kSeqALoads; ++j) {
      const int row = load_row + 8 * j;
      const float v = seq_load<A_F32>(A.ptr, (int64_t)(m0 + (row < a_last ? row : a_last)) * A.row_stride + (int64_t)k * A.k_stride);
      a_reg[j] = live ? v : 0.f;
    }
#pragma unroll
    for (int j = 0; j < kSeqBLoads; ++j) {
      const int row = load_row + 8 * j;
      const float v = seq_load<B_F32>(B.ptr, (int64_t)(n0 + (row < b_last ? row : b_last)) * B.row_stride + (int64_t)k * B.k_stride);
      b_reg[j] = live ? v : 0.f;
    }
  };
  auto deposit = [&](int buf) {
    float* as = stage[buf];
    float* bs = as + kSeqChunk * kSeqAStride;
#pragma unroll
    for (int j = 0; j < kSeqALoads; ++j) as[load_k * kSeqAStride + load_row + 8 * j] = a_reg[j];
#pragma unroll
    for (int j = 0; j < kSeqBLoads; ++j) bs[load_k * kSeqBStride + load_row + 8 * j] = b_reg[j];
  };

  float acc[4][8];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = 0.f;

  fetch(0);
  deposit(0);
  __syncthreads();
  const int chunks = (K + kSeqChunk - 1) / kSeqChunk;
  for (int c = 0; c < chunks; ++c) {
    const bool has_next = c + 1 < chunks;
    if (has_next) fetch((c + 1) * kSeqChunk);
    const float* as = stage[c & 1] + 4 * ty;
    const float* bs = stage[c & 1] + kSeqChunk * kSeqAStride + 4 * tx;
    // Only the steps below K run: a zero-filled step would still be a step of the chain (x + 0 keeps x, but
    // -0 + +0 does not keep -0), so the tail is cut rather than padded.
    const int len = (K - c * kSeqChunk) < kSeqChunk ? (K - c * kSeqChunk) : kSeqChunk;
#pragma unroll 4
    for (int k = 0; k < len; ++k) {
      const f32x4_t av = *reinterpret_cast<const f32x4_t*>(as + k * kSeqAStride);
      const f32x4_t b0 = *reinterpret_cast<const f32x4_t*>(bs + k * kSeqBStride);
      const f32x4_t b1 = *reinterpret_cast<const f32x4_t*>(bs + k * kSeqBStride + 64);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = __builtin_fmaf(av[i], b0[j], acc[i][j]);
          acc[i][4 + j] = __builtin_fmaf(av[i], b1[j], acc[i][4 + j]);
        }
      }
    }
    if (has_next) {
      deposit((c + 1) & 1);
      __syncthreads();
    }
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = m0 + 4 * ty + i;
    if (row >= M) continue;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int col = n0 + half * 64 + 4 * tx + j;
        if (col >= N) continue;
        const float v = acc[i][half * 4 + j];
        if constexpr (OUT_BF16) {
          reinterpret_cast<bf16_bits*>(C)[(int64_t)row * ldc + col] = to_bf16_bits(v);
        } else {
          reinterpret_cast<float*>(C)[(int64_t)row * ldc + col] = v;
        }
      }
    }
  }
}

template <bool A_F32, bool B_F32>
static void launch_seq(const SeqOperand& A, const SeqOperand& B, void* C, int64_t ldc, int M, int N, int K,
                       bool out_bf16, hipStream_t stream) {
  const int tiles_m = (M + kSeqBM - 1) / kSeqBM;
  const int tiles_n = (N + kSeqBN - 1) / kSeqBN;
  const dim3 grid((unsigned)(tiles_m * tiles_n));
  if (out_bf16) {
    hipLaunchKernelGGL((det_gemm_seq_kernel<A_F32, B_F32, true>), grid, dim3(kSeqThreads), 0, stream, A, B, C, ldc, M,
                       N, K, tiles_m);
  } else {
    hipLaunchKernelGGL((det_gemm_seq_kernel<A_F32, B_F32, false>), grid, dim3(kSeqThreads), 0, stream, A, B, C, ldc, M,
                       N, K, tiles_m);
  }
}

hipError_t det_gemm_seq_launch(const SeqOperand& A, bool a_f32, const SeqOperand& B, bool b_f32, void* C, int64_t ldc,
                               int M, int N, int K, bool out_bf16, hipStream_t stream) {
  if ((int64_t)((M + kSeqBM - 1) / kSeqBM) * ((N + kSeqBN - 1) / kSeqBN) > 0x7fffffffLL) return hipErrorInvalidValue;
  if (a_f32 && b_f32) launch_seq<true, true>(A, B, C, ldc, M, N, K, out_bf16, stream);
  else if (a_f32) launch_seq<true, false>(A, B, C, ldc, M, N, K, out_bf16, stream);
  else if (b_f32) launch_seq<false, true>(A, B, C, ldc, M, N, K, out_bf16, stream);
  else launch_seq<false, false>(A, B, C, ldc, M, N, K, out_bf16, stream);
  return hipGetLastError();
}

}  // namespace rlk
