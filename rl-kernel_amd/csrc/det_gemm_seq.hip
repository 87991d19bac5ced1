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
// The chain runs on the fp32 matrix pipe: an fp32 MFMA with reduction length one, v_mfma_f32_32x32x1_2b_f32, adds
// exactly one product to each of its accumulators with a single rounding - the fused multiply-add of the chain,
// also on fp32 operands (checked bit for bit against v_fma_f32 chains and the CPU's fmaf, fp32 denormal operands
// included) - at 64 flop per clock and SIMD, twice what the vector ALU does without packed instructions. A
// workgroup of four waves owns a 128 x 128 output tile, a wave 64 x 64 (two row halves; the instruction's two
// blocks sit side by side in the columns and take the same 32 rows); K is walked in chunks of 32 staged in LDS
// as fp32 [row][k] (144-byte rows: a lane's 16-byte read of four k of its own row is conflict free), the next
// chunk fetched while the current one is multiplied: 16-byte loads when both operands are K-contiguous with
// 16-byte aligned rows and 32 divides K, element loads with any non-negative strides otherwise. The row of a
// result depends on that row of A only. The tail of K is cut, never padded with zero steps (a padded step would
// turn an accumulator of -0 into +0). A vector-ALU form of the kernel (64 x 128 tiles, a thread 32 chains) ran at
// 80 TFLOP/s, the rate of unpacked v_fma_f32, and lost to this one at every size down to a single 64-row tile.
#include "rlk_device.h"
#include "rlk_host.h"

namespace rlk {

constexpr int kSeqChunk = 32;

template <bool F32>
__device__ __forceinline__ float seq_load(const void* base, int64_t index) {
  if constexpr (F32) {
    return reinterpret_cast<const float*>(base)[index];
  } else {
    return bf16_bits_to_float(reinterpret_cast<const bf16_bits*>(base)[index]);
  }
}

constexpr int kSeqMfmaBM = 128;
constexpr int kSeqMfmaBN = 128;
constexpr int kSeqMfmaThreads = 256;
constexpr int kSeqMfmaPitch = kSeqChunk + 4;  // floats per staged row: 144 bytes
constexpr int kSeqMfmaStageFloats = (kSeqMfmaBM + kSeqMfmaBN) * kSeqMfmaPitch;
constexpr int kSeqMfmaLdsBytes = 2 * kSeqMfmaStageFloats * 4;
constexpr int kSeqMfmaLoads = kSeqMfmaBM * kSeqChunk / kSeqMfmaThreads;  // 16 elements per thread, operand and chunk
typedef float f32x32_t __attribute__((ext_vector_type(32)));

// 16 bytes of a K-contiguous row (four fp32 or eight bf16 values) into the fp32 stage.
template <bool F32>
struct SeqUnit {
  static constexpr int kElems = F32 ? 4 : 8;                             // values per 16-byte unit
  static constexpr int kPerRow = kSeqChunk / kElems;                     // units of a row per chunk
  static constexpr int kPerThread = 128 * kPerRow / kSeqMfmaThreads;     // units per thread, operand and chunk
  u32x4_t raw;
  __device__ __forceinline__ void load(const void* row, int k) {
    raw = *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const char*>(row) + (int64_t)k * (F32 ? 4 : 2));
  }
  __device__ __forceinline__ void store(float* dst) const {
    if constexpr (F32) {
      *reinterpret_cast<u32x4_t*>(dst) = raw;
    } else {
      *reinterpret_cast<u32x4_t*>(dst) = u32x4_t{raw[0] << 16, raw[0] & 0xffff0000u, raw[1] << 16, raw[1] & 0xffff0000u};
      *reinterpret_cast<u32x4_t*>(dst + 4) = u32x4_t{raw[2] << 16, raw[2] & 0xffff0000u, raw[3] << 16, raw[3] & 0xffff0000u};
    }
  }
};

// VEC: both operands have unit K stride, 16-byte aligned rows and K % 32 == 0: 16-byte loads and LDS stores
// (a thread moves 2 to 4 units per operand and chunk instead of 16 elements).
template <bool A_F32, bool B_F32, bool OUT_BF16, bool VEC>
__global__ __launch_bounds__(kSeqMfmaThreads, 2) void det_gemm_seq_mfma_kernel(SeqOperand A, SeqOperand B,
                                                                               void* __restrict__ C, int64_t ldc, int M,
                                                                               int N, int K, int tiles_m) {
  extern __shared__ __attribute__((aligned(16))) float seq_stage[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave & 1, wave_n = wave >> 1;
  const int tile_m = blockIdx.x % tiles_m;
  const int tile_n = blockIdx.x / tiles_m;
  const int m0 = tile_m * kSeqMfmaBM;
  const int n0 = tile_n * kSeqMfmaBN;

  // Loader role: element (row, k) with k = tid % 32, rows tid / 32 + 8 j. Rows past the edge are clamped to the
  // last valid row (their results are never stored); k past K reads index K - 1 and its value is never multiplied.
  const int load_k = tid & 31;
  const int load_row = tid >> 5;
  const int a_last = M - 1 - m0, b_last = N - 1 - n0;
  float a_reg[VEC ? 1 : kSeqMfmaLoads], b_reg[VEC ? 1 : kSeqMfmaLoads];
  using UnitA = SeqUnit<A_F32>;
  using UnitB = SeqUnit<B_F32>;
  UnitA a_unit[UnitA::kPerThread];
  UnitB b_unit[UnitB::kPerThread];
  const void* a_row[UnitA::kPerThread];
  const void* b_row[UnitB::kPerThread];
  if constexpr (VEC) {
#pragma unroll
    for (int j = 0; j < UnitA::kPerThread; ++j) {
      const int row = (tid + j * kSeqMfmaThreads) / UnitA::kPerRow;
      a_row[j] = reinterpret_cast<const char*>(A.ptr) + (int64_t)(m0 + (row < a_last ? row : a_last)) * A.row_stride * (A_F32 ? 4 : 2);
    }
#pragma unroll
    for (int j = 0; j < UnitB::kPerThread; ++j) {
      const int row = (tid + j * kSeqMfmaThreads) / UnitB::kPerRow;
      b_row[j] = reinterpret_cast<const char*>(B.ptr) + (int64_t)(n0 + (row < b_last ? row : b_last)) * B.row_stride * (B_F32 ? 4 : 2);
    }
  }
  auto fetch = [&](int k0) {
    if constexpr (VEC) {
#pragma unroll
      for (int j = 0; j < UnitA::kPerThread; ++j) a_unit[j].load(a_row[j], k0 + ((tid + j * kSeqMfmaThreads) % UnitA::kPerRow) * UnitA::kElems);
#pragma unroll
      for (int j = 0; j < UnitB::kPerThread; ++j) b_unit[j].load(b_row[j], k0 + ((tid + j * kSeqMfmaThreads) % UnitB::kPerRow) * UnitB::kElems);
      return;
    }
    const int k = k0 + load_k < K ? k0 + load_k : K - 1;
#pragma unroll
    for (int j = 0; j < (VEC ? 1 : kSeqMfmaLoads); ++j) {
      const int row = load_row + 8 * j;
      a_reg[j] = seq_load<A_F32>(A.ptr, (int64_t)(m0 + (row < a_last ? row : a_last)) * A.row_stride + (int64_t)k * A.k_stride);
      b_reg[j] = seq_load<B_F32>(B.ptr, (int64_t)(n0 + (row < b_last ? row : b_last)) * B.row_stride + (int64_t)k * B.k_stride);
    }
  };
  auto deposit = [&](int buf) {
    float* as = seq_stage + buf * kSeqMfmaStageFloats;
    float* bs = as + kSeqMfmaBM * kSeqMfmaPitch;
    if constexpr (VEC) {
#pragma unroll
      for (int j = 0; j < UnitA::kPerThread; ++j) {
        const int idx = tid + j * kSeqMfmaThreads;
        a_unit[j].store(as + (idx / UnitA::kPerRow) * kSeqMfmaPitch + (idx % UnitA::kPerRow) * UnitA::kElems);
      }
#pragma unroll
      for (int j = 0; j < UnitB::kPerThread; ++j) {
        const int idx = tid + j * kSeqMfmaThreads;
        b_unit[j].store(bs + (idx / UnitB::kPerRow) * kSeqMfmaPitch + (idx % UnitB::kPerRow) * UnitB::kElems);
      }
      return;
    }
#pragma unroll
    for (int j = 0; j < (VEC ? 1 : kSeqMfmaLoads); ++j) {
      as[(load_row + 8 * j) * kSeqMfmaPitch + load_k] = a_reg[j];
      bs[(load_row + 8 * j) * kSeqMfmaPitch + load_k] = b_reg[j];
    }
  };

  // acc[h][r]: row m0 + 64 wave_m + 32 h + 8 ((r % 16) / 4) + 4 (lane / 32) + r % 4,
  //            column n0 + 64 wave_n + 32 (r / 16) + lane % 32.
  f32x32_t acc[2];
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int r = 0; r < 32; ++r) acc[h][r] = 0.f;

  // Four k at a time; both blocks of the instruction take the same 32 rows (lanes l and l + 32 read the same
  // address) and 32 columns each.
  const int a_frag = (wave_m * 64 + (lane & 31)) * kSeqMfmaPitch;
  const int b_frag = (kSeqMfmaBM + wave_n * 64 + lane) * kSeqMfmaPitch;
  auto four_steps = [&](const float* st, int k) __attribute__((always_inline)) {
    const f32x4_t a0 = *reinterpret_cast<const f32x4_t*>(st + a_frag + k);
    const f32x4_t a1 = *reinterpret_cast<const f32x4_t*>(st + a_frag + 32 * kSeqMfmaPitch + k);
    const f32x4_t bv = *reinterpret_cast<const f32x4_t*>(st + b_frag + k);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      acc[0] = __builtin_amdgcn_mfma_f32_32x32x1f32(a0[e], bv[e], acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_32x32x1f32(a1[e], bv[e], acc[1], 0, 0, 0);
    }
  };

  fetch(0);
  deposit(0);
  __syncthreads();
  const int chunks = (K + kSeqChunk - 1) / kSeqChunk;
  const int whole = K / kSeqChunk;  // chunks of 32 steps: a straight run of 64 MFMAs, no conditions
  for (int c = 0; c < whole; ++c) {
    const bool has_next = c + 1 < chunks;
    if (has_next) fetch((c + 1) * kSeqChunk);
    const float* st = seq_stage + (c & 1) * kSeqMfmaStageFloats;
#pragma unroll
    for (int k = 0; k < kSeqChunk; k += 4) four_steps(st, k);
    if (has_next) {
      deposit((c + 1) & 1);
      __syncthreads();
    }
  }
  if (whole < chunks) {  // the last chunk: only the steps below K run
    const float* st = seq_stage + (whole & 1) * kSeqMfmaStageFloats;
    const int len = K - whole * kSeqChunk;
    int k = 0;
    for (; k + 4 <= len; k += 4) four_steps(st, k);
    const f32x4_t a0 = *reinterpret_cast<const f32x4_t*>(st + a_frag + k);
    const f32x4_t a1 = *reinterpret_cast<const f32x4_t*>(st + a_frag + 32 * kSeqMfmaPitch + k);
    const f32x4_t bv = *reinterpret_cast<const f32x4_t*>(st + b_frag + k);
#pragma unroll
    for (int e = 0; e < 3; ++e) {
      if (k + e < len) {
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x1f32(a0[e], bv[e], acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_32x32x1f32(a1[e], bv[e], acc[1], 0, 0, 0);
      }
    }
  }

#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int r = 0; r < 32; ++r) {
      const int row = m0 + 64 * wave_m + 32 * h + 8 * ((r % 16) / 4) + 4 * (lane / 32) + r % 4;
      const int col = n0 + 64 * wave_n + 32 * (r / 16) + (lane & 31);
      if (row >= M || col >= N) continue;
      if constexpr (OUT_BF16) {
        reinterpret_cast<bf16_bits*>(C)[(int64_t)row * ldc + col] = to_bf16_bits(acc[h][r]);
      } else {
        reinterpret_cast<float*>(C)[(int64_t)row * ldc + col] = acc[h][r];
      }
    }
  }
}

template <bool A_F32, bool B_F32, bool OUT_BF16, bool VEC>
static hipError_t launch_seq_mfma_kernel(const SeqOperand& A, const SeqOperand& B, void* C, int64_t ldc, int M, int N,
                                         int K, hipStream_t stream) {
  auto kernel = det_gemm_seq_mfma_kernel<A_F32, B_F32, OUT_BF16, VEC>;
  static PerDeviceOnce once;
  hipError_t err = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kSeqMfmaLdsBytes, once);
  if (err != hipSuccess) return err;
  const int tiles_m = (M + kSeqMfmaBM - 1) / kSeqMfmaBM;
  const int tiles_n = (N + kSeqMfmaBN - 1) / kSeqMfmaBN;
  hipLaunchKernelGGL(kernel, dim3((unsigned)(tiles_m * tiles_n)), dim3(kSeqMfmaThreads), kSeqMfmaLdsBytes, stream, A, B,
                     C, ldc, M, N, K, tiles_m);
  return hipGetLastError();
}

template <bool A_F32, bool B_F32>
static hipError_t launch_seq_mfma(const SeqOperand& A, const SeqOperand& B, void* C, int64_t ldc, int M, int N, int K,
                                  bool out_bf16, hipStream_t stream) {
  auto whole_units = [](const SeqOperand& op, bool f32) {
    const int64_t elems = f32 ? 4 : 8;
    return op.k_stride == 1 && op.row_stride % elems == 0 && (reinterpret_cast<uintptr_t>(op.ptr) & 15) == 0;
  };
  const bool vec = K % kSeqChunk == 0 && whole_units(A, A_F32) && whole_units(B, B_F32);
  if (vec)
    return out_bf16 ? launch_seq_mfma_kernel<A_F32, B_F32, true, true>(A, B, C, ldc, M, N, K, stream)
                    : launch_seq_mfma_kernel<A_F32, B_F32, false, true>(A, B, C, ldc, M, N, K, stream);
  return out_bf16 ? launch_seq_mfma_kernel<A_F32, B_F32, true, false>(A, B, C, ldc, M, N, K, stream)
                  : launch_seq_mfma_kernel<A_F32, B_F32, false, false>(A, B, C, ldc, M, N, K, stream);
}

hipError_t det_gemm_seq_launch(const SeqOperand& A, bool a_f32, const SeqOperand& B, bool b_f32, void* C, int64_t ldc,
                               int M, int N, int K, bool out_bf16, hipStream_t stream) {
  if ((int64_t)((M + kSeqMfmaBM - 1) / kSeqMfmaBM) * ((N + kSeqMfmaBN - 1) / kSeqMfmaBN) > 0x7fffffffLL) return hipErrorInvalidValue;
  if (a_f32 && b_f32) return launch_seq_mfma<true, true>(A, B, C, ldc, M, N, K, out_bf16, stream);
  if (a_f32) return launch_seq_mfma<true, false>(A, B, C, ldc, M, N, K, out_bf16, stream);
  if (b_f32) return launch_seq_mfma<false, true>(A, B, C, ldc, M, N, K, out_bf16, stream);
  return launch_seq_mfma<false, false>(A, B, C, ldc, M, N, K, out_bf16, stream);
}

}  // namespace rlk
