// det_gemm for up to 64 tokens against few, long weight panels: one workgroup streams a
// 16-feature weight panel through a deep LDS ring while one wave per 16-token tile runs the
// MFMA chain.
//
// With M <= 64 the GEMM is a read of W at HBM speed. The contract allows no split-K, so the
// K/32 MFMA steps of an output element run one after the other in one wave, and a 16-row
// panel is the finest unit of work (N / 16 workgroups: 256 for the Qwen3-8B down projection,
// one per CU). To keep enough bytes in flight with one workgroup per CU, four producer waves
// issue direct-to-LDS loads several stages ahead; the consumer waves only read fragments and
// issue the dependent MFMA chain, which is short (K/32 steps of ~21 cycles). Measured on this
// part: L2 hits feed a CU's direct-to-LDS path at 64 bytes per clock (135 GB/s, two issuing
// waves suffice), data that comes through the fabric (infinity cache / HBM) arrives at about
// 6 TB/s chip-wide, i.e. 23 GB/s per CU: the weight panel is the slow stream, the activations
// (re-read by every workgroup, L2 hits) the wide one. Same instruction, same ascending K order,
// same zero start as every other det_gemm kernel, so the bits match.
#include "linear_logp_common.h"
#include "rlk_host.h"

namespace rlk {

// MT token tiles of 16 rows. Wave t < MT is the consumer of token tile t (its own MFMA chain
// over the shared weight fragments), the next four waves are the producers. A stage holds KT
// weight sub-tiles (64 K values each), then KT sub-tiles per token tile; a producer always
// fetches the same 8-row half (producer & 1) of the (tile, sub-tile) pairs
// (producer >> 1) + 2 j. Rows past M or N are clamped to the last valid row: computed, never
// stored (MFMA columns and rows are independent).
//
// GATED: W is a packed gate/up weight [2 I, K] (N = 2 I). The panel of workgroup b holds the gate
// rows of features 8 b .. 8 b + 7 in its first half and their up rows in the second, so gate and
// up of an output element sit 32 lanes apart in one accumulator; the epilogue brings them
// together, rounds both to bf16 as the unfused projection would, and stores swiglu(gate, up) into
// C[M, I] (bf16).
template <int KT, int RING, int MT, bool OUT_F32, bool GATED = false>
__global__ __launch_bounds__(64 * (MT + 4)) void det_gemm_stream_kernel(MatView W, MatView X,
                                                                              void* __restrict__ C, int64_t ldc, int M,
                                                                              int N, int K) {
  static_assert(!(GATED && OUT_F32), "the gated projection stores bf16");
  constexpr int kSubBytes = 16 * kRowBytes;
  constexpr int kPairs = KT * (1 + MT);
  constexpr int kStageBytes = kPairs * kSubBytes;
  constexpr int kLoads = kPairs / 2;  // per producer wave per stage
  static_assert(RING >= 2 && kPairs % 2 == 0 && MT >= 1 && MT <= 4, "ring geometry");
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // [0, MT): consumers, then 4 producers
  const int producer = wave - MT;
  const int n0 = blockIdx.x * (GATED ? 8 : 16);  // GATED: first feature of the workgroup
  const int nsub = K / kTileK;  // K % 64 == 0 on this path
  const int nstage = (nsub + KT - 1) / KT;

  // Producer: this lane's row inside a 16-row tile and its 16-byte chunk.
  const int rib = lane >> 3;
  const int chunk_elems = ((lane & 7) ^ rib) * kChunkElems;
  const int half = producer & 1;
  const int r16 = half * 8 + rib;
  int wr = n0 + r16 < N ? n0 + r16 : N - 1;  // rows past an edge are computed, never stored
  if constexpr (GATED) {
    const int features = N / 2;
    const int f = n0 + rib < features ? n0 + rib : features - 1;
    wr = half * features + f;  // producers with half == 0 fetch gate rows, the others up rows
  }
  const bf16_bits* w_base = W.ptr + (int64_t)wr * W.row_stride + chunk_elems;
  const bf16_bits* x_base[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int xr = t * 16 + r16 < M ? t * 16 + r16 : M - 1;
    x_base[t] = X.ptr + (int64_t)xr * X.row_stride + chunk_elems;
  }

  auto issue_stage = [&](int s) {
    if (producer < 0) return;
    char* base = lds + (s % RING) * kStageBytes;
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
      const int q = (producer >> 1) + 2 * j;  // pair: [0, KT) weights, then KT per token tile
      const bool is_w = q < KT;
      const int tile = is_w ? 0 : (q - KT) / KT;
      const int sub = is_w ? q : (q - KT) % KT;
      int ks = s * KT + sub;
      ks = ks < nsub ? ks : nsub - 1;  // past the end: re-fetch the last sub-tile (never consumed)
      const bf16_bits* row = w_base;
#pragma unroll
      for (int t = 0; t < MT; ++t) row = (!is_w && tile == t) ? x_base[t] : row;
      __builtin_amdgcn_global_load_lds((global_ptr_t)(row + ks * kTileK), (lds_ptr_t)(base + (2 * q + half) * 1024), 16,
                                       0, 0);
    }
  };

  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
  const int l16 = lane & 15;
  const int grp = lane >> 4;
  const int frag_lo = l16 * kRowBytes + ((grp ^ (l16 & 7)) << 4);  // K step 0 of a sub-tile
  const int frag_hi = frag_lo ^ 64;                                 // K step 1

#pragma unroll
  for (int s = 0; s < RING - 1; ++s) issue_stage(s);
  for (int s = 0; s < nstage; ++s) {
    __builtin_amdgcn_s_waitcnt(wait_vmcnt((RING - 2) * kLoads));  // my loads of stage s have landed
    wg_barrier();  // stage s is complete; the consumers are done with stage s - 1
    issue_stage(s + RING - 1);
    if (wave < MT) {
      const char* base = lds + (s % RING) * kStageBytes;
      const int remaining = nsub - s * KT;
      const int count = remaining < KT ? remaining : KT;
      u32x4_t wf[2 * KT], xf[2 * KT];
#pragma unroll
      for (int sub = 0; sub < KT; ++sub) {
        const char* wt = base + sub * kSubBytes;
        const char* xt = base + (KT + wave * KT + sub) * kSubBytes;
        wf[2 * sub] = *reinterpret_cast<const u32x4_t*>(wt + frag_lo);
        xf[2 * sub] = *reinterpret_cast<const u32x4_t*>(xt + frag_lo);
        wf[2 * sub + 1] = *reinterpret_cast<const u32x4_t*>(wt + frag_hi);
        xf[2 * sub + 1] = *reinterpret_cast<const u32x4_t*>(xt + frag_hi);
      }
      __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 2 * KT; ++i)
        if (i < 2 * count) acc = mfma_16x16x32(wf[i], xf[i], acc);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  __builtin_amdgcn_s_waitcnt(kWaitAll0);
  wg_barrier();

  const int m = wave * 16 + l16;
  if constexpr (GATED) {
    if (wave < MT) {
      // accumulator rows 4 grp + q: lane groups 0, 1 hold gate features n0 + 4 grp + q, groups 2, 3
      // the up projection of features n0 + 4 (grp - 2) + q
      float up[4];
#pragma unroll
      for (int q = 0; q < 4; ++q)
        up[q] = __int_as_float(__builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __float_as_int(acc[q])));
      const int f = n0 + grp * 4;
      if (grp < 2 && m < M) {
        bf16_bits* row = reinterpret_cast<bf16_bits*>(C) + (int64_t)m * ldc;
        uint32_t packed[2];
#pragma unroll
        for (int h = 0; h < 2; ++h)
          packed[h] = pack_bf16x2(swiglu_f32(round_through_bf16(acc[2 * h]), round_through_bf16(up[2 * h])),
                                  swiglu_f32(round_through_bf16(acc[2 * h + 1]), round_through_bf16(up[2 * h + 1])));
        if (f + 4 <= N / 2 && (reinterpret_cast<uintptr_t>(row + f) & 7) == 0) {
          *reinterpret_cast<u32x2_t*>(row + f) = u32x2_t{packed[0], packed[1]};
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (f + q < N / 2) row[f + q] = (bf16_bits)((packed[q >> 1] >> ((q & 1) * 16)) & 0xffffu);
        }
      }
    }
    return;
  }
  if (wave < MT && m < M) {
    const int n = n0 + grp * 4;
    if (OUT_F32) {
      float* row = reinterpret_cast<float*>(C) + (int64_t)m * ldc;
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (n + q < N) row[n + q] = acc[q];
    } else {
      bf16_bits* row = reinterpret_cast<bf16_bits*>(C) + (int64_t)m * ldc;
      const uint32_t lo = pack_bf16x2(acc[0], acc[1]);
      const uint32_t hi = pack_bf16x2(acc[2], acc[3]);
      if (n + 4 <= N && (reinterpret_cast<uintptr_t>(row + n) & 7) == 0) {
        *reinterpret_cast<u32x2_t*>(row + n) = u32x2_t{lo, hi};
      } else {
        const uint32_t packed[2] = {lo, hi};
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (n + q < N) row[n + q] = (bf16_bits)((packed[q >> 1] >> ((q & 1) * 16)) & 0xffffu);
      }
    }
  }
}

template <int KT, int RING, int MT, bool OUT_F32>
static hipError_t launch_stream(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                                      hipStream_t stream) {
  auto kernel = det_gemm_stream_kernel<KT, RING, MT, OUT_F32>;
  constexpr int kLds = RING * KT * (1 + MT) * 16 * kRowBytes;
  static_assert(kLds <= 160 * 1024, "ring exceeds the LDS");
  static PerDeviceOnce once;
  hipError_t err = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLds, once);
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL(kernel, dim3((N + 15) / 16), dim3(64 * (MT + 4)), kLds, stream, W, X, C, ldc, M, N, K);
  return hipGetLastError();
}

// Packed gate/up projection with the SwiGLU epilogue for up to 16 tokens (W.rows = 2 I, Y[M, I]):
// the two-workgroups-per-CU geometry, I / 8 workgroups.
hipError_t det_gemm_stream_gated_launch(const MatView& W, const MatView& X, void* Y, int64_t ldy, int M, int I, int K,
                                        hipStream_t stream) {
  auto kernel = det_gemm_stream_kernel<2, 8, 1, false, true>;
  constexpr int kLds = 8 * 2 * 2 * 16 * kRowBytes;
  static PerDeviceOnce once;
  hipError_t err = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLds, once);
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL(kernel, dim3((I + 7) / 8), dim3(64 * 5), kLds, stream, W, X, Y, ldy, M, 2 * I, K);
  return hipGetLastError();
}

// One to four token tiles; the ring takes 128 - 144 KiB (one workgroup per CU). `shallow`
// (M <= 16 only) halves the stage so that two workgroups share a CU.
hipError_t det_gemm_stream_launch(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                                  bool out_f32, bool shallow, hipStream_t stream) {
  if (M <= 16 && shallow)
    return out_f32 ? launch_stream<2, 8, 1, true>(W, X, C, ldc, M, N, K, stream)
                   : launch_stream<2, 8, 1, false>(W, X, C, ldc, M, N, K, stream);
  if (M <= 16)
    return out_f32 ? launch_stream<4, 8, 1, true>(W, X, C, ldc, M, N, K, stream)
                   : launch_stream<4, 8, 1, false>(W, X, C, ldc, M, N, K, stream);
  if (M <= 32)
    return out_f32 ? launch_stream<4, 6, 2, true>(W, X, C, ldc, M, N, K, stream)
                   : launch_stream<4, 6, 2, false>(W, X, C, ldc, M, N, K, stream);
  if (M <= 48)
    return out_f32 ? launch_stream<2, 9, 3, true>(W, X, C, ldc, M, N, K, stream)
                   : launch_stream<2, 9, 3, false>(W, X, C, ldc, M, N, K, stream);
  return out_f32 ? launch_stream<2, 7, 4, true>(W, X, C, ldc, M, N, K, stream)
                 : launch_stream<2, 7, 4, false>(W, X, C, ldc, M, N, K, stream);
}

}  // namespace rlk
