// det_gemm for decode-sized batches (M <= 16): one workgroup streams a 16-feature
// weight panel through a deep LDS ring while a single wave runs the MFMA chain.
//
// With M <= 16 the GEMM is a read of W at HBM speed. The contract allows no
// split-K, so the K/32 MFMA steps of an output element run one after the other
// in one wave, and a 16-row panel is the finest unit of work (N / 16 workgroups:
// 256 for the Qwen3-8B down projection, one per CU). To keep enough bytes in
// flight with one workgroup per CU, four producer waves issue direct-to-LDS loads
// several stages (of 256 or 512 K values) ahead; a fifth wave only reads fragments
// and issues the dependent MFMA chain, which is short (K/32 steps of ~21 cycles).
// The vector-memory front end of a CU retires about one 1 KiB load per 33 cycles,
// so the loop is bound by the number of loads: the consumer issues none, and for
// M <= 8 only half of each activation sub-tile is fetched (the upper eight MFMA
// columns then hold stale LDS; columns are independent and never stored).
// Same instruction, same ascending K order, same zero start as every other
// det_gemm kernel, so the bits match.
#include "det_gemm_tile.h"
#include "rlk_host.h"

namespace rlk {

// KT: 64-wide K sub-tiles per ring stage; RING: stages in the ring; HALF_X: M <= 8.
template <int KT, int RING, bool HALF_X, bool OUT_F32>
__global__ __launch_bounds__(320) void det_gemm_stream_kernel(MatView W, MatView X, void* __restrict__ C, int64_t ldc,
                                                               int M, int N, int K) {
  constexpr int kSubBytes = 16 * kRowBytes;        // one operand, one 64-wide sub-tile: 16 rows x 128 B
  constexpr int kStageBytes = 2 * KT * kSubBytes;  // W sub-tiles, then X sub-tiles
  constexpr int kProducers = 4;
  // 1 KiB blocks per stage: 2 KT of weights, then 2 KT (or, HALF_X, KT) of activations.
  constexpr int kBlocksPerStage = HALF_X ? 3 * KT : 4 * KT;
  constexpr int kLoads = kBlocksPerStage / kProducers;  // per producer wave per stage
  static_assert(RING >= 2 && kBlocksPerStage % kProducers == 0, "ring geometry");
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // 0: consumer, 1..4: producers
  const int producer = wave - 1;
  const int n0 = blockIdx.x * 16;
  const int nsub = K / kTileK;               // K % 64 == 0 on this path
  const int nstage = (nsub + KT - 1) / KT;

  // This lane's source row / chunk for a block of 8 rows.
  const int rib = lane >> 3;
  const int chunk_elems = ((lane & 7) ^ rib) * kChunkElems;
  const bf16_bits* w_src[2];
  const bf16_bits* x_src[2];
#pragma unroll
  for (int blk = 0; blk < 2; ++blk) {
    int wr = n0 + blk * 8 + rib;
    wr = wr < N ? wr : N - 1;  // rows past the edge are computed, never stored
    int xr = blk * 8 + rib;
    xr = xr < M ? xr : M - 1;
    w_src[blk] = W.ptr + (int64_t)wr * W.row_stride + chunk_elems;
    x_src[blk] = X.ptr + (int64_t)xr * X.row_stride + chunk_elems;
  }

  // Load j of producer p in a stage is entry p + 4 j of the stage's block list:
  // [0, 2 KT) weight blocks (sub-tile = e / 2, half = e % 2), then the token blocks
  // (both halves of every sub-tile, or with HALF_X only the lower half).
  auto issue_stage = [&](int s) {
    if (producer < 0) return;
    char* base = lds + (s % RING) * kStageBytes;
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
      const int e = producer + kProducers * j;
      const bool is_w = e < 2 * KT;
      const int local = is_w ? e : (HALF_X ? 2 * (e - 2 * KT) : e - 2 * KT);
      const int sub = local >> 1;
      const int blk = local & 1;
      const int idx = (is_w ? 0 : 2 * KT) + local;  // 1 KiB slot inside the stage
      int ks = s * KT + sub;
      ks = ks < nsub ? ks : nsub - 1;  // past the end: re-fetch the last sub-tile (never consumed)
      const bf16_bits* src = (is_w ? w_src[blk] : x_src[blk]) + ks * kTileK;
      __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(base + idx * 1024), 16, 0, 0);
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
    wg_barrier();  // stage s is complete; the consumer is done with stage s - 1
    issue_stage(s + RING - 1);
    if (wave == 0) {
      const char* base = lds + (s % RING) * kStageBytes;
      const int remaining = nsub - s * KT;
      const int count = remaining < KT ? remaining : KT;
      // All fragments of the stage first (2 KT reads per operand in flight at once), then the
      // dependent MFMA chain; the scheduling barrier keeps the compiler from serialising them.
      u32x4_t wf[2 * KT], xf[2 * KT];
#pragma unroll
      for (int sub = 0; sub < KT; ++sub) {
        const char* wt = base + sub * kSubBytes;
        const char* xt = base + (KT + sub) * kSubBytes;
        wf[2 * sub] = *reinterpret_cast<const u32x4_t*>(wt + frag_lo);
        xf[2 * sub] = *reinterpret_cast<const u32x4_t*>(xt + frag_lo);
        wf[2 * sub + 1] = *reinterpret_cast<const u32x4_t*>(wt + frag_hi);
        xf[2 * sub + 1] = *reinterpret_cast<const u32x4_t*>(xt + frag_hi);
      }
      __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
      __builtin_amdgcn_sched_barrier(0);
      if (count == KT) {
#pragma unroll
        for (int i = 0; i < 2 * KT; ++i) acc = mfma_16x16x32(wf[i], xf[i], acc);
      } else {
        // Last, partial stage: sub-tiles past K were re-fetched copies and must not be added.
#pragma unroll
        for (int i = 0; i < 2 * KT; ++i)
          if (i < 2 * count) acc = mfma_16x16x32(wf[i], xf[i], acc);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  __builtin_amdgcn_s_waitcnt(kWaitAll0);
  wg_barrier();

  if (wave == 0 && l16 < M) {
    const int n = n0 + grp * 4;
    if (OUT_F32) {
      float* row = reinterpret_cast<float*>(C) + (int64_t)l16 * ldc;
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (n + q < N) row[n + q] = acc[q];
    } else {
      bf16_bits* row = reinterpret_cast<bf16_bits*>(C) + (int64_t)l16 * ldc;
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

template <int KT, int RING, bool HALF_X, bool OUT_F32>
static hipError_t launch_stream(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                                hipStream_t stream) {
  auto kernel = det_gemm_stream_kernel<KT, RING, HALF_X, OUT_F32>;
  constexpr int kLds = RING * 2 * KT * 16 * kRowBytes;
  static PerDeviceOnce once;
  hipError_t err = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLds, once);
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL(kernel, dim3((N + 15) / 16), dim3(320), kLds, stream, W, X, C, ldc, M, N, K);
  return hipGetLastError();
}

// variant 0: 512-wide stages, ring of 4 (128 KiB, one workgroup per CU: few, long panels)
// variant 1: 256-wide stages, ring of 4 (64 KiB, two workgroups per CU: many, short panels)
hipError_t det_gemm_stream_launch(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                                  bool out_f32, int variant, hipStream_t stream) {
  const bool half = M <= 8;
  if (variant == 0) {
    if (half)
      return out_f32 ? launch_stream<8, 4, true, true>(W, X, C, ldc, M, N, K, stream)
                     : launch_stream<8, 4, true, false>(W, X, C, ldc, M, N, K, stream);
    return out_f32 ? launch_stream<8, 4, false, true>(W, X, C, ldc, M, N, K, stream)
                   : launch_stream<8, 4, false, false>(W, X, C, ldc, M, N, K, stream);
  }
  if (half)
    return out_f32 ? launch_stream<4, 4, true, true>(W, X, C, ldc, M, N, K, stream)
                   : launch_stream<4, 4, true, false>(W, X, C, ldc, M, N, K, stream);
  return out_f32 ? launch_stream<4, 4, false, true>(W, X, C, ldc, M, N, K, stream)
                 : launch_stream<4, 4, false, false>(W, X, C, ldc, M, N, K, stream);
}

}  // namespace rlk
