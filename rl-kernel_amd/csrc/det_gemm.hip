// Deterministic, batch-invariant bf16 GEMM for gfx950:  C[M,N] = X[M,K] * W[N,K]^T.
//
// Replaces the kernels behind rl_engine._C.det_gemm_* (reference
// csrc/cuda/gemm/det_gemm_kernel.cu:92-101, 250-402) and the Triton MFMA kernels of
// rl_engine/backends/rocm/gemm/mfma_gemm.py:135-274. No split-K, no atomics, no
// stream-K: one workgroup owns an output tile for the whole K range.
#include "det_gemm_tile.h"
#include "rlk_host.h"

namespace rlk {

// LOOP selects the main loop: kLoopGeneric (any strides, element loads),
// kLoopStaged (16-byte loads through registers) or kLoopPingPong (direct-to-LDS
// loads, two wave groups half an iteration apart). All three run the same MFMA chain.
// The K-major variants are the ping-pong loop with the weight operand (B[K,N], N contiguous),
// the activation operand (x[k * ld + m], tokens contiguous) or both read through transposing
// LDS loads.
enum : int {
  kLoopGeneric = 0,
  kLoopStaged = 1,
  kLoopPingPong = 2,
  kLoopPingPongKMajor = 3,   // weight K-major
  kLoopPingPongXKMajor = 4,  // activation K-major
  kLoopPingPongBothKMajor = 5,
  kLoopSolo = 6,  // four waves, one per SIMD
  kLoopStagedKMajor = 7,     // register-staged, weight K-major (the small tiles), K % 64 == 0
  kLoopStagedKMajorTail = 8  // the same with a zero-filled last K tile
};
constexpr bool loop_weight_kmajor(int loop) {
  return loop == kLoopPingPongKMajor || loop == kLoopPingPongBothKMajor || loop == kLoopStagedKMajor ||
         loop == kLoopStagedKMajorTail;
}
constexpr bool loop_act_kmajor(int loop) { return loop == kLoopPingPongXKMajor || loop == kLoopPingPongBothKMajor; }

template <class S, int LOOP, bool OUT_F32, int KS = 1, int NS = 2>
__global__ __launch_bounds__(S::kThreads) void det_gemm_kernel(MatView W, MatView X, void* __restrict__ C,
                                                                int64_t ldc, int M, int N, int K,
                                                                int tiles_m, int tiles_n, int group_m) {
  extern __shared__ __attribute__((aligned(16))) char lds[];

  // Tile raster: XCD-compact ids, then column groups of group_m token tiles so
  // the tiles resident on one XCD share weight and activation panels in its L2.
  const int total = tiles_m * tiles_n;
  const int id = xcd_compact_id(blockIdx.x, total);
  const int per_group = group_m * tiles_n;
  const int group = id / per_group;
  const int first_m = group * group_m;
  const int width = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
  const int within = id - group * per_group;
  const int tile_m = first_m + within % width;
  const int tile_n = within / width;
  const int n0 = tile_n * S::BN;
  const int m0 = tile_m * S::BM;

  f32x4_t acc[S::TN][S::TM];
  if constexpr (LOOP == kLoopSolo) {
    tile_mainloop_solo<S>(W, X, n0, m0, K, lds, acc);
  } else if constexpr (LOOP == kLoopStagedKMajor || LOOP == kLoopStagedKMajorTail) {
    tile_mainloop_staged_kmajor<S, KS, LOOP == kLoopStagedKMajorTail>(W, X, n0, m0, K, lds, acc);
  } else if constexpr (LOOP >= kLoopPingPongKMajor) {
    // whole K tiles through the ping-pong loop, the rest of a reduction length that 64 does not divide behind it
    const int k_whole = K & ~(kTileK - 1);
    if (k_whole > 0) {
      tile_mainloop_pingpong<S, loop_weight_kmajor(LOOP), loop_act_kmajor(LOOP), PlainRowMap<S>, KS, NS>(
          W, X, n0, m0, k_whole, lds, acc);
    } else {  // fewer than 64 K values: the tail step is the whole reduction
#pragma unroll
      for (int jn = 0; jn < S::TN; ++jn)
#pragma unroll
        for (int jm = 0; jm < S::TM; ++jm) acc[jn][jm] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    if (k_whole != K) tile_tail_step<S, loop_weight_kmajor(LOOP), loop_act_kmajor(LOOP)>(W, X, n0, m0, k_whole, K, lds, acc);
  } else if constexpr (LOOP == kLoopPingPong) {
    tile_mainloop_pingpong<S, false, false, PlainRowMap<S>, KS, NS>(W, X, n0, m0, K, lds, acc);
  } else {
    tile_mainloop_staged<S, LOOP == kLoopStaged>(W, X, n0, m0, K, lds, acc);
  }

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wave_n = wave % S::WN;
  const int wave_m = wave / S::WN;
  const int n_run = n0 + wave_n * 16 * S::TN + (lane >> 4) * S::kRun;  // first feature of this lane's run
  const int m_lane = m0 + wave_m * 16 * S::TM + (lane & 15);

  if constexpr (loop_weight_kmajor(LOOP)) {
    // No run permutation on this path: MFMA tile jn holds features jn*16 + (lane>>4)*4 + q.
    const int n_tile = n0 + wave_n * 16 * S::TN + (lane >> 4) * 4;
    if constexpr (!OUT_F32 && S::TN == 4) {
      // bf16 results of a wave whose 64 features all lie inside N, rows 16-byte aligned (both uniform over the
      // wave): a lane holds four 8-byte pieces of a token's row, 32 bytes apart. A 4 x 4 transpose of the pieces
      // between the four lanes of a token (two butterfly stages of lane swaps over distances 32 and 16: the
      // piece that lane g held at position c ends at lane c, position g) gives every lane the 16 consecutive
      // features 16 g .. 16 g + 15, stored as two 16-byte halves: 128 contiguous bytes per token and instruction
      // pair instead of 32 per instruction.
      // Ordinary stores. Non-temporal ones make a GEMM that is relaunched on the same operands 4-5 % faster (gate_up
      // at 4096 tokens 574 -> 550 us): the result then bypasses the 256 MB memory-side cache and the weights stay in
      // it from one launch to the next. With weights that come from HBM, as in a model with more than one layer,
      // they measured the same or 1 % slower, and gate_up and down launched alternately 0.6 % slower; not used.
      const int n_wave = n0 + wave_n * 64;
      const bool whole_span = n_wave + 64 <= N && (reinterpret_cast<uintptr_t>(C) & 15) == 0 && (ldc & 7) == 0;
      if (whole_span) {
        const int grp = lane >> 4;
#pragma unroll
        for (int jm = 0; jm < S::TM; ++jm) {
          uint32_t w[4][2];
#pragma unroll
          for (int jn = 0; jn < 4; ++jn) {
            w[jn][0] = pack_bf16x2(acc[jn][jm][0], acc[jn][jm][1]);
            w[jn][1] = pack_bf16x2(acc[jn][jm][2], acc[jn][jm][3]);
          }
#pragma unroll
          for (int c = 0; c < 2; ++c)  // lane bit 5 <-> piece bit 1
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              const auto r = __builtin_amdgcn_permlane32_swap(w[c][e], w[c + 2][e], false, false);
              w[c][e] = r[0];
              w[c + 2][e] = r[1];
            }
#pragma unroll
          for (int c = 0; c < 4; c += 2)  // lane bit 4 <-> piece bit 0
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              const auto r = __builtin_amdgcn_permlane16_swap(w[c][e], w[c + 1][e], false, false);
              w[c][e] = r[0];
              w[c + 1][e] = r[1];
            }
          const int m = m_lane + jm * 16;
          if (m < M) {
            bf16_bits* dst = reinterpret_cast<bf16_bits*>(C) + (int64_t)m * ldc + n_wave + grp * 16;
            *reinterpret_cast<u32x4_t*>(dst) = u32x4_t{w[0][0], w[0][1], w[1][0], w[1][1]};
            *reinterpret_cast<u32x4_t*>(dst + 8) = u32x4_t{w[2][0], w[2][1], w[3][0], w[3][1]};
          }
        }
        return;
      }
    }
#pragma unroll
    for (int jm = 0; jm < S::TM; ++jm) {
      const int m = m_lane + jm * 16;
      if (m >= M) continue;
#pragma unroll
      for (int jn = 0; jn < S::TN; ++jn) {
        const int n = n_tile + jn * 16;
        if (OUT_F32) {
          float* dst = reinterpret_cast<float*>(C) + (int64_t)m * ldc + n;
          if (n + 4 <= N && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
            *reinterpret_cast<f32x4_t*>(dst) = acc[jn][jm];
          } else {
#pragma unroll
            for (int q = 0; q < 4; ++q)
              if (n + q < N) dst[q] = acc[jn][jm][q];
          }
        } else {
          bf16_bits* dst = reinterpret_cast<bf16_bits*>(C) + (int64_t)m * ldc + n;
          const uint32_t lo = pack_bf16x2(acc[jn][jm][0], acc[jn][jm][1]);
          const uint32_t hi = pack_bf16x2(acc[jn][jm][2], acc[jn][jm][3]);
          if (n + 4 <= N && (reinterpret_cast<uintptr_t>(dst) & 7) == 0) {
            *reinterpret_cast<u32x2_t*>(dst) = u32x2_t{lo, hi};
          } else {
            const uint32_t packed[2] = {lo, hi};
#pragma unroll
            for (int q = 0; q < 4; ++q)
              if (n + q < N) dst[q] = (bf16_bits)((packed[q >> 1] >> ((q & 1) * 16)) & 0xffffu);
          }
        }
      }
    }
    return;
  }

  if constexpr (!OUT_F32 && S::TN == 4) {
    // bf16 results of a wave whose 64 features all lie inside N, rows 16-byte aligned (both uniform over the wave):
    // a lane holds the 16 consecutive features 16 g .. 16 g + 15 of a token as two 16-byte halves, so a store
    // instruction would write 16-byte pieces 32 bytes apart. Two lane swaps (over distance 16 between the halves,
    // then over distance 32) rotate (half, lane bit 5, lane bit 4) into (lane bit 4, half, lane bit 5): store s of
    // lane g then holds features 32 s + 8 g .. + 7, 64 contiguous bytes per token and instruction.
    const int n_wave = n0 + wave_n * 64;
    const bool whole_span = n_wave + 64 <= N && (reinterpret_cast<uintptr_t>(C) & 15) == 0 && (ldc & 7) == 0;
    if (whole_span) {
      const int grp = lane >> 4;
#pragma unroll
      for (int jm = 0; jm < S::TM; ++jm) {
        uint32_t half[2][4];
#pragma unroll
        for (int jn = 0; jn < 4; ++jn) {
          half[jn >> 1][2 * (jn & 1)] = pack_bf16x2(acc[jn][jm][0], acc[jn][jm][1]);
          half[jn >> 1][2 * (jn & 1) + 1] = pack_bf16x2(acc[jn][jm][2], acc[jn][jm][3]);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const auto r = __builtin_amdgcn_permlane16_swap(half[0][e], half[1][e], false, false);
          const auto t = __builtin_amdgcn_permlane32_swap(r[0], r[1], false, false);
          half[0][e] = t[0];
          half[1][e] = t[1];
        }
        const int m = m_lane + jm * 16;
        if (m < M) {
          bf16_bits* dst = reinterpret_cast<bf16_bits*>(C) + (int64_t)m * ldc + n_wave + grp * 8;
          *reinterpret_cast<u32x4_t*>(dst) = u32x4_t{half[0][0], half[0][1], half[0][2], half[0][3]};
          *reinterpret_cast<u32x4_t*>(dst + 32) = u32x4_t{half[1][0], half[1][1], half[1][2], half[1][3]};
        }
      }
      return;
    }
  }

#pragma unroll
  for (int jm = 0; jm < S::TM; ++jm) {
    const int m = m_lane + jm * 16;
    if (m >= M) continue;
    if (OUT_F32) {
      float* row = reinterpret_cast<float*>(C) + (int64_t)m * ldc;
      const bool vec_ok = (n_run + S::kRun <= N) && ((reinterpret_cast<uintptr_t>(row + n_run) & 15) == 0);
      if (vec_ok) {
#pragma unroll
        for (int jn = 0; jn < S::TN; ++jn) *reinterpret_cast<f32x4_t*>(row + n_run + jn * 4) = acc[jn][jm];
      } else {
#pragma unroll
        for (int jn = 0; jn < S::TN; ++jn)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (n_run + jn * 4 + q < N) row[n_run + jn * 4 + q] = acc[jn][jm][q];
      }
    } else {
      bf16_bits* row = reinterpret_cast<bf16_bits*>(C) + (int64_t)m * ldc;
      uint32_t packed[2 * S::TN];
#pragma unroll
      for (int jn = 0; jn < S::TN; ++jn) {
        packed[2 * jn] = pack_bf16x2(acc[jn][jm][0], acc[jn][jm][1]);
        packed[2 * jn + 1] = pack_bf16x2(acc[jn][jm][2], acc[jn][jm][3]);
      }
      // an odd number of MFMA tiles per wave makes a run an odd multiple of 8 bytes: 8-byte stores
      constexpr int kAlign = (S::TN % 2 == 0) ? 16 : 8;
      const bool vec_ok =
          (n_run + S::kRun <= N) && ((reinterpret_cast<uintptr_t>(row + n_run) & (kAlign - 1)) == 0);
      if (vec_ok) {
        if (S::TN % 2 == 1) {
#pragma unroll
          for (int v = 0; v < S::TN; ++v)
            *reinterpret_cast<u32x2_t*>(row + n_run + v * 4) = u32x2_t{packed[2 * v], packed[2 * v + 1]};
        } else if (S::TN >= 2) {
#pragma unroll
          for (int v = 0; v < S::TN / 2; ++v)
            *reinterpret_cast<u32x4_t*>(row + n_run + v * 8) =
                u32x4_t{packed[4 * v], packed[4 * v + 1], packed[4 * v + 2], packed[4 * v + 3]};
          if (S::TN % 2)
            *reinterpret_cast<u32x2_t*>(row + n_run + (S::TN - 1) * 4) =
                u32x2_t{packed[2 * S::TN - 2], packed[2 * S::TN - 1]};
        } else {
          *reinterpret_cast<u32x2_t*>(row + n_run) = u32x2_t{packed[0], packed[1]};
        }
      } else {
#pragma unroll
        for (int e = 0; e < S::kRun; ++e)
          if (n_run + e < N) row[n_run + e] = (bf16_bits)((packed[e >> 1] >> ((e & 1) * 16)) & 0xffffu);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------

template <class S, int LOOP, bool OUT_F32, int KS = 1, int NS = 2>
static hipError_t launch_tile(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                              hipStream_t stream) {
  auto kernel = det_gemm_kernel<S, LOOP, OUT_F32, KS, NS>;
  constexpr int kLds = NS * KS * S::kStageBytes;
  static_assert(kLds <= 160 * 1024, "stages exceed the LDS");
  static PerDeviceOnce once;
  hipError_t err = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLds, once);
  if (err != hipSuccess) return err;
  const int tiles_m = (M + S::BM - 1) / S::BM;
  const int tiles_n = (N + S::BN - 1) / S::BN;
  int group_m = tiles_m < 8 ? tiles_m : 8;
  hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n), dim3(S::kThreads), kLds, stream, W, X, C, ldc, M, N, K,
                     tiles_m, tiles_n, group_m);
  return hipGetLastError();
}

template <class S, int LOOP, int NS = 2>
static hipError_t launch_loop(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                              bool out_f32, hipStream_t stream) {
  return out_f32 ? launch_tile<S, LOOP, true, 1, NS>(W, X, C, ldc, M, N, K, stream)
                 : launch_tile<S, LOOP, false, 1, NS>(W, X, C, ldc, M, N, K, stream);
}

// LDS stages of the native ping-pong loop: 256 x 128 and 256 x 64 run three (144 / 120 KiB). With
// weights that come from HBM the extra K tile of lead is worth 8 % (gate_up at 256 tokens:
// 73 -> 68 us); on cache-resident operands it changes nothing. The smaller shapes have their
// deep-stage variants; the K-major loops measured no gain from a third stage and keep two.
template <class S>
constexpr int pingpong_stages() {
  return (S::BN >= 192 && S::BM <= 128) ? 3 : 2;
}

// kmajor_loop: 0, or the K-major ping-pong variant the operand layouts call for.
template <class S>
static hipError_t launch_shape(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                               bool vec, int kmajor_loop, bool allow_pingpong, bool out_f32, hipStream_t stream) {
  if constexpr (pingpong_supported<S>() && S::TN == 4) {
    if (kmajor_loop == kLoopPingPongKMajor)
      return launch_loop<S, kLoopPingPongKMajor>(W, X, C, ldc, M, N, K, out_f32, stream);
    if constexpr (S::BM % 128 == 0) {
      if (kmajor_loop == kLoopPingPongXKMajor)
        return launch_loop<S, kLoopPingPongXKMajor>(W, X, C, ldc, M, N, K, out_f32, stream);
      if (kmajor_loop == kLoopPingPongBothKMajor)
        return launch_loop<S, kLoopPingPongBothKMajor>(W, X, C, ldc, M, N, K, out_f32, stream);
    }
  }
  if (kmajor_loop != 0) return hipErrorInvalidValue;
  if constexpr (pingpong_supported<S>()) {
    if (vec && allow_pingpong && K % kTileK == 0) {
      return launch_loop<S, kLoopPingPong, pingpong_stages<S>()>(W, X, C, ldc, M, N, K, out_f32, stream);
    }
  }
  if (vec) return launch_loop<S, kLoopStaged>(W, X, C, ldc, M, N, K, out_f32, stream);
  return launch_loop<S, kLoopGeneric>(W, X, C, ldc, M, N, K, out_f32, stream);
}

constexpr int kDeep64 = 4;   // 64x64: 4 K tiles per stage, 2 x 64 KiB of LDS
constexpr int kDeep128 = 2;  // 128x64 / 128x128: 2 K tiles per stage, 3 x 48 / 2 x 64 KiB (three stages measured
                             // 8 % faster for 128x64; deeper rings did not pay for the other two)

// Deep-stage variant (KS K tiles per barrier pair) of a small tile; native layout only.
template <class S, int KS, int NS = 2>
static hipError_t launch_deep(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                              bool out_f32, hipStream_t stream) {
  return out_f32 ? launch_tile<S, kLoopPingPong, true, KS, NS>(W, X, C, ldc, M, N, K, stream)
                 : launch_tile<S, kLoopPingPong, false, KS, NS>(W, X, C, ldc, M, N, K, stream);
}

// The register-staged K-major-weight loop of a small tile with as many K tiles per stage as 128 KiB of LDS
// hold (four for 64 x 64, two for the 128-token tiles): a long reduction wants several K tiles in flight per
// workgroup.
template <class S>
static hipError_t launch_staged_kmajor(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                                       bool out_f32, hipStream_t stream) {
  // Whole stages of two K tiles: the direct-to-LDS ping-pong loop with a ring of as many stages as 128 KiB (144 for
  // the 128 x 64 tile) hold.
  constexpr int kDmaKs = 2;
  constexpr int kDmaNs = S::kStageBytes <= 16 * 1024 ? 4 : S::kStageBytes <= 24 * 1024 ? 3 : 2;
  if (K % (kTileK * kDmaKs) == 0 && K >= kTileK * kDmaKs * kDmaNs)
    return out_f32 ? launch_tile<S, kLoopPingPongKMajor, true, kDmaKs, kDmaNs>(W, X, C, ldc, M, N, K, stream)
                   : launch_tile<S, kLoopPingPongKMajor, false, kDmaKs, kDmaNs>(W, X, C, ldc, M, N, K, stream);
  constexpr int kKs = 128 * 1024 / (2 * S::kStageBytes) >= 4 ? 4 : 2;
  if (K % kTileK != 0)
    return out_f32 ? launch_tile<S, kLoopStagedKMajorTail, true, kKs, 2>(W, X, C, ldc, M, N, K, stream)
                   : launch_tile<S, kLoopStagedKMajorTail, false, kKs, 2>(W, X, C, ldc, M, N, K, stream);
  return out_f32 ? launch_tile<S, kLoopStagedKMajor, true, kKs, 2>(W, X, C, ldc, M, N, K, stream)
                 : launch_tile<S, kLoopStagedKMajor, false, kKs, 2>(W, X, C, ldc, M, N, K, stream);
}

// Tile shapes. Which one runs is a pure performance choice (see det_gemm_tile.h).
using Shape256x256 = TileShape<256, 256, 4, 2>;
using Shape256x256Solo = TileShape<256, 256, 2, 2>;
using Shape192x256 = TileShape<192, 256, 4, 2>;  // 192 features x 256 tokens: three MFMA tiles per wave along N
using Shape192x128 = TileShape<192, 128, 4, 2>;  // 192 features x 128 tokens
using Shape256x128 = TileShape<256, 128, 4, 2>;
using Shape256x64 = TileShape<256, 64, 4, 2>;
using Shape128x128 = TileShape<128, 128, 4, 2>;
using Shape128x64 = TileShape<128, 64, 4, 2>;
using Shape64x64 = TileShape<64, 64, 4, 2>;
using Shape64x16 = TileShape<64, 16, 4, 1>;
using Shape16x16 = TileShape<16, 16, 1, 1>;

static bool view_is_vectorizable(const MatView& v) {
  return v.k_stride == 1 && (v.row_stride % kChunkElems) == 0 && pitch_fits_lane_offsets(v.row_stride) &&
         (reinterpret_cast<uintptr_t>(v.ptr) & 15) == 0;
}

static int64_t tile_count(int M, int N, int bm, int bn) {
  return (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
}

int device_cu_count() {
  static std::atomic<int> cached[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return 256;
  }
  const bool tracked = dev >= 0 && dev < kMaxDevices;
  if (tracked) {
    const int have = cached[dev].load(std::memory_order_relaxed);
    if (have > 0) return have;
  }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess || prop.multiProcessorCount <= 0) {
    (void)hipGetLastError();
    return 256;
  }
  if (tracked) cached[dev].store(prop.multiProcessorCount, std::memory_order_relaxed);
  return prop.multiProcessorCount;
}

// Every tile shape the automatic choice weighs, in one table. `native` is the relative throughput of the shape on a
// full chip with both operands in the native (reduction-contiguous) layout, `w_kmajor` the same with a K-major weight
// (0: the shape has no such loop); `x_kmajor` says whether the shape also takes a K-major activation operand. The
// estimated time of a launch is rounds_of_workgroups(tiles) x tile area / quality; larger tiles win ties.
//
// Native column, fitted to sweeps over the Qwen3-8B projection shapes at 384 ... 6144 tokens: 192 x 256 (three
// quarters of the large tile at 0.89 of its throughput) fills the rounds that N / 256 leaves half empty - gate_up at
// 1024 tokens is 512 tiles = two full rounds instead of 384 = one and a half (169 -> 152 us), qkv at 3072 tokens
// 150 -> 128 us. Where 192 does not divide N its last feature tile is partly empty and the shape counts as
// `ragged192`: it still wins where it turns a round and a fraction into less (N = 5120 at 4096 tokens 293 -> 256 us,
// N = 10240 at 2048 tokens 190 -> 162 us) and loses the tie against 256 x 128 at N = 4096, 2048 tokens. 192 x 128
// (three stages) does the same one size down (weights from HBM: gate_up at 256 tokens 65.0 -> 62.2 us, N = 6144 at 768
// tokens 55.1 -> 49.1 us).
// K-major-weight column (`dY @ W`, `a @ b`, prepared weights): the 64- and 128-feature tiles give a long reduction
// against few output tiles - grad_hidden of the LogP backward up to about a thousand tokens (N = 4096, K = 151936) - a
// workgroup per CU, each streaming a narrow slice of the weight instead of a 256-column one (1.9 -> 0.8 ms at 256
// tokens, 1.8 -> 1.03 ms at 512, 1.65 -> 1.45 ms at 1024); their qualities are those of the direct-to-LDS loop.
struct TileCandidate {
  int config, bn, bm;
  double native, ragged192, w_kmajor;
  bool x_kmajor;
};
static const TileCandidate kTileCandidates[] = {
    {RLK_GEMM_CFG_256x256, 256, 256, 1.00, 0.00, 1.00, true},  {RLK_GEMM_CFG_192x256, 192, 256, 0.89, 0.85, 0.00, false},
    {RLK_GEMM_CFG_256x128, 256, 128, 0.65, 0.00, 0.70, true},  {RLK_GEMM_CFG_192x128, 192, 128, 0.56, 0.53, 0.00, false},
    {RLK_GEMM_CFG_256x64, 256, 64, 0.50, 0.00, 0.56, false},   {RLK_GEMM_CFG_128x128, 128, 128, 0.65, 0.00, 0.62, false},
    {RLK_GEMM_CFG_128x64, 128, 64, 0.45, 0.00, 0.40, false},   {RLK_GEMM_CFG_64x64, 64, 64, 0.42, 0.00, 0.25, false},
};

// The cheapest candidate by the estimate above. `w_kmajor` / `x_kmajor`: the operand layouts of the call.
static int pick_tile_candidate(int M, int N, int K, bool w_kmajor, bool x_kmajor) {
  const int cus = device_cu_count();
  int best = RLK_GEMM_CFG_64x64;
  double best_time = 1e300;
  for (const TileCandidate& c : kTileCandidates) {
    double quality;
    if (w_kmajor || x_kmajor) {
      if (c.w_kmajor == 0.0 || (x_kmajor && !c.x_kmajor)) continue;
      if (c.bn <= 128 && !w_kmajor) continue;  // the small K-major tiles exist for a K-major weight only
      quality = c.w_kmajor;
    } else {
      const bool wide192 = c.ragged192 != 0.0;
      if (wide192 && K % kTileK != 0) continue;
      quality = (wide192 && N % 192 != 0) ? c.ragged192 : c.native;
    }
    const double t = rounds_of_workgroups(tile_count(M, N, c.bm, c.bn), cus) * (double)(c.bn * c.bm) / quality;
    if (t < best_time * 0.999) {
      best_time = t;
      best = c.config;
    }
  }
  return best;
}

int pick_det_gemm_config(int M, int N, int K) {
  const int cus = device_cu_count();
  // Decode (weights fitted while they rotate through 1.3 GB, i.e. come from HBM as in a model with
  // many layers, not from the 256 MB memory-side cache): up to 16 tokens the streaming kernel with
  // two workgroups per CU is the fastest or equal for every Qwen3-8B projection (gate_up 52 -> 38 us,
  // qkv 14 -> 12 us against the one-wave tile kernel, which wins only when the weight is cache
  // resident). Up to 32 / 64 tokens it holds while there are at most 1.5 / 1 panels per CU: a
  // 64-token tile kernel would run on N / 64 CUs only.
  if (M <= 16) return (K >= 1024 && K % kTileK == 0) ? RLK_GEMM_CFG_STREAM16 : RLK_GEMM_CFG_16x16;
  if (K >= 1024 && K % kTileK == 0 && ((M <= 32 && N <= 24 * cus) || (M <= 64 && N <= 16 * cus)))
    return RLK_GEMM_CFG_STREAM64;
  // Problems that give the chip at most one small tile per CU: the deep-stage variants
  // (one workgroup per CU, several K tiles per barrier pair) beat the same tile run several
  // workgroups per CU. Smallest tile first: it spreads the weight stream over most CUs.
  if (K % (kTileK * kDeep64) == 0 && tile_count(M, N, 64, 64) <= cus) return RLK_GEMM_CFG_64x64_DEEP;
  if (K % (kTileK * kDeep128) == 0) {
    if (tile_count(M, N, 64, 128) <= cus) return RLK_GEMM_CFG_128x64_DEEP;
    if (tile_count(M, N, 128, 128) <= cus) return RLK_GEMM_CFG_128x128_DEEP;
  }
  return pick_tile_candidate(M, N, K, false, false);
}

// A K-major view (element [row, k] at ptr[k * k_stride + row], rows contiguous: B[K,N] as the
// weight operand, or the transposed operands of a weight gradient) that the transposing
// ping-pong loop can take.
static bool view_is_kmajor_fast(const MatView& v) {
  return v.row_stride == 1 && v.k_stride >= v.rows && (v.k_stride % kChunkElems) == 0 && pitch_fits_lane_offsets(v.k_stride) &&
         (reinterpret_cast<uintptr_t>(v.ptr) & 15) == 0 && (v.rows % kChunkElems) == 0;
}

// A token count just above a multiple of 256 (4097, 8200 ...) gives the large tiles a last row of token tiles that
// is nearly empty; when that row is what opens another round of workgroups, the few tokens cost a whole tile
// time (down at 4097 tokens: 272 tiles = two rounds instead of one, 0.54 against 0.27 ms). Rows are independent,
// so the remainder can run as a launch of its own on the few-token kernels without changing a bit. Returns
// whether that pays: the round the remainder opens, priced at 11 + 21 K / 1024 us for a 256 x 256 tile
// (measured on gate_up across K), against the few-token launch, which streams the weight once.
static bool remainder_launch_pays(int M, int N, int K, int rest, bool fast_few_tokens, bool w_kmajor) {
  const int64_t cus = device_cu_count();
  const int64_t feature_tiles = (N + 255) / 256;
  const int64_t rounds_all = (feature_tiles * ((M + 255) / 256) + cus - 1) / cus;
  const int64_t rounds_main = (feature_tiles * (M / 256) + cus - 1) / cus;
  if (rounds_all == rounds_main) return false;  // the remainder's tiles fit beside the last round
  const double round_us = 11.0 + 21.0 * K / 1024.0;
  double rest_us;
  if (w_kmajor) {
    rest_us = 10.0 + 0.4 * (K / 64.0);  // register-staged small tiles: a chain of K tiles
  } else if (fast_few_tokens) {
    rest_us = 8.0 + 2.0 * N * (double)K / 4.5e6 * (rest <= 16 ? 1.0 : 1.5);  // the weight once at 4.5 TB/s
  } else {
    return false;
  }
  return rest_us < 0.8 * round_us;
}

hipError_t det_gemm_launch(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                           bool out_f32, int config, hipStream_t stream) {
  if (config == RLK_GEMM_CFG_AUTO && M > 256 && M % 256 >= 1 && M % 256 <= 64) {
    const int rest = M % 256;
    const bool natives = view_is_vectorizable(W) && view_is_vectorizable(X) && K % kTileK == 0 && K >= 1024;
    const bool kmajor_w = !view_is_vectorizable(W) && view_is_kmajor_fast(W) && view_is_vectorizable(X) &&
                          K % kChunkElems == 0;
    if ((natives || kmajor_w) && remainder_launch_pays(M, N, K, rest, natives, kmajor_w)) {
      MatView head = X, tail = X;
      head.rows = M - rest;
      tail.rows = rest;
      tail.ptr = X.ptr + (int64_t)(M - rest) * X.row_stride;
      hipError_t err = det_gemm_launch(W, head, C, ldc, M - rest, N, K, out_f32, config, stream);
      if (err != hipSuccess) return err;
      char* c_tail = reinterpret_cast<char*>(C) + (int64_t)(M - rest) * ldc * (out_f32 ? 4 : 2);
      return det_gemm_launch(W, tail, c_tail, ldc, rest, N, K, out_f32, config, stream);
    }
  }
  if ((config & ~RLK_GEMM_CFG_FORCE_STAGED) == RLK_GEMM_CFG_SHORTK) {
    // Serves a K-major token operand with K <= 256 only (and has no register-staged form); anything else runs
    // the picked tile kernel (same bits).
    if (config == RLK_GEMM_CFG_SHORTK && det_gemm_shortk_supported(W, X, M, N, K))
      return det_gemm_shortk_launch(W, X, C, ldc, M, N, K, out_f32, stream);
    config = RLK_GEMM_CFG_AUTO | (config & RLK_GEMM_CFG_FORCE_STAGED);
  }
  // A weight gradient of up to 256 tokens with many output rows: the feature operand stays in registers.
  if (config == RLK_GEMM_CFG_AUTO && det_gemm_shortk_supported(W, X, M, N, K) && det_gemm_shortk_pays(M, N))
    return det_gemm_shortk_launch(W, X, C, ldc, M, N, K, out_f32, stream);
  const bool w_native = view_is_vectorizable(W), x_native = view_is_vectorizable(X);
  const bool vec = w_native && x_native && (K % kChunkElems) == 0;
  const bool allow_pingpong = (config & RLK_GEMM_CFG_FORCE_STAGED) == 0;
  config &= ~RLK_GEMM_CFG_FORCE_STAGED;
  const bool w_kmajor = !w_native && view_is_kmajor_fast(W), x_kmajor = !x_native && view_is_kmajor_fast(X);
  // A reduction length that 64 does not divide (the token count of a weight gradient) runs its whole K tiles in
  // the same loops and the rest in a register-staged step behind them; a native operand of the pair then
  // needs whole 16-byte chunks (K % 8 == 0).
  const bool k_fits = K >= 1 && ((K % kTileK) == 0 || (w_kmajor && x_kmajor) || (K % kChunkElems) == 0);
  if (allow_pingpong && k_fits && (w_kmajor || x_kmajor) && (w_native || w_kmajor) && (x_native || x_kmajor)) {
    const int loop = w_kmajor ? (x_kmajor ? kLoopPingPongBothKMajor : kLoopPingPongKMajor) : kLoopPingPongXKMajor;
    // Only the shapes with 64-feature wave columns have the transposing loop, and a K-major
    // activation needs at least 128 tokens per tile.
    // With few token tiles against a long reduction (grad_hidden of the LogP backward at 1024 tokens: N = 4096,
    // K = 151936) a smaller token tile doubles the workgroups, every one of which still streams its whole weight panel.
    if (config == RLK_GEMM_CFG_AUTO) config = pick_tile_candidate(M, N, K, w_kmajor, x_kmajor);
    switch (config) {
      case RLK_GEMM_CFG_256x256:
        return launch_shape<Shape256x256>(W, X, C, ldc, M, N, K, false, loop, true, out_f32, stream);
      case RLK_GEMM_CFG_256x128:
        return launch_shape<Shape256x128>(W, X, C, ldc, M, N, K, false, loop, true, out_f32, stream);
      case RLK_GEMM_CFG_256x64:
        if (!x_kmajor) return launch_shape<Shape256x64>(W, X, C, ldc, M, N, K, false, loop, true, out_f32, stream);
        break;
      case RLK_GEMM_CFG_64x64:
        if (w_kmajor && x_native) return launch_staged_kmajor<Shape64x64>(W, X, C, ldc, M, N, K, out_f32, stream);
        break;
      case RLK_GEMM_CFG_128x64:
        if (w_kmajor && x_native) return launch_staged_kmajor<Shape128x64>(W, X, C, ldc, M, N, K, out_f32, stream);
        break;
      case RLK_GEMM_CFG_128x128:
        if (w_kmajor && x_native) return launch_staged_kmajor<Shape128x128>(W, X, C, ldc, M, N, K, out_f32, stream);
        break;
      default:
        break;  // an explicitly requested other shape runs the element-wise loader below
    }
  }
  if (config == RLK_GEMM_CFG_AUTO) config = pick_det_gemm_config(M, N, K);
  if (config == RLK_GEMM_CFG_STREAM16_DEEP || config == RLK_GEMM_CFG_STREAM16 || config == RLK_GEMM_CFG_STREAM64) {
    // The streaming kernel serves up to 16 (STREAM16*) or 64 tokens and needs the fast layout;
    // otherwise a tile kernel computes the same bits.
    const int max_m = config == RLK_GEMM_CFG_STREAM64 ? 64 : 16;
    if (M <= max_m && vec && allow_pingpong && K % kTileK == 0)
      return det_gemm_stream_launch(W, X, C, ldc, M, N, K, out_f32, config == RLK_GEMM_CFG_STREAM16, stream);
    config = M <= 16 ? RLK_GEMM_CFG_16x16 : M <= 64 ? RLK_GEMM_CFG_64x64 : pick_det_gemm_config(M, N, K);
    if (config == RLK_GEMM_CFG_STREAM64) config = RLK_GEMM_CFG_64x64;
  }
  // Deep-stage variants need the fast layout and whole stages; otherwise the plain shape
  // computes the same bits.
  if (config == RLK_GEMM_CFG_64x64_DEEP || config == RLK_GEMM_CFG_128x64_DEEP || config == RLK_GEMM_CFG_128x128_DEEP) {
    const int ks = config == RLK_GEMM_CFG_64x64_DEEP ? kDeep64 : kDeep128;
    if (vec && allow_pingpong && K % (kTileK * ks) == 0) {
      if (config == RLK_GEMM_CFG_64x64_DEEP) return launch_deep<Shape64x64, kDeep64>(W, X, C, ldc, M, N, K, out_f32, stream);
      if (config == RLK_GEMM_CFG_128x64_DEEP) return launch_deep<Shape128x64, kDeep128, 3>(W, X, C, ldc, M, N, K, out_f32, stream);
      return launch_deep<Shape128x128, kDeep128>(W, X, C, ldc, M, N, K, out_f32, stream);
    }
    config = config == RLK_GEMM_CFG_64x64_DEEP    ? RLK_GEMM_CFG_64x64
             : config == RLK_GEMM_CFG_128x64_DEEP ? RLK_GEMM_CFG_128x64
                                                  : RLK_GEMM_CFG_128x128;
  }
  // The element-wise loader of the generic path keeps eight values per chunk in
  // flight; the largest shapes would spill registers with it.
  if (!vec && (config == RLK_GEMM_CFG_256x256 || config == RLK_GEMM_CFG_256x128 || config == RLK_GEMM_CFG_256x64))
    config = RLK_GEMM_CFG_128x128;
  if (config == RLK_GEMM_CFG_256x256_SOLO) {
    if (vec && allow_pingpong && K % kTileK == 0)
      return launch_loop<Shape256x256Solo, kLoopSolo>(W, X, C, ldc, M, N, K, out_f32, stream);
    config = RLK_GEMM_CFG_256x256;
  }
  if (config == RLK_GEMM_CFG_192x128) {
    if (vec && allow_pingpong && K % kTileK == 0)
      return launch_loop<Shape192x128, kLoopPingPong, pingpong_stages<Shape192x128>()>(W, X, C, ldc, M, N, K, out_f32, stream);
    config = RLK_GEMM_CFG_256x128;
  }
  if (config == RLK_GEMM_CFG_192x256) {
    if (vec && allow_pingpong && K % kTileK == 0)
      return launch_loop<Shape192x256, kLoopPingPong>(W, X, C, ldc, M, N, K, out_f32, stream);
    config = RLK_GEMM_CFG_256x256;
  }
  switch (config) {
    case RLK_GEMM_CFG_256x256:
      return launch_shape<Shape256x256>(W, X, C, ldc, M, N, K, vec, 0, allow_pingpong, out_f32, stream);
    case RLK_GEMM_CFG_256x128:
      return launch_shape<Shape256x128>(W, X, C, ldc, M, N, K, vec, 0, allow_pingpong, out_f32, stream);
    case RLK_GEMM_CFG_256x64:
      return launch_shape<Shape256x64>(W, X, C, ldc, M, N, K, vec, 0, allow_pingpong, out_f32, stream);
    case RLK_GEMM_CFG_128x128:
      return launch_shape<Shape128x128>(W, X, C, ldc, M, N, K, vec, 0, allow_pingpong, out_f32, stream);
    case RLK_GEMM_CFG_128x64:
      return launch_shape<Shape128x64>(W, X, C, ldc, M, N, K, vec, 0, allow_pingpong, out_f32, stream);
    case RLK_GEMM_CFG_64x64:
      return launch_shape<Shape64x64>(W, X, C, ldc, M, N, K, vec, 0, allow_pingpong, out_f32, stream);
    case RLK_GEMM_CFG_64x16:
      return launch_shape<Shape64x16>(W, X, C, ldc, M, N, K, vec, 0, allow_pingpong, out_f32, stream);
    case RLK_GEMM_CFG_16x16:
      return launch_shape<Shape16x16>(W, X, C, ldc, M, N, K, vec, 0, allow_pingpong, out_f32, stream);
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace rlk
