// det_gemm for a short reduction against many output rows: the weight gradient of a small batch,
// dW[N_out, N_in] = dY[T, N_out]^T x A[T, N_in] with T <= 256 tokens.
//
// Such a GEMM is a write of the output with a little arithmetic per element (at 256 tokens the 1.2 GB
// lm_head gradient is 0.18 ms of stores and 0.13 ms of MFMA work). The tile kernels spend most of their time
// per tile outside the K loop there (first loads, epilogue, workgroup turnover: 11 of 18 us for a
// 256 x 256 tile with four K tiles), and nothing overlaps those phases. Here a workgroup keeps the
// feature operand of 256 output columns in registers for the whole reduction (64 features x K per wave,
// gathered once), and streams the token operand through a ring of NS LDS stages (two; deeper rings measured the
// same), 64 tokens at a time: the loads of the following tile are in flight while a tile is multiplied and
// stored, and no phase waits for a workgroup to start. Same instruction, same ascending 32-wide K steps from a zero accumulator as every
// other det_gemm kernel, so the bits are the same.
//
// The token operand must be K-major (x[k * ld + m], tokens contiguous, as the transposed operand of a weight
// gradient is) with K % 64 == 0 and K <= 256; the feature operand may have any strides.
#include "det_gemm_tile.h"
#include "rlk_host.h"

namespace rlk {

constexpr int kShortKTokens = 64;     // tokens of one streamed tile (one K-major column)
constexpr int kShortKFeatures = 256;  // features of a workgroup: 64 per wave
constexpr int kShortKXcds = 8;

// The fragments of 16-token sub-tile j of a stage (KT K-major columns of 64 K rows, one per K tile).
template <int STEPS>
__device__ __forceinline__ void read_shortk_subtile(const char* stage, int j, int l16, int grp, u32x4_t (&dst)[STEPS]) {
#pragma unroll
  for (int s = 0; s < STEPS; ++s)
    dst[s] = read_kmajor_fragment(stage + (s >> 1) * (kTileK * kRowBytes), j, s & 1, l16, grp);
}

// KT = K / 64. Workgroup id -> (feature block, chunk of token tiles) such that the feature blocks of one chunk
// run on one XCD at the same time: they read the same token tiles, one from the fabric and the rest from L2.
template <int KT, bool OUT_F32, int NS>
__global__ __launch_bounds__(256, (NS * KT > 8 ? 1 : 2)) void det_gemm_shortk_kernel(MatView W, MatView X,
                                                                                      void* __restrict__ C, int64_t ldc,
                                                                                      int M, int N, int n_blocks,
                                                                                      int tiles_per_chunk,
                                                                                      int vec_store) {
  constexpr int kSteps = 2 * KT;                         // MFMA steps of the reduction
  constexpr int kStageBytes = KT * kTileK * kRowBytes;   // 64 tokens x K
  constexpr int kLoads = 2 * KT;                         // 1 KiB blocks per wave and stage
  constexpr int kStores = OUT_F32 ? 4 : 2;               // 16-byte stores per lane and 16-token sub-tile
  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15;
  const int grp = lane >> 4;

  const int xcd = blockIdx.x % kShortKXcds;
  const int slot = blockIdx.x / kShortKXcds;
  const int n_block = slot % n_blocks;
  const int chunk = xcd + kShortKXcds * (slot / n_blocks);
  const int m_tiles = (M + kShortKTokens - 1) / kShortKTokens;
  const int t_begin = chunk * tiles_per_chunk;
  const int t_end = t_begin + tiles_per_chunk < m_tiles ? t_begin + tiles_per_chunk : m_tiles;
  if (t_begin >= t_end) return;  // the whole workgroup leaves before any barrier

  const int n_wave = n_block * kShortKFeatures + wave * 64;
  const bool interior = vec_store != 0 && (n_block + 1) * kShortKFeatures <= N && t_end * kShortKTokens <= M;

  // The stationary operand. Which feature of the wave's 64 an MFMA tile takes as its row r is free; a lane
  // holds rows 4 grp .. 4 grp + 3 of every tile jn. bf16: tiles 2 h and 2 h + 1 give the lane the eight
  // consecutive features 32 h + 8 grp .. + 7, so one 16-byte store per lane writes 64 contiguous bytes per
  // token across the four lane groups. fp32: tile jn gives features 16 jn + 4 grp .. + 3, again 64 bytes per token
  // and store. Features past N are zeros.
  auto feature_of_row = [](int jn, int r) {
    return OUT_F32 ? jn * 16 + r : (jn >> 1) * 32 + (r >> 2) * 8 + (jn & 1) * 4 + (r & 3);
  };
  u32x4_t wf[kSteps][4];
#pragma unroll
  for (int jn = 0; jn < 4; ++jn) {
    const int f = n_wave + feature_of_row(jn, l16);
    const bool live = f < N;
    const bf16_bits* row = W.ptr + (int64_t)(live ? f : 0) * W.row_stride;
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      uint32_t v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int k = s * kMfmaK + grp * 8 + 2 * e;
        const uint32_t lo = row[(int64_t)k * W.k_stride];
        const uint32_t hi = row[(int64_t)(k + 1) * W.k_stride];
        v[e] = live ? (lo | (hi << 16)) : 0u;
      }
      wf[s][jn] = u32x4_t{v[0], v[1], v[2], v[3]};
    }
  }
  asm volatile("" ::: "memory");

  // Token tile t -> a stage: K tile kt is a K-major column (64 K rows of 128 bytes, the layout of
  // read_kmajor_fragment); a block is 8 K rows, lane -> (K row lane >> 3, chunk position lane & 7).
  const int rib = lane >> 3;
  const int kmajor_chunk = (lane & 7) ^ kmajor_swizzle_of_row_in_block(rib);
  const int64_t ldk = X.k_stride;
  auto issue = [&](int t, char* stage) {
    const int m0 = t * kShortKTokens;
    const int last = M - kChunkElems - m0;  // tokens past the edge are computed from valid data, never stored
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
      const int b = wave * kLoads + j;
      const int kt = b >> 3;
      const int kblk = b & 7;
      int at = (kmajor_chunk ^ kmajor_swizzle_of_block(kblk)) * kChunkElems;
      at = at < last ? at : last;
      const bf16_bits* src = X.ptr + (int64_t)(kt * kTileK + kblk * 8 + rib) * ldk + m0 + at;
      __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(stage + b * 1024), 16, 0, 0);
    }
  };
  auto clamped = [&](int t) { return t < t_end ? t : t_end - 1; };

  // A tile past the chunk re-fetches the last one into a stage nobody reads any more, so the number of
  // loads in flight is the same in every iteration.
#pragma unroll
  for (int i = 0; i < NS; ++i) issue(clamped(t_begin + i), lds + i * kStageBytes);
  __builtin_amdgcn_s_waitcnt(wait_vmcnt((NS - 1) * kLoads));  // my part of the first tile has landed

  // INTERIOR: every 16-byte store of the chunk lies inside the output, so the number of stores per tile is
  // fixed and the loads can be counted past them.
  auto stream_tiles = [&](auto interior_tag) {
    constexpr bool INTERIOR = decltype(interior_tag)::value;
    u32x4_t xf[2][kSteps];
    for (int t = t_begin; t < t_end; ++t) {
      char* stage = lds + ((t - t_begin) % NS) * kStageBytes;
      wg_barrier();  // every wave's part of tile t has landed
      read_shortk_subtile<kSteps>(stage, 0, l16, grp, xf[0]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (j < 3) {
          read_shortk_subtile<kSteps>(stage, j + 1, l16, grp, xf[(j + 1) & 1]);
        } else {
          __builtin_amdgcn_s_waitcnt(kWaitLgkm0);  // all my fragments of tile t are in registers
          wg_barrier();                            // ... and everybody else's: the stage is free
          issue(clamped(t + NS), stage);
        }
        f32x4_t acc[4];
#pragma unroll
        for (int jn = 0; jn < 4; ++jn) acc[jn] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < kSteps; ++s)
#pragma unroll
          for (int jn = 0; jn < 4; ++jn) acc[jn] = mfma_16x16x32(wf[s][jn], xf[j & 1][s], acc[jn]);

        const int m = t * kShortKTokens + j * 16 + l16;
        if constexpr (INTERIOR) {
          if constexpr (OUT_F32) {
            float* dst = reinterpret_cast<float*>(C) + (int64_t)m * ldc + n_wave + grp * 4;
#pragma unroll
            for (int jn = 0; jn < 4; ++jn) __builtin_nontemporal_store(acc[jn], reinterpret_cast<f32x4_t*>(dst + jn * 16));
          } else {
            // (Non-temporal stores: ordinary ones push the token tiles, which the 16 feature blocks of a chunk
            // share through the L2, out of it; every workgroup then waits for the tile to come through the
            // fabric again, and a slow load holds up the stores queued behind it: 462 -> 412 us at 256 tokens,
            // 292 -> 207 us at 64 for the lm_head gradient.)
            // The lane holds, of token l16, features 8 grp .. + 7 (lo) and 32 + 8 grp .. + 7 (hi). Lanes l16 and
            // l16 ^ 8 swap one of the two, so that a store writes whole 128-byte lines: the first one tokens
            // 0-7 of the sub-tile (lanes l16 >= 8 carry the upper 32 features), the second one tokens 8-15.
            const u32x4_t lo = {pack_bf16x2(acc[0][0], acc[0][1]), pack_bf16x2(acc[0][2], acc[0][3]),
                                pack_bf16x2(acc[1][0], acc[1][1]), pack_bf16x2(acc[1][2], acc[1][3])};
            const u32x4_t hi = {pack_bf16x2(acc[2][0], acc[2][1]), pack_bf16x2(acc[2][2], acc[2][3]),
                                pack_bf16x2(acc[3][0], acc[3][1]), pack_bf16x2(acc[3][2], acc[3][3])};
            const bool low_half = l16 < 8;
            u32x4_t first, second;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const uint32_t send = low_half ? hi[e] : lo[e];
              // row_ror:8 — lane i of a row of 16 reads lane i ^ 8
              const uint32_t got = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)send, 0x128, 0xf, 0xf, false);
              first[e] = low_half ? lo[e] : got;
              second[e] = low_half ? got : hi[e];
            }
            const int m8 = t * kShortKTokens + j * 16 + (l16 & 7);
            bf16_bits* dst = reinterpret_cast<bf16_bits*>(C) + (int64_t)m8 * ldc + n_wave + (l16 >> 3) * 32 + grp * 8;
            __builtin_nontemporal_store(first, reinterpret_cast<u32x4_t*>(dst));
            __builtin_nontemporal_store(second, reinterpret_cast<u32x4_t*>(dst + 8 * ldc));
          }
        } else if (m < M) {
#pragma unroll
          for (int jn = 0; jn < 4; ++jn)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int nn = n_wave + feature_of_row(jn, grp * 4 + q);
              if (nn >= N) continue;
              if constexpr (OUT_F32) {
                reinterpret_cast<float*>(C)[(int64_t)m * ldc + nn] = acc[jn][q];
              } else {
                reinterpret_cast<bf16_bits*>(C)[(int64_t)m * ldc + nn] = to_bf16_bits(acc[jn][q]);
              }
            }
        }
      }
      // My part of tile t + 1 has landed. Vector memory operations retire in order. Behind the loads of tile
      // t + 1 this wave has issued, per iteration since, the stores of sub-tiles 0-2, the loads of a later
      // tile and the stores of sub-tile 3: NS - 1 such iterations and one more set of last stores when those
      // loads came from the loop, the other prologue loads and at least one iteration when they came from the
      // prologue. With an unknown number of stores only the later tiles' loads may stay in flight.
      constexpr int kSteady = kStores + (NS - 1) * (4 * kStores + kLoads);
      constexpr int kEarly = (NS - 1) * kLoads + 4 * kStores;
      if (!INTERIOR) {
        __builtin_amdgcn_s_waitcnt(wait_vmcnt((NS - 1) * kLoads));
      } else if (t - t_begin >= NS - 1) {
        __builtin_amdgcn_s_waitcnt(wait_vmcnt(kSteady < 63 ? kSteady : 63));
      } else {
        __builtin_amdgcn_s_waitcnt(wait_vmcnt(kEarly < 63 ? kEarly : 63));
      }
    }
  };
  if (interior) {
    stream_tiles(BoolTag<true>{});
  } else {
    stream_tiles(BoolTag<false>{});
  }
  __builtin_amdgcn_s_waitcnt(kWaitAll0);  // no load may land in this LDS after the workgroup has left
}

bool det_gemm_shortk_supported(const MatView& W, const MatView& X, int M, int N, int K) {
  (void)W;
  (void)N;
  return K >= kTileK && K <= 4 * kTileK && K % kTileK == 0 && M >= kChunkElems && X.row_stride == 1 &&
         X.k_stride >= X.rows && (X.k_stride % kChunkElems) == 0 && (X.rows % kChunkElems) == 0 &&
         (reinterpret_cast<uintptr_t>(X.ptr) & 15) == 0;
}

// Token tiles per workgroup when the grid is two workgroups per CU (one for the deepest stages); chunks of token
// tiles come in eights, one per XCD.
static int shortk_tiles_per_chunk(int M, int N, int per_cu) {
  const int n_blocks = (N + kShortKFeatures - 1) / kShortKFeatures;
  const int m_tiles = (M + kShortKTokens - 1) / kShortKTokens;
  int chunks = (per_cu * device_cu_count() + n_blocks - 1) / n_blocks;
  chunks = (chunks + kShortKXcds - 1) / kShortKXcds * kShortKXcds;
  const int tiles = (m_tiles + chunks - 1) / chunks;
  return tiles < 1 ? 1 : tiles;
}

// Gathering the stationary operand and filling the ring cost a workgroup about as much as three token tiles:
// measured against the tile kernels the streaming kernel wins from six tiles per workgroup on (24576 x 4096 at
// 256 tokens 68 against 100 us, 12288 x 4096 at 128 tokens 26 against 43 us) and loses below (6144 x 4096 at 256
// tokens 38 against 34 us, 4096 x 12288 107 against 55 us).
bool det_gemm_shortk_pays(int M, int N) { return shortk_tiles_per_chunk(M, N, 2) >= 6; }

template <int KT, bool OUT_F32, int NS>
static hipError_t launch_shortk_ns(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N,
                                hipStream_t stream) {
  auto kernel = det_gemm_shortk_kernel<KT, OUT_F32, NS>;
  constexpr int kLds = NS * KT * kTileK * kRowBytes;
  constexpr int kPerCu = NS * KT > 8 ? 1 : 2;
  static PerDeviceOnce once;
  hipError_t err = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), kLds, once);
  if (err != hipSuccess) return err;
  const int n_blocks = (N + kShortKFeatures - 1) / kShortKFeatures;
  const int m_tiles = (M + kShortKTokens - 1) / kShortKTokens;
  const int tiles_per_chunk = shortk_tiles_per_chunk(M, N, kPerCu);
  const int chunks = (m_tiles + tiles_per_chunk - 1) / tiles_per_chunk;
  const int chunk_rounds = (chunks + kShortKXcds - 1) / kShortKXcds;
  const int elem = OUT_F32 ? 4 : 2;
  const int vec_store = (reinterpret_cast<uintptr_t>(C) % 16 == 0 && (ldc * elem) % 16 == 0) ? 1 : 0;
  hipLaunchKernelGGL(kernel, dim3(kShortKXcds * n_blocks * chunk_rounds), dim3(256), kLds, stream, W, X, C, ldc, M, N,
                     n_blocks, tiles_per_chunk, vec_store);
  return hipGetLastError();
}

template <int KT, bool OUT_F32>
static hipError_t launch_shortk(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N,
                                hipStream_t stream) {
  return launch_shortk_ns<KT, OUT_F32, 2>(W, X, C, ldc, M, N, stream);
}

hipError_t det_gemm_shortk_launch(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                                  bool out_f32, hipStream_t stream) {
  if (!det_gemm_shortk_supported(W, X, M, N, K)) return hipErrorInvalidValue;
  switch (K / kTileK) {
    case 1:
      return out_f32 ? launch_shortk<1, true>(W, X, C, ldc, M, N, stream)
                     : launch_shortk<1, false>(W, X, C, ldc, M, N, stream);
    case 2:
      return out_f32 ? launch_shortk<2, true>(W, X, C, ldc, M, N, stream)
                     : launch_shortk<2, false>(W, X, C, ldc, M, N, stream);
    case 3:
      return out_f32 ? launch_shortk<3, true>(W, X, C, ldc, M, N, stream)
                     : launch_shortk<3, false>(W, X, C, ldc, M, N, stream);
    default:
      return out_f32 ? launch_shortk<4, true>(W, X, C, ldc, M, N, stream)
                     : launch_shortk<4, false>(W, X, C, ldc, M, N, stream);
  }
}

}  // namespace rlk
