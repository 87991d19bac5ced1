// The LDS-tiled MFMA main loop shared by det_gemm and the fused linear-LogP.
//
// Arithmetic contract (the part that decides output bits):
//   * bf16 operands, products and sums in fp32 on v_mfma_f32_16x16x32_bf16;
//   * one fp32 accumulator per output element, started at +0, updated by
//     K/32 MFMA steps in ascending K order (the K tail is zero filled in both
//     operands up to the next multiple of 64);
//   * inside one step, k slot 8*(lane>>4)+e of the instruction always carries
//     element k0 + 8*(lane>>4) + e of both operands.
// Tile shape, wave count, pipelining, grid order and the row/column an element
// occupies inside a tile are not part of it: every configuration below runs the
// same chain for a given output element, so results do not depend on M, on the
// position of a row in the batch, or on the configuration picked.
//
// Orientation: the weight operand W[N,K] feeds the MFMA row side ("P"), the
// activation operand X[M,K] the column side ("Q"). A lane then owns one token
// (column) and a run of consecutive output features, which makes the C store a
// contiguous run per lane and keeps the LogP row reductions inside a lane.
#pragma once

#include "rlk_device.h"

namespace rlk {

template <int BN_, int BM_, int WN_, int WM_>
struct TileShape {
  static constexpr int BN = BN_;  // weight rows (output features) per workgroup
  static constexpr int BM = BM_;  // activation rows (tokens) per workgroup
  static constexpr int WN = WN_;  // waves along N
  static constexpr int WM = WM_;  // waves along M
  static constexpr int kThreads = kWave * WN * WM;
  static constexpr int TN = BN / (16 * WN);  // MFMA tiles per wave along N
  static constexpr int TM = BM / (16 * WM);  // MFMA tiles per wave along M
  static constexpr int kRun = 4 * TN;        // consecutive features one lane owns
  static constexpr int kWChunks = BN * kRowChunks;
  static constexpr int kXChunks = BM * kRowChunks;
  static constexpr int kWIters = (kWChunks + kThreads - 1) / kThreads;
  static constexpr int kXIters = (kXChunks + kThreads - 1) / kThreads;
  static constexpr int kStageBytes = (BN + BM) * kRowBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes;
  static_assert(BN % (16 * WN) == 0 && BM % (16 * WM) == 0, "wave tiles are whole MFMA tiles");
};

// A strided bf16 matrix whose rows are the non-reduction index.
struct MatView {
  const bf16_bits* ptr;
  int64_t row_stride;  // elements between consecutive rows
  int64_t k_stride;    // elements between consecutive k
  int rows;
};

// LDS row r of the weight stage holds feature perm(r) of the tile: lane group
// g = (lane>>4) of MFMA tile jn owns accumulator rows 4g..4g+3, and mapping them
// to features g*4*TN + jn*4 + q gives every lane one contiguous run of 4*TN.
template <class S>
__device__ __forceinline__ int weight_row_of_lds_row(int r) {
  constexpr int kWaveRows = 16 * S::TN;
  const int wn = r / kWaveRows;
  const int in_wave = r % kWaveRows;
  const int jn = in_wave / 16;
  const int i = in_wave % 16;
  return wn * kWaveRows + (i >> 2) * S::kRun + jn * 4 + (i & 3);
}

// Global -> register staging of one K tile of one operand.
template <int ITERS, int CHUNKS, int THREADS, bool VEC>
struct Stager {
  const bf16_bits* src[ITERS];  // row base pointers (k = 0) of this thread's chunks
  int lds_off[ITERS];
  int chunk_k[ITERS];  // first k of the chunk inside a tile
  u32x4_t regs[ITERS];
  int64_t k_stride;

  template <class RowMap>
  __device__ __forceinline__ void init(const MatView& m, int row0, int tid, RowMap row_map) {
    k_stride = m.k_stride;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      int ci = tid + i * THREADS;
      if (CHUNKS % THREADS != 0 && ci >= CHUNKS) ci = CHUNKS - 1;  // duplicate work, same value
      const int r = ci / kRowChunks;
      const int c = ci % kRowChunks;
      int grow = row0 + row_map(r);
      grow = grow < m.rows ? grow : m.rows - 1;  // rows past the edge are computed, never stored
      src[i] = m.ptr + (int64_t)grow * m.row_stride;
      lds_off[i] = lds_chunk_offset(r, c);
      chunk_k[i] = c * kChunkElems;
    }
  }

  // Issue the loads of K tile starting at k0. TAIL handles k >= K by zero fill.
  template <bool TAIL>
  __device__ __forceinline__ void load(int k0, int K) {
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int k = k0 + chunk_k[i];
      if (VEC) {
        if (TAIL) {
          const bool ok = k < K;  // K % 8 == 0 on this path: a chunk is all in or all out
          u32x4_t v = *reinterpret_cast<const u32x4_t*>(src[i] + (ok ? k : 0));
          const u32x4_t z = {0u, 0u, 0u, 0u};
          regs[i] = ok ? v : z;
        } else {
          regs[i] = *reinterpret_cast<const u32x4_t*>(src[i] + k);
        }
      } else {
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int ka = k + 2 * e, kb = k + 2 * e + 1;
          const uint32_t lo = (!TAIL || ka < K) ? src[i][(int64_t)(ka < K ? ka : 0) * k_stride] : 0;
          const uint32_t hi = (!TAIL || kb < K) ? src[i][(int64_t)(kb < K ? kb : 0) * k_stride] : 0;
          w[e] = lo | (hi << 16);
        }
        regs[i] = u32x4_t{w[0], w[1], w[2], w[3]};
      }
    }
  }

  __device__ __forceinline__ void store(char* lds_stage, int tid) {
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      if (CHUNKS % THREADS == 0 || tid + i * THREADS < CHUNKS)
        *reinterpret_cast<u32x4_t*>(lds_stage + lds_off[i]) = regs[i];
    }
  }
};

// Runs the whole K loop for one (feature tile, token tile) and leaves the fp32
// accumulators in registers. acc[jn][jm][q] is feature
//   n0 + wave_n*16*TN + (lane>>4)*4*TN + jn*4 + q
// of token
//   m0 + wave_m*16*TM + jm*16 + (lane&15).
template <class S, bool VEC>
__device__ __forceinline__ void tile_mainloop(const MatView& W, const MatView& X, int n0, int m0, int K,
                                              char* lds, f32x4_t (&acc)[S::TN][S::TM]) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_n = wave % S::WN;
  const int wave_m = wave / S::WN;

  Stager<S::kWIters, S::kWChunks, S::kThreads, VEC> sw;
  Stager<S::kXIters, S::kXChunks, S::kThreads, VEC> sx;
  sw.init(W, n0, tid, [](int r) { return weight_row_of_lds_row<S>(r); });
  sx.init(X, m0, tid, [](int r) { return r; });

#pragma unroll
  for (int jn = 0; jn < S::TN; ++jn)
#pragma unroll
    for (int jm = 0; jm < S::TM; ++jm) acc[jn][jm] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // Fragment read offsets: row (l&15) of each MFMA tile, chunk (s*4 + (l>>4)).
  const int l16 = lane & 15;
  const int grp = lane >> 4;
  const int frag_lo = (grp ^ (l16 & 7)) << 4;  // s = 0; s = 1 flips bit 6
  const int w_row_base = (wave_n * 16 * S::TN + l16) * kRowBytes;
  const int x_row_base = S::BN * kRowBytes + (wave_m * 16 * S::TM + l16) * kRowBytes;

  const int nk = (K + kTileK - 1) / kTileK;
  const bool ragged = (K % kTileK) != 0;

  if (nk == 1 && ragged) {
    sw.template load<true>(0, K);
    sx.template load<true>(0, K);
  } else {
    sw.template load<false>(0, K);
    sx.template load<false>(0, K);
  }
  sw.store(lds, tid);
  sx.store(lds + S::BN * kRowBytes, tid);
  __syncthreads();

  for (int kt = 0; kt < nk; ++kt) {
    char* cur = lds + (kt & 1) * S::kStageBytes;
    char* nxt = lds + ((kt + 1) & 1) * S::kStageBytes;
    const bool more = kt + 1 < nk;
    if (more) {
      const int k0 = (kt + 1) * kTileK;
      if (ragged && kt + 2 == nk) {
        sw.template load<true>(k0, K);
        sx.template load<true>(k0, K);
      } else {
        sw.template load<false>(k0, K);
        sx.template load<false>(k0, K);
      }
    }
#pragma unroll
    for (int s = 0; s < kTileK / kMfmaK; ++s) {
      const int frag = frag_lo ^ (s << 6);
      u32x4_t wf[S::TN], xf[S::TM];
#pragma unroll
      for (int jn = 0; jn < S::TN; ++jn)
        wf[jn] = *reinterpret_cast<const u32x4_t*>(cur + w_row_base + jn * 16 * kRowBytes + frag);
#pragma unroll
      for (int jm = 0; jm < S::TM; ++jm)
        xf[jm] = *reinterpret_cast<const u32x4_t*>(cur + x_row_base + jm * 16 * kRowBytes + frag);
#pragma unroll
      for (int jn = 0; jn < S::TN; ++jn)
#pragma unroll
        for (int jm = 0; jm < S::TM; ++jm) acc[jn][jm] = mfma_16x16x32(wf[jn], xf[jm], acc[jn][jm]);
    }
    if (more) {
      sw.store(nxt, tid);
      sx.store(nxt + S::BN * kRowBytes, tid);
    }
    __syncthreads();
  }
}

}  // namespace rlk
