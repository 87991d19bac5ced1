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

// Swizzle of the 16-byte chunk position inside a K row of a K-major stage (a 64-wide column of 64 K rows
// of 128 bytes): keeps both the 16-byte stores / direct loads and the transposing fragment reads free of
// bank conflicts. A transposing read takes 8 bytes per lane; of a fragment's lanes, lane group g reads K rows
// 8 g + 4 h + a (a = 0..3) and, in a row, the 32 bytes of its MFMA tile. The bank of a lane's 8 bytes is
// 32 (k & 1) + 4 chunk + 2 (lane & 1), so the 32 lanes the LDS serves together must differ in (k & 1, chunk): bit 2
// of the chunk position takes bit 1 of the K row and bit 1 takes the parity of the lane group, whichever two
// groups share a pass (0-1 / 2-3 or 0-2 / 1-3). (A swizzle that told apart only groups 0-2 / 1-3 measured one
// conflict cycle per read: SQ_LDS_BANK_CONFLICT equal to a third of the LDS-busy cycles with a K-major weight and
// to half of them with both operands K-major.)
__device__ __forceinline__ int kmajor_swizzle(int k_row) {
  return 4 * ((k_row >> 1) & 1) + 2 * (((k_row >> 3) ^ (k_row >> 4)) & 1);
}
// The same for the direct-to-LDS loads, which move blocks of 8 K rows (K row 8 kblk + rib of a tile): the part of
// the swizzle that depends on the lane's K row inside a block, and the part that depends on the block.
__device__ __forceinline__ int kmajor_swizzle_of_row_in_block(int rib) { return 4 * ((rib >> 1) & 1); }
__device__ __forceinline__ int kmajor_swizzle_of_block(int kblk) { return 2 * ((kblk ^ (kblk >> 1)) & 1); }

// The MFMA fragment of 16-row tile `j16` of a K-major column for K step `step`: ds_read_b64_tr_b16 hands lane r
// of a 16-lane group the four K values of row r out of 4 K rows x 16 rows.
// `col` is restrict-qualified (nothing writes the column while this function reads it) for what that does to the
// generated waits: in front of an LDS read that carries no alias information (this intrinsic, unlike a plain
// vector load) the compiler waits for every direct-to-LDS load in flight, which made a wave that prefetches the
// next stage wait for it before reading the current one. With the qualifier the reads carry an alias scope and
// only the hand-placed waits of the loops remain, as for the native layout.
__device__ __forceinline__ u32x4_t read_kmajor_fragment(const char* __restrict__ col, int j16, int step, int l16,
                                                        int grp) {
  typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
  typedef __attribute__((address_space(3))) bf16x4_t* lds_bf16x4_ptr_t;
  u32x2_t half[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int k_row = step * 32 + grp * 8 + h * 4 + (l16 >> 2);
    const int chunk = (2 * j16 + ((l16 & 3) >> 1)) ^ kmajor_swizzle(k_row);
    const char* p = col + k_row * kRowBytes + chunk * 16 + (l16 & 1) * 8;
    half[h] = __builtin_bit_cast(u32x2_t, __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4_ptr_t)p));
  }
  return u32x4_t{half[0].x, half[0].y, half[1].x, half[1].y};
}

// Global -> register staging of one K tile of a K-major operand (w[k * ld + n], rows contiguous; the weight
// B[K, N], or an activation stored token-contiguous): a thread's chunk is 8 consecutive rows at one k, stored
// into the K-major stage layout above. Needs rows % 8 == 0 and 16-byte aligned K rows. load<true> fills the
// K rows at and past K with zeros (their address is clamped to K row 0, which always exists).
template <int ITERS, int CHUNKS, int THREADS>
struct KMajorStager {
  const bf16_bits* src[ITERS];  // chunk source at K row 0
  int krow[ITERS];              // K row of the chunk inside a tile
  int lds_off[ITERS];
  u32x4_t regs[ITERS];
  int64_t ld;

  __device__ __forceinline__ void init(const MatView& w, int n0, int tid) {
    ld = w.k_stride;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      int ci = tid + i * THREADS;
      if (CHUNKS % THREADS != 0 && ci >= CHUNKS) ci = CHUNKS - 1;  // duplicate work, same value
      const int col = ci / (kTileK * kRowChunks);
      const int k = (ci / kRowChunks) % kTileK;
      const int c = ci % kRowChunks;
      int n = n0 + col * 64 + c * kChunkElems;
      n = n + kChunkElems <= w.rows ? n : w.rows - kChunkElems;  // features past the edge are computed, never stored
      src[i] = w.ptr + n;
      krow[i] = k;
      lds_off[i] = col * (kTileK * kRowBytes) + k * kRowBytes + ((c ^ kmajor_swizzle(k)) << 4);
    }
  }
  template <bool TAIL>
  __device__ __forceinline__ void load(int k0, int K) {
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int k = k0 + krow[i];
      if constexpr (TAIL) {
        const bool ok = k < K;
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(src[i] + (int64_t)(ok ? k : 0) * ld);
        const u32x4_t z = {0u, 0u, 0u, 0u};
        regs[i] = ok ? v : z;
      } else {
        regs[i] = *reinterpret_cast<const u32x4_t*>(src[i] + (int64_t)k * ld);
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

template <int V>
struct IntTag {
  static constexpr int value = V;
};

// The register-staged loop with a K-major weight operand (B[K, N], N contiguous) for the small tiles, which
// have no direct-to-LDS K-major loop: 16-byte loads of eight features at one k, the K-major stage layout and
// transposing fragment reads; activations as in tile_mainloop_staged. With this operand MFMA tile jn of a
// wave holds features (wave_n * TN + jn) * 16 + (lane >> 4) * 4 + q. Same MFMA chain: same bits.
// A stage holds KS consecutive K tiles, and the loads of two stages are in flight while a third is
// multiplied: these tiles serve long reductions against few outputs (one workgroup per CU), where one K
// tile in flight per workgroup would make every iteration a memory round trip. Every load is issued
// unconditionally (past the end it repeats the last K tile and its data is dropped), so the waits the
// compiler places count loads on one straight path.
// The last stage may hold fewer than KS tiles, and the last K tile fewer than 64 K values (the rest is
// filled with zeros in both operands, as in every other loop). Needs BN % 64 == 0, N % 8 == 0, K % 8 == 0
// (the activation chunks); 2 * KS * kStageBytes of LDS.
template <class S, int KS, bool RAGGED>
__device__ __forceinline__ void tile_mainloop_staged_kmajor(const MatView& W, const MatView& X, int n0, int m0, int K,
                                                            char* lds, f32x4_t (&acc)[S::TN][S::TM]) {
  static_assert(S::BN % 64 == 0, "whole 64-feature columns");
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_n = wave % S::WN;
  const int wave_m = wave / S::WN;

  // Addresses and LDS offsets of this thread's chunks; the data lives in the two register sets below.
  KMajorStager<S::kWIters, S::kWChunks, S::kThreads> sw;
  Stager<S::kXIters, S::kXChunks, S::kThreads, true> sx;
  sw.init(W, n0, tid);
  sx.init(X, m0, tid, [](int r) { return r; });
  u32x4_t wr[2][KS][S::kWIters], xr[2][KS][S::kXIters];

#pragma unroll
  for (int jn = 0; jn < S::TN; ++jn)
#pragma unroll
    for (int jm = 0; jm < S::TM; ++jm) acc[jn][jm] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int l16 = lane & 15;
  const int grp = lane >> 4;
  const int frag_lo = (grp ^ (l16 & 7)) << 4;
  const int x_row_base = S::BN * kRowBytes + (wave_m * 16 * S::TM + l16) * kRowBytes;
  constexpr int kSpan = KS * S::kStageBytes;
  const int k_tiles = (K + kTileK - 1) / kTileK;
  const int stages = (k_tiles + KS - 1) / KS;

  // RAGGED: K values at and past K (the tail of the last tile) read a clamped address and become zeros. The
  // choice is made at compile time: a select behind every load, or a branch around the loads, costs the loop
  // with whole tiles 15 % (the waits in front of the selects flatten its two stages of loads in flight).
  auto load_stage = [&](auto set, int st) __attribute__((always_inline)) {
    constexpr int R = decltype(set)::value;
    const u32x4_t zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int q = 0; q < KS; ++q) {
      int t = st * KS + q;
      t = t < k_tiles ? t : k_tiles - 1;
      const int k0 = t * kTileK;
#pragma unroll
      for (int i = 0; i < S::kWIters; ++i) {
        const int k = k0 + sw.krow[i];
        if constexpr (RAGGED) {
          const u32x4_t v = *reinterpret_cast<const u32x4_t*>(sw.src[i] + (int64_t)(k < K ? k : 0) * sw.ld);
          wr[R][q][i] = k < K ? v : zero;
        } else {
          wr[R][q][i] = *reinterpret_cast<const u32x4_t*>(sw.src[i] + (int64_t)k * sw.ld);
        }
      }
#pragma unroll
      for (int i = 0; i < S::kXIters; ++i) {
        const int k = k0 + sx.chunk_k[i];  // K % 8 == 0: a chunk is all in or all out
        if constexpr (RAGGED) {
          const u32x4_t v = *reinterpret_cast<const u32x4_t*>(sx.src[i] + (k < K ? k : 0));
          xr[R][q][i] = k < K ? v : zero;
        } else {
          xr[R][q][i] = *reinterpret_cast<const u32x4_t*>(sx.src[i] + k);
        }
      }
    }
  };
  // A tile past the end lands in a slot that is never multiplied.
  auto store_stage = [&](auto set, char* dst) __attribute__((always_inline)) {
    constexpr int R = decltype(set)::value;
#pragma unroll
    for (int q = 0; q < KS; ++q) {
      char* tile = dst + q * S::kStageBytes;
#pragma unroll
      for (int i = 0; i < S::kWIters; ++i)
        if (S::kWChunks % S::kThreads == 0 || tid + i * S::kThreads < S::kWChunks)
          *reinterpret_cast<u32x4_t*>(tile + sw.lds_off[i]) = wr[R][q][i];
#pragma unroll
      for (int i = 0; i < S::kXIters; ++i)
        if (S::kXChunks % S::kThreads == 0 || tid + i * S::kThreads < S::kXChunks)
          *reinterpret_cast<u32x4_t*>(tile + S::BN * kRowBytes + sx.lds_off[i]) = xr[R][q][i];
    }
  };
  auto multiply_stage = [&](const char* cur, int st) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < KS; ++q) {
      if (st * KS + q >= k_tiles) break;
      const char* tile = cur + q * S::kStageBytes;
#pragma unroll
      for (int s = 0; s < kTileK / kMfmaK; ++s) {
        u32x4_t wf[S::TN], xf[S::TM];
#pragma unroll
        for (int jn = 0; jn < S::TN; ++jn) {
          const int t16 = wave_n * S::TN + jn;  // 16-feature tile of the workgroup tile
          wf[jn] = read_kmajor_fragment(tile + (t16 >> 2) * (kTileK * kRowBytes), t16 & 3, s, l16, grp);
        }
#pragma unroll
        for (int jm = 0; jm < S::TM; ++jm)
          xf[jm] = *reinterpret_cast<const u32x4_t*>(tile + x_row_base + jm * 16 * kRowBytes + (frag_lo ^ (s << 6)));
#pragma unroll
        for (int jn = 0; jn < S::TN; ++jn)
#pragma unroll
          for (int jm = 0; jm < S::TM; ++jm) acc[jn][jm] = mfma_16x16x32(wf[jn], xf[jm], acc[jn][jm]);
      }
    }
  };

  using Set0 = IntTag<0>;
  using Set1 = IntTag<1>;
  load_stage(Set0{}, 0);
  load_stage(Set1{}, 1);
  store_stage(Set0{}, lds);
  __syncthreads();
  // Entering an even stage st: LDS half 0 holds it, register set 1 holds stage st + 1 (loads in flight).
  // The loop body has no exit in its middle: a path on which other loads are pending at the loop head
  // would make the compiler wait for all of them there.
  int st = 0;
  for (; st + 1 < stages; st += 2) {
    load_stage(Set0{}, st + 2);
    multiply_stage(lds, st);
    store_stage(Set1{}, lds + kSpan);
    __syncthreads();
    load_stage(Set1{}, st + 3);
    multiply_stage(lds + kSpan, st + 1);
    store_stage(Set0{}, lds);
    __syncthreads();
  }
  if (st < stages) multiply_stage(lds, st);
}

// Runs the whole K loop for one (feature tile, token tile) and leaves the fp32
// accumulators in registers. acc[jn][jm][q] is feature
//   n0 + wave_n*16*TN + (lane>>4)*4*TN + jn*4 + q
// of token
//   m0 + wave_m*16*TM + jm*16 + (lane&15).
template <class S, bool VEC>
__device__ __forceinline__ void tile_mainloop_staged(const MatView& W, const MatView& X, int n0, int m0, int K,
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

// ---------------------------------------------------------------------------
// Fast main loop: direct global -> LDS loads and an 8-wave ping-pong schedule.
//
// global_load_lds_dwordx4 moves 64 x 16 bytes from 64 independent global
// addresses into 1 KiB of consecutive LDS, i.e. eight 128-byte tile rows ("a
// block"). Lane i lands on row (i >> 3), chunk position (i & 7) of the block, so
// it fetches logical chunk (i & 7) ^ (i >> 3) of that row to reproduce the XOR
// swizzle of lds_chunk_offset(). No VGPR staging and no ds_write.
//
// The eight waves form two groups (waves 0-3 and 4-7; one wave of each group
// sits on every SIMD) that run half an iteration apart. While one group issues
// its MFMAs for a K tile out of registers, the other reads its fragments of the
// tile from LDS and starts the loads of a later tile, so the matrix pipe of a
// SIMD always has a wave whose operands are already in registers, and a wave
// that blocks on the memory pipeline never holds MFMAs back. Barriers are bare
// s_barrier instructions with hand-placed s_waitcnt: the fence of
// __syncthreads() would wait for every load in flight.
//
// Needs unit K stride, 16-byte aligned rows and K % 64 == 0. Same MFMA chain as
// the staged loop, so the same bits.
// ---------------------------------------------------------------------------

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* global_ptr_t;

// s_waitcnt immediates (gfx9 encoding: vmcnt [3:0]+[15:14], expcnt [6:4], lgkmcnt [11:8]).
constexpr int kWaitVm0 = 0x0f70;     // vmcnt(0)
constexpr int kWaitLgkm0 = 0xc07f;   // lgkmcnt(0)
constexpr int kWaitAll0 = 0x0070;    // vmcnt(0) lgkmcnt(0)
constexpr int wait_vmcnt(int n) { return 0x0f70 | (n & 15) | ((n >> 4) << 14); }
constexpr int wait_lgkmcnt(int n) { return 0xc07f | ((n & 15) << 8); }  // vmcnt / expcnt left at their maxima

// s_barrier without a fence; the empty asm statements only stop the compiler
// from moving memory operations across it.
__device__ __forceinline__ void wg_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// Who refills what. A block is 8 consecutive LDS rows of a stage (1 KiB, one
// load instruction). With waves laid out 4 (features) x 2 (tokens), wave j and
// wave 4 + j read the same 16*TN weight rows, waves 0-3 read token rows
// [0, BM/2) and waves 4-7 token rows [BM/2, BM). A wave may overwrite a row
// right after its own reads only if no other wave of its group reads that row
// (a barrier orders the two groups, nothing orders the waves inside a group):
//   late wave 4+j : the first half of the weight blocks of column j, right after its own reads
//                   of them, and a quarter of token rows [0, BM/2) at the start of its read phase
//                   (the early group finished with those one phase earlier)
//   early wave j  : the second half of the weight blocks of column j (the late wave read them one
//                   phase earlier, behind a barrier) and a quarter of token rows [BM/2, BM)
// so both groups issue the same number of loads and neither read phase outlasts a compute phase.
// For a block inside the matrix the 64 lane addresses are a uniform block base
// plus a per-lane offset that is the same for every block, so a wave keeps a few
// 32-bit lane offsets instead of one pointer per block; a block that crosses the
// last row takes a slower path with per-lane clamping (rows past the edge are
// computed and never stored).
//
// WK = true serves a weight operand stored K-major (B[K,N] with N contiguous, the
// `a @ b` and prepared-weight form). Its stage keeps, per 64-feature wave column,
// 64 K rows of 128 bytes (64 features); a block is 8 K rows of one column, so the
// ownership rule above is unchanged. Fragments come from ds_read_b64_tr_b16, which
// hands lane i of a 16-lane group the four K values of feature i out of 4 K rows x
// 16 features. The 16-byte chunk (8 features) at K row k sits at chunk position
// c ^ kmajor_swizzle(k), which keeps both the loads and the transposing reads
// free of bank conflicts. Needs TN == 4 (64-feature columns) and N % 8 == 0.
//
// XK = true is the same for the activation operand (X addressed as x[k * ldx + m],
// tokens contiguous: the transposed operands of a weight gradient). Its stage keeps
// 64-token columns of 64 K rows; a wave group must own whole columns, so BM % 128 == 0,
// and M % 8 == 0.
// (kmajor_swizzle is defined with the register-staged K-major loop above.)

// Which weight row an LDS row of the native (reduction-contiguous) weight stage holds, split
// into a block-uniform part and a part that depends on the lane's row inside the block.
// PlainRowMap is weight_row_of_lds_row(). GatedRowMap serves a packed gate/up weight
// [2 * I, K] (rows [0, I) gate, [I, 2 I) up): a tile covers BN / 2 features of both halves,
// MFMA tiles jn = 0, 1 of a wave hold gate features wave_n * 32 + (lane>>4) * 8 + jn * 4 + q
// and tiles jn = 2, 3 the up projection of the same features, so gate and up of one output
// element meet in one lane.
template <class S>
struct PlainRowMap {
  static constexpr bool kGated = false;
  static __device__ __forceinline__ int block_offset(int b) {
    constexpr int kWaveRows = 16 * S::TN;
    const int r0 = b * 8;
    return (r0 / kWaveRows) * kWaveRows + ((r0 % kWaveRows) / 16) * 4;
  }
  static __device__ __forceinline__ int block_half(int) { return 0; }
  static __device__ __forceinline__ int lane_offset(int parity, int rib) {
    const int i = parity * 8 + rib;
    return (i >> 2) * S::kRun + (i & 3);
  }
};

template <class S>
struct GatedRowMap {
  static_assert(S::TN == 4, "two gate and two up MFMA tiles per wave");
  static constexpr bool kGated = true;
  static __device__ __forceinline__ int block_offset(int b) {
    const int r0 = b * 8;
    return (r0 / 64) * 32 + (((r0 % 64) / 16) & 1) * 4;
  }
  static __device__ __forceinline__ int block_half(int b) { return ((b * 8 % 64) / 16) >> 1; }
  static __device__ __forceinline__ int lane_offset(int parity, int rib) {
    const int i = parity * 8 + rib;
    return (i >> 2) * 8 + (i & 3);
  }
};

// StridedColumnRowMap<S, STRIDE>: wave column c of the stage holds the 64 weight rows that
// start STRIDE * c after the tile origin (same order inside a column as PlainRowMap), so one
// workgroup covers a 64-row slice of four blocks of rows STRIDE apart.
template <class S, int STRIDE>
struct StridedColumnRowMap {
  static_assert(S::TN == 4, "64-row wave columns");
  static constexpr bool kGated = false;
  static __device__ __forceinline__ int block_offset(int b) {
    const int r0 = b * 8;
    return (r0 / 64) * STRIDE + ((r0 % 64) / 16) * 4;
  }
  static __device__ __forceinline__ int block_half(int) { return 0; }
  static __device__ __forceinline__ int lane_offset(int parity, int rib) {
    const int i = parity * 8 + rib;
    return (i >> 2) * S::kRun + (i & 3);
  }
};

template <class S, bool WK = false, bool XK = false, class Map = PlainRowMap<S>>
struct DmaLoader {
  static_assert(!(WK && Map::kGated), "the gated row map is for the native weight layout");
  static constexpr int kWaveRows = 16 * S::TN;
  static_assert(!WK || S::BN % 64 == 0, "K-major weights are staged in 64-feature columns");
  static_assert(!XK || S::BM % 128 == 0, "K-major activations need whole 64-token columns per wave group");
  static constexpr int kWBlocksPerWave = kWaveRows / 8;     // blocks of one weight column
  // A K-major weight of a tile whose waves cover fewer than 64 features each (TN < 4): the waves of several
  // wave columns read the same 64-feature stage column, so a block has no single pair of owners and may be
  // refilled only when every wave has read it, i.e. behind the barrier that ends the late group's read phase.
  static constexpr bool kSharedWColumn = WK && S::TN < 4;
  // Who refills a weight column. On the 256-token tiles, which are bound by the matrix pipe, its two waves split the
  // refill (native loop: MFMA utilisation 77 -> 82 %; K-major loops 4-6 %, lm_head weight gradient at 8192 tokens
  // 8.32 -> 7.77 ms, which had measured slower while the transposing reads still had bank conflicts and the compiler's
  // waits in front of them). The tiles of 128 and 64 tokens run where the weight stream bounds the time, and the half
  // of a column that the early wave refills starts one phase later: there the late wave refills the whole column as
  // soon as its weight fragments are in registers. Measured with weights from HBM, split -> whole column: the deep-stage
  // 64 x 64 / 128 x 64 / 128 x 128 tiles 6-13 % faster (down at 256 / 1024 tokens 57.6 -> 51.4 / 116 -> 101 us), native
  // 256 x 128 2-6 % faster, K-major 256 x 128 / 256 x 64 16-20 % faster; only the native 256 x 64 tile (three stages, one
  // token block per wave) is 3-8 % faster with the split and keeps it.
  static constexpr bool kSplitColumn = S::BM >= 256 || (!WK && !XK && S::BN == 256 && S::BM == 64);
  static_assert(!(kSharedWColumn && kSplitColumn), "a shared stage column is refilled by the late group alone");
  static constexpr int kWBlocksLate = kSplitColumn ? kWBlocksPerWave / 2 : kWBlocksPerWave;
  static constexpr int kWBlocksEarly = kWBlocksPerWave - kWBlocksLate;
  static constexpr int kXBlocksPerWave = (S::BM / 16) / 4;  // every wave
  static constexpr int kLateLoads = kWBlocksLate + kXBlocksPerWave;
  static constexpr int kEarlyLoads = kWBlocksEarly + kXBlocksPerWave;
  static constexpr int kBlocksW = S::BN / 8;

  const bf16_bits* w_base;  // W + n0 * ldw   (uniform)
  const bf16_bits* x_base;  // X + m0 * ldx   (uniform)
  int64_t ldw, ldx;
  int n0, m0, n_rows, m_rows;
  int rib;                 // row of this lane inside a block
  int chunk_elems;         // element offset of this lane's 16-byte chunk inside a 64-wide K tile
  uint32_t w_lane_off[2];  // by block parity: (feature offset of the lane) * ldw + chunk_elems
  uint32_t x_lane_off;     // rib * ldx + chunk_elems
  int kmajor_chunk;        // K-major operands: chunk position of this lane before the block part of the swizzle

  // Feature offset of lane row `rib` inside a weight block of parity p: LDS row
  // r = 8 b + rib holds a block-uniform feature plus Map::lane_offset(p, rib).
  static __device__ __forceinline__ int w_lane_row(int parity, int rib) { return Map::lane_offset(parity, rib); }

  __device__ __forceinline__ void init(const MatView& W, const MatView& X, int n0_, int m0_, int lane) {
    n0 = n0_;
    m0 = m0_;
    n_rows = Map::kGated ? W.rows / 2 : W.rows;  // rows of one half of a packed gate/up weight
    m_rows = X.rows;
    ldw = WK ? W.k_stride : W.row_stride;  // K-major: elements between consecutive K rows
    ldx = XK ? X.k_stride : X.row_stride;
    w_base = WK ? W.ptr + n0 : W.ptr + (int64_t)n0 * ldw;
    x_base = XK ? X.ptr + m0 : X.ptr + (int64_t)m0 * ldx;
    rib = lane >> 3;
    chunk_elems = ((lane & 7) ^ rib) * kChunkElems;
    // K-major: lane -> (K row rib of the block, chunk position lane & 7); the K-row part
    // of the swizzle that does not depend on the block is folded in here.
    kmajor_chunk = (lane & 7) ^ kmajor_swizzle_of_row_in_block(rib);
    if (WK) {
      w_lane_off[0] = (uint32_t)(rib * ldw);
      w_lane_off[1] = 0;
    } else {
      w_lane_off[0] = (uint32_t)(w_lane_row(0, rib) * ldw) + chunk_elems;
      w_lane_off[1] = (uint32_t)(w_lane_row(1, rib) * ldw) + chunk_elems;
    }
    x_lane_off = XK ? (uint32_t)(rib * ldx) : (uint32_t)(rib * ldx) + chunk_elems;
  }

  // Source of this lane's 16 bytes of K-major block `b` (8 K rows of one 64-wide column).
  static __device__ __forceinline__ const bf16_bits* kmajor_src(const bf16_bits* base, int64_t ld, uint32_t lane_off,
                                                                int kmajor_chunk, int first, int rows, int k0,
                                                                int b) {
    const int col = b >> 3;  // 64-wide column of the tile
    const int kblk = b & 7;  // K rows 8 kblk .. 8 kblk + 7 of the tile
    const int chunk = kmajor_chunk ^ kmajor_swizzle_of_block(kblk);
    int at = col * 64 + chunk * kChunkElems;  // offset inside the tile along the contiguous axis
    if (first + col * 64 + 64 > rows) {       // column crosses the edge (rows % 8 == 0 here)
      const int last = rows - kChunkElems - first;
      at = at < last ? at : last;
    }
    return base + (int64_t)(k0 + kblk * 8) * ld + lane_off + at;
  }

  __device__ __forceinline__ void load_w_block(char* stage, int k0, int b) const {
    if constexpr (WK) {
      const bf16_bits* src = kmajor_src(w_base, ldw, w_lane_off[0], kmajor_chunk, n0, n_rows, k0, b);
      __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(stage + b * 1024), 16, 0, 0);
      return;
    }
    const int row0 = Map::block_offset(b);  // block-uniform feature offset
    const int parity = b & 1;
    const bf16_bits* half_base = w_base + (int64_t)(Map::block_half(b) * n_rows) * ldw;
    const bf16_bits* src;
    if (n0 + row0 + w_lane_row(parity, 7) < n_rows) {
      src = half_base + (int64_t)row0 * ldw + k0 + w_lane_off[parity];
    } else {
      int g = n0 + row0 + w_lane_row(parity, rib);
      g = g < n_rows ? g : n_rows - 1;
      src = half_base + (int64_t)(g - n0) * ldw + k0 + chunk_elems;
    }
    __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(stage + b * 1024), 16, 0, 0);
  }

  __device__ __forceinline__ void load_x_block(char* stage, int k0, int xb) const {
    if constexpr (XK) {
      const bf16_bits* src = kmajor_src(x_base, ldx, x_lane_off, kmajor_chunk, m0, m_rows, k0, xb);
      __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(stage + (kBlocksW + xb) * 1024), 16, 0, 0);
      return;
    }
    const int row0 = xb * 8;
    const bf16_bits* src;
    if (m0 + row0 + 7 < m_rows) {
      src = x_base + (int64_t)row0 * ldx + k0 + x_lane_off;
    } else {
      int g = m0 + row0 + rib;
      g = g < m_rows ? g : m_rows - 1;
      src = x_base + (int64_t)(g - m0) * ldx + k0 + chunk_elems;
    }
    __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(stage + (kBlocksW + xb) * 1024), 16, 0, 0);
  }

  // The same for a native-layout tile that lies inside both matrices: no clamping.
  __device__ __forceinline__ void load_w_block_inside(char* stage, int k0, int b) const {
    const bf16_bits* src = w_base + (int64_t)(Map::block_half(b) * n_rows + Map::block_offset(b)) * ldw + k0 +
                           w_lane_off[b & 1];
    __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(stage + b * 1024), 16, 0, 0);
  }
  __device__ __forceinline__ void load_x_block_inside(char* stage, int k0, int xb) const {
    const bf16_bits* src = x_base + (int64_t)(xb * 8) * ldx + k0 + x_lane_off;
    __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(stage + (kBlocksW + xb) * 1024), 16, 0, 0);
  }

  // `wave` is the workgroup wave index 0..7.
  __device__ __forceinline__ void issue_early(char* stage, int k0, int wave) const {
#pragma unroll
    for (int j = kWBlocksLate; j < kWBlocksPerWave; ++j) load_w_block(stage, k0, wave * kWBlocksPerWave + j);
#pragma unroll
    for (int j = 0; j < kXBlocksPerWave; ++j) load_x_block(stage, k0, S::BM / 16 + wave * kXBlocksPerWave + j);
  }
  __device__ __forceinline__ void issue_late_x(char* stage, int k0, int wave) const {
    const int col = wave - 4;
#pragma unroll
    for (int j = 0; j < kXBlocksPerWave; ++j) load_x_block(stage, k0, col * kXBlocksPerWave + j);
  }
  __device__ __forceinline__ void issue_late_w(char* stage, int k0, int wave) const {
    const int col = wave - 4;
#pragma unroll
    for (int j = 0; j < kWBlocksLate; ++j) load_w_block(stage, k0, col * kWBlocksPerWave + j);
  }
};

template <class S>
constexpr bool pingpong_supported() {
  return S::WN == 4 && S::WM == 2 && S::BM % 64 == 0;
}

// With WK the accumulator of MFMA tile jn holds features wave_n*64 + jn*16 + (lane>>4)*4 + q
// (no run permutation: a K-major chunk is eight consecutive features).
//
// KS > 1 makes a stage KS consecutive 64-wide K tiles (each laid out as above), so a phase
// covers 64 * KS K values between two barriers: small tiles, whose phases would otherwise be
// shorter than a barrier, stay on the matrix pipe. Needs K % (64 * KS) == 0 and
// 2 * KS * S::kStageBytes of LDS; the MFMA chain is the same (K tiles ascending).
//
// NS is the number of stages (K tiles in LDS): tile t lives in stage t % NS and the loads of
// tile t + NS start as soon as tile t has been read, so NS - 1 tiles are in flight behind the
// one being read. Two stages cover the latency of L2 hits; a weight tile that is used by one
// workgroup only comes through the fabric and wants three. Needs NS * KS * S::kStageBytes of LDS.
template <class S, bool WK = false, bool XK = false, class Map = PlainRowMap<S>, int KS = 1, int NS = 2>
__device__ __forceinline__ void tile_mainloop_pingpong(const MatView& W, const MatView& X, int n0, int m0, int K,
                                                       char* lds, f32x4_t (&acc)[S::TN][S::TM]) {
  static_assert(pingpong_supported<S>(), "two groups of four waves, 4 x 2 wave layout");
  static_assert(KS >= 1 && NS >= 2 && (NS - 1) * KS * (DmaLoader<S, WK, XK, Map>::kLateLoads) <= 63 &&
                    KS * (DmaLoader<S, WK, XK, Map>::kLateLoads) <= 31,
                "loads in flight must fit vmcnt");
  using Loader = DmaLoader<S, WK, XK, Map>;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_n = wave % S::WN;
  const int wave_m = wave / S::WN;
  const bool late_group = wave >= 4;

  Loader loader;
  loader.init(W, X, n0, m0, lane);

#pragma unroll
  for (int jn = 0; jn < S::TN; ++jn)
#pragma unroll
    for (int jm = 0; jm < S::TM; ++jm) acc[jn][jm] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int l16 = lane & 15;
  const int grp = lane >> 4;
  const int frag_lo = (grp ^ (l16 & 7)) << 4;
  const int w_row_base = (wave_n * 16 * S::TN + l16) * kRowBytes;
  const int x_row_base = S::BN * kRowBytes + (wave_m * 16 * S::TM + l16) * kRowBytes;

  constexpr int kStageSpan = KS * S::kStageBytes;  // bytes of one stage (KS K tiles)
  constexpr int kStageK = KS * kTileK;             // K values of one stage
  const int nk = K / kStageK;
  // Loads past the last stage re-fetch the last one into a stage nobody reads
  // any more; that keeps the number of loads in flight (and so every s_waitcnt
  // immediate) the same in every iteration.
  auto tile_k = [&](int t) { return (t < nk ? t : nk - 1) * kStageK; };
  auto stage = [&](int t) { return lds + (t % NS) * kStageSpan; };
  auto issue_early = [&](char* st, int k0) {
#pragma unroll
    for (int s = 0; s < KS; ++s) loader.issue_early(st + s * S::kStageBytes, k0 + s * kTileK, wave);
  };
  auto issue_late_x = [&](char* st, int k0) {
#pragma unroll
    for (int s = 0; s < KS; ++s) loader.issue_late_x(st + s * S::kStageBytes, k0 + s * kTileK, wave);
  };
  auto issue_late_w = [&](char* st, int k0) {
#pragma unroll
    for (int s = 0; s < KS; ++s) loader.issue_late_w(st + s * S::kStageBytes, k0 + s * kTileK, wave);
  };

  // K-major fragments: the transposing read takes, from lane r of a 16-lane group, the address
  // of 4 features (tokens) at K row (r >> 2), positions 4 (r & 3) .. +3 of MFMA tile `j16` of a
  // 64-wide column.
  auto read_kmajor = [&](const char* col, int j16, int step) -> u32x4_t {
    return read_kmajor_fragment(col, j16, step, l16, grp);
  };
  auto read_w_kmajor = [&](const char* st, int jn, int step) -> u32x4_t {
    const int t16 = wave_n * S::TN + jn;  // 16-feature tile of the weight tile: column t16 / 4, tile t16 % 4 of it
    return read_kmajor(st + (t16 >> 2) * (64 * kRowBytes), t16 & 3, step);
  };
  auto read_x_kmajor = [&](const char* st, int jm, int step) -> u32x4_t {
    const int col = wave_m * (S::TM / 4) + (jm >> 2);
    return read_kmajor(st + S::BN * kRowBytes + col * (64 * kRowBytes), jm & 3, step);
  };

  u32x4_t w0[KS][S::TN], x0[KS][S::TM], w1[KS][S::TN], x1[KS][S::TM];
  // Weight fragments of both K steps (2 TN KS reads) ...
  auto read_w = [&](int t) {
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const char* st = stage(t) + s * S::kStageBytes;
#pragma unroll
      for (int jn = 0; jn < S::TN; ++jn) {
        if constexpr (WK) {
          w0[s][jn] = read_w_kmajor(st, jn, 0);
          w1[s][jn] = read_w_kmajor(st, jn, 1);
        } else {
          w0[s][jn] = *reinterpret_cast<const u32x4_t*>(st + w_row_base + jn * 16 * kRowBytes + frag_lo);
          w1[s][jn] = *reinterpret_cast<const u32x4_t*>(st + w_row_base + jn * 16 * kRowBytes + (frag_lo ^ 64));
        }
      }
    }
  };
  // ... and the token fragments of one K step (TM KS reads).
  auto read_x = [&](int t, int step) {
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const char* st = stage(t) + s * S::kStageBytes;
#pragma unroll
      for (int jm = 0; jm < S::TM; ++jm) {
        u32x4_t v;
        if constexpr (XK) {
          v = read_x_kmajor(st, jm, step);
        } else {
          v = *reinterpret_cast<const u32x4_t*>(st + x_row_base + jm * 16 * kRowBytes + (frag_lo ^ (step << 6)));
        }
        if (step == 0) {
          x0[s][jm] = v;
        } else {
          x1[s][jm] = v;
        }
      }
    }
  };
  auto read_tile = [&](int t) {
    read_w(t);
    read_x(t, 0);
    read_x(t, 1);
  };
  auto compute = [&]() {
    __builtin_amdgcn_s_setprio(2);
#pragma unroll
    for (int s = 0; s < KS; ++s) {
#pragma unroll
      for (int jn = 0; jn < S::TN; ++jn)
#pragma unroll
        for (int jm = 0; jm < S::TM; ++jm) acc[jn][jm] = mfma_16x16x32(w0[s][jn], x0[s][jm], acc[jn][jm]);
#pragma unroll
      for (int jn = 0; jn < S::TN; ++jn)
#pragma unroll
        for (int jm = 0; jm < S::TM; ++jm) acc[jn][jm] = mfma_16x16x32(w1[s][jn], x1[s][jm], acc[jn][jm]);
    }
    __builtin_amdgcn_s_setprio(0);
  };

  // Phases are the intervals between consecutive workgroup barriers:
  //   phase 2t     : early group reads tile t        | late group computes tile t-1
  //   phase 2t + 1 : early group computes tile t     | late group reads tile t
  // Tile t lives in stage t % NS, which is read in phases 2t and 2t + 1 and first
  // read again (tile t + NS) in phase 2t + 2 NS. The notes below are for NS = 2. Every wave waits for its own
  // fragment reads before the barrier that ends its read phase.
  //   late wave, phase 2t + 1: starts its token rows of tile t + 2 at once (the early group
  //     read them one phase earlier) and its weight blocks as soon as its own weight
  //     fragments are in registers; it confirms that part at the end of phase 2t + 3,
  //     behind the loads it starts there.
  //   early wave, phase 2t + 2: starts its part of tile t + 2 (rows the late group read one
  //     phase earlier); confirms it at the end of phase 2t + 3.
  if (!late_group) {
#pragma unroll
    for (int i = 0; i < NS; ++i) issue_early(stage(i), tile_k(i));
    __builtin_amdgcn_s_waitcnt(wait_vmcnt((NS - 1) * KS * Loader::kEarlyLoads));  // my part of tile 0 has landed
    wg_barrier();
    for (int t = 0; t < nk; ++t) {
      read_tile(t);
      if (t > 0) issue_early(stage(t - 1 + NS), tile_k(t - 1 + NS));  // the stage tile t - 1 has left
      __builtin_amdgcn_s_waitcnt(kWaitLgkm0);  // my fragments are in registers
      wg_barrier();
      compute();
      __builtin_amdgcn_s_waitcnt(wait_vmcnt((NS - 2) * KS * Loader::kEarlyLoads));  // my part of tile t+1 has landed
      wg_barrier();
    }
    wg_barrier();  // pairs with the late group's leading barrier
  } else {
#pragma unroll
    for (int i = 0; i < NS; ++i) {
      issue_late_x(stage(i), tile_k(i));
      issue_late_w(stage(i), tile_k(i));
    }
    __builtin_amdgcn_s_waitcnt(wait_vmcnt((NS - 1) * KS * Loader::kLateLoads));  // my part of tile 0 has landed
    wg_barrier();
    wg_barrier();  // half an iteration behind the early group
    // LDS reads return in order, so once at most kXReads of them are outstanding the weight
    // fragments (issued first) are in registers and their rows may be refilled.
    // (lgkmcnt is a 4-bit counter: with the 16 reads of eight K-major token tiles the wait for 15 also covers the
    // first of them; more reads per K step, i.e. several K tiles per stage, take the other order.) The order holds
    // whether the column's refill is split or not: the early wave of the column read it one phase earlier. On the
    // 128- and 64-token K-major tiles, which do not split, it is worth 1-7 % (12288 x 4096 at 2048 tokens, 256 x 128:
    // 181 -> 168 us).
    constexpr int kXReads = KS * S::TM * (XK ? 2 : 1);
    for (int t = 0; t < nk; ++t) {
      if constexpr (Loader::kSharedWColumn) {
        issue_late_x(stage(t), tile_k(t + NS));  // token rows the early group read one phase ago
        read_tile(t);
      } else if constexpr (kXReads <= 16) {
        issue_late_x(stage(t), tile_k(t + NS));  // token rows the early group read one phase ago
        read_w(t);
        read_x(t, 0);
        __builtin_amdgcn_s_waitcnt(wait_lgkmcnt(kXReads < 15 ? kXReads : 15));  // my weight fragments are in registers
        issue_late_w(stage(t), tile_k(t + NS));
        read_x(t, 1);
      } else {
        read_tile(t);
        __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
        issue_late_w(stage(t), tile_k(t + NS));
        issue_late_x(stage(t), tile_k(t + NS));
      }
      __builtin_amdgcn_s_waitcnt(kWaitLgkm0);  // all my fragments are in registers
      if constexpr (Loader::kSharedWColumn) {
        // Behind tile t + 1 this wave has started tiles t + 2 .. t + NS - 1 and the token rows of tile t + NS;
        // the weight blocks of tile t + NS follow the barrier, when every wave has read tile t.
        __builtin_amdgcn_s_waitcnt(wait_vmcnt((NS - 2) * KS * Loader::kLateLoads + KS * Loader::kXBlocksPerWave));
        wg_barrier();
        issue_late_w(stage(t), tile_k(t + NS));
      } else {
        __builtin_amdgcn_s_waitcnt(wait_vmcnt((NS - 1) * KS * Loader::kLateLoads));  // my part of tile t+1 has landed
        wg_barrier();
      }
      compute();
      wg_barrier();
    }
  }
  __builtin_amdgcn_s_waitcnt(kWaitAll0);
  wg_barrier();  // callers reuse the LDS after the loop
}

// ---------------------------------------------------------------------------
// The last, partial K tile behind a ping-pong loop that has a K-major operand.
//
// Direct-to-LDS loads move whole 64-wide K tiles; a reduction length that is not a multiple of 64 (the token
// count of a weight gradient) used to send the whole GEMM to the element-wise loader. Instead the ping-pong
// loop runs over the K / 64 whole tiles and this step adds the rest to the same accumulators: both operands of
// K values [k0, K) go through registers (16-byte chunks, zeros at and past K, addresses clamped into the
// matrix), into stage 0 in the layout the loop uses, and through the same fragment reads and two MFMA steps.
// The chain of an output element is the one every other loop runs: K tiles ascending, the tail zero-filled
// to a multiple of 64 in both operands. A native operand needs K % 8 == 0 (a chunk is all in or all out).
// Call it after the loop (which ends on a barrier); it ends on a barrier as well.
// ---------------------------------------------------------------------------
// Everything here is derived from a thread index the compiler cannot see through, so that none of the step's
// addresses is computed ahead of the main loop and kept alive across it (which made the 256 x 256 kernels
// spill hundreds of registers inside that loop).
template <class S, bool WK, bool XK>
__device__ __forceinline__ void tile_tail_step(const MatView& W, const MatView& X, int n0, int m0, int k0, int K,
                                               char* lds, f32x4_t (&acc)[S::TN][S::TM]) {
  static_assert(!WK || S::BN % 64 == 0, "K-major weights are staged in 64-feature columns");
  static_assert(!XK || S::BM % 128 == 0, "K-major activations need whole 64-token columns per wave group");
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_n = wave % S::WN;
  const int wave_m = wave / S::WN;
  char* x_stage = lds + S::BN * kRowBytes;

  if constexpr (WK) {
    KMajorStager<S::kWIters, S::kWChunks, S::kThreads> sw;
    sw.init(W, n0, tid);
    sw.template load<true>(k0, K);
    sw.store(lds, tid);
  } else {
    Stager<S::kWIters, S::kWChunks, S::kThreads, true> sw;
    sw.init(W, n0, tid, [](int r) { return weight_row_of_lds_row<S>(r); });
    sw.template load<true>(k0, K);
    sw.store(lds, tid);
  }
  if constexpr (XK) {
    KMajorStager<S::kXIters, S::kXChunks, S::kThreads> sx;
    sx.init(X, m0, tid);
    sx.template load<true>(k0, K);
    sx.store(x_stage, tid);
  } else {
    Stager<S::kXIters, S::kXChunks, S::kThreads, true> sx;
    sx.init(X, m0, tid, [](int r) { return r; });
    sx.template load<true>(k0, K);
    sx.store(x_stage, tid);
  }
  __syncthreads();

  const int l16 = lane & 15;
  const int grp = lane >> 4;
  const int frag_lo = (grp ^ (l16 & 7)) << 4;
  const int w_row_base = (wave_n * 16 * S::TN + l16) * kRowBytes;
  const int x_row_base = (wave_m * 16 * S::TM + l16) * kRowBytes;
#pragma unroll
  for (int s = 0; s < kTileK / kMfmaK; ++s) {
    u32x4_t wf[S::TN], xf[S::TM];
#pragma unroll
    for (int jn = 0; jn < S::TN; ++jn) {
      if constexpr (WK) {
        const int t16 = wave_n * S::TN + jn;
        wf[jn] = read_kmajor_fragment(lds + (t16 >> 2) * (64 * kRowBytes), t16 & 3, s, l16, grp);
      } else {
        wf[jn] = *reinterpret_cast<const u32x4_t*>(lds + w_row_base + jn * 16 * kRowBytes + (frag_lo ^ (s << 6)));
      }
    }
#pragma unroll
    for (int jm = 0; jm < S::TM; ++jm) {
      if constexpr (XK) {
        const int col = wave_m * (S::TM / 4) + (jm >> 2);
        xf[jm] = read_kmajor_fragment(x_stage + col * (64 * kRowBytes), jm & 3, s, l16, grp);
      } else {
        xf[jm] = *reinterpret_cast<const u32x4_t*>(x_stage + x_row_base + jm * 16 * kRowBytes + (frag_lo ^ (s << 6)));
      }
    }
#pragma unroll
    for (int jn = 0; jn < S::TN; ++jn)
#pragma unroll
      for (int jm = 0; jm < S::TM; ++jm) acc[jn][jm] = mfma_16x16x32(wf[jn], xf[jm], acc[jn][jm]);
  }
  __syncthreads();
}

// ---------------------------------------------------------------------------
// One wave per SIMD: four waves, each a 128 x 128 quarter of a 256 x 256 tile.
//
// A square wave tile reads 16 fragments from LDS per 64 MFMAs (the 64 x 128 wave tiles of
// the ping-pong loop: 12 per 32). Its 256 accumulator registers and two sets of 16
// fragments need the whole unified register file of a SIMD, so a wave has no partner to
// hide its stalls: fragment reads of K step s + 1 and the direct-to-LDS loads of K tile
// t + 2 are issued under the MFMAs of step s, and there is one barrier per K tile.
//
//   iteration t (tile t in stage t & 1; F0 = fragments of its first K step, already in registers)
//     read F1 (second K step of tile t)           | MFMAs on F0
//     wait: F1 in registers, my loads of tile t + 1 landed; barrier
//     start the loads of tile t + 2 into stage t & 1, read F0 of tile t + 1 | MFMAs on F1
//
// Same MFMA chain per output element as every other loop. Needs the native layouts,
// 16-byte aligned rows and K % 64 == 0.
// ---------------------------------------------------------------------------
template <class S>
constexpr bool solo_supported() {
  return S::WN == 2 && S::WM == 2 && S::BN == 256 && S::BM == 256;
}

template <bool V>
struct BoolTag {
  static constexpr bool value = V;
};

template <class S, bool INSIDE>
__device__ __forceinline__ void tile_mainloop_solo_impl(const MatView& W, const MatView& X, int n0, int m0, int K,
                                                        char* lds, f32x4_t (&acc)[S::TN][S::TM]) {
  static_assert(solo_supported<S>(), "four waves of 128 x 128");
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wave_n = wave % S::WN;
  const int wave_m = wave / S::WN;
  const int l16 = lane & 15;
  const int grp = lane >> 4;

  using Loader = DmaLoader<S>;
  Loader loader;
  loader.init(W, X, n0, m0, lane);
  constexpr int kBlocksW = S::BN / 8, kBlocksX = S::BM / 8;
  constexpr int kLoads = (kBlocksW + kBlocksX) / 4;  // blocks (load instructions) per wave and K tile
  static_assert(kBlocksW == 2 * kLoads && kBlocksX == 2 * kLoads, "waves 0, 1 load weight rows, waves 2, 3 token rows");
  // Inside the matrices a block's 64 addresses are a uniform base (operand, 128-row half of
  // the tile, block) plus one of two lane offsets, the same for every K tile.
  const bool loads_weights = wave < 2;
  const bf16_bits* my_base = (loads_weights ? loader.w_base : loader.x_base);
  const int64_t my_ld = loads_weights ? loader.ldw : loader.ldx;
  const uint32_t my_off[2] = {loads_weights ? loader.w_lane_off[0] : loader.x_lane_off,
                              loads_weights ? loader.w_lane_off[1] : loader.x_lane_off};
  my_base += (int64_t)((wave & 1) * (kLoads * 8)) * my_ld;
  auto issue_tile = [&](char* st, int k0) {
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
      const int b = wave * kLoads + j;
      if constexpr (INSIDE) {
        // weight block j of a 128-row wave column holds features 4 (j >> 1) + (lane part); token block j rows 8 j ..
        const int rows = loads_weights ? 4 * (j >> 1) : 8 * j;
        const bf16_bits* src = my_base + (int64_t)rows * my_ld + k0 + my_off[j & 1];
        __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(st + b * 1024), 16, 0, 0);
      } else if (loads_weights) {
        loader.load_w_block(st, k0, b);
      } else {
        loader.load_x_block(st, k0, b - kBlocksW);
      }
    }
  };

#pragma unroll
  for (int jn = 0; jn < S::TN; ++jn)
#pragma unroll
    for (int jm = 0; jm < S::TM; ++jm) acc[jn][jm] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int frag_lo = (grp ^ (l16 & 7)) << 4;
  const int w_row_base = (wave_n * 16 * S::TN + l16) * kRowBytes;
  const int x_row_base = S::BN * kRowBytes + (wave_m * 16 * S::TM + l16) * kRowBytes;
  u32x4_t w0[S::TN], x0[S::TM], w1[S::TN], x1[S::TM];
  auto read_step = [&](const char* st, int step, u32x4_t (&wf)[S::TN], u32x4_t (&xf)[S::TM]) {
    const int frag = frag_lo ^ (step << 6);
#pragma unroll
    for (int jn = 0; jn < S::TN; ++jn)
      wf[jn] = *reinterpret_cast<const u32x4_t*>(st + w_row_base + jn * 16 * kRowBytes + frag);
#pragma unroll
    for (int jm = 0; jm < S::TM; ++jm)
      xf[jm] = *reinterpret_cast<const u32x4_t*>(st + x_row_base + jm * 16 * kRowBytes + frag);
  };
  auto mfma_step = [&](const u32x4_t (&wf)[S::TN], const u32x4_t (&xf)[S::TM]) {
#pragma unroll
    for (int jn = 0; jn < S::TN; ++jn)
#pragma unroll
      for (int jm = 0; jm < S::TM; ++jm) acc[jn][jm] = mfma_16x16x32(wf[jn], xf[jm], acc[jn][jm]);
  };
  constexpr int kReads = S::TN + S::TM;    // fragment reads per K step
  constexpr int kMfmas = S::TN * S::TM;    // MFMAs per K step
  static_assert(kMfmas % kReads == 0 && kMfmas % (2 * kLoads) == 0, "whole interleave groups");

  const int nk = K / kTileK;
  char* const st0 = lds;
  char* const st1 = lds + S::kStageBytes;
  issue_tile(st0, 0);
  if (nk > 1) issue_tile(st1, kTileK);
  if (nk > 1) {
    __builtin_amdgcn_s_waitcnt(wait_vmcnt(kLoads));  // my part of tile 0 has landed
  } else {
    __builtin_amdgcn_s_waitcnt(kWaitVm0);
  }
  wg_barrier();
  read_step(st0, 0, w0, x0);
  __builtin_amdgcn_s_waitcnt(kWaitLgkm0);

  // One K tile. LOAD: tile t + 2 exists; READ: tile t + 1 exists. Written in issue order, one
  // row of MFMA tiles at a time with its share of the reads and loads in front; the fences keep
  // the compiler from regrouping them.
  static_assert(S::TN == S::TM && kLoads == 2 * S::TN, "one weight and one token fragment, two loads per MFMA row");
  auto read_one = [&](const char* st, int step, int j, u32x4_t (&wf)[S::TN], u32x4_t (&xf)[S::TM]) {
    const int frag = frag_lo ^ (step << 6);
    wf[j] = *reinterpret_cast<const u32x4_t*>(st + w_row_base + j * 16 * kRowBytes + frag);
    xf[j] = *reinterpret_cast<const u32x4_t*>(st + x_row_base + j * 16 * kRowBytes + frag);
  };
  auto issue_two = [&](char* st, int k0, int jn) {
#pragma unroll
    for (int j = 2 * jn; j < 2 * jn + 2; ++j) {
      const int b = wave * kLoads + j;
      if constexpr (INSIDE) {
        const int rows = loads_weights ? 4 * (j >> 1) : 8 * j;
        const bf16_bits* src = my_base + (int64_t)rows * my_ld + k0 + my_off[j & 1];
        __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(st + b * 1024), 16, 0, 0);
      } else if (loads_weights) {
        loader.load_w_block(st, k0, b);
      } else {
        loader.load_x_block(st, k0, b - kBlocksW);
      }
    }
  };
  auto iteration = [&](int t, auto load_tag, auto read_tag) {
    constexpr bool LOAD = decltype(load_tag)::value, READ = decltype(read_tag)::value;
    char* cur = (t & 1) ? st1 : st0;
    char* nxt = (t & 1) ? st0 : st1;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int jn = 0; jn < S::TN; ++jn) {
      read_one(cur, 1, jn, w1, x1);
#pragma unroll
      for (int jm = 0; jm < S::TM; ++jm) acc[jn][jm] = mfma_16x16x32(w0[jn], x0[jm], acc[jn][jm]);
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_waitcnt(kWaitAll0);  // F1 in registers, my part of tile t + 1 landed
    wg_barrier();
#pragma unroll
    for (int jn = 0; jn < S::TN; ++jn) {
      if constexpr (LOAD) issue_two(cur, (t + 2) * kTileK, jn);
      if constexpr (READ) read_one(nxt, 0, jn, w0, x0);
#pragma unroll
      for (int jm = 0; jm < S::TM; ++jm) acc[jn][jm] = mfma_16x16x32(w1[jn], x1[jm], acc[jn][jm]);
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (READ) __builtin_amdgcn_s_waitcnt(kWaitLgkm0);  // F0 of tile t + 1 in registers
  };
  int t = 0;
  for (; t + 2 < nk; ++t) iteration(t, BoolTag<true>{}, BoolTag<true>{});
  if (t + 1 < nk) iteration(t++, BoolTag<false>{}, BoolTag<true>{});
  iteration(t, BoolTag<false>{}, BoolTag<false>{});
  __builtin_amdgcn_s_waitcnt(kWaitAll0);
  wg_barrier();  // callers reuse the LDS after the loop
}

template <class S>
__device__ __forceinline__ void tile_mainloop_solo(const MatView& W, const MatView& X, int n0, int m0, int K,
                                                   char* lds, f32x4_t (&acc)[S::TN][S::TM]) {
  if (n0 + S::BN <= W.rows && m0 + S::BM <= X.rows) {
    tile_mainloop_solo_impl<S, true>(W, X, n0, m0, K, lds, acc);
  } else {
    tile_mainloop_solo_impl<S, false>(W, X, n0, m0, K, lds, acc);
  }
}

}  // namespace rlk
