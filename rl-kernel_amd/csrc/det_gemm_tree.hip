// det_gemm under the k-tree contract, for gfx950.
//
// The reference's second strict GEMM contract (its "triton_tree" backend,
// rl_engine/backends/shared/triton/gemm/det_gemm.py:218-258, 355-417; specification
// tests/ops/gemm/test_det_gemm.py:156-168; CUDA twin csrc/cuda/gemm/det_gemm_kernel.cu:74-85):
//
//   T(lo, hi) = bf16( sum_{k = lo .. hi-1} a_k * b_k )       if hi - lo <= 32,
//               fp32 accumulator from +0, k ascending, one fused multiply-add per term
//             = bf16( float(T(lo, mid)) + float(T(mid, hi)) ) otherwise,
//               mid = lo + (hi - lo) / 2                      (split in element space)
//   C = T(0, K).
//
// Every rounding point is a function of K alone, so the result is bit-identical for any
// M, batch or packing, and a K range that is a subtree (the contiguous half, quarter, ...
// a K-sharded rank holds) evaluates to exactly that tree node. The scalar chain of a leaf
// cannot go through the bf16 matrix instructions (a 16x16x32 step sums its 32 products in its
// own order). Two leaf loops evaluate it, bit for bit the same:
//   * vector ALU: a thread owns 4 rows x 8 columns and issues one v_fma_f32 per term;
//   * fp32 matrix pipe: a wave owns 32 rows x 64 columns and issues one
//     v_mfma_f32_32x32x1_2b_f32 per k. With a reduction length of one, an instruction adds
//     exactly one product to every accumulator, and the product of two bf16 values is exact
//     in fp32, so the step is the same single rounding as the fused multiply-add, at twice
//     the vector rate.
//
// A workgroup of 256 threads owns a 64 x 128 output tile.
// Leaves are visited left to right. The operands of a leaf are converted to fp32 on their
// way into LDS ([k][row], so a k step reads consecutive floats of one k row),
// the next leaf is fetched while the current one is summed. The tree is evaluated on the
// fly: a finished node waits in the register slot of its depth until its right sibling is
// finished, so a thread holds at most one bf16 node per tree level. Which slot is read or
// written is the same for every thread (it depends on K only), so the slot index is a
// uniform branch over compile-time register arrays, never an indexed register access.
#include "rlk_device.h"
#include "rlk_host.h"

namespace rlk {

constexpr int kTreeLeaf = 32;
constexpr int kTreeBM = 64;   // rows of A per workgroup
constexpr int kTreeBN = 128;  // columns (rows of the [N, K] operand) per workgroup
constexpr int kTreeThreads = 256;
constexpr int kTreeAStride = kTreeBM + 4;  // floats per k row in LDS (keeps 16-byte alignment, spreads banks)
constexpr int kTreeBStride = kTreeBN + 4;
constexpr int kTreeStageFloats = kTreeLeaf * (kTreeAStride + kTreeBStride);
constexpr int kTreeALoads = kTreeBM * kTreeLeaf / kTreeThreads;  // 8 elements per thread per leaf
constexpr int kTreeBLoads = kTreeBN * kTreeLeaf / kTreeThreads;  // 16
constexpr int kTreeRowBytes = 2 * kTreeLeaf + 16;                // bf16 stage of the matrix-pipe leaf

// Depth of the deepest leaf: sizes at depth d are floor or ceil of K / 2^d.
static int tree_depth(int K) {
  int depth = 0;
  for (int size = K; size > kTreeLeaf; size -= size / 2) ++depth;
  return depth;
}

__device__ __forceinline__ uint32_t bf16x2_add(uint32_t x, uint32_t y) {
  const float lo = __uint_as_float(x << 16) + __uint_as_float(y << 16);
  const float hi = __uint_as_float(x & 0xffff0000u) + __uint_as_float(y & 0xffff0000u);
  return pack_bf16x2(lo, hi);
}

// MAXD: number of tree levels below the root the kernel has slots for.
typedef float f32x32_t __attribute__((ext_vector_type(32)));

// MFMA: the leaf loop on the fp32 matrix pipe (else on the vector ALU).
template <int MAXD, bool MFMA>
__global__ __launch_bounds__(kTreeThreads, MAXD <= 10 ? 2 : 1) void det_gemm_tree_kernel(MatView A, MatView B, bf16_bits* __restrict__ C,
                                                                     int64_t ldc, int M, int N, int K, int tiles_m,
                                                                     int fast) {
  // Vector-ALU leaf: fp32 operands, [k][row]. Matrix-pipe leaf: bf16 operands as they lie in
  // memory, [row][k] with 80-byte rows (16-byte reads of consecutive rows fall on distinct banks).
  constexpr int kStageBytes = MFMA ? (kTreeBM + kTreeBN) * kTreeRowBytes : kTreeStageFloats * 4;
  __shared__ __attribute__((aligned(16))) char stage_bytes[2][kStageBytes];
  auto stage = [&](int buf) { return reinterpret_cast<float*>(stage_bytes[buf]); };

  const int tid = threadIdx.x;
  const int tile_m = blockIdx.x % tiles_m;
  const int tile_n = blockIdx.x / tiles_m;
  const int m0 = tile_m * kTreeBM;
  const int n0 = tile_n * kTreeBN;
  const int tx = tid & 15;  // columns 4 tx .. 4 tx + 3 and 64 + 4 tx .. 64 + 4 tx + 3
  const int ty = tid >> 4;  // rows 4 ty .. 4 ty + 3

  // Loader role: element (row, k) with k = tid % 32, rows tid / 32 + 8 j.
  const int load_k = tid & 31;
  const int load_row = tid >> 5;
  // Interior tiles address rows by a running offset; edge tiles clamp the row (rows past the
  // edge are computed from a valid row's data and never stored). k is clamped to K - 1: LDS
  // rows at and past a leaf's length are never used.
  const bool interior = m0 + kTreeBM <= M && n0 + kTreeBN <= N;
  const int a_last = M - 1 - m0, b_last = N - 1 - n0;
  const bf16_bits* a_tile = A.ptr + (int64_t)m0 * A.row_stride;
  const bf16_bits* b_tile = B.ptr + (int64_t)n0 * B.row_stride;
  bf16_bits a_reg[MFMA ? 1 : kTreeALoads], b_reg[MFMA ? 1 : kTreeBLoads];
  // Matrix-pipe kernel: 12 registers per thread. An operand with unit K stride, 16-byte aligned
  // rows and leaves that begin and end on multiples of 8 (bit 0 of `fast`: A, bit 1: B) is
  // fetched as 16-byte chunks (row tid / 4 (+ 64), chunk tid % 4 of the leaf); any other layout
  // element by element, two bf16 per register.
  uint32_t held[12];
  const bool a_fast = MFMA && (fast & 1), b_fast = MFMA && (fast & 2);
  const int chunk_row = tid >> 2, chunk = tid & 3;
  auto fetch = [&](int lo) {
    if constexpr (MFMA) {
      const int kc = lo + 8 * chunk < K ? lo + 8 * chunk : 0;  // a chunk past the leaf is not used
      if (a_fast) {
        const int row = chunk_row < a_last ? chunk_row : a_last;
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(a_tile + (int64_t)row * A.row_stride + kc);
        held[0] = v[0]; held[1] = v[1]; held[2] = v[2]; held[3] = v[3];
      }
      if (b_fast) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int row = chunk_row + 64 * j < b_last ? chunk_row + 64 * j : b_last;
          const u32x4_t v = *reinterpret_cast<const u32x4_t*>(b_tile + (int64_t)row * B.row_stride + kc);
          held[4 + 4 * j] = v[0]; held[5 + 4 * j] = v[1]; held[6 + 4 * j] = v[2]; held[7 + 4 * j] = v[3];
        }
      }
      const int k = (lo + load_k < K) ? lo + load_k : K - 1;
      if (!a_fast) {
        const bf16_bits* a_col = a_tile + (int64_t)k * A.k_stride;
#pragma unroll
        for (int j = 0; j < kTreeALoads; j += 2) {
          const int r0 = load_row + 8 * j, r1 = r0 + 8;
          const uint32_t e0 = a_col[(int64_t)(r0 < a_last ? r0 : a_last) * A.row_stride];
          const uint32_t e1 = a_col[(int64_t)(r1 < a_last ? r1 : a_last) * A.row_stride];
          held[j / 2] = e0 | (e1 << 16);
        }
      }
      if (!b_fast) {
        const bf16_bits* b_col = b_tile + (int64_t)k * B.k_stride;
#pragma unroll
        for (int j = 0; j < kTreeBLoads; j += 2) {
          const int r0 = load_row + 8 * j, r1 = r0 + 8;
          const uint32_t e0 = b_col[(int64_t)(r0 < b_last ? r0 : b_last) * B.row_stride];
          const uint32_t e1 = b_col[(int64_t)(r1 < b_last ? r1 : b_last) * B.row_stride];
          held[4 + j / 2] = e0 | (e1 << 16);
        }
      }
    } else {
      const int k = (lo + load_k < K) ? lo + load_k : K - 1;
      const bf16_bits* a_col = a_tile + (int64_t)k * A.k_stride;
      const bf16_bits* b_col = b_tile + (int64_t)k * B.k_stride;
      if (interior) {
        int64_t off = (int64_t)load_row * A.row_stride;
#pragma unroll
        for (int j = 0; j < kTreeALoads; ++j, off += 8 * A.row_stride) a_reg[j] = a_col[off];
        off = (int64_t)load_row * B.row_stride;
#pragma unroll
        for (int j = 0; j < kTreeBLoads; ++j, off += 8 * B.row_stride) b_reg[j] = b_col[off];
      } else {
#pragma unroll
        for (int j = 0; j < kTreeALoads; ++j) {
          const int row = load_row + 8 * j;
          a_reg[j] = a_col[(int64_t)(row < a_last ? row : a_last) * A.row_stride];
        }
#pragma unroll
        for (int j = 0; j < kTreeBLoads; ++j) {
          const int row = load_row + 8 * j;
          b_reg[j] = b_col[(int64_t)(row < b_last ? row : b_last) * B.row_stride];
        }
      }
    }
  };
  auto deposit = [&](int buf) {
    if constexpr (MFMA) {
      char* as = stage_bytes[buf];
      char* bs = as + kTreeBM * kTreeRowBytes;
      if (a_fast) {
        *reinterpret_cast<u32x4_t*>(as + chunk_row * kTreeRowBytes + 16 * chunk) = u32x4_t{held[0], held[1], held[2], held[3]};
      } else {
#pragma unroll
        for (int j = 0; j < kTreeALoads; ++j)
          *reinterpret_cast<bf16_bits*>(as + (load_row + 8 * j) * kTreeRowBytes + 2 * load_k) =
              (bf16_bits)((held[j / 2] >> (16 * (j & 1))) & 0xffffu);
      }
      if (b_fast) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
          *reinterpret_cast<u32x4_t*>(bs + (chunk_row + 64 * j) * kTreeRowBytes + 16 * chunk) =
              u32x4_t{held[4 + 4 * j], held[5 + 4 * j], held[6 + 4 * j], held[7 + 4 * j]};
      } else {
#pragma unroll
        for (int j = 0; j < kTreeBLoads; ++j)
          *reinterpret_cast<bf16_bits*>(bs + (load_row + 8 * j) * kTreeRowBytes + 2 * load_k) =
              (bf16_bits)((held[4 + j / 2] >> (16 * (j & 1))) & 0xffffu);
      }
    } else {
      float* as = stage(buf);
      float* bs = as + kTreeLeaf * kTreeAStride;
#pragma unroll
      for (int j = 0; j < kTreeALoads; ++j) as[load_k * kTreeAStride + load_row + 8 * j] = bf16_bits_to_float(a_reg[j]);
#pragma unroll
      for (int j = 0; j < kTreeBLoads; ++j) bs[load_k * kTreeBStride + load_row + 8 * j] = bf16_bits_to_float(b_reg[j]);
    }
  };

  // [lo, hi) of the node reached from the root by `path` (bit d set: right child at depth d).
  auto range_at = [&](int depth, uint32_t path, int& lo, int& hi) {
    lo = 0;
    hi = K;
    for (int d = 1; d <= depth; ++d) {
      const int mid = lo + (hi - lo) / 2;
      if ((path >> d) & 1u) lo = mid; else hi = mid;
    }
  };

  uint32_t slot[MAXD][16];  // slot[d - 1]: finished left child at depth d, waiting for its sibling
  uint32_t cur[16];

  int depth = 0, lo = 0, hi = K;
  uint32_t path = 0;
  while (hi - lo > kTreeLeaf) {
    hi = lo + (hi - lo) / 2;
    ++depth;
  }
  fetch(lo);
  deposit(0);
  __syncthreads();

  for (int leaf = 0;; ++leaf) {
    // The next leaf: climb while the current node is a right child, step to the right
    // sibling, descend along left children.
    int nd = depth;
    while (nd > 0 && ((path >> nd) & 1u)) --nd;
    const bool has_next = nd > 0;
    uint32_t npath = path;
    int nlo = 0, nhi = 0, ndepth = 0;
    if (has_next) {
      npath = (path & ((1u << nd) - 1u)) | (1u << nd);
      range_at(nd, npath, nlo, nhi);
      ndepth = nd;
      while (nhi - nlo > kTreeLeaf) {
        nhi = nlo + (nhi - nlo) / 2;
        ++ndepth;
      }
      fetch(nlo);
    }

    // The leaf: 32 independent chains per thread, k ascending.
    const float* as = stage(leaf & 1);
    const float* bs = as + kTreeLeaf * kTreeAStride;
    const int len = hi - lo;
    if constexpr (MFMA) {
      // Wave w: rows 32 (w & 1) ..., columns 64 (w >> 1) .... Block 0 of the instruction takes
      // columns 0..31, block 1 columns 32..63; the row operand of block 0 serves both (cbsz = 1).
      const int lane = tid & 63, wave = tid >> 6;
      const char* arow = stage_bytes[leaf & 1] + (32 * (wave & 1) + (lane & 31)) * kTreeRowBytes;
      const char* brow = stage_bytes[leaf & 1] + (kTreeBM + 64 * (wave >> 1) + lane) * kTreeRowBytes;
      f32x32_t acc;
#pragma unroll
      for (int r = 0; r < 32; ++r) acc[r] = 0.f;
      // Element 2 i of a chunk is the low half of word i, element 2 i + 1 the high half; either way
      // the fp32 operand is the bf16 pattern in the upper 16 bits.
      auto step = [&](const u32x4_t& av, const u32x4_t& bv, int e) {
        const float a = __uint_as_float((e & 1) ? (av[e >> 1] & 0xffff0000u) : (av[e >> 1] << 16));
        const float b = __uint_as_float((e & 1) ? (bv[e >> 1] & 0xffff0000u) : (bv[e >> 1] << 16));
        acc = __builtin_amdgcn_mfma_f32_32x32x1f32(a, b, acc, 1, 0, 0);
      };
      const int whole = len >> 3, rest = len & 7;
      for (int c = 0; c < whole; ++c) {
        const u32x4_t av = *reinterpret_cast<const u32x4_t*>(arow + 16 * c);
        const u32x4_t bv = *reinterpret_cast<const u32x4_t*>(brow + 16 * c);
#pragma unroll
        for (int e = 0; e < 8; ++e) step(av, bv, e);
      }
      if (rest) {  // the chunk is read whole (it lies inside the row); only its first `rest` elements count
        const u32x4_t av = *reinterpret_cast<const u32x4_t*>(arow + 16 * whole);
        const u32x4_t bv = *reinterpret_cast<const u32x4_t*>(brow + 16 * whole);
#pragma unroll
        for (int e = 0; e < 7; ++e)
          if (e < rest) step(av, bv, e);
      }
#pragma unroll
      for (int q = 0; q < 16; ++q) cur[q] = pack_bf16x2(acc[2 * q], acc[2 * q + 1]);
    } else {
    float acc[4][8];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = 0.f;
    // Operands of step k + 1 are read while step k is summed (one wave per SIMD: nothing else
    // hides the LDS latency). Row len of the stage is read and not used.
    const float* ap = as + 4 * ty;
    const float* bp = bs + 4 * tx;
    auto read_step = [&](int k, f32x4_t& av, f32x4_t& b0, f32x4_t& b1) {
      k = k < kTreeLeaf ? k : kTreeLeaf - 1;
      av = *reinterpret_cast<const f32x4_t*>(ap + k * kTreeAStride);
      b0 = *reinterpret_cast<const f32x4_t*>(bp + k * kTreeBStride);
      b1 = *reinterpret_cast<const f32x4_t*>(bp + k * kTreeBStride + 64);
      __builtin_amdgcn_sched_barrier(0);  // the reads stay above the multiply-adds that follow
    };
    auto fma_step = [&](const f32x4_t& av, const f32x4_t& b0, const f32x4_t& b1) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = __builtin_fmaf(av[i], b0[j], acc[i][j]);
          acc[i][4 + j] = __builtin_fmaf(av[i], b1[j], acc[i][4 + j]);
        }
      }
    };
    f32x4_t av0, b00, b10, av1, b01, b11;  // two operand sets, alternating
    read_step(0, av0, b00, b10);
    int k = 0;
    for (; k + 1 < len; k += 2) {
      read_step(k + 1, av1, b01, b11);
      fma_step(av0, b00, b10);
      read_step(k + 2, av0, b00, b10);
      fma_step(av1, b01, b11);
    }
    if (k < len) fma_step(av0, b00, b10);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) cur[i * 4 + j] = pack_bf16x2(acc[i][2 * j], acc[i][2 * j + 1]);

    }

    // Finished right children meet their waiting siblings.
    int d = depth;
    while (d > 0 && ((path >> d) & 1u)) {
#pragma unroll
      for (int s = 1; s <= MAXD; ++s) {
        if (s == d) {
#pragma unroll
          for (int r = 0; r < 16; ++r) cur[r] = bf16x2_add(slot[s - 1][r], cur[r]);
        }
      }
      --d;
    }
    if (d == 0) break;  // cur is the root
#pragma unroll
    for (int s = 1; s <= MAXD; ++s) {
      if (s == d) {
#pragma unroll
        for (int r = 0; r < 16; ++r) slot[s - 1][r] = cur[r];
      }
    }

    deposit((leaf + 1) & 1);
    __syncthreads();
    depth = ndepth;
    path = npath;
    lo = nlo;
    hi = nhi;
  }

  if constexpr (MFMA) {
    // Accumulator r of the instruction: block r / 16 (32 columns each); within a block
    // row 8 (q / 4) + 4 (lane / 32) + q % 4 with q = r % 16, column lane % 32. cur packs
    // accumulators 2 q', 2 q' + 1 (two consecutive rows of one column).
    const int lane = tid & 63, wave = tid >> 6;
    const int row_base = m0 + 32 * (wave & 1) + 4 * (lane >> 5);
    const int col_base = n0 + 64 * (wave >> 1) + (lane & 31);
#pragma unroll
    for (int r = 0; r < 32; ++r) {
      const int q = r & 15;
      const int row = row_base + 8 * (q >> 2) + (q & 3);
      const int col = col_base + 32 * (r >> 4);
      const uint32_t pair = cur[r >> 1];
      if (row < M && col < N) C[(int64_t)row * ldc + col] = (bf16_bits)((r & 1) ? (pair >> 16) : (pair & 0xffffu));
    }
    return;
  }
  // cur[i * 4 + j]: row 4 ty + i, column pair (j < 2 ? 4 tx + 2 j : 64 + 4 tx + 2 (j - 2)).
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = m0 + 4 * ty + i;
    if (row >= M) continue;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int col = n0 + half * 64 + 4 * tx;
      bf16_bits* dst = C + (int64_t)row * ldc + col;
      const uint32_t p0 = cur[i * 4 + 2 * half], p1 = cur[i * 4 + 2 * half + 1];
      if (col + 4 <= N && (reinterpret_cast<uintptr_t>(dst) & 7) == 0) {
        *reinterpret_cast<u32x2_t*>(dst) = u32x2_t{p0, p1};
      } else {
        if (col < N) dst[0] = (bf16_bits)(p0 & 0xffffu);
        if (col + 1 < N) dst[1] = (bf16_bits)(p0 >> 16);
        if (col + 2 < N) dst[2] = (bf16_bits)(p1 & 0xffffu);
        if (col + 3 < N) dst[3] = (bf16_bits)(p1 >> 16);
      }
    }
  }
}

int det_gemm_tree_max_k() { return kTreeLeaf << 20; }

template <bool MFMA>
static hipError_t launch_tree(const MatView& A, const MatView& B, bf16_bits* out, int64_t ldc, int M, int N, int K,
                              int depth, unsigned tiles, int tiles_m, int fast, hipStream_t stream) {
  if (depth <= 7) {  // K <= 4096: few enough slots for two workgroups per CU
    hipLaunchKernelGGL((det_gemm_tree_kernel<7, MFMA>), dim3(tiles), dim3(kTreeThreads), 0, stream, A, B, out, ldc, M, N,
                       K, tiles_m, fast);
  } else if (depth <= 10) {
    hipLaunchKernelGGL((det_gemm_tree_kernel<10, MFMA>), dim3(tiles), dim3(kTreeThreads), 0, stream, A, B, out, ldc, M,
                       N, K, tiles_m, fast);
  } else if (depth <= 20) {
    hipLaunchKernelGGL((det_gemm_tree_kernel<20, MFMA>), dim3(tiles), dim3(kTreeThreads), 0, stream, A, B, out, ldc, M,
                       N, K, tiles_m, fast);
  } else {
    return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

// A[M, K] and B as rows of output columns (B.rows = N), any strides; C[m * ldc + n].
// config: RLK_TREE_CFG_AUTO, or one of the two leaf loops (same bits).
hipError_t det_gemm_tree_launch(const MatView& A, const MatView& B, void* C, int64_t ldc, int M, int N, int K,
                                int config, hipStream_t stream) {
  const int tiles_m = (M + kTreeBM - 1) / kTreeBM;
  const int tiles_n = (N + kTreeBN - 1) / kTreeBN;
  const int64_t tiles = (int64_t)tiles_m * tiles_n;
  if (tiles > 0x7fffffff) return hipErrorInvalidValue;
  const int depth = tree_depth(K);
  bf16_bits* out = reinterpret_cast<bf16_bits*>(C);
  if (config == RLK_TREE_CFG_VALU)
    return launch_tree<false>(A, B, out, ldc, M, N, K, depth, (unsigned)tiles, tiles_m, 0, stream);
  if (config == RLK_TREE_CFG_AUTO || config == RLK_TREE_CFG_MFMA_F32) {
    // 16-byte chunks: every leaf begins and ends on a multiple of 8 (all leaves are K >> depth
    // long when that divides), rows contiguous in K and 16-byte aligned.
    const bool leaves_whole = depth <= 20 && K % (8 << depth) == 0;
    auto chunked = [&](const MatView& v) {
      return leaves_whole && v.k_stride == 1 && v.row_stride % 8 == 0 && (reinterpret_cast<uintptr_t>(v.ptr) & 15) == 0;
    };
    const int fast = (chunked(A) ? 1 : 0) | (chunked(B) ? 2 : 0);
    return launch_tree<true>(A, B, out, ldc, M, N, K, depth, (unsigned)tiles, tiles_m, fast, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace rlk
