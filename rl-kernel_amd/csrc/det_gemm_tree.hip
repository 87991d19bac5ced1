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
//   * vector ALU (det_gemm_tree_kernel): 256 threads per tile, a thread owns 4 rows x 8
//     columns and issues one v_fma_f32 per term; operands staged in LDS as fp32, [k][row];
//   * fp32 matrix pipe (det_gemm_tree_wide_kernel, the default for operands the node-per-wave kernel below
//     does not take): 512 threads per tile, a wave
//     owns 32 rows x 32 columns and issues one v_mfma_f32_16x16x1_4b_f32 per k. With a
//     reduction length of one, an instruction adds exactly one product to every accumulator,
//     and the product of two bf16 values is exact in fp32, so the step is the same single
//     rounding as the fused multiply-add, at twice the vector rate; operands staged in LDS
//     as fp32, [row][k].
//
// Two more kernels split K along the contract's own tree: the 16 nodes at depth 4 (8 at depth 3) are
// independent, a wave evaluates one of them for a block of outputs, and the bf16 nodes are folded in tree
// order: det_gemm_tree_nodes_kernel (fp32 matrix pipe, any row count; the fastest of all on K-contiguous aligned
// operands with equal leaves, and what RLK_TREE_CFG_AUTO picks for them) and det_gemm_tree_skinny_kernel (up to
// 16 rows, vector ALU; trees of 11 and 12 levels, which the former has no register slots for).
//
// Tiled kernels: a workgroup owns a 64 x 128 output tile. Leaves are visited left to right, the next leaf
// is fetched while the current one is summed. The tree is evaluated on the
// fly: a finished node waits in the register slot of its depth until its right sibling is
// finished, so a thread holds at most one bf16 node per tree level. Which slot is read or
// written is the same for every thread (it depends on K only), so the slot index is a
// uniform branch over compile-time register arrays, never an indexed register access.
#include "det_gemm_tile.h"
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
template <int MAXD>
__global__ __launch_bounds__(kTreeThreads, MAXD <= 10 ? 2 : 1) void det_gemm_tree_kernel(MatView A, MatView B, bf16_bits* __restrict__ C,
                                                                     int64_t ldc, int M, int N, int K, int tiles_m) {
  __shared__ __attribute__((aligned(16))) float stage[2][kTreeStageFloats];

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
  bf16_bits a_reg[kTreeALoads], b_reg[kTreeBLoads];
  auto fetch = [&](int lo) {
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
  };
  auto deposit = [&](int buf) {
    float* as = stage[buf];
    float* bs = as + kTreeLeaf * kTreeAStride;
#pragma unroll
    for (int j = 0; j < kTreeALoads; ++j) as[load_k * kTreeAStride + load_row + 8 * j] = bf16_bits_to_float(a_reg[j]);
#pragma unroll
    for (int j = 0; j < kTreeBLoads; ++j) bs[load_k * kTreeBStride + load_row + 8 * j] = bf16_bits_to_float(b_reg[j]);
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
    const float* as = stage[leaf & 1];
    const float* bs = as + kTreeLeaf * kTreeAStride;
    float acc[4][8];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = 0.f;
    const int len = hi - lo;
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

// The matrix-pipe leaf with eight waves per tile: a wave owns 32 rows x 32 columns (the four
// 16 x 16 blocks of v_mfma_f32_16x16x1_4b_f32), 16 accumulators and 8 packed tree registers per
// level per lane, so four waves fit on a SIMD. Measured, vector instructions do not run under this
// matrix instruction (matrix-pipe busy cycles and vector issue cycles add up to the kernel's time),
// so what the kernel saves is vector instructions: operands are converted to fp32 once, on their
// way into LDS ([row][k], 144-byte rows: a lane's 16-byte read of its own row is conflict free),
// and a k step needs none besides the MFMA.
constexpr int kTreeWideThreads = 512;
constexpr int kTreeWideRowBytes = 4 * kTreeLeaf + 16;
constexpr int kTreeWideRowBytesBf16 = 2 * kTreeLeaf + 16;
typedef float f32x16_t __attribute__((ext_vector_type(16)));

// F32_STAGE = false keeps the operands in LDS as bf16 (80-byte rows) and makes the fp32 pattern
// with one shift or mask per operand and k instead: fewer live registers, which is what decides
// between four waves per SIMD and spills when the tree has 8 to 10 levels.
template <int MAXD, bool F32_STAGE>
__global__ __launch_bounds__(kTreeWideThreads, MAXD <= 10 ? 4 : 2) void det_gemm_tree_wide_kernel(
    MatView A, MatView B, bf16_bits* __restrict__ C, int64_t ldc, int M, int N, int K, int tiles_m, int fast) {
  constexpr int kRowBytes = F32_STAGE ? kTreeWideRowBytes : kTreeWideRowBytesBf16;
  constexpr int kStageBytes = (kTreeBM + kTreeBN) * kRowBytes;
  __shared__ __attribute__((aligned(16))) char stage_bytes[2][kStageBytes];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int tile_m = blockIdx.x % tiles_m;
  const int tile_n = blockIdx.x / tiles_m;
  const int m0 = tile_m * kTreeBM;
  const int n0 = tile_n * kTreeBN;
  const int a_last = M - 1 - m0, b_last = N - 1 - n0;
  const bf16_bits* a_tile = A.ptr + (int64_t)m0 * A.row_stride;
  const bf16_bits* b_tile = B.ptr + (int64_t)n0 * B.row_stride;

  // Staging roles. Chunked operand (bit 0 of `fast`: A, bit 1: B): thread t holds chunk t % 4 of
  // row t / 4 (B: 128 rows, all threads; A: 64 rows, threads 0..255). Element-wise operand:
  // k = t % 32, rows t / 32 + 16 j, two bf16 per register.
  // Row-contiguous operand (K-major; bit 3: A, bit 4: B; rows a multiple of 8): thread t holds the
  // 16-byte chunk of eight rows at one k: A rows 8 (t % 8) ..., k = t / 8 (threads 0..255); B rows
  // 8 (t % 16) ..., k = t / 16.
  const bool a_fast = fast & 1, b_fast = fast & 2;
  const bool a_rows8 = fast & 8, b_rows8 = fast & 16;
  const int chunk_row = tid >> 2, chunk = tid & 3;
  const int load_k = tid & 31, load_row = tid >> 5;
  uint32_t held[8];  // [0, 4): A, [4, 8): B
  auto fetch = [&](int lo) {
    const int kc = lo + 8 * chunk < K ? lo + 8 * chunk : 0;  // a chunk past the leaf is not used
    const int k = (lo + load_k < K) ? lo + load_k : K - 1;
    if (a_fast) {
      if (tid < 256) {
        const int row = chunk_row < a_last ? chunk_row : a_last;
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(a_tile + (int64_t)row * A.row_stride + kc);
        held[0] = v[0]; held[1] = v[1]; held[2] = v[2]; held[3] = v[3];
      }
    } else if (a_rows8) {
      if (tid < 256) {
        const int kk = lo + (tid >> 3) < K ? lo + (tid >> 3) : K - 1;
        const int row = 8 * (tid & 7) <= a_last ? 8 * (tid & 7) : 0;  // a group past the edge is not stored
        const u32x4_t v = *reinterpret_cast<const u32x4_t*>(a_tile + (int64_t)kk * A.k_stride + row);
        held[0] = v[0]; held[1] = v[1]; held[2] = v[2]; held[3] = v[3];
      }
    } else {
      const bf16_bits* a_col = a_tile + (int64_t)k * A.k_stride;
#pragma unroll
      for (int j = 0; j < 4; j += 2) {
        const int r0 = load_row + 16 * j, r1 = r0 + 16;
        const uint32_t e0 = a_col[(int64_t)(r0 < a_last ? r0 : a_last) * A.row_stride];
        const uint32_t e1 = a_col[(int64_t)(r1 < a_last ? r1 : a_last) * A.row_stride];
        held[j / 2] = e0 | (e1 << 16);
      }
    }
    if (b_fast) {
      const int row = chunk_row < b_last ? chunk_row : b_last;
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(b_tile + (int64_t)row * B.row_stride + kc);
      held[4] = v[0]; held[5] = v[1]; held[6] = v[2]; held[7] = v[3];
    } else if (b_rows8) {
      const int kk = lo + (tid >> 4) < K ? lo + (tid >> 4) : K - 1;
      const int row = 8 * (tid & 15) <= b_last ? 8 * (tid & 15) : 0;
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(b_tile + (int64_t)kk * B.k_stride + row);
      held[4] = v[0]; held[5] = v[1]; held[6] = v[2]; held[7] = v[3];
    } else {
      const bf16_bits* b_col = b_tile + (int64_t)k * B.k_stride;
#pragma unroll
      for (int j = 0; j < 8; j += 2) {
        const int r0 = load_row + 16 * j, r1 = r0 + 16;
        const uint32_t e0 = b_col[(int64_t)(r0 < b_last ? r0 : b_last) * B.row_stride];
        const uint32_t e1 = b_col[(int64_t)(r1 < b_last ? r1 : b_last) * B.row_stride];
        held[4 + j / 2] = e0 | (e1 << 16);
      }
    }
  };
  // bf16 pair in one register -> two fp32 patterns
  auto lo_f32 = [](uint32_t v) { return v << 16; };
  auto hi_f32 = [](uint32_t v) { return v & 0xffff0000u; };
  auto deposit_chunk = [&](char* row, const uint32_t* v) {
    *reinterpret_cast<u32x4_t*>(row + 32 * chunk) = u32x4_t{lo_f32(v[0]), hi_f32(v[0]), lo_f32(v[1]), hi_f32(v[1])};
    *reinterpret_cast<u32x4_t*>(row + 32 * chunk + 16) = u32x4_t{lo_f32(v[2]), hi_f32(v[2]), lo_f32(v[3]), hi_f32(v[3])};
  };
  // eight rows of one k: element i of the chunk goes to row first + i, column k
  auto deposit_rows8 = [&](char* stage_rows, int first, int k, const uint32_t* v) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      char* at = stage_rows + (first + i) * kRowBytes;
      if constexpr (F32_STAGE) {
        *reinterpret_cast<uint32_t*>(at + 4 * k) = (i & 1) ? hi_f32(v[i / 2]) : lo_f32(v[i / 2]);
      } else {
        *reinterpret_cast<bf16_bits*>(at + 2 * k) = (bf16_bits)((v[i / 2] >> (16 * (i & 1))) & 0xffffu);
      }
    }
  };
  auto deposit = [&](int buf) {
    char* as = stage_bytes[buf];
    char* bs = as + kTreeBM * kRowBytes;
    if (a_rows8 && tid < 256) deposit_rows8(as, 8 * (tid & 7), tid >> 3, held);
    if (b_rows8) deposit_rows8(bs, 8 * (tid & 15), tid >> 4, held + 4);
    if constexpr (F32_STAGE) {
      if (a_fast) {
        if (tid < 256) deposit_chunk(as + chunk_row * kRowBytes, held);
      } else if (!a_rows8) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          *reinterpret_cast<uint32_t*>(as + (load_row + 16 * j) * kRowBytes + 4 * load_k) =
              (j & 1) ? hi_f32(held[j / 2]) : lo_f32(held[j / 2]);
      }
      if (b_fast) {
        deposit_chunk(bs + chunk_row * kRowBytes, held + 4);
      } else if (!b_rows8) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          *reinterpret_cast<uint32_t*>(bs + (load_row + 16 * j) * kRowBytes + 4 * load_k) =
              (j & 1) ? hi_f32(held[4 + j / 2]) : lo_f32(held[4 + j / 2]);
      }
    } else {
      if (a_fast) {
        if (tid < 256)
          *reinterpret_cast<u32x4_t*>(as + chunk_row * kRowBytes + 16 * chunk) = u32x4_t{held[0], held[1], held[2], held[3]};
      } else if (!a_rows8) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          *reinterpret_cast<bf16_bits*>(as + (load_row + 16 * j) * kRowBytes + 2 * load_k) =
              (bf16_bits)((held[j / 2] >> (16 * (j & 1))) & 0xffffu);
      }
      if (b_fast) {
        *reinterpret_cast<u32x4_t*>(bs + chunk_row * kRowBytes + 16 * chunk) = u32x4_t{held[4], held[5], held[6], held[7]};
      } else if (!b_rows8) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          *reinterpret_cast<bf16_bits*>(bs + (load_row + 16 * j) * kRowBytes + 2 * load_k) =
              (bf16_bits)((held[4 + j / 2] >> (16 * (j & 1))) & 0xffffu);
      }
    }
  };

  // A node is a range [lo, hi) of units, split at lo + (hi - lo) / 2. Element-space split (the contract of
  // rlk_det_gemm_tree_contract_id): a unit is one k, and a node of at most 32 units is a leaf. Leaf-space split
  // (bit 5 of `fast`): a unit is one of the fixed 32-wide K tiles [32 i, min(32 i + 32, K)), and a node of one
  // unit is a leaf. The two trees are the same when K / 32 is a power of two.
  const bool leaf_space = fast & 32;
  const int unit = leaf_space ? kTreeLeaf : 1;
  const int units = leaf_space ? (K + kTreeLeaf - 1) / kTreeLeaf : K;
  const int leaf_units = leaf_space ? 1 : kTreeLeaf;
  auto range_at = [&](int depth, uint32_t path, int& lo, int& hi) {
    lo = 0;
    hi = units;
    for (int d = 1; d <= depth; ++d) {
      const int mid = lo + (hi - lo) / 2;
      if ((path >> d) & 1u) lo = mid; else hi = mid;
    }
  };

  uint32_t slot[MAXD][8];  // slot[d - 1]: finished left child at depth d, waiting for its sibling
  uint32_t cur[8];

  // Wave w: rows 32 (w & 1) ..., columns 32 (w >> 1) .... Block b of the instruction is rows
  // 16 (b >> 1) ..., columns 16 (b & 1) ...: lane l feeds row 16 (l >> 5) + l % 16 and column
  // 16 ((l >> 4) & 1) + l % 16.
  const int a_row = 32 * (wave & 1) + 16 * (lane >> 5) + (lane & 15);
  const int b_row = kTreeBM + 32 * (wave >> 1) + 16 * ((lane >> 4) & 1) + (lane & 15);

  int depth = 0, lo = 0, hi = units;
  uint32_t path = 0;
  while (hi - lo > leaf_units) {
    hi = lo + (hi - lo) / 2;
    ++depth;
  }
  fetch(lo * unit);
  deposit(0);
  __syncthreads();

  for (int leaf = 0;; ++leaf) {
    bool has_next;
    uint32_t npath = path;
    int nlo = 0, nhi = 0, ndepth = 0;
    if (fast & 4) {
      // All leaves equally long (2^depth divides K): leaf i is [i * len, (i + 1) * len) at the
      // deepest level, and bit d of its path is bit depth - d of i.
      const int next = leaf + 1;
      has_next = next < (1 << depth);
      if (has_next) {
        nlo = next * (hi - lo);
        nhi = nlo + (hi - lo);
        ndepth = depth;
        npath = (__brev((uint32_t)next) >> (32 - depth)) << 1;
      }
    } else {
      int nd = depth;
      while (nd > 0 && ((path >> nd) & 1u)) --nd;
      has_next = nd > 0;
      if (has_next) {
        npath = (path & ((1u << nd) - 1u)) | (1u << nd);
        range_at(nd, npath, nlo, nhi);
        ndepth = nd;
        while (nhi - nlo > leaf_units) {
          nhi = nlo + (nhi - nlo) / 2;
          ++ndepth;
        }
      }
    }
    if (has_next) fetch(nlo * unit);

    const int len = (hi * unit < K ? hi * unit : K) - lo * unit;
    const char* arow = stage_bytes[leaf & 1] + a_row * kRowBytes;
    const char* brow = stage_bytes[leaf & 1] + b_row * kRowBytes;
    f32x16_t acc;
    if constexpr (F32_STAGE) {
      // Four k per 16-byte read. The first step of a leaf adds to a literal zero (no registers to
      // clear); a group past the leaf's length is read whole (it lies inside the row) and only its
      // first len % 4 elements count.
      auto read4 = [&](int g, f32x4_t& av, f32x4_t& bv) {
        av = *reinterpret_cast<const f32x4_t*>(arow + 16 * g);
        bv = *reinterpret_cast<const f32x4_t*>(brow + 16 * g);
      };
      f32x4_t av, bv;
      read4(0, av, bv);
      acc = __builtin_amdgcn_mfma_f32_16x16x1f32(av[0], bv[0], f32x16_t{}, 0, 0, 0);
      const int groups = len >> 2, rest = len & 3;
      if (groups > 0) {
#pragma unroll
        for (int e = 1; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x1f32(av[e], bv[e], acc, 0, 0, 0);
        for (int g = 1; g < groups; ++g) {
          read4(g, av, bv);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x1f32(av[e], bv[e], acc, 0, 0, 0);
        }
        if (rest) {
          read4(groups, av, bv);
#pragma unroll
          for (int e = 0; e < 3; ++e)
            if (e < rest) acc = __builtin_amdgcn_mfma_f32_16x16x1f32(av[e], bv[e], acc, 0, 0, 0);
        }
      } else {
#pragma unroll
        for (int e = 1; e < 3; ++e)
          if (e < rest) acc = __builtin_amdgcn_mfma_f32_16x16x1f32(av[e], bv[e], acc, 0, 0, 0);
      }
    } else {
      // Eight k per 16-byte read; element 2 i of a chunk is the low half of word i, element 2 i + 1
      // the high half, and the fp32 operand is that bf16 pattern in the upper 16 bits.
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.f;
      auto step = [&](const u32x4_t& av, const u32x4_t& bv, int e) {
        const float a = __uint_as_float((e & 1) ? (av[e >> 1] & 0xffff0000u) : (av[e >> 1] << 16));
        const float b = __uint_as_float((e & 1) ? (bv[e >> 1] & 0xffff0000u) : (bv[e >> 1] << 16));
        acc = __builtin_amdgcn_mfma_f32_16x16x1f32(a, b, acc, 0, 0, 0);
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
    }
#pragma unroll
    for (int q = 0; q < 8; ++q) cur[q] = pack_bf16x2(acc[2 * q], acc[2 * q + 1]);

    int d = depth;
    while (d > 0 && ((path >> d) & 1u)) {
#pragma unroll
      for (int s = 1; s <= MAXD; ++s) {
        if (s == d) {
#pragma unroll
          for (int r = 0; r < 8; ++r) cur[r] = bf16x2_add(slot[s - 1][r], cur[r]);
        }
      }
      --d;
    }
    if (d == 0) break;  // cur is the root
#pragma unroll
    for (int s = 1; s <= MAXD; ++s) {
      if (s == d) {
#pragma unroll
        for (int r = 0; r < 8; ++r) slot[s - 1][r] = cur[r];
      }
    }

    deposit((leaf + 1) & 1);
    __syncthreads();
    depth = ndepth;
    path = npath;
    lo = nlo;
    hi = nhi;
  }

  // Accumulator r: block r / 4; row 16 (block >> 1) + 4 (lane / 16) + r % 4, column 16 (block & 1) + lane % 16.
  // cur[q] packs accumulators 2 q, 2 q + 1 (two consecutive rows of one column).
  const int row_base = m0 + 32 * (wave & 1) + 4 * (lane >> 4);
  const int col_base = n0 + 32 * (wave >> 1) + (lane & 15);
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int block = r >> 2;
    const int row = row_base + 16 * (block >> 1) + (r & 3);
    const int col = col_base + 16 * (block & 1);
    const uint32_t pair = cur[r >> 1];
    if (row < M && col < N) C[(int64_t)row * ldc + col] = (bf16_bits)((r & 1) ? (pair >> 16) : (pair & 0xffffu));
  }
}

// Up to 16 rows of A (decode): the weight must stream at memory rate, and one chain per output
// is too little parallelism (N lanes in all). The contract's own tree supplies more: the 16 nodes
// at depth 4 are independent, so a workgroup of 16 waves takes 64 columns, wave w evaluates node w
// (a sixteenth of K) for them, one column per lane and MR fp32 chains per lane (plain v_fma_f32,
// A values uniform across the wave), and wave 0 folds the 16 bf16 nodes in tree order. Needs
// a uniform tree (every leaf K >> depth long, a multiple of 8), K-contiguous 16-byte aligned rows.
constexpr int kTreeSkinnySplit = 4;                       // depth of the nodes the waves take
constexpr int kTreeSkinnyWaves = 1 << kTreeSkinnySplit;   // 16
constexpr int kTreeSkinnyLevels = 8;                      // tree levels below a wave's node
constexpr int kTreeHalvesMaxN = 8192;                     // up to this many columns (and 8 rows) the wave halves split a node

// HALVES: the two halves of a wave take the two children of the wave's node (32 nodes at depth 5, 32
// columns per workgroup) and exchange them through a lane shuffle: twice the workgroups for narrow N.
template <int MR, bool HALVES>
__global__ __launch_bounds__(64 * kTreeSkinnyWaves) void det_gemm_tree_skinny_kernel(
    MatView A, MatView B, bf16_bits* __restrict__ C, int64_t ldc, int M, int N, int K, int depth) {
  static_assert(MR % 2 == 0 && MR <= 16, "rows are packed in pairs");
  constexpr int PR = MR / 2;
  __shared__ uint32_t nodes[kTreeSkinnyWaves][PR][64];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  constexpr int kCols = HALVES ? 32 : 64;
  const int col = blockIdx.x * kCols + (lane & (kCols - 1));
  const int node = HALVES ? 2 * wave + (lane >> 5) : wave;
  const int node_depth = HALVES ? kTreeSkinnySplit + 1 : kTreeSkinnySplit;
  const bf16_bits* wrow = B.ptr + (int64_t)(col < N ? col : N - 1) * B.row_stride;
  const int len = K >> depth;                              // leaf length, 8 ... 32, a multiple of 8
  const int leaves = 1 << (depth - node_depth);            // leaves under this lane's node
  const int first = node * leaves * len;                   // node j covers leaves [j * leaves, (j + 1) * leaves)
  const bf16_bits* arow[MR];
#pragma unroll
  for (int m = 0; m < MR; ++m) arow[m] = A.ptr + (int64_t)(m < M ? m : M - 1) * A.row_stride;

  uint32_t slot[kTreeSkinnyLevels][PR];  // slot[l]: finished left child l levels above the leaves
  uint32_t cur[PR];
  u32x4_t w_now[4], w_next[4];
  auto fetch = [&](int lo, u32x4_t (&w)[4]) {
#pragma unroll
    for (int c = 0; c < 4; ++c)
      if (8 * c < len) w[c] = *reinterpret_cast<const u32x4_t*>(wrow + lo + 8 * c);
  };
  fetch(first, w_now);
  for (int i = 0; i < leaves; ++i) {
    const int lo = first + i * len;
    if (i + 1 < leaves) fetch(lo + len, w_next);
    float acc[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[m] = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      if (8 * c < len) {
        u32x4_t a8[MR];  // eight k of every row of A: the same address in every lane
#pragma unroll
        for (int m = 0; m < MR; ++m) a8[m] = *reinterpret_cast<const u32x4_t*>(arow[m] + lo + 8 * c);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const uint32_t wb = w_now[c][e >> 1];
          const float b = __uint_as_float((e & 1) ? (wb & 0xffff0000u) : (wb << 16));
#pragma unroll
          for (int m = 0; m < MR; ++m) {
            const uint32_t ab = a8[m][e >> 1];
            const float a = __uint_as_float((e & 1) ? (ab & 0xffff0000u) : (ab << 16));
            acc[m] = __builtin_fmaf(a, b, acc[m]);
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < PR; ++r) cur[r] = pack_bf16x2(acc[2 * r], acc[2 * r + 1]);
    // Leaf i closes one node per trailing one bit of i; then it waits at the level of its lowest zero bit.
    int level = 0;
    for (int j = i; j & 1; j >>= 1, ++level) {
#pragma unroll
      for (int l = 0; l < kTreeSkinnyLevels; ++l) {
        if (l == level) {
#pragma unroll
          for (int r = 0; r < PR; ++r) cur[r] = bf16x2_add(slot[l][r], cur[r]);
        }
      }
    }
    if (i + 1 < leaves) {
#pragma unroll
      for (int l = 0; l < kTreeSkinnyLevels; ++l) {
        if (l == level) {
#pragma unroll
          for (int r = 0; r < PR; ++r) slot[l][r] = cur[r];
        }
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) w_now[c] = w_next[c];
    }
  }
  if constexpr (HALVES) {
    // left child in lanes 0..31, right child in lanes 32..63 of the same column
#pragma unroll
    for (int r = 0; r < PR; ++r) {
      const uint32_t other = (uint32_t)__shfl_xor((int)cur[r], 32, 64);
      cur[r] = lane < 32 ? bf16x2_add(cur[r], other) : bf16x2_add(other, cur[r]);
    }
  }
#pragma unroll
  for (int r = 0; r < PR; ++r) nodes[wave][r][lane] = cur[r];
  __syncthreads();
  if (wave != 0) return;
  // nodes 0..15 left to right at depth 4: pairs, then pairs of pairs, ... up to the root
#pragma unroll
  for (int r = 0; r < PR; ++r) {
    uint32_t v[kTreeSkinnyWaves];
#pragma unroll
    for (int w = 0; w < kTreeSkinnyWaves; ++w) v[w] = nodes[w][r][lane];
#pragma unroll
    for (int width = kTreeSkinnyWaves / 2; width >= 1; width /= 2)
#pragma unroll
      for (int w = 0; w < width; ++w) v[w] = bf16x2_add(v[2 * w], v[2 * w + 1]);
    if (col < N && lane < kCols) {
      if (2 * r < M) C[(int64_t)(2 * r) * ldc + col] = (bf16_bits)(v[0] & 0xffffu);
      if (2 * r + 1 < M) C[(int64_t)(2 * r + 1) * ldc + col] = (bf16_bits)(v[0] >> 16);
    }
  }
}

// The same split for more rows, on the matrix pipe: a workgroup of 8 waves takes 16 rows, wave w evaluates
// node w at depth 3 with one v_mfma_f32_16x16x1_4b_f32 per k, and wave 0 folds the 8 bf16 nodes in tree order.
// Many more workgroups than the tiled kernel has tiles: for row counts whose tiles do not fill the chip. Two
// workgroups fit a CU (LDS, registers), so one computes while the other starts or folds. The four 16 x 16
// blocks of the instruction are
//   KB = 1: four groups of 16 columns (64 columns per workgroup), the row operand of block 0 broadcast;
//   KB = 4: the four grandchildren (depth 5) of the wave's node for one group of 16 columns, every block
//           with its own k range; the lane then folds its four blocks in tree order. Four times the
//           workgroups and a quarter of the leaves per lane: for narrow N, where 64-column workgroups
//           would leave most CUs idle and a lane's chain of leaves (one memory round trip each) decides.
// CHUNKS = leaf length / 8.
// Operand path: a lane's operand is 16 bytes per 8 k of ITS column, so loads into registers would touch 64
// different lines per instruction and the address pipe, not memory or the matrix pipe, would set the pace. A
// wave therefore brings its leaf in through LDS: direct-to-LDS loads whose lanes walk the 16-byte granules
// (column, chunk) in order - 4 / CHUNKS columns' worth of contiguous bytes per line touched - into a region of
// LDS that belongs to the wave alone (two leaves: one landing while the other is read), then every lane reads
// its own column back with ds_read_b128. No barrier: the wave waits for its own loads. The rows of A go the
// same way for KB = 1 (16 rows of one k range: one load instruction per leaf); for KB = 4 the four blocks
// need four k ranges of A, which would not fit beside the weight, and those stay register loads.
// Every load is issued unconditionally (past the node's end it repeats the last leaf), so that the waits
// count loads along one straight path.
// Workgroup ids are dealt so that the row groups of one column group run on the same XCD at the same time and
// share that L2's copy of the weight.
constexpr int kTreeNodeSplit = 3;                     // depth of the nodes the waves take
constexpr int kTreeNodeWaves = 1 << kTreeNodeSplit;   // 8: two workgroups per CU, one starts while the other folds
constexpr int kTreeNodeLevels = 7;                    // tree levels below a node, KB = 1 (K <= 32768)

template <int KB, int CHUNKS>
struct TreeNodesLds {
  static constexpr int kABytes = KB == 1 ? 1024 : 0;  // a leaf of the 16 rows: one load instruction whatever CHUNKS
  static constexpr int kWBytes = 1024 * CHUNKS;       // a leaf of the wave's 64 (column, k range) pairs, behind the rows
  static constexpr int kLeafBytes = kABytes + kWBytes;
  static constexpr int kWaveBytes = 2 * kLeafBytes;
  static constexpr int kNodesBytes = kTreeNodeWaves * (KB == 4 ? 2 : 8) * 64 * 4;
  static constexpr int kStageBytes = kTreeNodeWaves * kWaveBytes;
  static constexpr int kBytes = kStageBytes > kNodesBytes ? kStageBytes : kNodesBytes;
};

// On this chip a vector-ALU instruction is not hidden behind the fp32 matrix instructions of the other waves of
// its SIMD: each one adds about three cycles to the 32 of a 16x16x1 step. The leaf loop is therefore written
// for few of them: two per step to widen the bf16 operands, addresses as a scalar base plus a lane offset that
// never changes, LDS reads at immediate offsets (the loop handles an even and an odd leaf per turn, so the
// staging region of each is known at compile time), and the tree bookkeeping once per pair of leaves.
template <int KB, int CHUNKS>
__global__ __launch_bounds__(64 * kTreeNodeWaves, 4) void det_gemm_tree_nodes_kernel(
    MatView A, MatView B, bf16_bits* __restrict__ C, int64_t ldc, int M, int N, int K, int depth, int row_groups) {
  using L = TreeNodesLds<KB, CHUNKS>;
  constexpr int kLevels = KB == 4 ? kTreeNodeLevels - 2 : kTreeNodeLevels;
  constexpr int kKeep = KB == 4 ? 2 : 8;  // packed registers a wave hands to the fold
  constexpr int kAAhead = 2;              // KB = 4: leaves of A in flight in registers
  constexpr int kLoadsPerLeaf = CHUNKS + (KB == 1 ? 1 : CHUNKS);
  extern __shared__ __attribute__((aligned(16))) char tree_lds[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int id = xcd_compact_id(blockIdx.x, gridDim.x);
  const int n0 = (id / row_groups) * (KB == 4 ? 16 : 64), m0 = (id % row_groups) * 16;
  constexpr int len = 8 * CHUNKS;  // leaf length
  const int node_depth = kTreeNodeSplit + (KB == 4 ? 2 : 0);
  const int leaves = 1 << (depth - node_depth);  // leaves under one block's node: a power of two, at least 2
  // The k range of block b of this wave starts at (KB * wave + b) * leaves * len; block_k = leaves * len.
  const int block_k = leaves * len;
  const int wave_k = (KB == 4 ? 4 * wave : wave) * block_k;  // uniform

  // Granule g = 64 j + lane of a leaf: pair g / CHUNKS (KB = 1: column; KB = 4: column % 16 and block), position
  // g % CHUNKS, which holds chunk position ^ swizzle(pair): the lanes of a ds_read_b128 then spread over the banks.
  // Addresses are a uniform base (the workgroup's first column or row, the wave's k range, the leaf) plus a lane
  // offset in bytes that fits 32 bits (the launcher checks the strides).
  static_assert(CHUNKS == 3 || CHUNKS == 4, "leaves of 24 or 32");
  auto swizzle = [](int pair) { return CHUNKS == 4 ? (pair >> 2) & 3 : 0; };  // 48-byte pairs spread by themselves
  const char* const w_base = reinterpret_cast<const char*>(B.ptr + (int64_t)n0 * B.row_stride + wave_k);
  const char* const a_base = reinterpret_cast<const char*>(A.ptr + (int64_t)m0 * A.row_stride + wave_k);
  uint32_t w_off[CHUNKS];
#pragma unroll
  for (int j = 0; j < CHUNKS; ++j) {
    const int g = 64 * j + lane, pair = g / CHUNKS, chunk = (g % CHUNKS) ^ swizzle(pair);
    const int col = KB == 4 ? (pair & 15) : pair;
    const int col_in = n0 + col < N ? col : N - 1 - n0;
    w_off[j] = 2u * (uint32_t)(col_in * (int)B.row_stride + (KB == 4 ? (pair >> 4) * block_k : 0) + 8 * chunk);
  }
  uint32_t a_off;
  if constexpr (KB == 1) {  // lanes past the 16 rows repeat the last granule; their 16 bytes land in the spare of the region
    const int g = lane < 16 * CHUNKS ? lane : 16 * CHUNKS - 1, row = g / CHUNKS;
    const int row_in = m0 + row < M ? row : M - 1 - m0;
    a_off = 2u * (uint32_t)(row_in * (int)A.row_stride + 8 * ((g % CHUNKS) ^ swizzle(row)));
  } else {
    const int row = lane & 15;
    const int row_in = m0 + row < M ? row : M - 1 - m0;
    a_off = 2u * (uint32_t)(row_in * (int)A.row_stride + (lane >> 4) * block_k);
  }
  char* const mine = tree_lds + wave * L::kWaveBytes;
  // Lane l reads chunk c of its pair l at read_at[c] (+ kABytes for the weight): rows and columns use the same
  // lane offsets, lanes 16 .. 63 read rows that do not exist (inside the region; the instruction broadcasts block 0).
  const char* read_at[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) read_at[c] = mine + lane * (16 * CHUNKS) + 16 * (c ^ swizzle(lane));

  u32x4_t wq[CHUNKS], aq[KB == 1 ? 1 : kAAhead + 1][CHUNKS];
  // leaf: which leaf of the node (past the end: the last one again); stage: 0 or 1
  auto issue = [&](int leaf, int stage_index, u32x4_t (&a)[CHUNKS]) __attribute__((always_inline)) {
    const int lo = (leaf < leaves ? leaf : leaves - 1) * (2 * len);  // uniform, bytes
    char* const stage = mine + stage_index * L::kLeafBytes;
    // the leaf's bases stay in scalar registers (the empty statements keep the compiler from folding the leaf
    // into the lane offsets, which would cost a 64-bit vector add per load)
    const char* w_leaf = w_base + lo;
    const char* a_leaf = a_base + lo;
    asm volatile("" : "+s"(w_leaf));
    asm volatile("" : "+s"(a_leaf));
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
      uint32_t off = w_off[j];
      asm volatile("" : "+v"(off));  // widened here, next to the scalar base, not once outside the loop
      __builtin_amdgcn_global_load_lds((global_ptr_t)(w_leaf + off), (lds_ptr_t)(stage + L::kABytes + 1024 * j), 16, 0, 0);
    }
    uint32_t off = a_off;
    asm volatile("" : "+v"(off));
    if constexpr (KB == 1) {
      __builtin_amdgcn_global_load_lds((global_ptr_t)(a_leaf + off), (lds_ptr_t)stage, 16, 0, 0);
    } else {
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c) a[c] = *reinterpret_cast<const u32x4_t*>(a_leaf + off + 16 * c);
    }
  };
  auto take = [&](int stage_index) __attribute__((always_inline)) {  // the landed leaf out of LDS into registers
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      wq[c] = *reinterpret_cast<const u32x4_t*>(read_at[c] + stage_index * L::kLeafBytes + L::kABytes);
      if constexpr (KB == 1) aq[0][c] = *reinterpret_cast<const u32x4_t*>(read_at[c] + stage_index * L::kLeafBytes);
    }
  };
  // Leaf i (stage i & 1, a compile-time constant at every call): start the load of leaf i + 2 into the region leaf i
  // came from, sum the leaf, round it to bf16, and bring leaf i + 1 into registers.
  auto leaf_sum = [&](int i, int stage_index, uint32_t (&node)[8]) __attribute__((always_inline)) {
    __builtin_amdgcn_s_waitcnt(kWaitLgkm0);  // leaf i is in registers: its region is free
    asm volatile("" ::: "memory");
    issue(i + 2, stage_index, aq[KB == 1 ? 0 : kAAhead]);
    f32x16_t acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t wb = wq[c][e >> 1], ab = aq[0][c][e >> 1];
        const float b = __uint_as_float((e & 1) ? (wb & 0xffff0000u) : (wb << 16));
        const float a = __uint_as_float((e & 1) ? (ab & 0xffff0000u) : (ab << 16));
        if constexpr (KB == 4) {
          acc = __builtin_amdgcn_mfma_f32_16x16x1f32(a, b, acc, 0, 0, 0);
        } else {
          acc = __builtin_amdgcn_mfma_f32_16x16x1f32(a, b, acc, 2, 0, 0);
        }
      }
    }
#pragma unroll
    for (int q = 0; q < 8; ++q) node[q] = pack_bf16x2(acc[2 * q], acc[2 * q + 1]);
    __builtin_amdgcn_s_waitcnt(wait_vmcnt(kLoadsPerLeaf));  // leaf i + 1 has landed (leaf i + 2 may be on its way)
    asm volatile("" ::: "memory");
    take(stage_index ^ 1);
    if constexpr (KB == 4) {
#pragma unroll
      for (int p = 0; p < kAAhead; ++p)
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) aq[p][c] = aq[p + 1][c];
    }
  };

  uint32_t slot[kLevels - 1][8];  // slot[l]: a finished left child l + 1 levels above the leaves
  uint32_t left[8], cur[8];
  issue(0, 0, aq[0]);
  issue(1, 1, aq[KB == 1 ? 0 : 1]);
  __builtin_amdgcn_s_waitcnt(wait_vmcnt(kLoadsPerLeaf));  // leaf 0 has landed
  asm volatile("" ::: "memory");
  take(0);
  for (int i = 0; i < leaves; i += 2) {
    leaf_sum(i, 0, left);
    leaf_sum(i + 1, 1, cur);
#pragma unroll
    for (int r = 0; r < 8; ++r) cur[r] = bf16x2_add(left[r], cur[r]);
    // Pair i / 2 closes one node per trailing one bit of i / 2; then it waits at the level of its lowest zero bit.
    int level = 0;
    for (int j = i >> 1; j & 1; j >>= 1, ++level) {
#pragma unroll
      for (int l = 0; l < kLevels - 1; ++l) {
        if (l == level) {
#pragma unroll
          for (int r = 0; r < 8; ++r) cur[r] = bf16x2_add(slot[l][r], cur[r]);
        }
      }
    }
    if (i + 2 < leaves) {
#pragma unroll
      for (int l = 0; l < kLevels - 1; ++l) {
        if (l == level) {
#pragma unroll
          for (int r = 0; r < 8; ++r) slot[l][r] = cur[r];
        }
      }
    }
  }
  // The fold's table takes the place of the staging regions: every wave's loads must have landed first.
  __builtin_amdgcn_s_waitcnt(kWaitAll0);
  __syncthreads();
  uint32_t(*nodes)[kKeep][64] = reinterpret_cast<uint32_t(*)[kKeep][64]>(tree_lds);
  // Accumulator r: block r / 4; row 4 (lane / 16) + r % 4, column lane % 16 of the block.
  // cur[q] packs accumulators 2 q, 2 q + 1 (two consecutive rows of one column), block q / 2.
  if constexpr (KB == 4) {
    // blocks 0..3 are the node's grandchildren left to right: (0 + 1) + (2 + 3)
#pragma unroll
    for (int h = 0; h < 2; ++h)
      nodes[wave][h][lane] = bf16x2_add(bf16x2_add(cur[h], cur[2 + h]), bf16x2_add(cur[4 + h], cur[6 + h]));
  } else {
#pragma unroll
    for (int r = 0; r < 8; ++r) nodes[wave][r][lane] = cur[r];
  }
  __syncthreads();
  if (wave != 0) return;
  const int out_col = n0 + (lane & 15);
  const int out_row = m0 + 4 * (lane >> 4);
#pragma unroll
  for (int q = 0; q < kKeep; ++q) {
    uint32_t v[kTreeNodeWaves];
#pragma unroll
    for (int w = 0; w < kTreeNodeWaves; ++w) v[w] = nodes[w][q][lane];
#pragma unroll
    for (int width = kTreeNodeWaves / 2; width >= 1; width /= 2)
#pragma unroll
      for (int w = 0; w < width; ++w) v[w] = bf16x2_add(v[2 * w], v[2 * w + 1]);
    const int c = out_col + (KB == 4 ? 0 : 16 * (q >> 1));
    const int r = out_row + 2 * (q & 1);
    if (c < N) {
      if (r < M) C[(int64_t)r * ldc + c] = (bf16_bits)(v[0] & 0xffffu);
      if (r + 1 < M) C[(int64_t)(r + 1) * ldc + c] = (bf16_bits)(v[0] >> 16);
    }
  }
}

template <int KB, int CHUNKS>
static hipError_t launch_nodes_leaf(const MatView& A, const MatView& B, bf16_bits* out, int64_t ldc, int M, int N, int K,
                                    int depth, hipStream_t stream) {
  using L = TreeNodesLds<KB, CHUNKS>;
  static PerDeviceOnce once;
  auto kernel = det_gemm_tree_nodes_kernel<KB, CHUNKS>;
  hipError_t err = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), L::kBytes, once);
  if (err != hipSuccess) return err;
  constexpr int kCols = KB == 4 ? 16 : 64;
  const int row_groups = (M + 15) / 16;
  const int64_t groups = (int64_t)((N + kCols - 1) / kCols) * row_groups;
  if (groups > 0x7fffffff) return hipErrorInvalidValue;
  hipLaunchKernelGGL(kernel, dim3((unsigned)groups), dim3(64 * kTreeNodeWaves), L::kBytes, stream, A, B, out, ldc, M, N,
                     K, depth, row_groups);
  return hipGetLastError();
}

template <int KB>
static hipError_t launch_nodes(const MatView& A, const MatView& B, bf16_bits* out, int64_t ldc, int M, int N, int K,
                               int depth, hipStream_t stream) {
  // equal leaves that are a multiple of 8 long are 24 or 32 long: a tree stops splitting at 32, so its leaves are
  // longer than 16
  return (K >> depth) == 24 ? launch_nodes_leaf<KB, 3>(A, B, out, ldc, M, N, K, depth, stream)
                            : launch_nodes_leaf<KB, 4>(A, B, out, ldc, M, N, K, depth, stream);
}

int det_gemm_tree_max_k() { return kTreeLeaf << 20; }

template <int MAXD>
static void launch_valu(const MatView& A, const MatView& B, bf16_bits* out, int64_t ldc, int M, int N, int K,
                        unsigned tiles, int tiles_m, hipStream_t stream) {
  hipLaunchKernelGGL(det_gemm_tree_kernel<MAXD>, dim3(tiles), dim3(kTreeThreads), 0, stream, A, B, out, ldc, M, N, K,
                     tiles_m);
}

template <int MAXD>
static void launch_wide(const MatView& A, const MatView& B, bf16_bits* out, int64_t ldc, int M, int N, int K,
                        unsigned tiles, int tiles_m, int fast, hipStream_t stream) {
  // fp32 staging except for 8 to 10 tree levels, where its extra live registers would spill
  hipLaunchKernelGGL((det_gemm_tree_wide_kernel<MAXD, MAXD != 10>), dim3(tiles), dim3(kTreeWideThreads), 0, stream, A, B,
                     out, ldc, M, N, K, tiles_m, fast);
}

// A[M, K] and B as rows of output columns (B.rows = N), any strides; C[m * ldc + n].
// config: RLK_TREE_CFG_AUTO, or one of the two leaf loops (same bits).
hipError_t det_gemm_tree_launch(const MatView& A, const MatView& B, void* C, int64_t ldc, int M, int N, int K,
                                int config, hipStream_t stream, bool leaf_space) {
  const int tiles_m = (M + kTreeBM - 1) / kTreeBM;
  const int tiles_n = (N + kTreeBN - 1) / kTreeBN;
  const int64_t tiles64 = (int64_t)tiles_m * tiles_n;
  if (tiles64 > 0x7fffffff) return hipErrorInvalidValue;
  const unsigned tiles = (unsigned)tiles64;
  bf16_bits* out = reinterpret_cast<bf16_bits*>(C);
  if (leaf_space) {
    // With a power-of-two number of whole leaves the leaf-space tree is the element-space tree: every kernel
    // below serves it. Otherwise the tiled matrix-pipe kernel walks the tree in units of leaves.
    const int leaves = (K + kTreeLeaf - 1) / kTreeLeaf;
    if (K % kTreeLeaf != 0 || (leaves & (leaves - 1)) != 0) {
      int levels = 0;
      while ((1 << levels) < leaves) ++levels;
      if (levels > 20) return hipErrorInvalidValue;
      auto chunked = [&](const MatView& v) {  // leaves start on multiples of 32; the last one ends at K
        return K % 8 == 0 && v.k_stride == 1 && v.row_stride % 8 == 0 && (reinterpret_cast<uintptr_t>(v.ptr) & 15) == 0;
      };
      auto rows8 = [&](const MatView& v, int rows) {
        return v.row_stride == 1 && rows % 8 == 0 && v.k_stride >= rows && v.k_stride % 8 == 0 &&
               (reinterpret_cast<uintptr_t>(v.ptr) & 15) == 0;
      };
      const bool a_chunked = chunked(A), b_chunked = chunked(B);
      const int fast = 32 | (a_chunked ? 1 : 0) | (b_chunked ? 2 : 0) | (!a_chunked && rows8(A, M) ? 8 : 0) |
                       (!b_chunked && rows8(B, N) ? 16 : 0);
      if (levels <= 7) launch_wide<7>(A, B, out, ldc, M, N, K, tiles, tiles_m, fast, stream);
      else if (levels <= 10) launch_wide<10>(A, B, out, ldc, M, N, K, tiles, tiles_m, fast, stream);
      else launch_wide<20>(A, B, out, ldc, M, N, K, tiles, tiles_m, fast, stream);
      return hipGetLastError();
    }
  }
  const int depth = tree_depth(K);
  if (depth > 20) return hipErrorInvalidValue;
  // Register slots for 7 levels (K <= 4096), 10 (K <= 32768) or 20: the fewer, the more waves per SIMD.
  if (config == RLK_TREE_CFG_VALU) {
    if (depth <= 7) launch_valu<7>(A, B, out, ldc, M, N, K, tiles, tiles_m, stream);
    else if (depth <= 10) launch_valu<10>(A, B, out, ldc, M, N, K, tiles, tiles_m, stream);
    else launch_valu<20>(A, B, out, ldc, M, N, K, tiles, tiles_m, stream);
    return hipGetLastError();
  }
  if (config != RLK_TREE_CFG_AUTO && config != RLK_TREE_CFG_MFMA_F32 && config != RLK_TREE_CFG_SKINNY &&
      config != RLK_TREE_CFG_NODES)
    return hipErrorInvalidValue;
  // 16-byte chunks: every leaf begins and ends on a multiple of 8 (all leaves are K >> depth long
  // when that divides), rows contiguous in K and 16-byte aligned. Uniform tree: 2^depth divides K.
  const bool leaves_whole = K % (8 << depth) == 0;
  auto chunked = [&](const MatView& v) {
    return leaves_whole && v.k_stride == 1 && v.row_stride % 8 == 0 && (reinterpret_cast<uintptr_t>(v.ptr) & 15) == 0;
  };
  const bool uniform = depth >= 1 && K % (1 << depth) == 0;
  // Row-contiguous (K-major) operand: 16-byte chunks of eight rows at one k.
  auto rows8 = [&](const MatView& v, int rows) {
    return v.row_stride == 1 && rows % 8 == 0 && v.k_stride >= rows && v.k_stride % 8 == 0 &&
           (reinterpret_cast<uintptr_t>(v.ptr) & 15) == 0;
  };
  const bool a_chunked = chunked(A), b_chunked = chunked(B);
  // Up to 16 rows: the kernel that gives each of the 16 depth-4 nodes to a wave of its own.
  const bool skinny_ok = M <= 16 && a_chunked && b_chunked && depth >= kTreeSkinnySplit &&
                         depth - kTreeSkinnySplit <= kTreeSkinnyLevels;
  if (config == RLK_TREE_CFG_SKINNY && !skinny_ok) return hipErrorInvalidValue;
  // (at least two leaves under a wave's node; lane offsets of up to 64 rows and the reduction length in 32 bits)
  const bool nodes_ok = a_chunked && b_chunked && depth > kTreeNodeSplit && depth - kTreeNodeSplit <= kTreeNodeLevels &&
                        ((K >> depth) == 24 || (K >> depth) == 32) && A.row_stride < (1 << 24) && B.row_stride < (1 << 24);
  if (config == RLK_TREE_CFG_NODES && !nodes_ok) return hipErrorInvalidValue;
  // The node-per-wave kernel splits a node over the four blocks of its instruction where 64-column workgroups
  // would not give every CU one; that needs two more tree levels above the leaves.
  const int64_t wide_groups = (int64_t)((N + 63) / 64) * ((M + 15) / 16);
  const bool split_blocks = nodes_ok && wide_groups < 256 && depth > kTreeNodeSplit + 2;
  // The node-per-wave kernel wherever it is eligible. Measured on the Qwen3-8B projections it is ahead of the tiled
  // kernel at every row count (gate_up: 58 against 279 us at 16 rows, 157 against 281 us at 64, 8.8 against 9.6 ms at
  // 4096; down 4.7 against 6.2 ms at 4096): its waves never meet at a barrier inside a node and its operands need no
  // conversion pass. Up to 8 rows it is ahead of the vector-ALU kernel below as well, with weights that come from HBM
  // (gate_up at one token 59 against 84 us, the lm_head 287 against 403 us, down 33 against 75 us).
  if (config == RLK_TREE_CFG_AUTO && nodes_ok) config = RLK_TREE_CFG_NODES;
  if (config == RLK_TREE_CFG_NODES) {
    return split_blocks ? launch_nodes<4>(A, B, out, ldc, M, N, K, depth, stream)
                        : launch_nodes<1>(A, B, out, ldc, M, N, K, depth, stream);
  }
  // Up to 16 rows of a tree the node kernel does not take (11 or 12 levels): the vector-ALU node kernel.
  if (skinny_ok && (config == RLK_TREE_CFG_SKINNY || config == RLK_TREE_CFG_AUTO)) {
    // Narrow N: 32 columns per workgroup and the wave halves on the two children of a node (down at one
    // token 78 -> 61 us, o_proj 24 -> 20 us; gate_up 66 -> 73 us, and 16 rows twice as slow: not there).
    const bool halves = depth > kTreeSkinnySplit && depth - kTreeSkinnySplit - 1 <= kTreeSkinnyLevels && M <= 8 &&
                        N <= kTreeHalvesMaxN;
    const dim3 grid((unsigned)(halves ? (N + 31) / 32 : (N + 63) / 64)), block(64 * kTreeSkinnyWaves);
    auto launch = [&](auto kernel) { hipLaunchKernelGGL(kernel, grid, block, 0, stream, A, B, out, ldc, M, N, K, depth); };
    if (M <= 4) {
      if (halves) launch(det_gemm_tree_skinny_kernel<4, true>); else launch(det_gemm_tree_skinny_kernel<4, false>);
    } else if (M <= 8) {
      if (halves) launch(det_gemm_tree_skinny_kernel<8, true>); else launch(det_gemm_tree_skinny_kernel<8, false>);
    } else {
      launch(det_gemm_tree_skinny_kernel<16, false>);
    }
    return hipGetLastError();
  }
  const int fast = (a_chunked ? 1 : 0) | (b_chunked ? 2 : 0) | (uniform ? 4 : 0) |
                   (!a_chunked && rows8(A, M) ? 8 : 0) | (!b_chunked && rows8(B, N) ? 16 : 0);
  if (depth <= 7) launch_wide<7>(A, B, out, ldc, M, N, K, tiles, tiles_m, fast, stream);
  else if (depth <= 10) launch_wide<10>(A, B, out, ldc, M, N, K, tiles, tiles_m, fast, stream);
  else launch_wide<20>(A, B, out, ldc, M, N, K, tiles, tiles_m, fast, stream);
  return hipGetLastError();
}

}  // namespace rlk
