/*
 * CPU oracle for the deterministic dense path - TEST INFRASTRUCTURE ONLY.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load
 * this file's library; the product (librlk_gfx950.so and the rl_engine package)
 * never does. It restates, in scalar C, the arithmetic of the reference
 * (ryankert01/RL-Kernel) GEMM contracts so the HIP kernels can be checked
 * against them. Every matrix is bf16 as raw uint16 bit patterns; A is [M,K]
 * row major, Bt is the right-hand side stored [N,K] row major.
 *
 * Build: gcc -O2 -fPIC -shared -ffp-contract=off -o librlk_oracle.so rlk_oracle.c -lm
 * (-ffp-contract=off so a*b+c is never fused: products of two bf16 values are
 * exact in fp32 either way, but the k-tree adds must round exactly once each.)
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bf16_to_f32(uint16_t b) {
  uint32_t u = ((uint32_t)b) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* fp32 -> bf16, round to nearest even; NaN -> quiet NaN keeping the sign. */
static uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

uint16_t oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }
float oracle_bf16_to_f32(uint16_t b) { return bf16_to_f32(b); }

/*
 * Round-once GEMM with strictly sequential fp32 accumulation:
 *   C[i,j] = bf16( ((a_i0*b_0j + a_i1*b_1j) + a_i2*b_2j) + ... ).
 * Follows the reference's native twin of the round-once contract,
 * csrc/musa/det_gemm.mu:25-48 (one thread per C element, float acc = 0, k
 * ascending, one cast to bf16), whose own test demands equality with
 * (a.float() @ w.float().t()).to(bf16) at [4,16]x[9,16]
 * (tests/test_musa_det_gemm.py:133-140).
 */
void oracle_gemm_seq_f32(const uint16_t* a, const uint16_t* bt, uint16_t* c, int M, int N, int K) {
  for (int i = 0; i < M; ++i)
    for (int j = 0; j < N; ++j) {
      float acc = 0.0f;
      for (int k = 0; k < K; ++k) {
        const float p = bf16_to_f32(a[(size_t)i * K + k]) * bf16_to_f32(bt[(size_t)j * K + k]);
        acc = acc + p;
      }
      c[(size_t)i * N + j] = f32_to_bf16(acc);
    }
}

/*
 * The sequential chain on fp32 operands with an fp32 result: acc = fmaf(a_ik, b_kj, acc), k ascending
 * from +0, nothing rounded below fp32. Follows the same kernel with float inputs and a float output
 * (csrc/musa/det_gemm.mu:25-48 instantiated for float, its det_gemm_fwd_fp32) and the role of the
 * reference's fp32-output strict GEMM, rl_engine/backends/shared/triton/gemm/det_gemm.py:680-749. The
 * step is written as one fused multiply-add (for bf16-valued operands the product is exact, so the fused
 * step equals multiply-then-add; for general fp32 operands this is the stated choice: the reference's sources leave
 * fusion to their compilers and hold no fp32-operand fixture, so against the reference that case is PARITY UNPINNED).
 */
void oracle_gemm_seq_fma_f32in(const float* a, const float* bt, float* c, int M, int N, int K) {
  for (int i = 0; i < M; ++i)
    for (int j = 0; j < N; ++j) {
      float acc = 0.0f;
      for (int k = 0; k < K; ++k) acc = fmaf(a[(size_t)i * K + k], bt[(size_t)j * K + k], acc);
      c[(size_t)i * N + j] = acc;
    }
}

/* The same sum accumulated in fp64 (every product is exact; the fp64 sum of
 * K <= 2^20 such products is exact to far below one fp32 ulp). Output is the
 * unrounded double, for tests that bound the distance to the true value. */
void oracle_gemm_f64(const uint16_t* a, const uint16_t* bt, double* c, int M, int N, int K) {
  for (int i = 0; i < M; ++i)
    for (int j = 0; j < N; ++j) {
      double acc = 0.0;
      for (int k = 0; k < K; ++k)
        acc += (double)bf16_to_f32(a[(size_t)i * K + k]) * (double)bf16_to_f32(bt[(size_t)j * K + k]);
      c[(size_t)i * N + j] = acc;
    }
}

/*
 * Legacy k-tree contract: leaves of at most 32 K values summed sequentially in
 * fp32 and rounded to bf16; inner nodes are bf16 adds (fp32 add of the two
 * children, rounded to bf16); the split point is the midpoint in ELEMENT space.
 * Follows tests/ops/gemm/test_det_gemm.py:156-168 (_k_tree_gemm) and
 * csrc/cuda/gemm/det_gemm_kernel.cu:74-85 (k_tree_naive).
 * A leaf term is one fused multiply-add, as in the reference's GPU kernels ("scalar-FMA
 * leaves", rl_engine/backends/rocm/gemm/det_gemm.py:35-36; nvcc contracts acc += a*b).
 * The product of two bf16 values is exact in fp32 unless it underflows below 2^-126,
 * so fmaf and multiply-then-add differ only there.
 */
static uint16_t k_tree_element(const uint16_t* arow, const uint16_t* brow, int lo, int hi) {
  if (hi - lo <= 32) {
    float acc = 0.0f;
    for (int k = lo; k < hi; ++k) acc = fmaf(bf16_to_f32(arow[k]), bf16_to_f32(brow[k]), acc);
    return f32_to_bf16(acc);
  }
  const int mid = lo + (hi - lo) / 2;
  const float l = bf16_to_f32(k_tree_element(arow, brow, lo, mid));
  const float r = bf16_to_f32(k_tree_element(arow, brow, mid, hi));
  return f32_to_bf16(l + r);
}

/*
 * Leaf-space variant: leaves are the fixed 32-wide K tiles [32t, 32t+32) and the
 * midpoint split runs over leaf indices. Follows DetGemmTreeReferenceOp,
 * rl_engine/reference/gemm/det_gemm.py:29-60. Equal to the element-space tree
 * when K/32 is a power of two, different otherwise (e.g. K = 12288).
 */
static uint16_t k_tree_leaf(const uint16_t* arow, const uint16_t* brow, int K, int leaf_lo, int leaf_hi) {
  if (leaf_hi - leaf_lo <= 1) {
    const int lo = leaf_lo * 32;
    const int hi = (lo + 32 < K) ? lo + 32 : K;
    float acc = 0.0f;
    for (int k = lo; k < hi; ++k) acc = fmaf(bf16_to_f32(arow[k]), bf16_to_f32(brow[k]), acc);
    return f32_to_bf16(acc);
  }
  const int mid = leaf_lo + (leaf_hi - leaf_lo) / 2;
  const float l = bf16_to_f32(k_tree_leaf(arow, brow, K, leaf_lo, mid));
  const float r = bf16_to_f32(k_tree_leaf(arow, brow, K, mid, leaf_hi));
  return f32_to_bf16(l + r);
}

void oracle_gemm_ktree(const uint16_t* a, const uint16_t* bt, uint16_t* c, int M, int N, int K, int leaf_space) {
  const int leaves = (K + 31) / 32;
  for (int i = 0; i < M; ++i)
    for (int j = 0; j < N; ++j) {
      const uint16_t* arow = a + (size_t)i * K;
      const uint16_t* brow = bt + (size_t)j * K;
      c[(size_t)i * N + j] = (K == 0) ? 0
                             : leaf_space ? k_tree_leaf(arow, brow, K, 0, leaves)
                                          : k_tree_element(arow, brow, 0, K);
    }
}
