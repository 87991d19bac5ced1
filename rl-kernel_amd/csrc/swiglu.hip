// SwiGLU for gfx950: the elementwise activation between the two FFN GEMMs, and the
// packed gate/up projection with the activation fused into its epilogue.
//
// Stands in for swiglu_forward / swiglu_backward / swiglu_packed_forward /
// swiglu_packed_backward (reference csrc/cuda/activation/activation.cu:20-31, 62-135;
// csrc/bindings/ops.cpp:400-419) and for the fused decode projection
// rl_engine/backends/rocm/gemm/swiglu_gemm.py:13-86.
//
// Arithmetic (token-local, so batch invariant):
//   g, u  = the bf16-ROUNDED gate and up projections, widened to fp32
//   s     = rcp(1 + e(-g))             v_rcp_f32 (within 1 ulp of the quotient);
//                                      e(x) = v_exp_f32(x * log2(e))
//   y     = bf16((g * s) * u)
//   d_up  = bf16(dy * (g * s));   d_gate = bf16((dy * u) * (s * (1 + g * (1 - s))))
// The elementwise kernels also serve fp16 and fp32 tensors (the reference dispatches on the
// element type, activation.cu:240-284): same fp32 arithmetic, one rounding to the element type.
// The fused kernel rounds its two fp32 accumulators to bf16 before the activation, so it
// returns exactly what the GEMM followed by the elementwise kernel returns.
#include "linear_logp_common.h"
#include "rlk_host.h"

namespace rlk {

// ---------------------------------------------------------------------------
// Elementwise kernels: eight features per thread, 16-byte accesses.
// gate[m * ld_g + c], up[m * ld_u + c]: a packed [T, 2 I] buffer is the case
// up = gate + I, ld_g = ld_u = 2 I.
// ---------------------------------------------------------------------------

struct SwigluArgs {
  const char* gate;
  const char* up;
  const char* dy;  // backward only
  char* y;         // forward: y; backward: d_gate
  char* y2;        // backward: d_up
  int64_t ld_g, ld_u, ld_dy, ld_y, ld_y2;  // in elements
  int rows, cols;
};

// ELEM: rlk_dtype of the tensors. Arithmetic is fp32 for every type; results are rounded to
// the element type once (round to nearest even), fp32 results are stored as they are.
template <int ELEM>
struct ActElem;
template <>
struct ActElem<RLK_DTYPE_BF16> {
  typedef bf16_bits type;
  static __device__ __forceinline__ float widen(bf16_bits v) { return bf16_to_f32(v); }
  static __device__ __forceinline__ bf16_bits narrow(float v) { return to_bf16_bits(v); }
};
template <>
struct ActElem<RLK_DTYPE_FP16> {
  typedef _Float16 type;
  static __device__ __forceinline__ float widen(_Float16 v) { return (float)v; }
  static __device__ __forceinline__ _Float16 narrow(float v) { return (_Float16)v; }
};
template <>
struct ActElem<RLK_DTYPE_FP32> {
  typedef float type;
  static __device__ __forceinline__ float widen(float v) { return v; }
  static __device__ __forceinline__ float narrow(float v) { return v; }
};

template <int ELEM>
__device__ __forceinline__ void load8(const char* base, int64_t index, bool vec, int valid, float (&out)[8]) {
  typedef typename ActElem<ELEM>::type T;
  const T* p = reinterpret_cast<const T*>(base) + index;
  if (vec && valid >= 8) {
    T raw[8];
    constexpr int kVecs = (int)sizeof(T) * 8 / 16;  // 16-byte accesses
#pragma unroll
    for (int i = 0; i < kVecs; ++i)
      reinterpret_cast<u32x4_t*>(raw)[i] = reinterpret_cast<const u32x4_t*>(p)[i];
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = ActElem<ELEM>::widen(raw[i]);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = i < valid ? ActElem<ELEM>::widen(p[i]) : 0.f;
  }
}

template <int ELEM>
__device__ __forceinline__ void store8(char* base, int64_t index, bool vec, int valid, const float (&v)[8]) {
  typedef typename ActElem<ELEM>::type T;
  T* p = reinterpret_cast<T*>(base) + index;
  T raw[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) raw[i] = ActElem<ELEM>::narrow(v[i]);
  if (vec && valid >= 8) {
    constexpr int kVecs = (int)sizeof(T) * 8 / 16;
#pragma unroll
    for (int i = 0; i < kVecs; ++i) reinterpret_cast<u32x4_t*>(p)[i] = reinterpret_cast<const u32x4_t*>(raw)[i];
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (i < valid) p[i] = raw[i];
  }
}

template <bool BACKWARD, int ELEM>
__global__ __launch_bounds__(256) void swiglu_kernel(SwigluArgs a, bool vec) {
  const int groups = (a.cols + 7) / 8;
  const int64_t total = (int64_t)a.rows * groups;
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
    const int row = (int)(idx / groups);
    const int col = (int)(idx - (int64_t)row * groups) * 8;
    const int valid = a.cols - col;
    float g[8], u[8];
    load8<ELEM>(a.gate, (int64_t)row * a.ld_g + col, vec, valid, g);
    load8<ELEM>(a.up, (int64_t)row * a.ld_u + col, vec, valid, u);
    if (!BACKWARD) {
      float y[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] = swiglu_f32(g[i], u[i]);
      store8<ELEM>(a.y, (int64_t)row * a.ld_y + col, vec, valid, y);
    } else {
      float dy[8], dg[8], du[8];
      load8<ELEM>(a.dy, (int64_t)row * a.ld_dy + col, vec, valid, dy);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float s = sigmoid_f32(g[i]);
        du[i] = dy[i] * (g[i] * s);
        dg[i] = (dy[i] * u[i]) * (s * (1.0f + g[i] * (1.0f - s)));
      }
      store8<ELEM>(a.y, (int64_t)row * a.ld_y + col, vec, valid, dg);
      store8<ELEM>(a.y2, (int64_t)row * a.ld_y2 + col, vec, valid, du);
    }
  }
}

// Rows start on 16-byte boundaries and hold whole 16-byte vectors.
static bool rows_aligned16(const void* p, int64_t ld, int elem_bytes) {
  return (reinterpret_cast<uintptr_t>(p) & 15) == 0 && (ld * elem_bytes) % 16 == 0;
}

template <int ELEM>
static void launch_swiglu_typed(const SwigluArgs& a, bool vec, bool backward, unsigned blocks, hipStream_t stream) {
  if (backward) {
    hipLaunchKernelGGL((swiglu_kernel<true, ELEM>), dim3(blocks), dim3(256), 0, stream, a, vec);
  } else {
    hipLaunchKernelGGL((swiglu_kernel<false, ELEM>), dim3(blocks), dim3(256), 0, stream, a, vec);
  }
}

hipError_t swiglu_launch(const void* gate, int64_t ld_g, const void* up, int64_t ld_u, const void* dy, int64_t ld_dy,
                         void* out, int64_t ld_out, void* out2, int64_t ld_out2, int rows, int cols, bool backward,
                         int dtype, hipStream_t stream) {
  if (rows == 0 || cols == 0) return hipSuccess;
  SwigluArgs a;
  a.gate = reinterpret_cast<const char*>(gate);
  a.up = reinterpret_cast<const char*>(up);
  a.dy = reinterpret_cast<const char*>(dy);
  a.y = reinterpret_cast<char*>(out);
  a.y2 = reinterpret_cast<char*>(out2);
  a.ld_g = ld_g;
  a.ld_u = ld_u;
  a.ld_dy = ld_dy;
  a.ld_y = ld_out;
  a.ld_y2 = ld_out2;
  a.rows = rows;
  a.cols = cols;
  const int eb = dtype == RLK_DTYPE_FP32 ? 4 : 2;
  bool vec = rows_aligned16(gate, ld_g, eb) && rows_aligned16(up, ld_u, eb) && rows_aligned16(out, ld_out, eb);
  if (backward) vec = vec && rows_aligned16(dy, ld_dy, eb) && rows_aligned16(out2, ld_out2, eb);
  const int64_t total = (int64_t)rows * ((cols + 7) / 8);
  int64_t blocks = (total + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  switch (dtype) {
    case RLK_DTYPE_BF16:
      launch_swiglu_typed<RLK_DTYPE_BF16>(a, vec, backward, (unsigned)blocks, stream);
      break;
    case RLK_DTYPE_FP16:
      launch_swiglu_typed<RLK_DTYPE_FP16>(a, vec, backward, (unsigned)blocks, stream);
      break;
    case RLK_DTYPE_FP32:
      launch_swiglu_typed<RLK_DTYPE_FP32>(a, vec, backward, (unsigned)blocks, stream);
      break;
    default:
      return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Packed gate/up projection with the activation in the epilogue.
// W is the packed weight [2 * I, K]; a workgroup owns S::BN / 2 features of both halves.
// ---------------------------------------------------------------------------

template <class S>
__global__ __launch_bounds__(S::kThreads) void det_gemm_swiglu_kernel(MatView W, MatView X, bf16_bits* __restrict__ Y,
                                                                       int64_t ldy, int M, int I, int K, int tiles_m,
                                                                       int tiles_n, int group_m) {
  static_assert(S::TN == 4 && pingpong_supported<S>(), "gated tiles use the 4 x 2 ping-pong layout");
  extern __shared__ __attribute__((aligned(16))) char lds[];
  constexpr int kTileFeatures = S::BN / 2;

  const int total = tiles_m * tiles_n;
  const int id = xcd_compact_id(blockIdx.x, total);
  const int per_group = group_m * tiles_n;
  const int group = id / per_group;
  const int first_m = group * group_m;
  const int width = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
  const int within = id - group * per_group;
  const int tile_m = first_m + within % width;
  const int tile_n = within / width;
  const int f0 = tile_n * kTileFeatures;
  const int m0 = tile_m * S::BM;

  f32x4_t acc[S::TN][S::TM];
  tile_mainloop_pingpong<S, false, false, GatedRowMap<S>>(W, X, f0, m0, K, lds, acc);

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wave_n = wave % S::WN;
  const int wave_m = wave / S::WN;
  const int f_run = f0 + wave_n * 32 + (lane >> 4) * 8;  // first of this lane's 8 consecutive features
  const int m_lane = m0 + wave_m * 16 * S::TM + (lane & 15);
#pragma unroll
  for (int jm = 0; jm < S::TM; ++jm) {
    const int m = m_lane + jm * 16;
    if (m >= M) continue;
    float y[8];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        y[h * 4 + q] = swiglu_f32(round_through_bf16(acc[h][jm][q]), round_through_bf16(acc[h + 2][jm][q]));
    const int64_t at = (int64_t)m * ldy + f_run;
    store8<RLK_DTYPE_BF16>(reinterpret_cast<char*>(Y), at, (reinterpret_cast<uintptr_t>(Y + at) & 15) == 0, I - f_run, y);
  }
}

using GatedShape256 = TileShape<256, 256, 4, 2>;
using GatedShape128 = TileShape<256, 128, 4, 2>;
using GatedShape64 = TileShape<256, 64, 4, 2>;

template <class S>
static hipError_t launch_gated(const MatView& W, const MatView& X, void* Y, int64_t ldy, int M, int I, int K,
                               hipStream_t stream) {
  auto kernel = det_gemm_swiglu_kernel<S>;
  static PerDeviceOnce once;
  hipError_t err = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), S::kLdsBytes, once);
  if (err != hipSuccess) return err;
  const int tiles_m = (M + S::BM - 1) / S::BM;
  const int tiles_n = (I + S::BN / 2 - 1) / (S::BN / 2);
  const int group_m = tiles_m < 8 ? tiles_m : 8;
  hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n), dim3(S::kThreads), S::kLdsBytes, stream, W, X,
                     reinterpret_cast<bf16_bits*>(Y), ldy, M, I, K, tiles_m, tiles_n, group_m);
  return hipGetLastError();
}

// Up to 16 tokens the streaming kernel serves the packed projection (the same panels of 16 weight
// rows, eight gate and eight up), from 129 tokens on the gated tile kernels; between them the
// projection and the activation run as two kernels (the weight read bounds the time there and the
// GEMM kernels for few tokens spread it over more CUs than a gated 128-feature tile).
static bool streams_gated(int M, int K) { return M <= 16 && K >= 1024; }

bool det_gemm_swiglu_fused_supported(const MatView& W, const MatView& X, int M, int K) {
  auto native = [](const MatView& v) {
    return v.k_stride == 1 && (v.row_stride % kChunkElems) == 0 && pitch_fits_lane_offsets(v.row_stride) &&
           (reinterpret_cast<uintptr_t>(v.ptr) & 15) == 0;
  };
  return native(W) && native(X) && (K % kTileK) == 0 && (M > 128 || streams_gated(M, K));
}

// Y[M, I] = swiglu(X @ W[0:I]^T, X @ W[I:2I]^T). `workspace` ([M, 2 I] bf16) is used only when
// the fused kernel does not apply (other layouts, ragged K, up to 128 tokens: there the weight read bounds the time and the
// GEMM kernels for few tokens spread it over more CUs than a gated 128-feature tile), where the
// projection and the activation run as two kernels with the same result.
hipError_t det_gemm_swiglu_launch(const MatView& W, const MatView& X, void* Y, int64_t ldy, void* workspace, int M,
                                  int I, int K, hipStream_t stream) {
  if (det_gemm_swiglu_fused_supported(W, X, M, K)) {
    if (streams_gated(M, K)) return det_gemm_stream_gated_launch(W, X, Y, ldy, M, I, K, stream);
    const int64_t t256 = (int64_t)((M + 255) / 256) * ((I + 127) / 128);
    const int64_t t128 = (int64_t)((M + 127) / 128) * ((I + 127) / 128);
    // Rounds of workgroups x tokens per tile / relative throughput, as in pick_det_gemm_config:
    // a partly filled last round costs little more than its share, so the large tile wins early.
    const int cus = device_cu_count();
    auto cost = [cus](int64_t tiles, double tokens, double quality) {
      return rounds_of_workgroups(tiles, cus) * tokens / quality;
    };
    if (M > 128 && cost(t256, 256.0, 1.0) <= cost(t128, 128.0, 0.65))
      return launch_gated<GatedShape256>(W, X, Y, ldy, M, I, K, stream);
    if (M > 64 && t128 >= 128) return launch_gated<GatedShape128>(W, X, Y, ldy, M, I, K, stream);
    return launch_gated<GatedShape64>(W, X, Y, ldy, M, I, K, stream);
  }
  if (workspace == nullptr) return hipErrorInvalidValue;
  hipError_t err = det_gemm_launch(W, X, workspace, 2 * (int64_t)I, M, 2 * I, K, false, RLK_GEMM_CFG_AUTO, stream);
  if (err != hipSuccess) return err;
  const bf16_bits* gu = reinterpret_cast<const bf16_bits*>(workspace);
  return swiglu_launch(gu, 2 * (int64_t)I, gu + I, 2 * (int64_t)I, nullptr, 0, Y, ldy, nullptr, 0, M, I, false,
                       RLK_DTYPE_BF16, stream);
}

}  // namespace rlk
