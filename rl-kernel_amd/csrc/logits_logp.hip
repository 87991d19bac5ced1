// Log-probabilities from materialised logits for gfx950: the stage the sampler path uses
// when the LM-head logits already exist and must not be recomputed.
//
// Stands in for hip_deterministic_logp_tile_stats / hip_deterministic_logp_backward
// (reference csrc/rocm/logprob/hip_deterministic_logp_kernel.hip:389-467, 472-540,
// 550-640; csrc/bindings/ops.cpp:122-135), for _merge_tile_partials
// (rl_engine/reference/logprob/vocab_parallel_logp.py:355-363) and for the ROCm branch
// of LinearLogpWrapper.from_local_logits
// (rl_engine/integrations/common/linear_logp.py:750-815, 817-923).
//
// HBM-bound: every logit is read once (2 or 4 bytes), nothing [T, V]-sized is written
// by the forward; the temperature division happens in registers instead of through an
// fp32 copy of the logits.
//
// Reduction contract (per row; a function of the row's values and the tile geometry
// only, never of the token count or of where the row sits in the batch):
//   y_c     = float(z_c) * (1 / temperature)      (plain float(z_c) without a temperature;
//             the same scaling as the fused linear-LogP)
//   tile t  = columns [t * V / tiles, (t + 1) * V / tiles) cut at the real vocabulary
//   vector g = columns [8 g, 8 g + 8) of the row;
//             columns outside the tile count as -inf
//   lane l of the tile's wave takes vectors g0 + l, g0 + l + 64, ... ascending
//             (g0 = first vector touching the tile) with state (m, s) = (-inf, 0):
//             t = max of the vector;  n = max(m, t);
//             if n > -inf: s = s * e(m - n) + ((e(y0 - n) + e(y1 - n)) + ...);  m = n
//   the 64 lane states merge in an xor butterfly (offsets 32, 16, 8, 4, 2, 1):
//             M = max(m_a, m_b);  S = s_a * e(m_a - M) + s_b * e(m_b - M)   (-inf sides skipped)
//   tile_max = M, tile_sum = S (0 when M is not finite)
//   lse = merge over tiles ascending (same formula as the fused forward's split merge)
//   e(x) = v_exp_f32(x * log2(e)) with an unfused fp32 multiply.
#include "linear_logp_common.h"
#include "rlk_host.h"

namespace rlk {

template <int ELEM>
struct LogitElem;

template <>
struct LogitElem<RLK_DTYPE_BF16> {
  using type = uint16_t;
  static constexpr int kVec = 8;
  static __device__ __forceinline__ float to_float(uint16_t v) { return __uint_as_float((uint32_t)v << 16); }
  static __device__ __forceinline__ uint16_t from_float(float f) {
    return (uint16_t)(pack_bf16x2(f, 0.f) & 0xffffu);
  }
};
template <>
struct LogitElem<RLK_DTYPE_FP16> {
  using type = _Float16;
  static constexpr int kVec = 8;
  static __device__ __forceinline__ float to_float(_Float16 v) { return (float)v; }
  static __device__ __forceinline__ _Float16 from_float(float f) { return (_Float16)f; }
};
template <>
struct LogitElem<RLK_DTYPE_FP32> {
  using type = float;
  static constexpr int kVec = 8;
  static __device__ __forceinline__ float to_float(float v) { return v; }
  static __device__ __forceinline__ float from_float(float f) { return f; }
};

// Columns [g * VEC, g * VEC + VEC) of a row as floats; `aligned` says the row base is 16-byte
// aligned, `cols` bounds the row (a vector that would run past it is read element by element).
template <int ELEM>
__device__ __forceinline__ void load_logit_vector(const typename LogitElem<ELEM>::type* row, int col, int cols,
                                                  bool aligned, float (&out)[LogitElem<ELEM>::kVec]) {
  using L = LogitElem<ELEM>;
  using E = typename L::type;
  constexpr int kBytes = L::kVec * (int)sizeof(E);
  if (aligned && col + L::kVec <= cols) {
    E vals[L::kVec];
    const u32x4_t* src = reinterpret_cast<const u32x4_t*>(row + col);
    u32x4_t raw[kBytes / 16];
#pragma unroll
    for (int i = 0; i < kBytes / 16; ++i) raw[i] = src[i];
    __builtin_memcpy(vals, raw, kBytes);
#pragma unroll
    for (int i = 0; i < L::kVec; ++i) out[i] = L::to_float(vals[i]);
  } else {
#pragma unroll
    for (int i = 0; i < L::kVec; ++i) out[i] = (col + i < cols) ? L::to_float(row[col + i]) : 0.f;
  }
}

struct TileStatsArgs {
  const void* logits;
  int64_t row_stride;  // elements
  const int64_t* target;     // [T] global ids, or null (no target plane)
  const float* temperature;  // [T] or null
  float* out_max;            // element (row, tile) at out_max[row * out_row_stride + tile * out_tile_stride]
  float* out_sum;
  float* out_target;         // or null
  int64_t out_row_stride, out_tile_stride;
  int T;
  int64_t V, vocab_start, real_vocab;
  int num_tiles, tiles_per_group;
};

// The (m, s) state of one lane over its vectors of one tile. FAST: every vector of the row is
// a whole, 16-byte aligned vector (decided per row, so the branch is uniform).
template <int ELEM, bool HAS_TEMP, bool FAST>
__device__ __forceinline__ void tile_lane_state(const typename LogitElem<ELEM>::type* row_ptr, int cols, int lo_col,
                                                int hi_col, float inv_t, int lane, float& m, float& s) {
  constexpr int VEC = LogitElem<ELEM>::kVec;
  constexpr int kBatch = 4;
  const int g0 = lo_col / VEC;
  const int g1 = (hi_col + VEC - 1) / VEC;
  // Four vectors of a lane are loaded before any is folded, so a wave keeps 4 KiB (8 KiB for
  // fp32) in flight; the folds still run in ascending vector order. A lane past the last
  // vector re-reads the last one with every column masked, which leaves (m, s) untouched.
  for (int base = g0; base < g1; base += 64 * kBatch) {
    float y[kBatch][VEC];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      if (base + 64 * u >= g1) break;  // uniform
      const int g = base + 64 * u + lane;
      const int gc = g < g1 ? g : g1 - 1;
      load_logit_vector<ELEM>(row_ptr, gc * VEC, cols, FAST, y[u]);
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      if (base + 64 * u >= g1) break;  // uniform
      const int g = base + 64 * u + lane;
      const int lo = lo_col - g * VEC;
      const int hi = g < g1 ? hi_col - g * VEC : lo;  // columns [lo, hi) of the vector count
      if (lo > 0 || hi < VEC) {                        // only vectors that straddle a tile edge
#pragma unroll
        for (int i = 0; i < VEC; ++i) y[u][i] = (i >= lo && i < hi) ? y[u][i] : kNegInf;
      }
      float vmax = kNegInf;
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const float v = HAS_TEMP ? y[u][i] * inv_t : y[u][i];  // -inf stays -inf (temperature > 0)
        y[u][i] = v;
        vmax = fmaxf(vmax, v);
      }
      const float n = fmaxf(m, vmax);
      float sum = pinned_exp(y[u][0] - n);
#pragma unroll
      for (int i = 1; i < VEC; ++i) sum = sum + pinned_exp(y[u][i] - n);
      const float scaled = s * pinned_exp(m - n);
      s = (n > kNegInf) ? (scaled + sum) : s;
      m = n;
    }
  }
}

template <int ELEM, bool HAS_TEMP>
__global__ __launch_bounds__(256) void logits_tile_stats_kernel(TileStatsArgs a) {
  using L = LogitElem<ELEM>;
  using E = typename L::type;
  constexpr int VEC = L::kVec;
  const int row = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const E* row_ptr = reinterpret_cast<const E*>(a.logits) + (int64_t)row * a.row_stride;
  const int cols = (int)a.V;
  const bool fast = (reinterpret_cast<uintptr_t>(row_ptr) & 15) == 0 && (cols % VEC) == 0;
  const float inv_t = HAS_TEMP ? 1.0f / a.temperature[row] : 1.0f;
  const int tile_size = cols / a.num_tiles;
  const int64_t real_span = a.real_vocab - a.vocab_start;
  const int real_cols = real_span <= 0 ? 0 : (real_span < cols ? (int)real_span : cols);
  const int64_t target_span = a.target ? a.target[row] - a.vocab_start : -1;
  const int target_local = (target_span >= 0 && target_span < real_cols) ? (int)target_span : -1;

  const int tile_first = blockIdx.y * a.tiles_per_group;
  const int tile_last = tile_first + a.tiles_per_group < a.num_tiles ? tile_first + a.tiles_per_group : a.num_tiles;
  for (int tile = tile_first + wave; tile < tile_last; tile += 4) {
    const int col_begin = tile * tile_size;
    const int col_end = col_begin + tile_size;
    const int real_end = col_end < real_cols ? col_end : real_cols;
    float m = kNegInf, s = 0.f;
    if (real_end > col_begin) {
      if (fast) {
        tile_lane_state<ELEM, HAS_TEMP, true>(row_ptr, cols, col_begin, real_end, inv_t, lane, m, s);
      } else {
        tile_lane_state<ELEM, HAS_TEMP, false>(row_ptr, cols, col_begin, real_end, inv_t, lane, m, s);
      }
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
      const float om = __shfl_xor(m, offset, 64);
      const float os = __shfl_xor(s, offset, 64);
      const float n = fmaxf(m, om);
      const float mine = (m > kNegInf) ? s * pinned_exp(m - n) : 0.f;
      const float theirs = (om > kNegInf) ? os * pinned_exp(om - n) : 0.f;
      // The lower lane's term goes first on both sides, so both lanes add in the same order.
      s = (lane & offset) ? (theirs + mine) : (mine + theirs);
      m = n;
    }
    if (lane == 0) {
      const bool finite = m > kNegInf && m < -kNegInf;
      const int64_t at = (int64_t)row * a.out_row_stride + (int64_t)tile * a.out_tile_stride;
      a.out_max[at] = m;
      a.out_sum[at] = finite ? s : 0.f;
      if (a.out_target) {
        float zt = 0.f;
        if (target_local >= col_begin && target_local < real_end) {
          zt = L::to_float(row_ptr[target_local]);
          if (HAS_TEMP) zt = zt * inv_t;
        }
        a.out_target[at] = zt;
      }
    }
  }
}

// grad = coef_logp * (onehot - p) + coef_lse * p with p = e(y - lse) (0 when lse is not
// finite), 0 on padded columns, multiplied by 1 / temperature once more when one is given.
// Elementwise; written in the dtype of the logits.
struct LogitsBackwardArgs {
  const void* logits;
  int64_t row_stride;
  const float* lse;
  const float* coef_logp;
  const float* coef_lse;  // or null
  const int64_t* target_local;  // [T] local column or -1
  const float* temperature;     // or null
  void* grad;
  int64_t grad_row_stride;
  int T;
  int64_t V, vocab_start, real_vocab;
};

template <int ELEM>
__global__ __launch_bounds__(256) void logits_backward_kernel(LogitsBackwardArgs a) {
  using L = LogitElem<ELEM>;
  using E = typename L::type;
  constexpr int VEC = L::kVec;
  const int row = blockIdx.x;
  const E* row_in = reinterpret_cast<const E*>(a.logits) + (int64_t)row * a.row_stride;
  E* row_out = reinterpret_cast<E*>(a.grad) + (int64_t)row * a.grad_row_stride;
  const bool aligned_in = (reinterpret_cast<uintptr_t>(row_in) & 15) == 0;
  const bool aligned_out = (reinterpret_cast<uintptr_t>(row_out) & 15) == 0;
  const float row_lse = a.lse[row];
  const bool finite_row = row_lse > kNegInf && row_lse < -kNegInf;
  const float lse_safe = finite_row ? row_lse : 0.f;
  const float g_logp = a.coef_logp[row];
  const float g_lse = a.coef_lse ? a.coef_lse[row] : 0.f;
  const bool has_temp = a.temperature != nullptr;
  const float inv_t = has_temp ? 1.0f / a.temperature[row] : 1.0f;
  const int64_t hit = a.target_local[row];
  const int64_t real_cols = a.real_vocab - a.vocab_start > 0 ? a.real_vocab - a.vocab_start : 0;
  const int64_t real_end = a.V < real_cols ? a.V : real_cols;
  const int64_t vectors = (a.V + VEC - 1) / VEC;
  for (int64_t g = (int64_t)blockIdx.y * 256 + threadIdx.x; g < vectors; g += (int64_t)gridDim.y * 256) {
    const int64_t col = g * VEC;
    float z[VEC];
    load_logit_vector<ELEM>(row_in, (int)col, (int)a.V, aligned_in, z);
    E out[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      const int64_t c = col + i;
      float value = 0.f;
      if (c < real_end) {
        const float y = has_temp ? z[i] * inv_t : z[i];
        const float p = finite_row ? pinned_exp(y - lse_safe) : 0.f;
        const float onehot = (c == hit) ? 1.0f : 0.0f;
        value = g_logp * (onehot - p);
        if (a.coef_lse) value = value + g_lse * p;
        if (has_temp) value = value * inv_t;
      }
      out[i] = L::from_float(value);
    }
    if (aligned_out && col + VEC <= a.V) {
      constexpr int kBytes = VEC * (int)sizeof(E);
      u32x4_t raw[kBytes / 16];
      __builtin_memcpy(raw, out, kBytes);
#pragma unroll
      for (int i = 0; i < kBytes / 16; ++i) reinterpret_cast<u32x4_t*>(row_out + col)[i] = raw[i];
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        if (col + i < a.V) row_out[col + i] = out[i];
    }
  }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------

static int tiles_per_group_for(int T, int num_tiles) {
  // Enough workgroups to fill 256 CUs several times over when T is small; one workgroup
  // (4 waves) per row once T alone does that. A group is a multiple of 4 tiles (one per wave).
  int groups = 1;
  while ((int64_t)T * groups < 4096 && groups * 4 < num_tiles) groups *= 2;
  int per = (num_tiles + groups - 1) / groups;
  per = (per + 3) / 4 * 4;
  return per;
}

hipError_t logits_tile_stats_launch(const void* logits, int dtype, int64_t row_stride, const int64_t* target,
                                    const float* temperature, int T, int64_t V, int64_t vocab_start,
                                    int64_t real_vocab, int num_tiles, float* out_max, float* out_sum,
                                    float* out_target, int64_t out_row_stride, int64_t out_tile_stride,
                                    hipStream_t stream) {
  TileStatsArgs a;
  a.logits = logits;
  a.row_stride = row_stride;
  a.target = target;
  a.temperature = temperature;
  a.out_max = out_max;
  a.out_sum = out_sum;
  a.out_target = out_target;
  a.out_row_stride = out_row_stride;
  a.out_tile_stride = out_tile_stride;
  a.T = T;
  a.V = V;
  a.vocab_start = vocab_start;
  a.real_vocab = real_vocab;
  a.num_tiles = num_tiles;
  a.tiles_per_group = tiles_per_group_for(T, num_tiles);
  const int groups = (num_tiles + a.tiles_per_group - 1) / a.tiles_per_group;
  const dim3 grid((unsigned)T, (unsigned)groups);
  const bool has_temp = temperature != nullptr;
#define RLK_LAUNCH_TILE_STATS(ELEM)                                                                          \
  if (has_temp) {                                                                                            \
    hipLaunchKernelGGL((logits_tile_stats_kernel<ELEM, true>), grid, dim3(256), 0, stream, a);               \
  } else {                                                                                                   \
    hipLaunchKernelGGL((logits_tile_stats_kernel<ELEM, false>), grid, dim3(256), 0, stream, a);              \
  }
  switch (dtype) {
    case RLK_DTYPE_BF16:
      RLK_LAUNCH_TILE_STATS(RLK_DTYPE_BF16)
      break;
    case RLK_DTYPE_FP16:
      RLK_LAUNCH_TILE_STATS(RLK_DTYPE_FP16)
      break;
    case RLK_DTYPE_FP32:
      RLK_LAUNCH_TILE_STATS(RLK_DTYPE_FP32)
      break;
    default:
      return hipErrorInvalidValue;
  }
#undef RLK_LAUNCH_TILE_STATS
  return hipGetLastError();
}

hipError_t logits_backward_launch(const void* logits, int dtype, int64_t row_stride, const float* lse,
                                  const float* coef_logp, const float* coef_lse, const int64_t* target_local,
                                  const float* temperature, void* grad, int64_t grad_row_stride, int T, int64_t V,
                                  int64_t vocab_start, int64_t real_vocab, hipStream_t stream) {
  LogitsBackwardArgs a;
  a.logits = logits;
  a.row_stride = row_stride;
  a.lse = lse;
  a.coef_logp = coef_logp;
  a.coef_lse = coef_lse;
  a.target_local = target_local;
  a.temperature = temperature;
  a.grad = grad;
  a.grad_row_stride = grad_row_stride;
  a.T = T;
  a.V = V;
  a.vocab_start = vocab_start;
  a.real_vocab = real_vocab;
  const int vec = 8;
  const int64_t vectors = (V + vec - 1) / vec;
  int64_t chunks = (vectors + 255) / 256;
  // a few vectors per thread; the result is elementwise, so the geometry is free
  chunks = (chunks + 3) / 4;
  if (chunks < 1) chunks = 1;
  if (chunks > 65535) chunks = 65535;
  const dim3 grid((unsigned)T, (unsigned)chunks);
  switch (dtype) {
    case RLK_DTYPE_BF16:
      hipLaunchKernelGGL(logits_backward_kernel<RLK_DTYPE_BF16>, grid, dim3(256), 0, stream, a);
      break;
    case RLK_DTYPE_FP16:
      hipLaunchKernelGGL(logits_backward_kernel<RLK_DTYPE_FP16>, grid, dim3(256), 0, stream, a);
      break;
    case RLK_DTYPE_FP32:
      hipLaunchKernelGGL(logits_backward_kernel<RLK_DTYPE_FP32>, grid, dim3(256), 0, stream, a);
      break;
    default:
      return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace rlk
