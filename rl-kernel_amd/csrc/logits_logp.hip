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
//   a tile belongs to 16 lanes; lane l of them takes vectors g0 + l, g0 + l + 16, ... ascending
//             (g0 = first vector touching the tile) with state (m, s) = (-inf, 0):
//             n = max(m, the eight y);
//             if n > -inf: s = s * e(m - n) + ((e(y0 - n) + e(y1 - n)) + ...);  m = n
//   the 16 lane states merge in an xor butterfly (offsets 8, 4, 2, 1):
//             M = max(m_a, m_b);  S = s_a * e(m_a - M) + s_b * e(m_b - M)   (-inf sides skipped,
//             the lower lane's term first)
//   tile_max = M, tile_sum = S (0 when M is not finite)
//   lse = merge over tiles ascending (same formula as the fused forward's split merge)
//   e(x) = v_exp_f32(x * log2(e)) with an unfused fp32 multiply.
// (Four tiles share a wave, so one butterfly serves four tiles; a wave per tile spent as many
// instructions on its 64-lane butterfly as on the tile's logits.)
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

// The eight values of vector g of a row, widened to fp32. ALIGNED: every row is made of whole,
// 16-byte aligned vectors (decided once on the host), so a vector is one or two 16-byte loads from a
// uniform row base plus a 32-bit lane offset; otherwise element by element, columns past the row as 0.
template <int ELEM, bool ALIGNED>
struct RawVector;

template <bool ALIGNED>
struct RawVector<RLK_DTYPE_BF16, ALIGNED> {
  u32x4_t w;
  __device__ __forceinline__ void load(const uint16_t* row, int g, int cols) {
    if constexpr (ALIGNED) {
      w = *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const char*>(row) + (uint32_t)g * 16u);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = g * 8 + 2 * i;
        const uint32_t lo = c < cols ? row[c] : 0u, hi = c + 1 < cols ? row[c + 1] : 0u;
        w[i] = lo | (hi << 16);
      }
    }
  }
  __device__ __forceinline__ void unpack(float (&y)[8]) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      y[2 * i] = __uint_as_float(w[i] << 16);
      y[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

template <bool ALIGNED>
struct RawVector<RLK_DTYPE_FP16, ALIGNED> {
  _Float16 h[8];
  __device__ __forceinline__ void load(const _Float16* row, int g, int cols) {
    if constexpr (ALIGNED) {
      const u32x4_t w = *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const char*>(row) + (uint32_t)g * 16u);
      __builtin_memcpy(h, &w, 16);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) h[i] = g * 8 + i < cols ? row[g * 8 + i] : (_Float16)0.f;
    }
  }
  __device__ __forceinline__ void unpack(float (&y)[8]) const {
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = (float)h[i];
  }
};

template <bool ALIGNED>
struct RawVector<RLK_DTYPE_FP32, ALIGNED> {
  f32x4_t lo, hi;
  __device__ __forceinline__ void load(const float* row, int g, int cols) {
    if constexpr (ALIGNED) {
      const char* p = reinterpret_cast<const char*>(row) + (uint32_t)g * 32u;
      lo = reinterpret_cast<const f32x4_t*>(p)[0];
      hi = reinterpret_cast<const f32x4_t*>(p)[1];
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        lo[i] = g * 8 + i < cols ? row[g * 8 + i] : 0.f;
        hi[i] = g * 8 + 4 + i < cols ? row[g * 8 + 4 + i] : 0.f;
      }
    }
  }
  __device__ __forceinline__ void unpack(float (&y)[8]) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      y[i] = lo[i];
      y[4 + i] = hi[i];
    }
  }
};

// max(a, b, c) in one instruction. (fmaxf on values that come out of integer shifts costs an extra
// canonicalising instruction per operand; v_max3_f32 needs none. For the non-NaN values of this contract it
// returns what nested fmaxf returns.)
__device__ __forceinline__ float max3_f32(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// One step of a lane's online chain: the eight scaled logits of a vector folded into (m, s).
// (Measured without effect on the kernel's time once its instruction count was halved: a fused
// exp2(y * log2e - n * log2e), and skipping the rescale of s while no lane's maximum moves.)
__device__ __forceinline__ void fold_logit_vector(const float (&y)[8], float& m, float& s) {
  const float n = max3_f32(max3_f32(max3_f32(max3_f32(y[0], y[1], y[2]), y[3], y[4]), y[5], y[6]), y[7], m);
  float sum = pinned_exp(y[0] - n);
#pragma unroll
  for (int i = 1; i < 8; ++i) sum = sum + pinned_exp(y[i] - n);
  const float scaled = s * pinned_exp(m - n);
  s = (n > kNegInf) ? (scaled + sum) : s;
  m = n;
}

// Value of lane (l ^ OFFSET) for OFFSET 1, 2 (DPP quad permutes) and 4, 8 (ds_swizzle xor mode).
template <int OFFSET>
__device__ __forceinline__ float xor_lane(float v) {
  const int bits = __float_as_int(v);
  int out;
  if constexpr (OFFSET == 1) {
    out = __builtin_amdgcn_update_dpp(bits, bits, 0xB1, 0xf, 0xf, false);  // quad_perm [1, 0, 3, 2]
  } else if constexpr (OFFSET == 2) {
    out = __builtin_amdgcn_update_dpp(bits, bits, 0x4E, 0xf, 0xf, false);  // quad_perm [2, 3, 0, 1]
  } else {
    out = __builtin_amdgcn_ds_swizzle(bits, (OFFSET << 10) | 0x1f);  // and 0x1f, or 0, xor OFFSET
  }
  return __int_as_float(out);
}

template <int OFFSET>
__device__ __forceinline__ void merge_lane_states(int lane, float& m, float& s) {
  const float om = xor_lane<OFFSET>(m);
  const float os = xor_lane<OFFSET>(s);
  const float n = fmaxf(m, om);
  const float mine = (m > kNegInf) ? s * pinned_exp(m - n) : 0.f;
  const float theirs = (om > kNegInf) ? os * pinned_exp(om - n) : 0.f;
  // The lower lane's term goes first on both sides, so both lanes add in the same order.
  s = (lane & OFFSET) ? (theirs + mine) : (mine + theirs);
  m = n;
}

template <bool V>
struct BoolConstant {
  static constexpr bool value = V;
};

constexpr int kTileLanes = 16;                    // lanes that share a tile
constexpr int kTilesPerWave = kWave / kTileLanes;  // 4

template <int ELEM, bool HAS_TEMP, bool ALIGNED>
__global__ __launch_bounds__(256) void logits_tile_stats_kernel(TileStatsArgs a) {
  using L = LogitElem<ELEM>;
  using E = typename L::type;
  constexpr int VEC = 8, kBatch = 4;
  constexpr int kStep = kTileLanes * kBatch;  // vectors of a tile per batch
  const int row = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l16 = lane & (kTileLanes - 1);
  const int grp = lane / kTileLanes;
  const E* row_ptr = reinterpret_cast<const E*>(a.logits) + (int64_t)row * a.row_stride;
  const int cols = (int)a.V;
  const float inv_t = HAS_TEMP ? 1.0f / a.temperature[row] : 1.0f;
  const int tile_size = cols / a.num_tiles;
  const int64_t real_span = a.real_vocab - a.vocab_start;
  const int real_cols = real_span <= 0 ? 0 : (real_span < cols ? (int)real_span : cols);
  const int64_t target_span = a.target ? a.target[row] - a.vocab_start : -1;
  const int target_local = (target_span >= 0 && target_span < real_cols) ? (int)target_span : -1;

  const int tile_first = blockIdx.y * a.tiles_per_group;
  const int tile_last = tile_first + a.tiles_per_group < a.num_tiles ? tile_first + a.tiles_per_group : a.num_tiles;
  // A wave takes four consecutive tiles at a time, one per group of 16 lanes.
  for (int t0 = tile_first + wave * kTilesPerWave; t0 < tile_last; t0 += 4 * kTilesPerWave) {
    const int tile = t0 + grp;
    const bool have = tile < tile_last;
    const int lo_col = tile * tile_size;
    const int col_end = lo_col + tile_size;
    int hi_col = col_end < real_cols ? col_end : real_cols;
    if (!have || hi_col < lo_col) hi_col = lo_col;  // no columns: every vector below is masked out
    const int g0 = lo_col / VEC;
    const int g1 = hi_col > lo_col ? (hi_col + VEC - 1) / VEC : g0;
    const int g_last = g1 > g0 ? g1 - 1 : (have ? g0 : 0);  // a valid vector to clamp loads to
    // Batches in which all four vectors of every lane are whole vectors of the lane's tile (only the very
    // first vector of a tile may start inside the vector) run without clamps and with one mask.
    const int g_whole = (hi_col % VEC) ? g1 - 1 : g1;
    const int my_clean = g_whole > g0 ? (g_whole - g0) / kStep : 0;
    const int my_slots = (g1 - g0 + kTileLanes - 1) / kTileLanes;  // vector slots of 16 lanes this tile needs
    int clean = __builtin_amdgcn_readlane(my_clean, 0), slots = __builtin_amdgcn_readlane(my_slots, 0);
#pragma unroll
    for (int other = kTileLanes; other < kWave; other += kTileLanes) {  // uniform over the wave's four tiles
      const int c = __builtin_amdgcn_readlane(my_clean, other), t = __builtin_amdgcn_readlane(my_slots, other);
      clean = c < clean ? c : clean;
      slots = t > slots ? t : slots;
    }

    float m = kNegInf, s = 0.f;
    int g = g0 + l16;  // this lane's next vector
    // Clean batches, the loads rotating through the four raw vectors: a vector's registers are free once it is
    // unpacked, and the same vector of the next batch is fetched into them before the fold, so a lane always
    // has three or four loads in flight instead of none while it folds the end of a batch.
    RawVector<ELEM, ALIGNED> raw[kBatch];
    if (clean > 0) {
#pragma unroll
      for (int u = 0; u < kBatch; ++u) raw[u].load(row_ptr, g + u * kTileLanes, cols);
    }
    auto clean_batch = [&](auto more, bool first) __attribute__((always_inline)) {
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        float y[VEC];
        raw[u].unpack(y);
        if constexpr (decltype(more)::value) raw[u].load(row_ptr, g + kStep + u * kTileLanes, cols);
        if (u == 0 && first) {  // the tile may start inside its first vector (lane 0 of the 16)
          const int lo = lo_col - g * VEC;
#pragma unroll
          for (int i = 0; i < VEC; ++i) y[i] = (i >= lo) ? y[i] : kNegInf;
        }
        if (HAS_TEMP) {
#pragma unroll
          for (int i = 0; i < VEC; ++i) y[i] = y[i] * inv_t;  // -inf stays -inf (temperature > 0)
        }
        fold_logit_vector(y, m, s);
      }
    };
    for (int b = 0; b + 1 < clean; ++b, g += kStep) clean_batch(BoolConstant<true>{}, b == 0);
    if (clean > 0) {
      clean_batch(BoolConstant<false>{}, clean == 1);
      g += kStep;
    }
    for (int b = clean; b * kBatch < slots; ++b, g += kStep) {  // the rest: clamped loads, both edges masked
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int gu = g + u * kTileLanes;
        raw[u].load(row_ptr, gu < g1 ? gu : g_last, cols);
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        if (b * kBatch + u >= slots) break;  // uniform: no tile of this wave reaches this slot
        const int gu = g + u * kTileLanes;
        float y[VEC];
        raw[u].unpack(y);
        const int lo = lo_col - gu * VEC;
        const int hi = gu < g1 ? hi_col - gu * VEC : lo;  // columns [lo, hi) of the vector count
#pragma unroll
        for (int i = 0; i < VEC; ++i) y[i] = (i >= lo && i < hi) ? y[i] : kNegInf;
        if (HAS_TEMP) {
#pragma unroll
          for (int i = 0; i < VEC; ++i) y[i] = y[i] * inv_t;
        }
        fold_logit_vector(y, m, s);  // a vector of -inf leaves (m, s) as they are
      }
    }
    merge_lane_states<8>(lane, m, s);
    merge_lane_states<4>(lane, m, s);
    merge_lane_states<2>(lane, m, s);
    merge_lane_states<1>(lane, m, s);
    if (l16 == 0 && have) {
      const bool finite = m > kNegInf && m < -kNegInf;
      const int64_t at = (int64_t)row * a.out_row_stride + (int64_t)tile * a.out_tile_stride;
      a.out_max[at] = m;
      a.out_sum[at] = finite ? s : 0.f;
      if (a.out_target) {
        float zt = 0.f;
        if (target_local >= lo_col && target_local < hi_col) {
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
  // (4 waves) per row once T alone does that. A group is a multiple of 16 tiles (four per wave).
  int groups = 1;
  while ((int64_t)T * groups < 4096 && groups * 16 < num_tiles) groups *= 2;
  int per = (num_tiles + groups - 1) / groups;
  per = (per + 15) / 16 * 16;
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
  // every row made of whole, 16-byte aligned vectors: vector loads (the same arithmetic either way)
  const int64_t elem_bytes = dtype == RLK_DTYPE_FP32 ? 4 : 2;
  const bool aligned = (reinterpret_cast<uintptr_t>(logits) & 15) == 0 && (row_stride * elem_bytes) % 16 == 0 && V % 8 == 0;
#define RLK_LAUNCH_TILE_STATS(ELEM)                                                                          \
  if (aligned && has_temp) {                                                                                 \
    hipLaunchKernelGGL((logits_tile_stats_kernel<ELEM, true, true>), grid, dim3(256), 0, stream, a);         \
  } else if (aligned) {                                                                                      \
    hipLaunchKernelGGL((logits_tile_stats_kernel<ELEM, false, true>), grid, dim3(256), 0, stream, a);        \
  } else if (has_temp) {                                                                                     \
    hipLaunchKernelGGL((logits_tile_stats_kernel<ELEM, true, false>), grid, dim3(256), 0, stream, a);        \
  } else {                                                                                                   \
    hipLaunchKernelGGL((logits_tile_stats_kernel<ELEM, false, false>), grid, dim3(256), 0, stream, a);       \
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
