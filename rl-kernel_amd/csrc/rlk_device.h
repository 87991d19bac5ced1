// Device-side building blocks shared by the gfx950 kernels of this library.
//
// Everything here is written for CDNA4 (gfx950) only: 64-wide wavefronts, the
// v_mfma_f32_16x16x32_bf16 matrix instruction and v_cvt_pk_bf16_f32.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rlk {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;
typedef uint16_t bf16_bits;

constexpr int kWave = 64;
// K extent of one MFMA step and of one LDS tile (the pinned arithmetic order:
// ascending 32-wide MFMA steps over the whole K range into one fp32 accumulator).
constexpr int kMfmaK = 32;
constexpr int kTileK = 64;
// One 16-byte chunk carries 8 bf16 values; an LDS tile row holds 8 chunks.
constexpr int kChunkElems = 8;
constexpr int kRowChunks = kTileK / kChunkElems;
constexpr int kRowBytes = kTileK * 2;

// The one matrix instruction every det_gemm / linear-LogP kernel uses.
//   P operand (MFMA "A"): lane l holds row (l & 15), k slots 8*(l >> 4) .. +7
//   Q operand (MFMA "B"): lane l holds col (l & 15), k slots 8*(l >> 4) .. +7
//   accumulator:          lane l holds rows 4*(l >> 4) .. +3 of col (l & 15)
// An output element's value depends only on its own P row, Q column and the
// accumulator chain, never on what the other 15 rows / columns hold.
__device__ __forceinline__ f32x4_t mfma_16x16x32(const u32x4_t p, const u32x4_t q, const f32x4_t acc) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, p),
                                                 __builtin_bit_cast(bf16x8_t, q), acc, 0, 0, 0);
}

// fp32 -> bf16, round to nearest even (v_cvt_pk_bf16_f32), two values packed low/high.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  bf16x2_t r;
  r.x = (__bf16)lo;
  r.y = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, r);
}

__device__ __forceinline__ bf16_bits to_bf16_bits(float v) {
  return (bf16_bits)(pack_bf16x2(v, 0.0f) & 0xffffu);
}

__device__ __forceinline__ float bf16_bits_to_float(bf16_bits b) {
  return __uint_as_float(((uint32_t)b) << 16);
}

// XOR swizzle of the 16-byte chunk position inside a 128-byte LDS tile row.
// Eight consecutive rows at the same logical chunk land on eight different
// chunk positions, so the ds_read_b128 of an MFMA fragment is conflict free.
__device__ __forceinline__ int lds_chunk_offset(int row, int chunk) {
  return row * kRowBytes + ((chunk ^ (row & 7)) << 4);
}

// Workgroup id -> tile id such that the workgroups one XCD runs together cover
// a compact range of tiles. The hardware deals consecutive workgroup ids to the
// eight XCDs round robin; each XCD has its own L2.
__device__ __forceinline__ int xcd_compact_id(int wg, int total) {
  constexpr int kXcds = 8;
  const int per = total / kXcds;
  const int rem = total % kXcds;
  const int xcd = wg % kXcds;
  const int slot = wg / kXcds;
  // XCDs [0, rem) own per+1 ids, the rest own per ids.
  const int base = xcd * per + (xcd < rem ? xcd : rem);
  return base + slot;
}

}  // namespace rlk
