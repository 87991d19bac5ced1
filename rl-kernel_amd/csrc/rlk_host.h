// Host-side declarations shared by the translation units of librlk_gfx950.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/rlk.h"
#include "det_gemm_tile.h"

namespace rlk {

constexpr int kMaxDevices = 64;

int pick_det_gemm_config(int M, int N, int K);

// W[N,K] is the operand whose rows are output features, X[M,K] the one whose
// rows are tokens; C[m*ldc + n].
hipError_t det_gemm_launch(const MatView& W, const MatView& X, void* C, int64_t ldc, int M, int N, int K,
                           bool out_f32, int config, hipStream_t stream);

hipError_t fill_zero_launch(void* dst, int64_t rows, int64_t cols, int64_t ld, int elem_bytes,
                            hipStream_t stream);

void set_last_error(const char* fmt, ...);

}  // namespace rlk
