// Load-path probe for MI355X (gfx950): what the memory system delivers to the CUs, measured with kernels that
// only load. A diagnostic, not part of librlk_gfx950.so: it prices the load side of the tile kernels
// (det_gemm_tile.h) so that their measured times can be compared with what the hardware allows.
//
//   1. ceilings: bytes per second out of the L2, the memory-side cache and HBM with every CU loading
//   2. rate of one workgroup against the bytes it keeps in flight (few workgroups: nothing else is busy)
//   3. the load side of a small-tile GEMM without its arithmetic: npanels weight panels, each read at the same
//      pace by the workgroups of its token tiles (all on one XCD), plus the token rows, which stay in the L2
//   4. L2-resident matrix rows read 128 bytes at a time, by the distance between the rows
//   5. the load side of the 256 x 256 tile GEMM at its headline shape
//   6. the other side: the matrix pipe alone, the same MFMA sequence out of registers, at the power cap
//   7. that sequence with the kernel's LDS reads, L2 loads and barriers added, and the shader clock each variant sees
//   8. a K-major weight streamed as column slabs by one workgroup per slab (decode against a prepared weight)
//
// Loads are the direct-to-LDS DMA form the tile kernels use (or ordinary vector loads, "vgpr"). Build:
//   hipcc --offload-arch=gfx950 -O3 -o load_path_probe load_path_probe.hip     (rl-kernel_amd/build.py does it)
// Run without arguments for every section, or with one section number.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* global_ptr_t;

#define CK(x)                                                                 \
  do {                                                                        \
    hipError_t e_ = (x);                                                      \
    if (e_ != hipSuccess) {                                                   \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);   \
      exit(1);                                                                \
    }                                                                         \
  } while (0)

static void require(bool ok, const char* what) {
  if (!ok) {
    printf("refused: %s\n", what);
    exit(1);
  }
}

constexpr int kWaitAllVm = 0x0f70;  // s_waitcnt vmcnt(0); low four bits = loads allowed to stay in flight

// ---- 1 and 2: streams ------------------------------------------------------------------------------------
// Workgroup w reads stream w % nstreams, `steps` steps of NW * U KiB, wrapping inside the stream; each wave
// issues U loads of 1 KiB per step and waits until the previous step's loads have landed (2U in flight).
template <int MODE, int NW, int U>
__global__ __launch_bounds__(NW * 64) void stream_kernel(const char* base, size_t stream_bytes, int nstreams,
                                                          int steps, unsigned* sink) {
  extern __shared__ __align__(1024) char lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wg = blockIdx.x;
  const size_t step_bytes = (size_t)NW * U * 1024;
  const size_t steps_in_stream = stream_bytes / step_bytes;
  const char* stream = base + (size_t)(wg % nstreams) * stream_bytes;
  size_t pos = ((size_t)(wg / nstreams) * 7) % steps_in_stream;  // readers of one stream start apart
  unsigned acc = 0;
  if constexpr (MODE == 0) {
    char* mine = lds + wave * (2 * U * 1024);
    for (int s = 0; s < steps; ++s) {
      const char* src = stream + pos * step_bytes + (size_t)wave * U * 1024 + lane * 16;
      char* dst = mine + (s & 1) * (U * 1024);
#pragma unroll
      for (int u = 0; u < U; ++u)
        __builtin_amdgcn_global_load_lds((global_ptr_t)(src + u * 1024), (lds_ptr_t)(dst + u * 1024), 16, 0, 0);
      __builtin_amdgcn_s_waitcnt(kWaitAllVm | U);
      if (++pos == steps_in_stream) pos = 0;
    }
    __builtin_amdgcn_s_waitcnt(kWaitAllVm);
    __syncthreads();
    acc = *(unsigned*)(lds + threadIdx.x * 4);
  } else {
    uint4 v[U];
    for (int s = 0; s < steps; ++s) {
      const char* src = stream + pos * step_bytes + (size_t)wave * U * 1024 + lane * 16;
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = *(const uint4*)(src + u * 1024);
#pragma unroll
      for (int u = 0; u < U; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
      if (++pos == steps_in_stream) pos = 0;
    }
  }
  if (acc == 0x12345678u) sink[0] = acc;  // never true for the 0x01 fill; keeps the loads alive
}

static size_t g_buffer_bytes = 0;

template <int MODE, int NW, int U>
static void run_streams(const char* name, const char* buf, size_t stream_bytes, int nstreams, int nwg, int steps,
                        unsigned* sink) {
  static_assert(U <= 8 && NW * 2 * U * 1024 <= 128 * 1024, "LDS ring of a workgroup");
  require((size_t)nstreams * stream_bytes <= g_buffer_bytes, "streams exceed the buffer");
  require(stream_bytes % ((size_t)NW * U * 1024) == 0 && stream_bytes >= (size_t)NW * U * 1024, "stream size");
  const size_t lds = MODE == 0 ? (size_t)NW * 2 * U * 1024 : 0;
  CK(hipFuncSetAttribute((const void*)stream_kernel<MODE, NW, U>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  for (int i = 0; i < 2; ++i) stream_kernel<MODE, NW, U><<<nwg, NW * 64, lds>>>(buf, stream_bytes, nstreams, steps, sink);
  CK(hipEventRecord(a));
  const int reps = 5;
  for (int i = 0; i < reps; ++i) stream_kernel<MODE, NW, U><<<nwg, NW * 64, lds>>>(buf, stream_bytes, nstreams, steps, sink);
  CK(hipEventRecord(b));
  CK(hipEventSynchronize(b));
  float ms;
  CK(hipEventElapsedTime(&ms, a, b));
  ms /= reps;
  const double bytes = (double)nwg * steps * NW * U * 1024;
  printf("%-40s %s %3d KB in flight per workgroup, %4d workgroups, %4d streams x %7.2f MB: %7.1f us  %6.2f TB/s  %6.1f GB/s per workgroup\n",
         name, MODE == 0 ? "dma " : "vgpr", NW * 2 * U, nwg, nstreams, stream_bytes / 1e6, ms * 1e3,
         bytes / ms * 1e-9, bytes / ms * 1e-6 / nwg);
  fflush(stdout);
}

// ---- 3: the load side of a small-tile GEMM ---------------------------------------------------------------
// Workgroup w loads weight panel w % npanels and token tile w / npanels, 32 KiB of each per step, and waits for
// the previous step (128 KiB in flight per workgroup, more than the tile kernels keep). Consecutive workgroup
// ids go round the eight XCDs, so with npanels a multiple of 8 the readers of a panel share an L2.
// PREFETCH (four token tiles only): each reader also touches its quarter of the panel's step LEAD steps ahead,
// one dword per 128-byte line, into a spare 256 bytes of LDS - a load with no register destination.
template <int PREFETCH, int LEAD>
__global__ __launch_bounds__(512) void panel_kernel(const char* weights, const char* tokens, size_t panel_bytes,
                                                    int npanels, int steps, unsigned* sink) {
  extern __shared__ __align__(1024) char lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int panel = blockIdx.x % npanels, ttile = blockIdx.x / npanels;
  const char* w = weights + (size_t)panel * panel_bytes;
  const char* x = tokens + (size_t)ttile * panel_bytes;
  char* mine = lds + wave * 16384;
  for (int s = 0; s < steps; ++s) {
    const char* ws = w + (size_t)s * 32768 + wave * 4096 + lane * 16;
    const char* xs = x + (size_t)s * 32768 + wave * 4096 + lane * 16;
    char* dst = mine + (s & 1) * 8192;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      __builtin_amdgcn_global_load_lds((global_ptr_t)(ws + u * 1024), (lds_ptr_t)(dst + u * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((global_ptr_t)(xs + u * 1024), (lds_ptr_t)(dst + 4096 + u * 1024), 16, 0, 0);
    }
    if (PREFETCH && wave == 0) {
      if (s + LEAD < steps) {
        const char* p = w + (size_t)(s + LEAD) * 32768 + ttile * 8192 + lane * 128;
        __builtin_amdgcn_global_load_lds((global_ptr_t)p, (lds_ptr_t)(lds + 131072), 4, 0, 0);
      }
      __builtin_amdgcn_s_waitcnt(kWaitAllVm | 9);
    } else {
      __builtin_amdgcn_s_waitcnt(kWaitAllVm | 8);
    }
  }
  __builtin_amdgcn_s_waitcnt(kWaitAllVm);
  __syncthreads();
  const unsigned acc = *(unsigned*)(lds + threadIdx.x * 4);
  if (acc == 0x12345678u) sink[0] = acc;
}

// The same with the addresses of the real operands: the weight [4096, 12288] and the token rows [T, 12288] are
// row-major bf16 (rows 24576 bytes apart), a panel is R consecutive rows, a step covers 32 KiB of it (KT K tiles of
// 128 bytes per row, R * KT = 256) and a load instruction moves 8 rows x 128 bytes, as in the tile kernels.
template <int R>
__global__ __launch_bounds__(512) void panel_rows_kernel(const char* weights, const char* tokens, int npanels, int steps,
                                                         unsigned* sink) {
  extern __shared__ __align__(1024) char lds[];
  constexpr int kRowBytes = 24576, kRowBlocks = R / 8, kKt = 256 / R;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int panel = blockIdx.x % npanels, ttile = blockIdx.x / npanels;
  const char* w = weights + (size_t)panel * R * kRowBytes + (size_t)(lane >> 3) * kRowBytes + (lane & 7) * 16;
  const char* x = tokens + (size_t)ttile * R * kRowBytes + (size_t)(lane >> 3) * kRowBytes + (lane & 7) * 16;
  char* mine = lds + wave * 16384;
  for (int s = 0; s < steps; ++s) {
    char* dst = mine + (s & 1) * 8192;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = wave * 4 + u;  // block j of the step: rows 8 (j % kRowBlocks) .., K tile j / kRowBlocks
      const size_t off = (size_t)(8 * (j % kRowBlocks)) * kRowBytes + (size_t)(s * kKt + j / kRowBlocks) * 128;
      __builtin_amdgcn_global_load_lds((global_ptr_t)(w + off), (lds_ptr_t)(dst + u * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((global_ptr_t)(x + off), (lds_ptr_t)(dst + 4096 + u * 1024), 16, 0, 0);
    }
    __builtin_amdgcn_s_waitcnt(kWaitAllVm | 8);
  }
  __builtin_amdgcn_s_waitcnt(kWaitAllVm);
  __syncthreads();
  const unsigned acc = *(unsigned*)(lds + threadIdx.x * 4);
  if (acc == 0x12345678u) sink[0] = acc;
}

template <int R>
static void run_panel_rows(const char* name, const char* buf, int token_tiles, int ncopies, unsigned* sink) {
  constexpr size_t kRowBytes = 24576;
  const int npanels = 4096 / R, steps = (int)(kRowBytes / ((256 / R) * 128));
  const size_t copy_bytes = 4096 * kRowBytes, token_bytes = (size_t)token_tiles * R * kRowBytes;
  require((size_t)ncopies * copy_bytes + token_bytes <= g_buffer_bytes, "operands exceed the buffer");
  const char* tokens = buf + (size_t)ncopies * copy_bytes;
  const int lds = 131072, nwg = npanels * token_tiles;
  CK(hipFuncSetAttribute((const void*)panel_rows_kernel<R>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  int c = 0;
  for (int i = 0; i < 5; ++i, c = (c + 1) % ncopies)
    panel_rows_kernel<R><<<nwg, 512, lds>>>(buf + (size_t)c * copy_bytes, tokens, npanels, steps, sink);
  CK(hipEventRecord(a));
  const int reps = 40;
  for (int i = 0; i < reps; ++i, c = (c + 1) % ncopies)
    panel_rows_kernel<R><<<nwg, 512, lds>>>(buf + (size_t)c * copy_bytes, tokens, npanels, steps, sink);
  CK(hipEventRecord(b));
  CK(hipEventSynchronize(b));
  float ms;
  CK(hipEventElapsedTime(&ms, a, b));
  ms /= reps;
  printf("%-58s %3d panels x %d token tiles, weights %s: %6.1f us per launch\n", name, npanels, token_tiles,
         ncopies == 1 ? "relaunched (memory-side cache)" : "rotating (from HBM)          ", ms * 1e3);
  fflush(stdout);
}

template <int PREFETCH, int LEAD>
static void run_panels(const char* name, const char* buf, int npanels, int token_tiles, size_t panel_bytes,
                       int ncopies, unsigned* sink) {
  const int steps = (int)(panel_bytes / 32768);
  const size_t copy_bytes = (size_t)npanels * panel_bytes;
  require(panel_bytes % 32768 == 0 && npanels % 8 == 0, "panel size / count");
  require(!PREFETCH || token_tiles == 4, "the quarter touch needs four readers per panel");
  require((size_t)ncopies * copy_bytes + (size_t)token_tiles * panel_bytes <= g_buffer_bytes, "panels exceed the buffer");
  const char* tokens = buf + (size_t)ncopies * copy_bytes;
  const int lds = 131072 + 256, nwg = npanels * token_tiles;
  CK(hipFuncSetAttribute((const void*)panel_kernel<PREFETCH, LEAD>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  int c = 0;
  for (int i = 0; i < 5; ++i, c = (c + 1) % ncopies)
    panel_kernel<PREFETCH, LEAD><<<nwg, 512, lds>>>(buf + (size_t)c * copy_bytes, tokens, panel_bytes, npanels, steps, sink);
  CK(hipEventRecord(a));
  const int reps = 40;
  for (int i = 0; i < reps; ++i, c = (c + 1) % ncopies)
    panel_kernel<PREFETCH, LEAD><<<nwg, 512, lds>>>(buf + (size_t)c * copy_bytes, tokens, panel_bytes, npanels, steps, sink);
  CK(hipEventRecord(b));
  CK(hipEventSynchronize(b));
  float ms;
  CK(hipEventElapsedTime(&ms, a, b));
  ms /= reps;
  printf("%-58s %3d panels x %d token tiles, weights %s: %6.1f us per launch\n", name, npanels, token_tiles,
         ncopies == 1 ? "relaunched (memory-side cache)" : "rotating (from HBM)          ", ms * 1e3);
  fflush(stdout);
}

// ---- 4: rows of a matrix, 128 bytes at a time ------------------------------------------------------------
// What a tile kernel's loads look like: a workgroup reads 256 rows x 128 bytes per step (wave w, load u covers
// rows 32 w + 8 u .. + 7, a lane takes 16 bytes of row lane / 8), rows `row_stride` bytes apart, and moves 128
// bytes along the rows per step, wrapping after `row_steps`. The workgroups of an XCD read the same 256 rows
// (L2 hits); the question is whether the distance between rows (pages, DRAM rows, channels) limits a CU.
__global__ __launch_bounds__(512) void rows_kernel(const char* base, size_t row_stride, int row_steps, int steps,
                                                   unsigned* sink) {
  extern __shared__ __align__(1024) char lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const char* mine = base + (size_t)(blockIdx.x % 8) * 256 * row_stride +
                     (size_t)(32 * wave + (lane >> 3)) * row_stride + (lane & 7) * 16;
  char* dst = lds + wave * 8192;
  int pos = (blockIdx.x / 8) % row_steps;
  for (int s = 0; s < steps; ++s) {
    const char* src = mine + (size_t)pos * 128;
    char* d = dst + (s & 1) * 4096;
#pragma unroll
    for (int u = 0; u < 4; ++u)
      __builtin_amdgcn_global_load_lds((global_ptr_t)(src + (size_t)(8 * u) * row_stride), (lds_ptr_t)(d + u * 1024), 16, 0, 0);
    __builtin_amdgcn_s_waitcnt(kWaitAllVm | 4);
    if (++pos == row_steps) pos = 0;
  }
  __builtin_amdgcn_s_waitcnt(kWaitAllVm);
  __syncthreads();
  const unsigned acc = *(unsigned*)(lds + threadIdx.x * 4);
  if (acc == 0x12345678u) sink[0] = acc;
}

static void run_rows(const char* name, const char* buf, size_t row_stride, int row_steps, int nwg, unsigned* sink) {
  require((size_t)(8 * 256) * row_stride <= g_buffer_bytes, "rows exceed the buffer");
  require((size_t)row_steps * 128 <= row_stride && row_steps >= 1, "row length");
  const int steps = 2048, lds = 65536;
  CK(hipFuncSetAttribute((const void*)rows_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  for (int i = 0; i < 2; ++i) rows_kernel<<<nwg, 512, lds>>>(buf, row_stride, row_steps, steps, sink);
  CK(hipEventRecord(a));
  const int reps = 5;
  for (int i = 0; i < reps; ++i) rows_kernel<<<nwg, 512, lds>>>(buf, row_stride, row_steps, steps, sink);
  CK(hipEventRecord(b));
  CK(hipEventSynchronize(b));
  float ms;
  CK(hipEventElapsedTime(&ms, a, b));
  ms /= reps;
  const double bytes = (double)nwg * steps * 32768;
  printf("%-40s rows %8zu B apart, %2d steps along a row, %3d workgroups: %6.2f TB/s  %6.1f GB/s per workgroup\n", name,
         row_stride, row_steps, nwg, bytes / ms * 1e-9, bytes / ms * 1e-6 / nwg);
  fflush(stdout);
}

// ---- 5: the load side of the 256 x 256 tile GEMM at its headline shape ------------------------------------
// gate_up at 4096 tokens (W [24576, 4096], X [4096, 4096], bf16, rows of 8 KiB): 1536 workgroups, each 64 steps
// of (256 weight rows + 256 token rows) x 128 bytes with the previous step awaited before the next is issued
// (one K tile of lead, as in the kernel), and the kernel's raster (XCD-compact ids, groups of eight token tiles).
__global__ __launch_bounds__(512) void big_tile_kernel(const char* weights, const char* tokens, int tiles_m, int tiles_n,
                                                       unsigned* sink) {
  extern __shared__ __align__(1024) char lds[];
  constexpr int kRowBytes = 8192;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int per_xcd = tiles_m * tiles_n / 8;
  const int id = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  const int group_m = 8, per_group = group_m * tiles_n;
  const int group = id / per_group, within = id - group * per_group;
  const int tile_m = group * group_m + within % group_m, tile_n = within / group_m;
  const char* w = weights + (size_t)tile_n * 256 * kRowBytes + (size_t)(lane >> 3) * kRowBytes + (lane & 7) * 16;
  const char* x = tokens + (size_t)tile_m * 256 * kRowBytes + (size_t)(lane >> 3) * kRowBytes + (lane & 7) * 16;
  char* mine = lds + wave * 16384;
  for (int s = 0; s < 64; ++s) {
    char* dst = mine + (s & 1) * 8192;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t off = (size_t)(8 * (wave * 4 + u)) * kRowBytes + (size_t)s * 128;
      __builtin_amdgcn_global_load_lds((global_ptr_t)(w + off), (lds_ptr_t)(dst + u * 1024), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((global_ptr_t)(x + off), (lds_ptr_t)(dst + 4096 + u * 1024), 16, 0, 0);
    }
    __builtin_amdgcn_s_waitcnt(kWaitAllVm | 8);
  }
  __builtin_amdgcn_s_waitcnt(kWaitAllVm);
  __syncthreads();
  const unsigned acc = *(unsigned*)(lds + threadIdx.x * 4);
  if (acc == 0x12345678u) sink[0] = acc;
}

static void run_big_tile(const char* buf, unsigned* sink) {
  const int tiles_m = 16, tiles_n = 96, lds = 131072;
  const size_t wbytes = (size_t)24576 * 8192, xbytes = (size_t)4096 * 8192;
  require(wbytes + xbytes <= g_buffer_bytes, "operands exceed the buffer");
  CK(hipFuncSetAttribute((const void*)big_tile_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  for (int i = 0; i < 5; ++i) big_tile_kernel<<<tiles_m * tiles_n, 512, lds>>>(buf, buf + wbytes, tiles_m, tiles_n, sink);
  CK(hipEventRecord(a));
  const int reps = 20;
  for (int i = 0; i < reps; ++i) big_tile_kernel<<<tiles_m * tiles_n, 512, lds>>>(buf, buf + wbytes, tiles_m, tiles_n, sink);
  CK(hipEventRecord(b));
  CK(hipEventSynchronize(b));
  float ms;
  CK(hipEventElapsedTime(&ms, a, b));
  ms /= reps;
  printf("gate_up at 4096 tokens, 256x256 tiles, loads only: %6.1f us per launch (%.1f TB/s out of the L2s)\n", ms * 1e3,
         1536.0 * 64 * 65536 / ms * 1e-9);
  fflush(stdout);
}

// ---- 6: the matrix pipe alone ----------------------------------------------------------------------------
// The MFMA sequence of the 256 x 256 tile kernel out of registers: per wave and K tile 64 v_mfma_f32_16x16x32_bf16
// (4 weight x 8 token fragments, two K steps), eight waves per CU, no loads, no LDS. One launch is the matrix work
// of gate_up at 4096 tokens. With random bf16 operand values (weights scaled by 0.02, as in the benchmark) and
// with zeros: what the part sustains at its power cap when nothing but the matrix pipe runs.
typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float probe_f32x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t probe_u32x4_t;

__global__ __launch_bounds__(512) void mfma_only_kernel(const probe_u32x4_t* frags, int ktiles, float* sink) {
  const int lane = threadIdx.x & 63;
  probe_u32x4_t w[2][4], x[2][8];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
#pragma unroll
    for (int j = 0; j < 4; ++j) w[s][j] = frags[(s * 12 + j) * 64 + lane];
#pragma unroll
    for (int j = 0; j < 8; ++j) x[s][j] = frags[(s * 12 + 4 + j) * 64 + lane];
  }
  probe_f32x4_t acc[4][8];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 8; ++b) acc[a][b] = probe_f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int t = 0; t < ktiles; ++t) {
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 8; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(probe_bf16x8_t, w[s][a]),
                                                               __builtin_bit_cast(probe_bf16x8_t, x[s][b]), acc[a][b], 0, 0, 0);
#pragma unroll
    for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(w[0][j]), "+v"(w[1][j]));  // the loop is not collapsed
  }
  float r = 0.f;
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 8; ++b) r += acc[a][b][0] + acc[a][b][1] + acc[a][b][2] + acc[a][b][3];
  if (r == 123.456f) sink[0] = r;
}

static uint16_t probe_bf16_of(float f) {
  uint32_t u;
  __builtin_memcpy(&u, &f, 4);
  return (uint16_t)((u + 0x7fff + ((u >> 16) & 1)) >> 16);
}

static void run_mfma_only(char* buf, unsigned* sink) {
  constexpr int kFrags = 24 * 64;  // 24 fragments of 64 lanes x 16 bytes
  static uint16_t host[kFrags * 8];
  for (int mode = 0; mode < 2; ++mode) {
    srand(7);
    for (int i = 0; i < kFrags * 8; ++i) {
      float g = 0.f;  // a sum of 12 uniforms: about normal
      for (int q = 0; q < 12; ++q) g += (float)(rand() % 65536) / 65536.f;
      g -= 6.f;
      const int frag = (i / 8 / 64) % 12;
      host[i] = mode == 0 ? probe_bf16_of(frag < 4 ? 0.02f * g : g) : 0;
    }
    CK(hipMemcpy(buf, host, sizeof(host), hipMemcpyHostToDevice));
    const int ktiles = 64 * 6;  // 256 workgroups x 6 tiles x 64 K tiles = the 1536 tiles of gate_up at 4096 tokens
    hipEvent_t a, b;
    CK(hipEventCreate(&a));
    CK(hipEventCreate(&b));
    for (int i = 0; i < 100; ++i)  // the clocks settle
      mfma_only_kernel<<<256, 512>>>(reinterpret_cast<const probe_u32x4_t*>(buf), ktiles, reinterpret_cast<float*>(sink));
    CK(hipEventRecord(a));
    const int reps = 200;
    for (int i = 0; i < reps; ++i)
      mfma_only_kernel<<<256, 512>>>(reinterpret_cast<const probe_u32x4_t*>(buf), ktiles, reinterpret_cast<float*>(sink));
    CK(hipEventRecord(b));
    CK(hipEventSynchronize(b));
    float ms;
    CK(hipEventElapsedTime(&ms, a, b));
    ms /= reps;
    const double flops = 256.0 * 8 * ktiles * 64 * (2.0 * 16 * 16 * 32);
    printf("matrix pipe only, %s operands: %6.1f us per launch of %.1f GFLOP = %6.1f TFLOP/s (%.1f %% of 2.5 PFLOP/s)\n",
           mode == 0 ? "random" : "zero  ", ms * 1e3, flops * 1e-9, flops / ms * 1e-9, flops / ms * 1e-9 / 25.0);
    fflush(stdout);
  }
}

// ---- 7: what the data movement of the tile kernel costs the matrix pipe ------------------------------------
// The MFMA sequence of section 6 with, one after the other, the kernel's LDS fragment reads (24 ds_read_b128 per
// wave and K tile at the kernel's addresses), its direct-to-LDS loads (8 per wave and K tile = 64 KiB per workgroup,
// from 4 MiB that stay in the L2) and two barriers per K tile; every wave reads, loads and multiplies (no roles).
// Workgroup 0 also reports the shader clock it saw (clock64 against the 100 MHz wall clock): on zero operands the
// clock stays at its maximum and the cost is cycles, on random operands the power cap turns bytes into clock.
// MODE bit 0: fragment reads, bit 1: loads, bit 2: barriers.
template <int MODE>
__global__ __launch_bounds__(512) void mfma_with_traffic_kernel(const char* src, int ktiles, float* sink) {
  extern __shared__ __align__(1024) char lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wave_n = wave & 3, wave_m = wave >> 2;
  const int l16 = lane & 15, grp = lane >> 4;
  for (int i = tid; i < 131072 / 16; i += 512)
    reinterpret_cast<probe_u32x4_t*>(lds)[i] = reinterpret_cast<const probe_u32x4_t*>(src)[i];
  __syncthreads();
  const int frag_lo = (grp ^ (l16 & 7)) << 4;
  const int w_row = (wave_n * 64 + l16) * 128, x_row = 256 * 128 + (wave_m * 128 + l16) * 128;
  probe_u32x4_t w[2][4], x[2][8];
  auto read_frags = [&](const char* st) {
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        w[s][j] = *reinterpret_cast<const probe_u32x4_t*>(st + w_row + j * 16 * 128 + (frag_lo ^ (s << 6)));
#pragma unroll
      for (int j = 0; j < 8; ++j)
        x[s][j] = *reinterpret_cast<const probe_u32x4_t*>(st + x_row + j * 16 * 128 + (frag_lo ^ (s << 6)));
    }
  };
  read_frags(lds);
  const long long c0 = clock64(), r0 = wall_clock64();
  probe_f32x4_t acc[4][8];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 8; ++b) acc[a][b] = probe_f32x4_t{0.f, 0.f, 0.f, 0.f};
  const char* gsrc = src + (size_t)(blockIdx.x % 32) * 131072 + wave * 8192 + lane * 16;  // 4 MiB per 32 workgroups
  for (int t = 0; t < ktiles; ++t) {
    char* st = lds + (t & 1) * 65536;
    if (MODE & 2) {
#pragma unroll
      for (int u = 0; u < 8; ++u)
        __builtin_amdgcn_global_load_lds((global_ptr_t)(gsrc + (t & 1) * 65536 + u * 1024),
                                         (lds_ptr_t)(st + wave * 8192 + u * 1024), 16, 0, 0);
    }
    if (MODE & 1) read_frags(lds + ((t + 1) & 1) * 65536);
    if (MODE & 4) __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 8; ++b)
          acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(probe_bf16x8_t, w[s][a]),
                                                               __builtin_bit_cast(probe_bf16x8_t, x[s][b]), acc[a][b], 0, 0, 0);
    if (MODE & 4) __builtin_amdgcn_s_barrier();
    if (!(MODE & 1)) {
#pragma unroll
      for (int j = 0; j < 4; ++j) asm volatile("" : "+v"(w[0][j]), "+v"(w[1][j]));
    }
    if (MODE & 2) __builtin_amdgcn_s_waitcnt(kWaitAllVm | 8);
  }
  __builtin_amdgcn_s_waitcnt(kWaitAllVm);
  float r = 0.f;
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 8; ++b) r += acc[a][b][0] + acc[a][b][1] + acc[a][b][2] + acc[a][b][3];
  if (r == 123.456f) sink[0] = r;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    const long long c1 = clock64(), r1 = wall_clock64();
    reinterpret_cast<long long*>(sink)[1] = c1 - c0;
    reinterpret_cast<long long*>(sink)[2] = r1 - r0;
  }
}

template <int MODE>
static void run_mfma_with_traffic(const char* name, const char* buf, float* sink) {
  CK(hipFuncSetAttribute((const void*)mfma_with_traffic_kernel<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, 131072));
  const int ktiles = 64 * 6;
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  for (int i = 0; i < 100; ++i) mfma_with_traffic_kernel<MODE><<<256, 512, 131072>>>(buf, ktiles, sink);
  CK(hipEventRecord(a));
  const int reps = 200;
  for (int i = 0; i < reps; ++i) mfma_with_traffic_kernel<MODE><<<256, 512, 131072>>>(buf, ktiles, sink);
  CK(hipEventRecord(b));
  CK(hipEventSynchronize(b));
  float ms;
  CK(hipEventElapsedTime(&ms, a, b));
  ms /= reps;
  long long rec[4];
  CK(hipMemcpy(rec, sink, 32, hipMemcpyDeviceToHost));
  const double flops = 256.0 * 8 * ktiles * 64 * (2.0 * 16 * 16 * 32);
  printf("%-50s %6.1f us  %6.1f TFLOP/s  shader clock %.2f GHz\n", name, ms * 1e3, flops / ms * 1e-9,
         (double)rec[1] / (double)rec[2] * 0.1);
  fflush(stdout);
}

static void run_traffic_cost(char* buf, char* sink_bytes) {
  constexpr size_t kBytes = (size_t)8 << 20;  // 4 MiB are read; stages of 64 KiB: weight rows first (scaled by 0.02)
  static uint16_t host[kBytes / 2];
  float* sink = reinterpret_cast<float*>(sink_bytes);
  for (int mode = 0; mode < 2; ++mode) {
    srand(7);
    for (size_t i = 0; i < kBytes / 2; ++i) {
      float g = 0.f;
      for (int q = 0; q < 12; ++q) g += (float)(rand() % 65536) / 65536.f;
      g -= 6.f;
      host[i] = mode == 0 ? probe_bf16_of(((i * 2) % 65536) < 32768 ? 0.02f * g : g) : 0;
    }
    CK(hipMemcpy(buf, host, kBytes, hipMemcpyHostToDevice));
    printf("   %s operands\n", mode == 0 ? "random" : "zero");
    run_mfma_with_traffic<0>("matrix pipe only", buf, sink);
    run_mfma_with_traffic<1>("+ LDS fragment reads", buf, sink);
    run_mfma_with_traffic<3>("+ fragment reads + direct-to-LDS loads from L2", buf, sink);
    run_mfma_with_traffic<7>("+ reads + loads + two barriers per K tile", buf, sink);
    run_mfma_with_traffic<2>("matrix pipe + direct-to-LDS loads only", buf, sink);
  }
}

// ---- 8: column slabs of a K-major weight ------------------------------------------------------------------
// Decode against a prepared weight B[K = 12288][N = 4096] (rows of 8 KiB): with no split-K a workgroup owns its
// features for the whole reduction, i.e. it streams a column slab of `slab_bytes` per K row (128 bytes = 64 features:
// 64 workgroups; 64 bytes: 128; 32 bytes: 256), 32 KiB per step, the previous step awaited. Copies of the weight
// rotate, so it comes from HBM, or one copy is relaunched (memory-side cache).
__global__ __launch_bounds__(512) void column_slab_kernel(const char* w, int slab_bytes, int nslabs, int krows, unsigned* sink) {
  extern __shared__ __align__(1024) char lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const size_t row_bytes = (size_t)slab_bytes * nslabs;
  const int lanes_per_row = slab_bytes / 16;      // 8, 4, 2
  const int rows_per_instr = 64 / lanes_per_row;  // 8, 16, 32
  const int rows_per_step = 8 * 4 * rows_per_instr;
  const char* mine = w + (size_t)blockIdx.x * slab_bytes + (size_t)(lane / lanes_per_row) * row_bytes + (lane % lanes_per_row) * 16;
  char* dst = lds + wave * 8192;
  const int steps = krows / rows_per_step;
  for (int s = 0; s < steps; ++s) {
    const char* src = mine + (size_t)(s * rows_per_step + wave * 4 * rows_per_instr) * row_bytes;
    char* d = dst + (s & 1) * 4096;
#pragma unroll
    for (int u = 0; u < 4; ++u)
      __builtin_amdgcn_global_load_lds((global_ptr_t)(src + (size_t)(u * rows_per_instr) * row_bytes), (lds_ptr_t)(d + u * 1024), 16, 0, 0);
    __builtin_amdgcn_s_waitcnt(kWaitAllVm | 4);
  }
  __builtin_amdgcn_s_waitcnt(kWaitAllVm);
  __syncthreads();
  const unsigned acc = *(unsigned*)(lds + threadIdx.x * 4);
  if (acc == 0x12345678u) sink[0] = acc;
}

static void run_column_slabs(const char* buf, int slab_bytes, int ncopies, unsigned* sink) {
  const int krows = 12288, row_bytes = 8192, nslabs = row_bytes / slab_bytes, lds = 65536;
  const size_t copy_bytes = (size_t)krows * row_bytes;
  require(slab_bytes == 128 || slab_bytes == 64 || slab_bytes == 32, "slab width");
  require((size_t)ncopies * copy_bytes <= g_buffer_bytes, "copies exceed the buffer");
  CK(hipFuncSetAttribute((const void*)column_slab_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  int c = 0;
  for (int i = 0; i < 5; ++i, c = (c + 1) % ncopies)
    column_slab_kernel<<<nslabs, 512, lds>>>(buf + (size_t)c * copy_bytes, slab_bytes, nslabs, krows, sink);
  CK(hipEventRecord(a));
  const int reps = 40;
  for (int i = 0; i < reps; ++i, c = (c + 1) % ncopies)
    column_slab_kernel<<<nslabs, 512, lds>>>(buf + (size_t)c * copy_bytes, slab_bytes, nslabs, krows, sink);
  CK(hipEventRecord(b));
  CK(hipEventSynchronize(b));
  float ms;
  CK(hipEventElapsedTime(&ms, a, b));
  ms /= reps;
  printf("slabs of %3d bytes per K row, %3d workgroups, weight %s: %6.1f us  %5.2f TB/s\n", slab_bytes, nslabs,
         ncopies == 1 ? "relaunched (memory-side cache)" : "rotating (from HBM)          ", ms * 1e3, copy_bytes / ms * 1e-9);
  fflush(stdout);
}

// Without arguments every section runs; with a section number (1 .. 8) only that one.
int main(int argc, char** argv) {
  const int only = argc > 1 ? atoi(argv[1]) : 0;
  auto want = [&](int section) { return only == 0 || only == section; };
  g_buffer_bytes = (size_t)4 << 30;
  char* buf;
  unsigned* sink;
  CK(hipMalloc(&buf, g_buffer_bytes));
  CK(hipMalloc(&sink, 4));
  char* scratch;
  CK(hipMalloc(&scratch, 32));
  CK(hipMemset(buf, 1, g_buffer_bytes));
  CK(hipDeviceSynchronize());

  if (want(1)) {
    printf("== 1. ceilings, every CU loading\n");
    run_streams<0, 8, 8>("L2: all workgroups cycle over 1 MB", buf, 1 << 20, 1, 256, 400, sink);
    run_streams<1, 8, 8>("L2: all workgroups cycle over 1 MB", buf, 1 << 20, 1, 256, 400, sink);
    run_streams<0, 8, 8>("memory-side cache: 128 MB cycled", buf, 1 << 19, 256, 256, 400, sink);
    run_streams<1, 8, 8>("memory-side cache: 128 MB cycled", buf, 1 << 19, 256, 256, 400, sink);
    run_streams<0, 8, 8>("HBM: 4 GB once, 16 MB per workgroup", buf, 16 << 20, 256, 256, 256, sink);
    run_streams<1, 8, 8>("HBM: 4 GB once, 16 MB per workgroup", buf, 16 << 20, 256, 256, 256, sink);
    run_streams<1, 4, 8>("HBM: 4 GB once, 2 MB per workgroup", buf, 2 << 20, 2048, 2048, 64, sink);
  }
  if (want(2)) {
    printf("== 2. one workgroup's rate against its bytes in flight (each streams its own 16 MB from HBM)\n");
    for (int nwg : {32, 256}) {
      run_streams<0, 1, 1>("HBM", buf, 16 << 20, nwg, nwg, 2048, sink);
      run_streams<0, 1, 4>("HBM", buf, 16 << 20, nwg, nwg, 2048, sink);
      run_streams<0, 2, 4>("HBM", buf, 16 << 20, nwg, nwg, 2048, sink);
      run_streams<0, 4, 4>("HBM", buf, 16 << 20, nwg, nwg, 1024, sink);
      run_streams<0, 8, 4>("HBM", buf, 16 << 20, nwg, nwg, 512, sink);
      run_streams<0, 8, 8>("HBM", buf, 16 << 20, nwg, nwg, 256, sink);
    }
    for (int nwg : {8, 256}) {
      printf("   (each workgroup cycles over its own 64 KB: L2 hits)\n");
      run_streams<0, 1, 1>("L2", buf, 64 << 10, nwg, nwg, 4096, sink);
      run_streams<0, 1, 4>("L2", buf, 64 << 10, nwg, nwg, 4096, sink);
      run_streams<0, 2, 4>("L2", buf, 64 << 10, nwg, nwg, 4096, sink);
      run_streams<0, 4, 4>("L2", buf, 64 << 10, nwg, nwg, 4096, sink);
      run_streams<0, 8, 8>("L2", buf, 64 << 10, nwg, nwg, 4096, sink);
    }
  }
  if (want(3)) {
    printf("== 3. load side of the small-tile GEMMs of the down projection (4096 features, K = 12288), no arithmetic\n");
    for (int ncopies : {1, 14}) {
      // 256 tokens, 64 x 64 tiles: 64 panels of 64 features (1.5 MB), four token tiles of 64 tokens (1.5 MB each)
      run_panels<0, 0>("256 tokens, 64x64 tiles", buf, 64, 4, 3 << 19, ncopies, sink);
      run_panels<1, 2>("256 tokens, 64x64 tiles, quarter touch 2 steps ahead", buf, 64, 4, 3 << 19, ncopies, sink);
      run_panels<1, 6>("256 tokens, 64x64 tiles, quarter touch 6 steps ahead", buf, 64, 4, 3 << 19, ncopies, sink);
      // 1024 tokens, 128 x 128 tiles: 32 panels of 128 features (3 MB), eight token tiles of 128 tokens (3 MB each)
      run_panels<0, 0>("1024 tokens, 128x128 tiles", buf, 32, 8, 3 << 20, ncopies, sink);
      // and with the row-major addresses of the operands themselves
      run_panel_rows<64>("256 tokens, 64x64 tiles, row-major operands", buf, 4, ncopies, sink);
      run_panel_rows<128>("1024 tokens, 128x128 tiles, row-major operands", buf, 8, ncopies, sink);
    }
  }
  if (want(4)) {
    printf("== 4. 256 rows x 128 bytes per step out of the L2, by the distance between rows\n");
    for (int nwg : {8, 256}) {
      run_rows("rows back to back (8 KB each)", buf, 8192, 64, nwg, sink);
      run_rows("rows of K = 12288 bf16", buf, 24576, 64, nwg, sink);
      run_rows("rows of V = 151936 bf16", buf, 303872, 64, nwg, sink);
      run_rows("rows 1 MB apart", buf, 1 << 20, 64, nwg, sink);
    }
  }
  if (want(5)) {
    printf("== 5. load side of the 256 x 256 tile GEMM at the headline shape, no arithmetic\n");
    run_big_tile(buf, sink);
  }
  if (want(6)) {
    printf("== 6. the matrix pipe alone: the MFMA sequence of the 256 x 256 tile kernel out of registers\n");
    run_mfma_only(buf, sink);
  }
  if (want(7)) {
    printf("== 7. the same sequence with the kernel's LDS reads, L2 loads and barriers added one after the other\n");
    run_traffic_cost(buf, scratch);
  }
  if (want(8)) {
    printf("== 8. a K-major weight [12288][4096] streamed as column slabs, one workgroup per slab (decode against a prepared weight)\n");
    for (int ncopies : {1, 14})
      for (int slab : {128, 64, 32}) run_column_slabs(buf, slab, ncopies, sink);
  }
  return 0;
}
