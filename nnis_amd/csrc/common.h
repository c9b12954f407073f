// Shared helpers of the gfx950 kernels: element types, loads that widen to
// 32-bit, wave and block reductions, and the error channel of the C entry
// points.  Every entry point returns 0 on success; on refusal it returns a
// non-zero code and leaves a message for nnis_last_error().
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

typedef __bf16 bf16_t;

// element type codes shared with the Python side
enum : int { NNIS_F32 = 0, NNIS_BF16 = 1 };

constexpr int kWave = 64;        // lanes of a gfx950 wavefront
constexpr int kPageTokens = 64;  // tokens a cache page holds

// Where a page keeps its 64 tokens of one key/value head, in elements.  Both orders are those in which the
// attention kernels' wave-wide 16-byte loads read: consecutive lanes, consecutive memory.
//   keys    [chunk of 8 channels][token][8 channels]
//   values  [tile of 16 channels][half of 32 tokens][group of 8 tokens][channel of the tile][8 tokens]
// A head size that is no multiple of 8 (16) leaves the last chunk (tile) partly unused.
__host__ __device__ constexpr size_t nnis_k_page_elems(int head_dim) { return (size_t)((head_dim + 7) / 8) * kPageTokens * 8; }
__host__ __device__ constexpr size_t nnis_v_page_elems(int head_dim) { return (size_t)((head_dim + 15) / 16) * kPageTokens * 16; }
__host__ __device__ constexpr size_t nnis_k_offset(int token, int channel) {
  return (size_t)(channel / 8) * (kPageTokens * 8) + (size_t)token * 8 + channel % 8;
}
__host__ __device__ constexpr size_t nnis_v_offset(int channel, int token) {
  return ((((size_t)(channel / 16) * 2 + token / 32) * 4 + (token % 32) / 8) * 16 + channel % 16) * 8 + token % 8;
}

// The weights of the matrix-core products are kept packed (nnis_pack_weight): rows in strips of 16, K in
// chunks of 64, both padded with zeros, and a strip's chunk (2 KB) in the order in which a wave's two
// 16-byte loads take it as the first operand of v_mfma_f32_16x16x32_bf16:
//   [strip][chunk][half][lane = 16 * (k % 64 / 16) + row % 16][8 elements],  half = k % 16 / 8
// so that a load instruction of a wave reads 1 KB of consecutive memory whatever K is (rows of the
// checkpoint's order are K * 2 bytes apart: 16 pieces of 64 bytes an instruction, measured at 55 to 80% of the
// packed order's bandwidth on weights of 8 to 200 MB).
// A strip is an odd number of chunks long (one chunk of padding where K gives an even number, never read), so
// that the strips' first chunks, which a kernel's waves all ask for at once, do not lie a power of two apart
// and meet in the same memory channels.
constexpr int kPackedChunkElems = 1024;  // a strip's chunk
constexpr int kPackedHalfElems = 512;
__host__ __device__ constexpr int nnis_packed_chunks(int k) { return (k + 63) / 64; }
__host__ __device__ constexpr size_t nnis_packed_strip_elems(int k) { return (size_t)(nnis_packed_chunks(k) | 1) * kPackedChunkElems; }
__host__ __device__ constexpr size_t nnis_packed_elems(int n, int k) { return (size_t)((n + 15) / 16) * nnis_packed_strip_elems(k); }
// where the lane that multiplies `row` with k group g (k % 64 / 16) finds its 8 elements of chunk 0, half 0
__host__ __device__ constexpr size_t nnis_packed_lane(int row, int g, int k) {
  return (size_t)(row >> 4) * nnis_packed_strip_elems(k) + (size_t)(g * 16 + (row & 15)) * 8;
}

extern thread_local char g_nnis_error[512];

static inline int nnis_fail(const char* fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(g_nnis_error, sizeof(g_nnis_error), fmt, args);
  va_end(args);
  return 1;
}

#define NNIS_REQUIRE(cond, ...)                  \
  do {                                           \
    if (!(cond)) return nnis_fail(__VA_ARGS__);  \
  } while (0)

#define NNIS_LAUNCH_CHECK(name)                                                        \
  do {                                                                                 \
    hipError_t launch_error = hipGetLastError();                                       \
    if (launch_error != hipSuccess)                                                    \
      return nnis_fail("%s: launch failed: %s", name, hipGetErrorString(launch_error)); \
  } while (0)

static inline bool nnis_dtype_ok(int dtype) { return dtype == NNIS_F32 || dtype == NNIS_BF16; }
static inline int nnis_dtype_size(int dtype) { return dtype == NNIS_F32 ? 4 : 2; }

// ---- typed access -----------------------------------------------------------

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }  // round to nearest even

// element `index` of an array whose element type is only known at run time;
// the branch is uniform over a launch
__device__ __forceinline__ float load_as_f32(const void* base, int dtype, size_t index) {
  return dtype == NNIS_F32 ? ((const float*)base)[index] : (float)((const bf16_t*)base)[index];
}

__device__ __forceinline__ void store_from_f32(void* base, int dtype, size_t index, float value) {
  if (dtype == NNIS_F32) {
    ((float*)base)[index] = value;
  } else {
    ((bf16_t*)base)[index] = (bf16_t)value;
  }
}

// ---- reductions ---------------------------------------------------------------

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int offset = kWave / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int offset = kWave / 2; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, kWave));
  return v;
}

// sum over a block of up to 1024 threads; `scratch` holds at least 16 floats;
// every thread gets the result
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();  // scratch may still be read from a previous call
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.0f;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  return total;
}

// Blocks go to the chip's 8 dies in turn (block i to die i % 8), each die with an L2 of its own.  A kernel
// for few tokens whose blocks are (unit of weight rows) x (tile of 16 * MT tokens) deals them so that all
// token tiles of a unit run on one die, one after the other: the unit's weight rows come from memory once.
// Launch ((units + 7) / 8) * 8 * tiles blocks; a block whose unit is beyond the last leaves.
__device__ __forceinline__ void nnis_deal_tiles(int block, int tiles, int& unit_block, int& tile) {
  const int die = block % 8, nth = block / 8;
  unit_block = (nth / tiles) * 8 + die;
  tile = nth % tiles;
}
