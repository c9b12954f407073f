// bfloat16 matrix products on the matrix cores: Y[M, N] = X[M, K] * W[N, K]^T,
// 32-bit accumulation, output bfloat16 or 32-bit.  K is contiguous in both
// operands, so a lane's 16-byte load is 8 consecutive k of one row, which is
// what v_mfma_f32_16x16x32_bf16 wants of either operand: lane l holds row
// (l % 16), k-group (l / 16) of 8.  The instruction sums over the 4 groups x 8
// elements; which k each (group, element) stands for is free as long as both
// operands agree.  Its result D[i][j] (i: row of the first operand, j: row of
// the second) lies with lane l as D[4 * (l / 16) + e][l % 16], e = 0..3.
//
//  * gemm_skinny_kernel: M <= 64 (decode).  The weight is streamed once from
//    memory straight into operand registers; a wave owns a strip of 16 weight
//    rows; X (small, shared by all waves) comes through the caches.  Waves of
//    a block may split K and add their parts through LDS.
//  * gemm_tiled_kernel: any M (prefill).  128x128 or 64x128 or 64x64 output
//    tiles, K staged through LDS in steps of 64 with an XOR swizzle of the
//    16-byte chunks so that operand reads are free of bank conflicts, global
//    loads of the next step in flight while the current one is multiplied.
//
// Both need K % 8 == 0 and 16-byte aligned operands (the host checks) and take
// any M and N.
#include "common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ bf16x8 load_chunk(const bf16_t* p) { return *(const bf16x8*)p; }

__device__ __forceinline__ bf16x8 zero_chunk() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

__device__ __forceinline__ f32x4 mfma(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

template <typename OutT>
__device__ __forceinline__ void store4(OutT* y, size_t index, f32x4 v, int valid, bool vector_ok);

template <>
__device__ __forceinline__ void store4<float>(float* y, size_t index, f32x4 v, int valid, bool vector_ok) {
  if (valid == 4 && vector_ok) {
    *(f32x4*)(y + index) = v;
  } else {
    for (int e = 0; e < valid; ++e) y[index + e] = v[e];
  }
}

template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* y, size_t index, f32x4 v, int valid, bool vector_ok) {
  if (valid == 4 && vector_ok) {
    typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
    bf16x4 packed;
#pragma unroll
    for (int e = 0; e < 4; ++e) packed[e] = (__bf16)v[e];
    *(bf16x4*)(y + index) = packed;
  } else {
    for (int e = 0; e < valid; ++e) y[index + e] = (bf16_t)v[e];
  }
}

// -----------------------------------------------------------------------------
// skinny: MT token tiles of 16 (M <= 16 * MT); KSPLIT waves share one strip's K.
// A decode-sized product is bound by memory latency, not bandwidth: a wave
// issues the loads of DEPTH steps of 64 k (weights and activations) before the
// first multiply, so its whole share of K is usually one round trip.
// -----------------------------------------------------------------------------
template <int MT, int KSPLIT, typename OutT>
__global__ __launch_bounds__(KSPLIT > 4 ? 64 * KSPLIT : 256) void gemm_skinny_kernel(const bf16_t* __restrict__ x,
                                                                                   const bf16_t* __restrict__ w,
                                                                                   OutT* __restrict__ y, int m, int n,
                                                                                   int k) {
  constexpr int kWaves = KSPLIT > 4 ? KSPLIT : 4;
  constexpr int kStrips = kWaves / KSPLIT;  // strips of 16 weight rows per block
  constexpr int DEPTH = MT <= 2 ? 4 : 2;
  __shared__ float partial[KSPLIT > 1 ? kWaves : 1][MT][kWave][4];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int strip = blockIdx.x * kStrips + wave / KSPLIT;
  const int part = wave % KSPLIT;
  const int r = lane % 16, g = lane / 16;
  const int strips = (n + 15) / 16;
  const bool active = strip < strips;

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};

  if (active) {
    int w_row = strip * 16 + r;
    w_row = w_row < n ? w_row : n - 1;  // rows beyond N read a valid row and are not stored
    const bf16_t* w_ptr = w + (size_t)w_row * k;
    const bf16_t* x_ptr[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      int token = t * 16 + r;
      token = token < m ? token : m - 1;
      x_ptr[t] = x + (size_t)token * k;
    }
    const int chunks = (k + 63) / 64;
    for (int base = part; base < chunks; base += KSPLIT * DEPTH) {
      bf16x8 wa[DEPTH], wb[DEPTH], xa[DEPTH][MT], xb[DEPTH][MT];
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int ka = (base + d * KSPLIT) * 64 + g * 16, kb = ka + 8;
        const bool in_a = ka + 8 <= k, in_b = kb + 8 <= k;  // false also for steps beyond the last
        wa[d] = in_a ? load_chunk(w_ptr + ka) : zero_chunk();
        wb[d] = in_b ? load_chunk(w_ptr + kb) : zero_chunk();
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          xa[d][t] = in_a ? load_chunk(x_ptr[t] + ka) : zero_chunk();
          xb[d][t] = in_b ? load_chunk(x_ptr[t] + kb) : zero_chunk();
        }
      }
#pragma unroll
      for (int d = 0; d < DEPTH; ++d)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          acc[t] = mfma(wa[d], xa[d][t], acc[t]);
          acc[t] = mfma(wb[d], xb[d][t], acc[t]);
        }
    }
  }

  if constexpr (KSPLIT > 1) {
    if (part != 0) {
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) partial[wave][t][lane][e] = acc[t][e];
    }
    __syncthreads();
    if (part != 0) return;
#pragma unroll
    for (int other = 1; other < KSPLIT; ++other)
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[t][e] += partial[wave + other][t][lane][e];
  }
  if (!active) return;

  // lane holds D[weight row 4g + e][token r]: four consecutive outputs of one token
  const int n0 = strip * 16 + g * 4;
  const int valid = n - n0 >= 4 ? 4 : (n - n0 > 0 ? n - n0 : 0);
  const bool vector_ok = (n % 4) == 0;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int token = t * 16 + r;
    if (token < m && valid > 0) store4<OutT>(y, (size_t)token * n + n0, acc[t], valid, vector_ok);
  }
}

// -----------------------------------------------------------------------------
// tiled: BM x BN output tile per block of 4 waves (2 x 2), K in steps of 64
// -----------------------------------------------------------------------------
constexpr int kBK = 64;  // k per stage: 8 chunks of 16 bytes per row

// chunk c (0..7) of row `row` of a staged tile lives at chunk (c ^ (row & 7))
__device__ __forceinline__ int swizzled(int row, int chunk) { return row * 8 + (chunk ^ (row & 7)); }

template <int BM, int BN, typename OutT>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                         OutT* __restrict__ y, int m, int n, int k) {
  constexpr int WM = BM / 2, WN = BN / 2;  // a wave's part of the tile
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int A_CHUNKS = BM * 8 / 256, B_CHUNKS = BN * 8 / 256;  // 16-byte chunks a thread stages per step
  // Global loads run PF steps ahead of the multiply, in registers; the step after
  // the current one lies in the other LDS buffer.  With few blocks on a compute
  // unit nothing else hides the latency of a load, so short products need depth.
  constexpr int PF = (BM * BN >= 128 * 128) ? 3 : 4;
  __shared__ bf16x8 a_tile[2][BM * 8];
  __shared__ bf16x8 b_tile[2][BN * 8];

  const int tid = threadIdx.x;
  const int wave = tid / kWave, lane = tid % kWave;
  const int wave_m = wave / 2, wave_n = wave % 2;
  const int r = lane % 16, g = lane / 16;
  const int row0 = blockIdx.y * BM, col0 = blockIdx.x * BN;

  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};

  // what this thread stages: rows and chunk of each of its 16-byte pieces
  const bf16_t* a_src[A_CHUNKS];
  const bf16_t* b_src[B_CHUNKS];
  int a_dst[A_CHUNKS], b_dst[B_CHUNKS];
  const int chunk_k = (tid % 8) * 8;
#pragma unroll
  for (int c = 0; c < A_CHUNKS; ++c) {
    const int index = tid + c * 256;  // row = index / 8, chunk = index % 8
    int row = row0 + index / 8;
    row = row < m ? row : m - 1;
    a_src[c] = x + (size_t)row * k + chunk_k;
    a_dst[c] = swizzled(index / 8, index % 8);
  }
#pragma unroll
  for (int c = 0; c < B_CHUNKS; ++c) {
    const int index = tid + c * 256;
    int row = col0 + index / 8;
    row = row < n ? row : n - 1;
    b_src[c] = w + (size_t)row * k + chunk_k;
    b_dst[c] = swizzled(index / 8, index % 8);
  }

  bf16x8 a_stage[PF][A_CHUNKS], b_stage[PF][B_CHUNKS];
  const int steps = (k + kBK - 1) / kBK;

#define NNIS_FETCH(slot, step)                                                                   \
  do {                                                                                           \
    const int k0 = (step) * kBK;                                                                 \
    const bool in = k0 + chunk_k + 8 <= k;                                                       \
    _Pragma("unroll") for (int c = 0; c < A_CHUNKS; ++c) a_stage[slot][c] = in ? load_chunk(a_src[c] + k0) : zero_chunk(); \
    _Pragma("unroll") for (int c = 0; c < B_CHUNKS; ++c) b_stage[slot][c] = in ? load_chunk(b_src[c] + k0) : zero_chunk(); \
  } while (0)
#define NNIS_STAGE(slot, buffer)                                                                 \
  do {                                                                                           \
    _Pragma("unroll") for (int c = 0; c < A_CHUNKS; ++c) a_tile[buffer][a_dst[c]] = a_stage[slot][c]; \
    _Pragma("unroll") for (int c = 0; c < B_CHUNKS; ++c) b_tile[buffer][b_dst[c]] = b_stage[slot][c]; \
  } while (0)

#pragma unroll
  for (int s = 0; s < PF; ++s)
    if (s < steps) NNIS_FETCH(s, s);
  NNIS_STAGE(0, 0);
  __syncthreads();
  for (int base = 0; base < steps; base += PF) {
#pragma unroll
    for (int j = 0; j < PF; ++j) {
      const int step = base + j;
      if (step < steps) {  // uniform over the block
        const int buffer = step & 1;
        // slot j went to LDS a step ago: refill it with the step PF ahead
        if (step + PF < steps) NNIS_FETCH(j, step + PF);
#pragma unroll
        for (int half = 0; half < 2; ++half) {  // two instructions of 32 k per stage
          bf16x8 a_frag[TM], b_frag[TN];
#pragma unroll
          for (int i = 0; i < TM; ++i) a_frag[i] = a_tile[buffer][swizzled(wave_m * WM + i * 16 + r, half * 4 + g)];
#pragma unroll
          for (int jj = 0; jj < TN; ++jj) b_frag[jj] = b_tile[buffer][swizzled(wave_n * WN + jj * 16 + r, half * 4 + g)];
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int jj = 0; jj < TN; ++jj) acc[i][jj] = mfma(b_frag[jj], a_frag[i], acc[i][jj]);
        }
        if (step + 1 < steps) NNIS_STAGE((j + 1) % PF, buffer ^ 1);
        __syncthreads();
      }
    }
  }
#undef NNIS_FETCH
#undef NNIS_STAGE

  // first operand = weight rows: lane holds D[n = 4g + e][token = r]
  const bool vector_ok = (n % 4) == 0;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int token = row0 + wave_m * WM + i * 16 + r;
    if (token >= m) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n0 = col0 + wave_n * WN + j * 16 + g * 4;
      const int valid = n - n0 >= 4 ? 4 : (n - n0 > 0 ? n - n0 : 0);
      if (valid > 0) store4<OutT>(y, (size_t)token * n + n0, acc[i][j], valid, vector_ok);
    }
  }
}

template <int MT, int KSPLIT, typename OutT>
void launch_skinny(const bf16_t* x, const bf16_t* w, OutT* y, int m, int n, int k, hipStream_t stream) {
  const int strips = (n + 15) / 16;
  const int waves = KSPLIT > 4 ? KSPLIT : 4;
  const int per_block = waves / KSPLIT;
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, KSPLIT, OutT>), dim3((strips + per_block - 1) / per_block),
                     dim3(64 * waves), 0, stream, x, w, y, m, n, k);
}

template <int MT, typename OutT>
void dispatch_skinny_split(const bf16_t* x, const bf16_t* w, OutT* y, int m, int n, int k, int split, hipStream_t stream) {
  if (split == 8) launch_skinny<MT, 8, OutT>(x, w, y, m, n, k, stream);
  else if (split == 4) launch_skinny<MT, 4, OutT>(x, w, y, m, n, k, stream);
  else if (split == 2) launch_skinny<MT, 2, OutT>(x, w, y, m, n, k, stream);
  else launch_skinny<MT, 1, OutT>(x, w, y, m, n, k, stream);
}

template <typename OutT>
void dispatch_skinny(const bf16_t* x, const bf16_t* w, OutT* y, int m, int n, int k, int split, hipStream_t stream) {
  const int tiles = (m + 15) / 16;
  if (tiles == 1) dispatch_skinny_split<1, OutT>(x, w, y, m, n, k, split, stream);
  else if (tiles == 2) dispatch_skinny_split<2, OutT>(x, w, y, m, n, k, split, stream);
  else if (tiles == 3) dispatch_skinny_split<3, OutT>(x, w, y, m, n, k, split, stream);
  else dispatch_skinny_split<4, OutT>(x, w, y, m, n, k, split, stream);
}

template <int BM, int BN, typename OutT>
void launch_tiled(const bf16_t* x, const bf16_t* w, OutT* y, int m, int n, int k, hipStream_t stream) {
  hipLaunchKernelGGL((gemm_tiled_kernel<BM, BN, OutT>), dim3((n + BN - 1) / BN, (m + BM - 1) / BM), dim3(256), 0, stream,
                     x, w, y, m, n, k);
}

template <typename OutT>
void dispatch_tiled(const bf16_t* x, const bf16_t* w, OutT* y, int m, int n, int k, int tile_hint, hipStream_t stream) {
  // the largest tile that still gives every compute unit a block or two
  const long long blocks_128 = (long long)((m + 127) / 128) * ((n + 127) / 128);
  const long long blocks_64_128 = (long long)((m + 63) / 64) * ((n + 127) / 128);
  int tile = blocks_128 >= 384 ? 1 : (blocks_64_128 >= 256 ? 2 : 3);
  if (tile_hint >= 1 && tile_hint <= 3) tile = tile_hint;  // for tuning runs
  if (tile == 1) launch_tiled<128, 128, OutT>(x, w, y, m, n, k, stream);
  else if (tile == 2) launch_tiled<64, 128, OutT>(x, w, y, m, n, k, stream);
  else launch_tiled<64, 64, OutT>(x, w, y, m, n, k, stream);
}

}  // namespace

// y_dtype: NNIS_BF16 or NNIS_F32.  Picks the skinny kernel for M <= 64.  split_hint: 0, or the number of
// waves (1, 2, 4, 8) that share a strip's K in the skinny kernel, overriding the choice made here.
extern "C" int nnis_gemm_bf16(const void* x, const void* w, void* y, int y_dtype, int m, int n, int k, int split_hint,
                              void* stream_ptr) {
  NNIS_REQUIRE(nnis_dtype_ok(y_dtype), "gemm_bf16: unknown output dtype %d", y_dtype);
  NNIS_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm_bf16: bad sizes m=%d n=%d k=%d", m, n, k);
  NNIS_REQUIRE(k % 8 == 0, "gemm_bf16: K=%d is not a multiple of 8 (16-byte loads); use the ordered kernel", k);
  NNIS_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0) && ((uintptr_t)y % 16 == 0),
               "gemm_bf16: operands must be 16-byte aligned");
  if (m == 0) return 0;
  hipStream_t stream = (hipStream_t)stream_ptr;
  const bf16_t* xp = (const bf16_t*)x;
  const bf16_t* wp = (const bf16_t*)w;
  if (m <= 64) {
    // With few strips the waves of a block share a strip's K, so that each wave's
    // share is one round of loads (4 steps of 64 for up to 32 tokens, 2 beyond);
    // with thousands of strips there are waves enough to hide the latency.
    const int strips = (n + 15) / 16;
    const int chunks = (k + 63) / 64;
    const int depth = m <= 32 ? 4 : 2;
    int split = 1;
    if (strips < 2048) {
      while (split < 8 && chunks > split * depth) split *= 2;
    }
    if (split_hint == 1 || split_hint == 2 || split_hint == 4 || split_hint == 8) split = split_hint;  // for tuning runs
    if (y_dtype == NNIS_F32) dispatch_skinny<float>(xp, wp, (float*)y, m, n, k, split, stream);
    else dispatch_skinny<bf16_t>(xp, wp, (bf16_t*)y, m, n, k, split, stream);
    NNIS_LAUNCH_CHECK("gemm_skinny");
  } else {
    NNIS_REQUIRE((m + 63) / 64 <= 65535, "gemm_bf16: %d rows exceed the grid limit", m);
    const int tile_hint = split_hint >= 16 ? split_hint / 16 : 0;  // hints of 16, 32, 48 pick the tile: 128x128, 64x128, 64x64
    if (y_dtype == NNIS_F32) dispatch_tiled<float>(xp, wp, (float*)y, m, n, k, tile_hint, stream);
    else dispatch_tiled<bf16_t>(xp, wp, (bf16_t*)y, m, n, k, tile_hint, stream);
    NNIS_LAUNCH_CHECK("gemm_tiled");
  }
  return 0;
}
