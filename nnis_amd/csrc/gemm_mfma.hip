// bfloat16 matrix products on the matrix cores: Y[M, N] = X[M, K] * W[N, K]^T,
// 32-bit accumulation, output bfloat16 or 32-bit.  K is contiguous in both
// operands, so a lane's 16-byte load is 8 consecutive k of one row, which is
// what v_mfma_f32_16x16x32_bf16 wants of either operand: lane l holds row
// (l % 16), k-group (l / 16) of 8.  The instruction sums over the 4 groups x 8
// elements; which k each (group, element) stands for is free as long as both
// operands agree.  Its result D[i][j] (i: row of the first operand, j: row of
// the second) lies with lane l as D[4 * (l / 16) + e][l % 16], e = 0..3.
//
//  * gemm_skinny_kernel: few tokens (decode; nnis_gemm_takes_few_tokens says
//    how many).  The weight is streamed from memory straight into operand
//    registers; a wave owns a strip of 16 weight rows; X (small, shared by all
//    waves) comes through the caches.  Waves of a block may split K and add
//    their parts through LDS.
//  * gemm_tiled_kernel: any M (prefill).  64x128 or 64x64 output tiles of 4
//    waves, or, where a product still fills the chip with them, 256x256 or
//    256x192 tiles of 8 waves; K in steps of 64 that go from memory straight
//    into LDS, a ring of stages deep, with an XOR swizzle of the 16-byte
//    chunks so that operand reads are free of bank conflicts.
//
// Both need K % 8 == 0 and 16-byte aligned operands (the host checks) and take
// any M and N.
#include "common.h"
#include "epilogue.h"

#include <type_traits>

#ifndef NNIS_FEW_TOKENS
#define NNIS_FEW_TOKENS 256
#endif

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ bf16x8 load_chunk(const bf16_t* p) { return *(const bf16x8*)p; }
// Weights that a kernel reads once and that are too large to be found in a cache by the next step: loaded past
// the caches' keeping.  Measured with 1 token, microseconds, plain against streamed: 25 MB 7.5 / 7.0, 67 MB 14.4 /
// 13.6, 201 MB 39.9 / 36.5; but 8.4 MB 3.9 / 4.4 and 1.8 MB 3.2 / 3.6, hence the limit.
constexpr size_t kStreamWeightBytes = 16u << 20;
__device__ __forceinline__ bf16x8 load_stream(const bf16_t* p) { return __builtin_nontemporal_load((const bf16x8*)p); }

__device__ __forceinline__ bf16x8 zero_chunk() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

__device__ __forceinline__ f32x4 mfma(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ void store4(float* y, size_t index, f32x4 v, int valid, bool vector_ok) {
  if (valid == 4 && vector_ok) {
    *(f32x4*)(y + index) = v;
  } else {
    for (int e = 0; e < valid; ++e) y[index + e] = v[e];
  }
}

__device__ __forceinline__ void store4(bf16_t* y, size_t index, f32x4 v, int valid, bool vector_ok) {
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
// Weights up to this size stay in the dies' L2 over a kernel: reading them again costs little
constexpr size_t kRereadWeightBytes = 8u << 20;
constexpr int kFewTokens = NNIS_FEW_TOKENS;

// What a projection that ends a part of a pre-norm block does with its result instead of storing it
// (OutT = ResidualOut): the residual stream takes it in, and the norm that follows is prepared.
//   v = resid + y (32-bit, in place);  scaled = bf16(v * gain);  ss[part][token] = sum over the part's
//   columns of v * v.  The norm's 1 / sqrt(mean + eps) is left to the kernel that reads `scaled`: it needs
//   the whole row, and the parts of a row are spread over the blocks.  Statistics as in
//   /root/reference/crates/nnis-model/src/kernels.rs:15-48.
struct ResidualOut {
  float* resid;      // [m, n]
  const void* gain;  // [n], the following norm's weight
  int gain_dtype;
  bf16_t* scaled;    // [m, n]
  float* ss;         // [parts, m]; a part is 16 columns (skinny kernel) or a wave's columns (tiled kernel)
};

// four consecutive columns of a token: what the stream and the gain hold there, asked for early.  A gain in
// bfloat16 stays as it was loaded (two words in g) until it is taken: arithmetic on it here would make the
// kernel wait for the load before its main loop.
struct ResidualHeld {
  f32x4 v, g;
};

__device__ __forceinline__ ResidualHeld residual_ask(const ResidualOut& o, size_t index, int column, int valid, bool vector_ok) {
  ResidualHeld h;
  h.v = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
  h.g = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
  if (valid == 4 && vector_ok) {
    h.v = *(const f32x4*)(o.resid + index);
    if (o.gain_dtype == NNIS_F32) {
      h.g = *(const f32x4*)((const float*)o.gain + column);
    } else {
      const float2 packed = *(const float2*)((const bf16_t*)o.gain + column);
      h.g[0] = packed.x;
      h.g[1] = packed.y;
    }
  } else {
    for (int e = 0; e < valid; ++e) {
      h.v[e] = o.resid[index + e];
      h.g[e] = load_as_f32(o.gain, o.gain_dtype, column + e);
    }
  }
  return h;
}

// ... and the lane's accumulator acc taken in; returns the lane's part of the row's sum of squares
__device__ __forceinline__ float residual_take(const ResidualOut& o, const ResidualHeld& h, size_t index, f32x4 acc, int valid,
                                               bool vector_ok) {
  typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
  float sq = 0.0f;
  f32x4 v = h.v, gain = h.g;
  if (valid == 4 && vector_ok && o.gain_dtype != NNIS_F32) {  // four bfloat16 in two words: a float's upper half each
    const unsigned lo = __float_as_uint(h.g[0]), hi = __float_as_uint(h.g[1]);
    gain[0] = __uint_as_float(lo << 16);
    gain[1] = __uint_as_float(lo & 0xffff0000u);
    gain[2] = __uint_as_float(hi << 16);
    gain[3] = __uint_as_float(hi & 0xffff0000u);
  }
  bf16x4 scaled;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    v[e] += acc[e];
    if (e < valid) sq = fmaf(v[e], v[e], sq);
    scaled[e] = (__bf16)(v[e] * gain[e]);
  }
  if (valid == 4 && vector_ok) {
    *(f32x4*)(o.resid + index) = v;
    *(bf16x4*)(o.scaled + index) = scaled;
  } else {
    for (int e = 0; e < valid; ++e) {
      o.resid[index + e] = v[e];
      o.scaled[index + e] = scaled[e];
    }
  }
  return sq;
}

// What the tiled kernel does for a projection that starts a part of a pre-norm block (OutT = ScaledOut<EPI>):
// its operand is the `scaled` that a ResidualOut left, the row's 1 / sqrt(mean of squares + eps) is taken
// from the parts of ss and applied to the product, then the epilogue stores, gates or rotates.  For the
// two epilogues that need pairs of weight rows in one lane (gate and up of the same channels; the two
// halves of a head that rotate into each other), the tile's strips of 16 weight rows alternate between the
// two: strips 2u and 2u+1 of a wave are the lower and upper rows of pair unit u.
template <int EPI>
struct ScaledOut {
  bf16_t* y;  // store: [m, n]; silu: [m, n / 2]; rope: the queries (= rope.q_out)
  const float* ss_parts;  // [parts, m]
  int parts;
  float eps;
  RopeTarget rope;
};
template <typename T> struct scaled_epilogue { static constexpr int value = -1; };
template <int EPI> struct scaled_epilogue<ScaledOut<EPI>> { static constexpr int value = EPI; };

// the weight row that strip row `tile_row` (0 .. BN-1) of column block `block` multiplies; -1 beyond the end
template <int EPI, int BN, int WGN = 2>
__device__ __forceinline__ int paired_weight_row(const RopeTarget& rope, int block, int tile_row, int n) {
  constexpr int WN = BN / WGN;
  const int wave_n = tile_row / WN, strip = (tile_row % WN) / 16, rr = tile_row % 16;
  const int unit = block * (BN / 32) + wave_n * (WN / 32) + strip / 2;
  const bool upper = strip % 2;
  if (EPI == EPI_SILU) {
    const int inner = n / 2, channel = unit * 16 + rr;
    return channel < inner ? (upper ? inner : 0) + channel : -1;
  }
  const int per_head = rope.head_dim / 32;
  if (unit >= (rope.heads + 2 * rope.kv_heads) * per_head) return -1;
  return (unit / per_head) * rope.head_dim + (unit % per_head) * 16 + rr + (upper ? rope.head_dim / 2 : 0);
}

// The activations as the decode attention leaves them when it cuts a sequence's keys into runs: per (token,
// head, run) head_dim outputs, the run's softmax reference (a power of two's exponent) and its sum, in rows of
// head_dim + 4 floats.  x[token][head * head_dim + d] = sum_s O_s[d] 2^(m_s - M) / sum_s l_s 2^(m_s - M), M the
// largest m_s: what attention_combine_kernel computes, term by term in the same order.
struct RunsIn {
  const float* partial;  // [tokens, heads, runs, head_dim + 4]
  const int* tok_slot;   // [tokens]; a negative slot is a padding row: its activations count as zeros
  int runs, heads, head_dim;
};
constexpr int kMostRuns = 8;

extern __shared__ __align__(16) char skinny_lds[];  // RUNS: the block's activations, [16 * MT][k + 8] bfloat16

// The block's threads make the activations of `tokens` tokens from token0 on, [tokens][k] in rows of x_row
// elements at x_tile, from up to MOST runs.  A thread's loads of two items (4 channels of a token each) are
// asked for together, before any is used; a run beyond the last reads the last again and counts for nothing.
template <int MOST>
__device__ __forceinline__ void make_activations(const RunsIn& runs, bf16_t* x_tile, int x_row, int token0, int tokens, int k) {
  typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
  typedef __attribute__((ext_vector_type(2))) float f32x2;
  const int groups = k / 4, row_floats = runs.head_dim + 4;
  const int items = tokens > 0 ? tokens * groups : 0;
  constexpr int kTogether = 2;
  for (int first = threadIdx.x; first < items; first += kTogether * blockDim.x) {
    f32x2 state[kTogether][MOST];  // a run's reference and sum
    f32x4 out[kTogether][MOST];
    bool live[kTogether];
#pragma unroll
    for (int i = 0; i < kTogether; ++i) {
      int item = first + i * blockDim.x;
      item = item < items ? item : items - 1;  // (the last again: stored twice, the same)
      const int local = item / groups, channel = (item % groups) * 4;
      const int token = token0 + local;
      live[i] = runs.tok_slot[token] >= 0;
      const int head = channel / runs.head_dim, d = channel % runs.head_dim;
      const float* base = runs.partial + ((size_t)token * runs.heads + head) * runs.runs * row_floats;
#pragma unroll
      for (int s = 0; s < MOST; ++s) {
        const float* p = base + (size_t)(s < runs.runs ? s : runs.runs - 1) * row_floats;
        state[i][s] = *(const f32x2*)(p + runs.head_dim);
        out[i][s] = *(const f32x4*)(p + d);
      }
    }
#pragma unroll
    for (int i = 0; i < kTogether; ++i) {
      int item = first + i * blockDim.x;
      item = item < items ? item : items - 1;
      const int local = item / groups, channel = (item % groups) * 4;
      float top = -INFINITY;
#pragma unroll
      for (int s = 0; s < MOST; ++s) top = s < runs.runs ? fmaxf(top, state[i][s][0]) : top;
      f32x4 num = {0.0f, 0.0f, 0.0f, 0.0f};
      float den = 0.0f;
#pragma unroll
      for (int s = 0; s < MOST; ++s) {
        if (s < runs.runs) {
          const float weight = state[i][s][0] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(state[i][s][0] - top);
          num += out[i][s] * weight;
          den += state[i][s][1] * weight;
        }
      }
      bf16x4 made;
#pragma unroll
      for (int e = 0; e < 4; ++e) made[e] = live[i] ? (__bf16)(num[e] / den) : (__bf16)0.0f;  // a padding row: zeros
      *(bf16x4*)(x_tile + (size_t)local * x_row + channel) = made;
    }
  }
}

// RUNS: x is not read but made, by the block for its 16 * MT tokens, from `runs` into LDS (every block makes
// the same few KB again: cheaper than a kernel of its own between the attention and this projection).
// PAIR: two blocks share a strip's K (block 2 s takes the even shares, 2 s + 1 the odd ones).  Each leaves its sums
// in `pair.sums`; the one that finds the other's already there (a count per strip in `pair.count`, which it sets
// back to zero) adds them to its own and ends the strip.  Nobody waits for anybody.  For strips so few that they
// leave half the chip without a block, on a K long enough that a compute unit's own rate of reading bounds the kernel.
struct PairScratch {
  float* sums;  // [strips][2][MT][64 lanes][4]
  int* count;   // [strips], zero between calls
};

template <int MT, int KSPLIT, bool RUNS, typename OutT, bool PAIR = false>
__global__ __launch_bounds__(KSPLIT > 4 ? 64 * KSPLIT : 256) void gemm_skinny_kernel(const bf16_t* __restrict__ x,
                                                                                   const bf16_t* __restrict__ w,
                                                                                   OutT y, int m, int n, int k, int tiles,
                                                                                   int stream_weights, RunsIn runs,
                                                                                   PairScratch pair) {
  constexpr int kWaves = KSPLIT > 4 ? KSPLIT : 4;
  constexpr int kStrips = kWaves / KSPLIT;  // strips of 16 weight rows per block
  constexpr int kShares = PAIR ? 2 * KSPLIT : KSPLIT;  // waves that share a strip's K
  static_assert(!PAIR || (!RUNS && kStrips == 1), "paired blocks: one strip a block, activations from memory");
  constexpr int DEPTH = MT <= 2 ? 4 : 2;
  __shared__ float partial[KSPLIT > 1 ? kWaves : 1][MT][kWave][4];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  int strip_block, tile;
  if constexpr (PAIR) {
    strip_block = blockIdx.x / 2;  // (one tile of tokens)
    tile = 0;
  } else {
    nnis_deal_tiles(blockIdx.x, tiles, strip_block, tile);
  }
  const int strip = strip_block * kStrips + wave / KSPLIT;
  const int token0 = tile * 16 * MT;  // this block's tokens: token0 + (0 .. 16 * MT - 1)
  const int x_row = k + 8;  // elements of a row of the activations in LDS: 16 rows apart fall into different banks
  const int part = wave % KSPLIT;
  const int share = PAIR ? 2 * part + (int)(blockIdx.x % 2) : part;  // this wave's place among those that share the strip's K
  const int r = lane % 16, g = lane / 16;
  const int strips = (n + 15) / 16;
  const bool active = strip < strips;

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};

  // lane holds D[weight row 4g + e][token r]: four consecutive outputs of one token
  const int n0 = strip * 16 + g * 4;
  const int valid = n - n0 >= 4 ? 4 : (n - n0 > 0 ? n - n0 : 0);
  const bool vector_ok = (n % 4) == 0;
  constexpr bool kResidual = std::is_same<OutT, ResidualOut>::value;
  ResidualHeld held[kResidual ? MT : 1];
  if constexpr (kResidual) {
    if (active && part == 0) {  // the wave that ends the strip asks for the stream before its weights
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int token = token0 + t * 16 + r;
        held[t] = residual_ask(y, (size_t)(token < m ? token : 0) * n + n0, n0, (token < m) ? valid : 0, vector_ok);
      }
    }
  }

  const int chunks = nnis_packed_chunks(k);
  // packed weights: the strip's padding rows and the last chunk's padding are zeros that are there to read
  const bf16_t* w_ptr = w + nnis_packed_lane(active ? strip * 16 + r : 0, g, k);
  // a round: DEPTH steps of 64 k of this wave (base, base + kShares, ..): their weights ...
  auto ask_weights = [&](int base, bf16x8 (&wa)[DEPTH], bf16x8 (&wb)[DEPTH]) {
    if (stream_weights) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int c = base + d * kShares;
        wa[d] = c < chunks ? load_stream(w_ptr + (size_t)c * kPackedChunkElems) : zero_chunk();  // zeros for steps beyond the last
        wb[d] = c < chunks ? load_stream(w_ptr + (size_t)c * kPackedChunkElems + kPackedHalfElems) : zero_chunk();
      }
    } else {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int c = base + d * kShares;
        wa[d] = c < chunks ? load_chunk(w_ptr + (size_t)c * kPackedChunkElems) : zero_chunk();
        wb[d] = c < chunks ? load_chunk(w_ptr + (size_t)c * kPackedChunkElems + kPackedHalfElems) : zero_chunk();
      }
    }
  };
  const bf16_t* x_ptr[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    int token = token0 + t * 16 + r;
    token = token < m ? token : m - 1;
    x_ptr[t] = x + (size_t)token * k;
  }
  auto load_x = [&](int t, int kk) -> bf16x8 {
    if constexpr (RUNS) return *(const bf16x8*)(skinny_lds + ((size_t)(t * 16 + r) * x_row + kk) * sizeof(bf16_t));
    else return load_chunk(x_ptr[t] + kk);
  };
  // ... and their activations and products
  auto multiply = [&](int base, const bf16x8 (&wa)[DEPTH], const bf16x8 (&wb)[DEPTH]) {
    bf16x8 xa[DEPTH][MT], xb[DEPTH][MT];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int ka = (base + d * kShares) * 64 + g * 16, kb = ka + 8;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        xa[d][t] = ka + 8 <= k ? load_x(t, ka) : zero_chunk();
        xb[d][t] = kb + 8 <= k ? load_x(t, kb) : zero_chunk();
      }
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        acc[t] = mfma(wa[d], xa[d][t], acc[t]);
        acc[t] = mfma(wb[d], xb[d][t], acc[t]);
      }
  };
  int base = share;
  if constexpr (RUNS) {
    // the first round's weights are asked for before the block makes its activations: the two latencies overlap
    bf16x8 wa[DEPTH], wb[DEPTH];
    if (active && base < chunks) ask_weights(base, wa, wb);
    const int tokens_here = min(16 * MT, m - token0);  // rows beyond them are never multiplied into a stored result
    if (runs.runs <= 4) make_activations<4>(runs, (bf16_t*)skinny_lds, x_row, token0, tokens_here, k);
    else make_activations<kMostRuns>(runs, (bf16_t*)skinny_lds, x_row, token0, tokens_here, k);
    __syncthreads();
    if (active && base < chunks) {
      multiply(base, wa, wb);
      base += kShares * DEPTH;
    }
  }
  if (active) {
    for (; base < chunks; base += kShares * DEPTH) {
      bf16x8 wa[DEPTH], wb[DEPTH];
      ask_weights(base, wa, wb);
      multiply(base, wa, wb);
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
  if constexpr (PAIR) {
    // (one wave of the block is left.)  The sums go out past the caches, are waited for, and then the count:
    // who finds it at one has the other block's sums in memory.  All of it with relaxed order at agent scope,
    // which rests on three facts of this chip and not on the language's memory model: (1) a wave's stores are
    // counted by vmcnt, and `s_waitcnt vmcnt(0)` below ends only when they have been written where agent-scope
    // accesses see them; (2) atomic loads and stores at agent scope go past the dies' own L2 (each die has
    // one), so the second block reads what the first wrote and not a line its die had kept; (3) a wave issues
    // no load before the branch it stands behind is decided, so the sums are not read before the count.  The
    // same with a release on the count and an acquire fence for the second block (the compiler then writes
    // back and invalidates the L2 around them) was measured: 2048 x 5632 at 1 / 8 / 16 tokens 7.8 / 8.3 / 9.7
    // -> 10.1 / 10.4 / 12.0 us, 2048 x 8192 9.7 / 10.2 / 11.7 -> 12.4 / 13.3 / 15.2: more than the second
    // block gains.  The asm statements keep the compiler from moving memory accesses across them.
    float* mine = pair.sums + ((size_t)strip * 2 + blockIdx.x % 2) * (MT * kWave * 4);
    const float* theirs = pair.sums + ((size_t)strip * 2 + 1 - blockIdx.x % 2) * (MT * kWave * 4);
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        __hip_atomic_store(mine + (t * kWave + lane) * 4 + e, acc[t][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    int before = 0;
    if (lane == 0) before = __hip_atomic_fetch_add(pair.count + strip, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    before = __builtin_amdgcn_readfirstlane(before);
    asm volatile("" ::: "memory");
    if (before == 0) return;  // the first of the two: the other ends the strip
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        acc[t][e] += __hip_atomic_load(theirs + (t * kWave + lane) * 4 + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (lane == 0) __hip_atomic_store(pair.count + strip, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int token = token0 + t * 16 + r;
    if constexpr (kResidual) {
      float sq = 0.0f;
      if (token < m && valid > 0) sq = residual_take(y, held[t], (size_t)token * n + n0, acc[t], valid, vector_ok);
      sq += __shfl_xor(sq, 16, kWave);
      sq += __shfl_xor(sq, 32, kWave);
      if (g == 0 && token < m) y.ss[(size_t)strip * m + token] = sq;
    } else {
      if (token < m && valid > 0) store4(y, (size_t)token * n + n0, acc[t], valid, vector_ok);
    }
  }
}

// -----------------------------------------------------------------------------
// tiled: BM x BN output tile per block of 4 waves (2 x 2), K in steps of BK = 64.  The operands go from
// memory straight into LDS (no registers between), a ring of NS stages deep.  Measured on products from
// 2048 x 576 x 576 to 2048 x 6144 x 2048, in place of loads through registers: 10 to 17% less time; steps of
// 32 k, and frags of the next step read before the barrier, were slower; tiles of 128 x 256 and 256 x 256
// with 8 waves gain only where they still make 500 blocks and more.
// -----------------------------------------------------------------------------
// chunk c of row `row` of a staged tile (CHUNKS chunks of 16 bytes a row) lives at chunk c ^ (row % CHUNKS)
template <int CHUNKS>
__device__ __forceinline__ int swizzled(int row, int chunk) { return row * CHUNKS + (chunk ^ (row & (CHUNKS - 1))); }

typedef __attribute__((address_space(1))) const void* global_ptr_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;
// The loads into LDS are not the compiler's to wait for: the kernel counts them itself.
template <int N>
__device__ __forceinline__ void wait_loads_but() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

extern __shared__ __align__(16) char tile_lds[];  // NS stages of BM + BN rows of BK

#ifndef NNIS_TILE_GROUP_ROWS
#define NNIS_TILE_GROUP_ROWS 512
#endif
#ifndef NNIS_LARGE_TILE_GROUP_ROWS
#define NNIS_LARGE_TILE_GROUP_ROWS 512  // (2048, every row block of a 2,048-token product with a column block: no faster)
#endif
// NS stages: 2 for the 64 x 128 tile where the grid gives a compute unit three blocks and more (48 KB of LDS a
// block instead of 72: three fit, and 2048 x 3072 x 576 takes 15.3 us instead of 17.5, 2048 x 6144 x 2048 68.5
// instead of 75); 3 where a compute unit runs fewer; 6 where the grid leaves it one block at most and K is
// long, so that the loads in flight are all that hides the memory's latency (64 tokens x 11264 x 2048: 20.9 us
// with 3, 19.7 with 6; a K of 9 steps in 256 blocks took 13.4 us with 6 against 11.7)
// SPLIT: K is cut into ksplit parts, a block leaves its part's sums in `partial` and gemm_reduce_kernel does the
// rest (a variant of its own, so that the other has no branch around the loads that prepare its epilogue).
// WGM x WGN: the block's waves, each with BM / WGM rows and BN / WGN columns of the tile.  2 x 2 for the tiles of 64
// rows; 4 x 2 for the tile of 256 x 256, which a product takes when it still gives most compute units a block: a
// step of such a tile brings 64 KB from L2 for 8.4 MFLOP where four tiles of 64 x 128 bring 96 KB for 2.1 (measured
// on 2048 x 16384 x 2048: 117 us against 171; 2048 x 6144 x 2048: 57 against 68; 6224 x 2048 x 8192: 188 against 308).
template <int BM, int BN, int BK, int NS, bool SPLIT, typename OutT, int WGM = 2, int WGN = 2>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_tiled_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                    OutT y, int m, int n, int k, int col_blocks, int ksplit,
                                                                    float* __restrict__ partial) {
  constexpr int W = WGM * WGN;
  constexpr int WM = BM / WGM, WN = BN / WGN;  // a wave's part of the tile
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int CH = BK / 8;  // 16-byte chunks per staged row
  static_assert(CH == 8, "a load instruction of a wave fills 8 rows of 8 chunks");
  // One load instruction of a wave moves 64 x 16 bytes into 1 KB of LDS that is contiguous.  Of the activations
  // that is 8 rows of a stage, lane l to row l / 8, place l % 8; the swizzle is made on the way in by the
  // choice of the source: place p of row r holds chunk p ^ (r % 8).
  constexpr int A_LOADS = BM / (8 * W), B_LOADS = BN / (8 * W);  // a wave's load instructions per step (8 rows each)
  static_assert(A_LOADS * 8 * W == BM && B_LOADS * 8 * W == BN && (64 * W) % BM == 0, "the tile must divide among the waves");
  constexpr int LOADS = A_LOADS + B_LOADS;
  constexpr int A_BYTES = BM * BK * 2, STAGE_BYTES = (BM + BN) * BK * 2;

  const int tid = threadIdx.x;
  const int wave = tid / kWave, lane = tid % kWave;
  const int wave_m = wave / WGN, wave_n = wave % WGN;
  const int r = lane % 16, g = lane / 16;
  // Blocks go to the chip's 8 dies in turn (block i to die i % 8), and each die has an L2 of its own: the
  // tiles are dealt so that a die's blocks cover a band of consecutive rows of X with all their column
  // blocks, and each die reads its band once instead of every die reading all of X.
  // With ksplit > 1 the grid holds every tile ksplit times, part p of K for each (tiles of a part together).
  int col_block, row_block, part;
  {
    const int total = gridDim.x, die = blockIdx.x % 8, nth = blockIdx.x / 8;
    const int each = total / 8, more = total % 8;  // the first `more` dies have one block more
    const int item = die * each + (die < more ? die : more) + nth;
    const int tiles = total / ksplit;
    part = item / tiles;
    const int tile = item % tiles;
    // within the order of the tiles, kGroup row blocks go through the column blocks together, rows fastest:
    // a column block of W serves them all while it is near
    constexpr int kGroup = (BM >= 256 ? NNIS_LARGE_TILE_GROUP_ROWS : NNIS_TILE_GROUP_ROWS) / BM;
    const int row_blocks = tiles / col_blocks;
    const int group = tile / (kGroup * col_blocks), within = tile % (kGroup * col_blocks);
    const int rows_here = min(kGroup, row_blocks - group * kGroup);
    row_block = group * kGroup + within % rows_here;
    col_block = within / rows_here;
  }
  const int row0 = row_block * BM, col0 = col_block * BN;

  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};

  // what this lane loads: its chunk (the same for every load: rows 8 apart) of rows 8 (W o + wave) + lane / 8
  const bf16_t* a_src[A_LOADS];
  const bf16_t* b_src[B_LOADS];
  const int chunk_k = ((lane % 8) ^ (lane / 8)) * 8;
#pragma unroll
  for (int o = 0; o < A_LOADS; ++o) {
    int row = row0 + (o * W + wave) * 8 + lane / 8;
    row = row < m ? row : m - 1;
    a_src[o] = x + (size_t)row * k + chunk_k;
  }
  constexpr int EPI = scaled_epilogue<OutT>::value;  // -1: the product is stored or added as it is
  constexpr bool kPaired = EPI == EPI_SILU || EPI == EPI_ROPE;
  // The weights are packed in the order the matrix instruction takes them: a load instruction copies one half of
  // a strip's chunk (1 KB, lane l's 16 bytes to place l) and the stage holds [strip of the tile][half][lane].
  const int chunks = nnis_packed_chunks(k);
#pragma unroll
  for (int o = 0; o < B_LOADS; ++o) {
    const int piece = o * W + wave;  // (strip of the tile, half)
    const int tile_row = (piece / 2) * 16 + r;
    int row;
    if constexpr (kPaired) {
      row = paired_weight_row<EPI, BN, WGN>(y.rope, col_block, tile_row, n);
      row = row >= 0 ? row : 0;  // rows beyond the end read a valid row and are not stored
    } else {
      row = col0 + tile_row;
      row = row < n ? row : n - 1;
    }
    b_src[o] = w + nnis_packed_lane(row, g, k) + (piece % 2) * kPackedHalfElems;
  }
  // Step s lies in stage s % NS.  A step first asks for the step NS - 1 ahead, into the
  // stage that was read a step ago (every wave is past the barrier that ended that step, and what it read
  // there its matrix instructions have taken); then multiplies its own stage; then waits until all but the
  // newest NS - 2 steps' loads of this wave have arrived (loads arrive in the order they were
  // asked for), and for the other waves' at the barrier.  A step beyond the end of K is asked for all the
  // same, so that the count holds: from the row's last whole chunk, a valid address, and nobody reads it.
  // In the last step of a K that is no multiple of BK the same holds for the activations' chunks beyond K;
  // they meet the zeros that pad the packed weights' last chunk (finite times zero: the row's own last values).
  const int steps = (k + BK - 1) / BK;
  const int steps_a_part = (steps + ksplit - 1) / ksplit;
  const int step0 = part * steps_a_part;  // this block multiplies steps step0 .. step1 - 1 (none, for a part beyond the end)
  const int step1 = step0 + steps_a_part < steps ? step0 + steps_a_part : steps;
  int last_chunk = k - 8 - chunk_k;  // offset of the row's last whole chunk from this lane's first
  last_chunk = last_chunk > -chunk_k ? last_chunk : -chunk_k;
  auto ask = [&](int step, int stage) {
    char* base = tile_lds + stage * STAGE_BYTES + wave * 1024;
    const int k0 = step * BK;
    const int from = k0 <= last_chunk ? k0 : last_chunk;
#pragma unroll
    for (int o = 0; o < A_LOADS; ++o)
      __builtin_amdgcn_global_load_lds((global_ptr_t)(a_src[o] + from), (lds_ptr_t)(base + o * W * 1024), 16, 0, 0);
    const size_t from_chunk = (size_t)(step < chunks ? step : chunks - 1) * kPackedChunkElems;
#pragma unroll
    for (int o = 0; o < B_LOADS; ++o)
      __builtin_amdgcn_global_load_lds((global_ptr_t)(b_src[o] + from_chunk), (lds_ptr_t)(base + A_BYTES + o * W * 1024), 16, 0, 0);
  };

#pragma unroll
  for (int s = 0; s < NS - 1; ++s) ask(step0 + s, s);

  // Behind the first steps' loads, so that one wait covers both: a prepared operand's row scales, for the
  // epilogue, and what the rotation needs of each token
  constexpr int PG = 64 * W / BM;  // threads a row of the tile has for the parts of its sum of squares
  __shared__ float row_scale[EPI >= 0 ? PG : 1][EPI >= 0 ? BM : 1];  // each thread's share of a row's sum of squares
  int tok_pos[TM], tok_page[TM];
  if constexpr (EPI >= 0 && !SPLIT) {  // (with K in parts the reduce kernel does this)
    // a thread takes the parts pg, pg + PG, .. of its row: eight loads at a time, none waiting for another
    const int tile_row = tid % BM, pg = tid / BM;
    const int token = row0 + tile_row < m ? row0 + tile_row : m - 1;
    float total = 0.0f;
    if (y.parts <= 8 * PG) {
      for (int p0 = pg; p0 < y.parts; p0 += 8 * PG) {
        float part[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int p = p0 + PG * u;
          part[u] = y.ss_parts[(size_t)(p < y.parts ? p : y.parts - 1) * m + token];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) total += p0 + PG * u < y.parts ? part[u] : 0.0f;
      }
    } else {  // a wide row that the kernel for few tokens prepared (a part per 16 columns): 32 loads at a time
      for (int p0 = pg; p0 < y.parts; p0 += 32 * PG) {
        float part[32];
#pragma unroll
        for (int u = 0; u < 32; ++u) {
          const int p = p0 + PG * u;
          part[u] = y.ss_parts[(size_t)(p < y.parts ? p : y.parts - 1) * m + token];
        }
#pragma unroll
        for (int u = 0; u < 32; ++u) total += p0 + PG * u < y.parts ? part[u] : 0.0f;
      }
    }
    row_scale[pg][tile_row] = total;
    if constexpr (EPI == EPI_ROPE) {
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        int token = row0 + wave_m * WM + i * 16 + r;
        token = token < m ? token : m - 1;
        const int slot = y.rope.tok_page ? 0 : y.rope.tok_slot[token];
        tok_pos[i] = y.rope.tok_pos[token];
        tok_page[i] = rope_page(y.rope, token, slot, tok_pos[i]);
      }
    }
  }

  // a residual epilogue asks for the stream and the gain before the product (small tiles: registers)
  constexpr bool kResidual = std::is_same<OutT, ResidualOut>::value;
  constexpr bool kAskEarly = kResidual && TM * TN <= 8;
  ResidualHeld held[kAskEarly ? TM : 1][kAskEarly ? TN : 1];
  if constexpr (kAskEarly && !SPLIT) {
    const bool vector_ok = (n % 4) == 0;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int token = row0 + wave_m * WM + i * 16 + r;
        const int n0 = col0 + wave_n * WN + j * 16 + g * 4;
        const int valid = (token < m) ? (n - n0 >= 4 ? 4 : (n - n0 > 0 ? n - n0 : 0)) : 0;
        held[i][j] = residual_ask(y, (size_t)(token < m ? token : 0) * n + (valid > 0 ? n0 : 0), valid > 0 ? n0 : 0, valid, vector_ok);
      }
  }

  wait_loads_but<(NS - 2) * LOADS>();
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  int stage = 0;
  // One block of 8 waves a compute unit (the tiles of 128 and 256 x 128): the two waves of a SIMD leave a step's barrier
  // together, and with reads first and products after, the matrix unit would wait at the head of every step.  So a
  // step's second half is multiplied after the barrier, while the next step's first half is read, and its first
  // half before it, while the second is read: the operands of a half are in registers one barrier ahead.  Every
  // read of a stage is still waited for before the barrier that lets the stage be filled again, and a sum takes
  // its halves in the same order as before.
  constexpr bool kCarry = TM * TN <= 16 && W == 8;
  if constexpr (kCarry) {
    static_assert(BK == 64, "two halves of 32 k a step");
    bf16x8 a0[TM], b0[TN], a1[TM], b1[TN];
    auto read_half = [&](int from, int half, bf16x8 (&a)[TM], bf16x8 (&b)[TN]) {
      const bf16x8* a_tile = (const bf16x8*)(tile_lds + from * STAGE_BYTES);
      const bf16x8* b_tile = (const bf16x8*)(tile_lds + from * STAGE_BYTES + A_BYTES);
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = a_tile[swizzled<CH>(wave_m * WM + i * 16 + r, g * 2 + half)];
#pragma unroll
      for (int jj = 0; jj < TN; ++jj) b[jj] = b_tile[((wave_n * TN + jj) * 2 + half) * kWave + lane];
    };
    auto multiply = [&](const bf16x8 (&a)[TM], const bf16x8 (&b)[TN]) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int jj = 0; jj < TN; ++jj) acc[i][jj] = mfma(b[jj], a[i], acc[i][jj]);
    };
    // for the scheduler: a read behind each of the first products, then the rest of the products
    auto interleave = [&]() {
#pragma unroll
      for (int n = 0; n < TM + TN; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - (TM + TN), 0);
    };
    static_assert(TM * TN >= TM + TN, "a product for every read");
    if (step0 < step1) read_half(0, 0, a0, b0);
    for (int step = step0; step < step1; ++step) {
      ask(step + NS - 1, stage == 0 ? NS - 1 : stage - 1);
      read_half(stage, 1, a1, b1);
      multiply(a0, b0);
      interleave();
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      wait_loads_but<(NS - 2) * LOADS>();
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("" ::: "memory");
      stage = stage + 1 == NS ? 0 : stage + 1;
      read_half(stage, 0, a0, b0);  // (after the last step: of a stage that nobody multiplies; no branch in the loop's body)
      multiply(a1, b1);
      interleave();
    }
  } else {
  for (int step = step0; step < step1; ++step) {
    // The tile of 256 x 256 asks for the next step between its two halves, under the first half's products
    // (2048 x 16384 x 2048 137 us against 141, 6224 x 11264 x 2048 277 against 294); the tile of 256 x 192, whose
    // steps are shorter, loses by the later start of its loads (2048 x 11264 x 2048 105 against 95).
    constexpr bool kAskBetween = TM * TN > 16 && BN >= 256;
    if constexpr (!kAskBetween) ask(step + NS - 1, stage == 0 ? NS - 1 : stage - 1);
    const bf16x8* a_tile = (const bf16x8*)(tile_lds + stage * STAGE_BYTES);
    const bf16x8* b_tile = (const bf16x8*)(tile_lds + stage * STAGE_BYTES + A_BYTES);
    static_assert(BK == 64, "two halves of 32 k a step");
    if constexpr (TM * TN <= 16) {
      bf16x8 a_frag[2][TM], b_frag[2][TN];  // an instruction takes 32 k: the operands of both halves of the step
#pragma unroll
      for (int half = 0; half < 2; ++half) {
#pragma unroll
        for (int i = 0; i < TM; ++i) a_frag[half][i] = a_tile[swizzled<CH>(wave_m * WM + i * 16 + r, g * 2 + half)];  // k as the weights are packed
#pragma unroll
        for (int jj = 0; jj < TN; ++jj) b_frag[half][jj] = b_tile[((wave_n * TN + jj) * 2 + half) * kWave + lane];
      }
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int jj = 0; jj < TN; ++jj) acc[i][jj] = mfma(b_frag[half][jj], a_frag[half][i], acc[i][jj]);
      // the order for the compiler's scheduler: the first half's reads, then the first half's products each with a read of
      // the second half behind it, then the rest of the products -- so that no wave waits for all its reads before it multiplies
      __builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0);
#pragma unroll
      for (int n = 0; n < TM + TN; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 2 * TM * TN - (TM + TN), 0);
    } else {
      // a wave tile of 64 x 128: the operands of one half at a time (registers); the other wave of the SIMD
      // multiplies while this one reads.  (The reads of a half spread between its products, each two groups of
      // four products ahead of its use, by scheduling barriers: 136 us against 139 on 2048 x 16384 x 2048.)
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        bf16x8 a_frag[TM], b_frag[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) a_frag[i] = a_tile[swizzled<CH>(wave_m * WM + i * 16 + r, g * 2 + half)];
#pragma unroll
        for (int jj = 0; jj < TN; ++jj) b_frag[jj] = b_tile[((wave_n * TN + jj) * 2 + half) * kWave + lane];
#pragma unroll
        for (int jj = 0; jj < TN; ++jj)
#pragma unroll
          for (int i = 0; i < TM; ++i) acc[i][jj] = mfma(b_frag[jj], a_frag[i], acc[i][jj]);
        if constexpr (kAskBetween) {
          if (half == 0) ask(step + NS - 1, stage == 0 ? NS - 1 : stage - 1);
        }
      }
    }
    // what this wave read of its stage has arrived too: the stage is the next step's to fill
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    wait_loads_but<(NS - 2) * LOADS>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    stage = stage + 1 == NS ? 0 : stage + 1;
  }
  }
  wait_loads_but<0>();  // the steps asked for beyond the end: nothing of this block is in flight when it ends

  // A part of K: the sums go to `partial` [part][token][grid column] as they are; gemm_reduce_kernel adds the
  // parts and does what would follow here.
  if constexpr (SPLIT) {
    const size_t width = (size_t)col_blocks * BN;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int token = row0 + wave_m * WM + i * 16 + r;
      if (token >= m) continue;
#pragma unroll
      for (int j = 0; j < TN; ++j)
        *(f32x4*)(partial + ((size_t)part * m + token) * width + col0 + wave_n * WN + j * 16 + g * 4) = acc[i][j];
    }
    return;
  } else {
  // a prepared operand's norm: 1 / sqrt(mean of squares + eps) of a tile row
  auto scale_of = [&](int row) -> float {
    if constexpr (EPI >= 0) {
      float total;
      if constexpr (PG == 4) total = (row_scale[0][row] + row_scale[1][row]) + (row_scale[2][row] + row_scale[3][row]);
      else if constexpr (PG == 2) total = row_scale[0][row] + row_scale[1][row];
      else total = row_scale[0][row];
      return 1.0f / sqrtf(total / (float)k + y.eps);
    } else {
      return 1.0f;
    }
  };
  // first operand = weight rows: lane holds D[n = 4g + e][token = r]
  const bool vector_ok = (n % 4) == 0;
  if constexpr (kPaired) {
    // strips 2u and 2u+1 of this wave: lower and upper rows of a pair unit
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int token = row0 + wave_m * WM + i * 16 + r;
      if (token >= m) continue;
      const float scale = scale_of(wave_m * WM + i * 16 + r);
#pragma unroll
      for (int u = 0; u < TN / 2; ++u) {
        const int first = paired_weight_row<EPI, BN, WGN>(y.rope, col_block, wave_n * WN + 32 * u, n);  // the unit's first lower row
        if (first < 0) continue;
        float lo[4], hi[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          lo[e] = acc[i][2 * u][e] * scale;
          hi[e] = acc[i][2 * u + 1][e] * scale;
        }
        if constexpr (EPI == EPI_SILU) {
          epilogue_silu(y.y, token, n / 2, first + 4 * g, lo, hi);
        } else {
          const int hd = y.rope.head_dim, head = first / hd, f0 = first % hd + 4 * g;
          epi_f32x4 c = {1.0f, 1.0f, 1.0f, 1.0f}, sn = {0.0f, 0.0f, 0.0f, 0.0f};
          if (head < y.rope.heads + y.rope.kv_heads) {
            c = *(const epi_f32x4*)(rope_cos_row(y.rope, token, tok_pos[i]) + f0);
            sn = *(const epi_f32x4*)(rope_sin_row(y.rope, token, tok_pos[i]) + f0);
          }
          epilogue_rope(y.rope, token, tok_pos[i], head >= y.rope.heads ? tok_page[i] : -1, head, f0, lo, hi, c, sn);
        }
      }
    }
  } else {
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int token = row0 + wave_m * WM + i * 16 + r;
    float sq = 0.0f;
    float scale = 1.0f;
    if constexpr (EPI == EPI_STORE) scale = scale_of(wave_m * WM + i * 16 + r);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n0 = col0 + wave_n * WN + j * 16 + g * 4;
      const int valid = n - n0 >= 4 ? 4 : (n - n0 > 0 ? n - n0 : 0);
      if (token >= m || valid <= 0) continue;
      if constexpr (kResidual) {
        if constexpr (kAskEarly) sq += residual_take(y, held[i][j], (size_t)token * n + n0, acc[i][j], valid, vector_ok);
        else sq += residual_take(y, residual_ask(y, (size_t)token * n + n0, n0, valid, vector_ok), (size_t)token * n + n0, acc[i][j], valid, vector_ok);
      } else if constexpr (EPI == EPI_STORE) store4(y.y, (size_t)token * n + n0, acc[i][j] * scale, valid, vector_ok);
      else store4(y, (size_t)token * n + n0, acc[i][j], valid, vector_ok);
    }
    if constexpr (kResidual) {
      // a part of the row's sum of squares: this wave's columns
      sq += __shfl_xor(sq, 16, kWave);
      sq += __shfl_xor(sq, 32, kWave);
      if (g == 0 && token < m) y.ss[(size_t)(col_block * WGN + wave_n) * m + token] = sq;
    }
  }
  }
  }  // !SPLIT
}

// The parts of K that gemm_tiled_kernel left in `partial` [ksplit][m][width], added in the order of the parts,
// and the product's epilogue: stored, or taken into the residual stream with the next norm prepared (a part of
// a row's sum of squares per 64 columns).  A thread has 4 columns of a token, a block 16 tokens x 64 columns.
template <typename OutT>
__global__ __launch_bounds__(256) void gemm_reduce_kernel(const float* __restrict__ partial, OutT y, int m, int n, int width,
                                                          int ksplit) {
  constexpr bool kResidual = std::is_same<OutT, ResidualOut>::value;
  const int token = blockIdx.y * 16 + threadIdx.x / 16;
  const int n0 = blockIdx.x * 64 + (threadIdx.x % 16) * 4;
  const int valid = token < m ? (n - n0 >= 4 ? 4 : (n - n0 > 0 ? n - n0 : 0)) : 0;
  const bool vector_ok = (n % 4) == 0;
  const size_t index = (size_t)(valid > 0 ? token : 0) * n + (valid > 0 ? n0 : 0);
  ResidualHeld held;
  if constexpr (kResidual) held = residual_ask(y, index, valid > 0 ? n0 : 0, valid, vector_ok);
  // every load is asked for before any is used: none stands behind a branch (a part beyond the last reads
  // the last again and counts as zero)
  f32x4 part[8];
  const float* from = partial + (size_t)(valid > 0 ? token : 0) * width + (valid > 0 ? n0 : 0);
#pragma unroll
  for (int p = 0; p < 8; ++p) part[p] = *(const f32x4*)(from + (size_t)(p < ksplit ? p : ksplit - 1) * m * width);
  f32x4 sum = part[0];
#pragma unroll
  for (int p = 1; p < 8; ++p) {
    const float keep = p < ksplit ? 1.0f : 0.0f;
    sum += part[p] * keep;
  }
  if constexpr (kResidual) {
    float sq = valid > 0 ? residual_take(y, held, index, sum, valid, vector_ok) : 0.0f;
#pragma unroll
    for (int offset = 1; offset < 16; offset <<= 1) sq += __shfl_xor(sq, offset, kWave);
    if (threadIdx.x % 16 == 0 && token < m) y.ss[(size_t)blockIdx.x * m + token] = sq;
  } else {
    if (valid > 0) store4(y, index, sum, valid, vector_ok);
  }
}

// The same for a prepared operand (ScaledOut): a thread has the four lower and the four upper sums of a pair
// unit (32 grid columns: 16 lower, then 16 upper rows; for EPI_STORE simply 2 x 4 columns 16 apart) of one
// token, a block 16 tokens x 4 units.  The 16 lanes of a token add the parts of its sum of squares.
template <int EPI>
__global__ __launch_bounds__(256) void gemm_reduce_scaled_kernel(const float* __restrict__ partial, ScaledOut<EPI> y, int m, int n,
                                                                 int k, int width, int ksplit) {
  const int token = blockIdx.y * 16 + threadIdx.x / 16;
  const int sub = threadIdx.x % 16;
  const int unit = blockIdx.x * 4 + sub / 4, quad = sub % 4;
  const int safe_token = token < m ? token : m - 1;
  float squares = 0.0f;
  for (int p0 = sub; p0 < y.parts; p0 += 64) {
    float part[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int p = p0 + 16 * u;
      part[u] = y.ss_parts[(size_t)(p < y.parts ? p : y.parts - 1) * m + safe_token];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) squares += p0 + 16 * u < y.parts ? part[u] : 0.0f;
  }
  int pos = 0, page = -1;
  if constexpr (EPI == EPI_ROPE) {
    const int slot = y.rope.tok_page ? 0 : y.rope.tok_slot[safe_token];
    pos = y.rope.tok_pos[safe_token];
    page = rope_page(y.rope, safe_token, slot, pos);
  }
  const int column = unit * 32 + quad * 4;  // the lower four; the upper four are 16 on
  const bool inside = token < m && column + 16 < width;
  // every load is asked for before any is used: none stands behind a branch (a part beyond the last reads
  // the last again and counts as zero)
  f32x4 lo_part[8], hi_part[8];
  const float* from = partial + (size_t)safe_token * width + (inside ? column : 0);
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    const float* at = from + (size_t)(p < ksplit ? p : ksplit - 1) * m * width;
    lo_part[p] = *(const f32x4*)at;
    hi_part[p] = *(const f32x4*)(at + 16);
  }
#pragma unroll
  for (int offset = 1; offset < 16; offset <<= 1) squares += __shfl_xor(squares, offset, kWave);
  const float scale = 1.0f / sqrtf(squares / (float)k + y.eps);
  f32x4 lo_sum = lo_part[0], hi_sum = hi_part[0];
#pragma unroll
  for (int p = 1; p < 8; ++p) {
    const float keep = p < ksplit ? 1.0f : 0.0f;
    lo_sum += lo_part[p] * keep;
    hi_sum += hi_part[p] * keep;
  }
  if (!inside) return;
  float lo[4], hi[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    lo[e] = lo_sum[e] * scale;
    hi[e] = hi_sum[e] * scale;
  }
  if constexpr (EPI == EPI_STORE) {
    const bool vector_ok = (n % 4) == 0;
    const int rest_lo = n - column, rest_hi = n - column - 16;
    if (rest_lo > 0) store4(y.y, (size_t)token * n + column, (f32x4){lo[0], lo[1], lo[2], lo[3]}, rest_lo >= 4 ? 4 : rest_lo, vector_ok);
    if (rest_hi > 0) store4(y.y, (size_t)token * n + column + 16, (f32x4){hi[0], hi[1], hi[2], hi[3]}, rest_hi >= 4 ? 4 : rest_hi, vector_ok);
  } else if constexpr (EPI == EPI_SILU) {
    if (unit * 16 < n / 2) epilogue_silu(y.y, token, n / 2, unit * 16 + quad * 4, lo, hi);
  } else {
    const int hd = y.rope.head_dim, per_head = hd / 32;
    if (unit >= (y.rope.heads + 2 * y.rope.kv_heads) * per_head) return;
    const int head = unit / per_head, f0 = (unit % per_head) * 16 + quad * 4;
    epi_f32x4 c = {1.0f, 1.0f, 1.0f, 1.0f}, sn = {0.0f, 0.0f, 0.0f, 0.0f};
    if (head < y.rope.heads + y.rope.kv_heads) {
      c = *(const epi_f32x4*)(rope_cos_row(y.rope, token, pos) + f0);
      sn = *(const epi_f32x4*)(rope_sin_row(y.rope, token, pos) + f0);
    }
    epilogue_rope(y.rope, token, pos, head >= y.rope.heads ? page : -1, head, f0, lo, hi, c, sn);
  }
}

// bytes of LDS the kernel's RUNS variant needs for the activations of 16 * MT tokens
size_t skinny_runs_lds(int token_tiles, int k) { return (size_t)16 * token_tiles * (k + 8) * sizeof(bf16_t); }

// runs: null, or where the activations come from instead of x (the variant of the kernel that makes them)
template <int MT, int KSPLIT, typename OutT>
void launch_skinny(const bf16_t* x, const bf16_t* w, OutT y, int m, int n, int k, const RunsIn* runs, hipStream_t stream) {
  const int strips = (n + 15) / 16;
  const int waves = KSPLIT > 4 ? KSPLIT : 4;
  const int per_block = waves / KSPLIT;
  const int strip_blocks = (strips + per_block - 1) / per_block;
  const int tiles = (m + 16 * MT - 1) / (16 * MT);
  const dim3 grid(tiles == 1 ? strip_blocks : (strip_blocks + 7) / 8 * 8 * tiles), block(64 * waves);
  const int stream_weights = (size_t)n * k * sizeof(bf16_t) > kStreamWeightBytes;
  if constexpr (std::is_same<OutT, ResidualOut>::value) {
    if (runs) {
      hipLaunchKernelGGL((gemm_skinny_kernel<MT, KSPLIT, true, OutT>), grid, block, skinny_runs_lds(MT, k), stream, x, w, y, m, n, k,
                         tiles, stream_weights, *runs, PairScratch{});
      return;
    }
  }
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, KSPLIT, false, OutT>), grid, block, 0, stream, x, w, y, m, n, k, tiles, stream_weights,
                     RunsIn{}, PairScratch{});
}

// Two blocks a strip (see PairScratch), for up to 16 tokens into the stream: where the strips leave half the chip
// without a block and each block's share of the weights is long -- a compute unit reads about 30 GB/s whatever its
// waves, so 128 blocks read 2048 x 8192 no faster than 3.7 TB/s.
constexpr int kPairStripsMost = 128, kPairChunksLeast = 80;
bool takes_paired_blocks(int m, int n, int k, const float* workspace, size_t workspace_bytes, const int* pair_count) {
  const int strips = (n + 15) / 16;
  return pair_count && workspace && m <= 16 && strips <= kPairStripsMost && nnis_packed_chunks(k) >= kPairChunksLeast &&
         (size_t)strips * 2 * kWave * 4 * sizeof(float) <= workspace_bytes;
}

void launch_skinny_paired(const bf16_t* x, const bf16_t* w, ResidualOut y, int m, int n, int k, float* workspace, int* pair_count,
                          hipStream_t stream) {
  const int strips = (n + 15) / 16;
  const int stream_weights = (size_t)n * k * sizeof(bf16_t) > kStreamWeightBytes;
  hipLaunchKernelGGL((gemm_skinny_kernel<1, 8, false, ResidualOut, true>), dim3(2 * strips), dim3(64 * 8), 0, stream, x, w, y, m, n, k, 1,
                     stream_weights, RunsIn{}, PairScratch{workspace, pair_count});
}

template <int MT, typename OutT>
void dispatch_skinny_split(const bf16_t* x, const bf16_t* w, OutT y, int m, int n, int k, int split, const RunsIn* runs,
                           hipStream_t stream) {
  if (split == 8) launch_skinny<MT, 8, OutT>(x, w, y, m, n, k, runs, stream);
  else if (split == 4) launch_skinny<MT, 4, OutT>(x, w, y, m, n, k, runs, stream);
  else if (split == 2) launch_skinny<MT, 2, OutT>(x, w, y, m, n, k, runs, stream);
  else launch_skinny<MT, 1, OutT>(x, w, y, m, n, k, runs, stream);
}

// token tiles a wave of the skinny kernel takes: all of them (up to 4) when the weights are large and
// should be read once; one, with the other tiles in blocks of their own on the same die, when the dies' L2
// keep the weights (a few MB) and a wave's work is what the kernel's time hangs on
int skinny_tiles_per_wave(int m, int n, int k) {
  return (size_t)n * k * sizeof(bf16_t) <= kRereadWeightBytes ? 1 : (m + 15) / 16;
}

template <typename OutT>
void dispatch_skinny(const bf16_t* x, const bf16_t* w, OutT y, int m, int n, int k, int split, hipStream_t stream,
                     const RunsIn* runs = nullptr) {
  const int tiles = skinny_tiles_per_wave(m, n, k);
  if (tiles == 1) dispatch_skinny_split<1, OutT>(x, w, y, m, n, k, split, runs, stream);
  else if (tiles == 2) dispatch_skinny_split<2, OutT>(x, w, y, m, n, k, split, runs, stream);
  else if (tiles == 3) dispatch_skinny_split<3, OutT>(x, w, y, m, n, k, split, runs, stream);
  else dispatch_skinny_split<4, OutT>(x, w, y, m, n, k, split, runs, stream);
}

#ifndef NNIS_DEEP_RING_BLOCKS
#define NNIS_DEEP_RING_BLOCKS 256
#endif
constexpr int kDeepRingBlocks = NNIS_DEEP_RING_BLOCKS;  // grids up to this many blocks take the ring of 6 stages
#ifndef NNIS_SHALLOW_RING_BLOCKS
#define NNIS_SHALLOW_RING_BLOCKS 513
#endif
constexpr int kShallowRingBlocks = NNIS_SHALLOW_RING_BLOCKS;  // grids of 64 x 128 tiles from this many blocks on: 2 stages

// Scratch for the parts of a K that is cut among blocks (the caller's; nothing is allocated here)
struct Workspace {
  float* floats;
  size_t bytes;
};

// Parts of K for a tiled product of `tiles` tiles: a power of two up to 8, as long as the chip still has
// compute units without a block, a part keeps at least 4 steps of 64, and the parts fit the workspace.
int tiled_ksplit(int tiles, int m, int width, int k, size_t workspace_bytes) {
  const int steps = (k + 63) / 64;
  int ksplit = 1;
  while (ksplit < 8 && tiles * ksplit * 2 <= 256 && steps / (ksplit * 2) >= 4) ksplit *= 2;
  while (ksplit > 1 && (size_t)ksplit * m * width * sizeof(float) > workspace_bytes) ksplit /= 2;
  return ksplit;
}

template <int BM, int BN, int BK, int NS, bool SPLIT, typename OutT, int WGM = 2, int WGN = 2>
void launch_tiled_kernel(const bf16_t* x, const bf16_t* w, OutT y, int m, int n, int k, int col_blocks, int row_blocks, int ksplit,
                         Workspace ws, hipStream_t stream) {
  constexpr int lds_bytes = NS * (BM + BN) * BK * 2;
  // beyond 64 KB a kernel has to be told once; a refusal shows as the launch's failure
  static const hipError_t allowed = hipFuncSetAttribute((const void*)gemm_tiled_kernel<BM, BN, BK, NS, SPLIT, OutT, WGM, WGN>,
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
  (void)allowed;
  hipLaunchKernelGGL((gemm_tiled_kernel<BM, BN, BK, NS, SPLIT, OutT, WGM, WGN>), dim3((unsigned)col_blocks * row_blocks * ksplit),
                     dim3(64 * WGM * WGN), lds_bytes, stream, x, w, y, m, n, k, col_blocks, ksplit, ws.floats);
}

// the tile of 256 x 256 (8 waves, 2 stages of 64 KB, one block a compute unit); returns the parts of a row's sum of
// squares that a residual epilogue wrote: one per wave column
template <int BN, typename OutT>
int launch_tiled_large(const bf16_t* x, const bf16_t* w, OutT y, int m, int n, int k, int columns, hipStream_t stream) {
  const int col_blocks = (columns + BN - 1) / BN, row_blocks = (m + 255) / 256;
  launch_tiled_kernel<256, BN, 64, 2, false, OutT, 4, 2>(x, w, y, m, n, k, col_blocks, row_blocks, 1, {nullptr, 0}, stream);
  return 2 * col_blocks;
}

// the tiles of 128 x 128, 128 x 192 and 256 x 128 (8 waves as 4 x 2, a wave tile of 32 x 64, 32 x 96 or 64 x 64; 3 stages
// of 32, 40 or 48 KB:
// one block a compute unit, whose row blocks share each column block's weights); returns the parts of a row's
// sum of squares written
template <int BM, int BN, typename OutT>
int launch_tiled_medium(const bf16_t* x, const bf16_t* w, OutT y, int m, int n, int k, int columns, hipStream_t stream) {
  const int col_blocks = (columns + BN - 1) / BN, row_blocks = (m + BM - 1) / BM;
  launch_tiled_kernel<BM, BN, 64, 3, false, OutT, 4, 2>(x, w, y, m, n, k, col_blocks, row_blocks, 1, {nullptr, 0}, stream);
  return 2 * col_blocks;
}

template <int BM, int BN, int BK, int NS, typename OutT>
int launch_tiled_staged(const bf16_t* x, const bf16_t* w, OutT y, int m, int n, int k, int col_blocks, int row_blocks, int ksplit,
                        Workspace ws, hipStream_t stream) {
  if (ksplit > 1) {
    launch_tiled_kernel<BM, BN, BK, NS, true, OutT>(x, w, y, m, n, k, col_blocks, row_blocks, ksplit, ws, stream);
    constexpr int EPI = scaled_epilogue<OutT>::value;
    if constexpr (EPI >= 0) {
      hipLaunchKernelGGL((gemm_reduce_scaled_kernel<EPI>), dim3((col_blocks * BN + 127) / 128, (m + 15) / 16), dim3(256), 0, stream,
                         ws.floats, y, m, n, k, col_blocks * BN, ksplit);
    } else {
      hipLaunchKernelGGL((gemm_reduce_kernel<OutT>), dim3((n + 63) / 64, (m + 15) / 16), dim3(256), 0, stream, ws.floats, y, m, n,
                         col_blocks * BN, ksplit);
    }
    return (n + 63) / 64;
  }
  launch_tiled_kernel<BM, BN, BK, NS, false, OutT>(x, w, y, m, n, k, col_blocks, row_blocks, 1, ws, stream);
  return 2 * col_blocks;  // a part per wave column
}

// `columns`: the weight rows the grid covers (n, or the rows of all pair units).  Returns the parts of a
// row's sum of squares that a residual epilogue wrote.
template <int BM, int BN, int BK, typename OutT>
int launch_tiled(const bf16_t* x, const bf16_t* w, OutT y, int m, int n, int k, int columns, Workspace ws, hipStream_t stream) {
  const int col_blocks = (columns + BN - 1) / BN, row_blocks = (m + BM - 1) / BM;
  const int ksplit = ws.floats ? tiled_ksplit(col_blocks * row_blocks, m, col_blocks * BN, k, ws.bytes) : 1;
  const int steps_a_part = ((k + BK - 1) / BK + ksplit - 1) / ksplit;
  const int blocks = col_blocks * row_blocks * ksplit;
  if (blocks <= kDeepRingBlocks && steps_a_part >= 16)
    return launch_tiled_staged<BM, BN, BK, 6, OutT>(x, w, y, m, n, k, col_blocks, row_blocks, ksplit, ws, stream);
  if (BN == 128 && ksplit == 1 && blocks >= kShallowRingBlocks)
    return launch_tiled_staged<BM, BN, BK, 2, OutT>(x, w, y, m, n, k, col_blocks, row_blocks, 1, ws, stream);
  return launch_tiled_staged<BM, BN, BK, 3, OutT>(x, w, y, m, n, k, col_blocks, row_blocks, ksplit, ws, stream);
}

// The tile of a product: 2: 64x128, 3: 64x64 (4 waves, several blocks a compute unit), and five tiles of 8 waves that
// a compute unit runs one at a time -- 4: 256x256, 5: 256x192 (two stages), 7: 256x128, 8: 128x192, 6: 128x128 (three
// stages, a step's second half multiplied behind the barrier).
//
// Among the five the one whose rounds of blocks (blocks / 256 compute units, rounded up) come to the least tile area
// over the tile's rate.  Rates, from full rounds at K = 2048 over weights from memory, relative to 256x128 (32768
// outputs in 35.5 us): 256x256 1.10, 256x192 1.08, 128x192 0.91, 128x128 0.82.  The rule names the fastest tile, or
// one within a few per cent of it, on all of 77 products of 256 to 4,096 rows with 2,048 to 16,384 columns (auto
// against each tile asked for); a few of them, microseconds: 2048 x 16384 in 512 tiles of 256x256 128 (256x128: 141);
// 2048 x 6144 in 256 of 256x192 49 (256x256, 192 tiles: 56); 3072 x 6144 in 768 of 128x192 80 (384 of 256x192: 92);
// 1536 x 16384 in 768 of 256x128 99 (384 of 256x256: 113); 4096 x 2048 in 256 of 256x128 35.5 (512 of 128x128: 43);
// 2048 x 2560 in 224 of 128x192 26.5 (64x128: 29); 2048 x 2048 in 256 of 128x128 21.6 (64x128: 23.6).  At a K of
// 8,192 the three-stage tiles gain on the others (4096 x 2048 x 8192 in 256 of 256x128: 117 us, 1.18 PFLOP/s): from
// a K of 8,192 on the rates are 256x256 0.97, 256x192 0.93, 128x192 0.90, 128x128 0.80 of 256x128, from 4,096 on
// the same but 256x256 1.03 (4096 x 6144 x 8192 in 768 tiles of 256x128 347 us against 383 in 512 of 256x192; 2048 x 28672 x
// 4096 in 1792 of them 438 against 473 in 896 of 256x256); there the rule is within a tenth of the fastest tile on
// the same 77 products but one (1536 x 6144 x 8192: 190 in 192 tiles of 256x192, 162 in 384 of 128x192, a round and
// a half that the rule below keeps out).
//
// What keeps a tile out:
//  * rows that do not fill its row blocks: 300 rows would be multiplied as 512.  Three quarters for the three-stage
//    tiles (384 x 16384 x 4096 as 512 rows in 256 tiles of 256x128: 61 us against 75 in tiles of 64x128); for the two-stage ones three quarters from 1,024 rows on and fifteen sixteenths below (384 x 16384 x
//    2048 as 512 rows of 256x192 took 44.5 us against 34.2 in tiles of 64x128);
//  * blocks too few for the chip, against the 4-wave tiles, which several of fit a compute unit: the two-stage tiles
//    want 160 blocks (1024 x 6144 x 2048 in 128 tiles: 44 us against 34), a single round of the others five eighths
//    of the compute units (1024 x 2560 x 2048 in 160 tiles of 128x128: 20.0 against 21.6; 1024 x 2048 x 8192 in 128:
//    58 against 51; in 144, 768 x 3072 60 against 67 but 384 x 6144 77 against 68), two rounds seven eighths of them (3072 x 2048 x 4096 in 384 tiles of 128x128: 81 against 69),
//    more rounds a last one that is half full (1280 x 16384 x 8192 in 640 tiles of 256x128: 334 against 372);
//  * a short K: the three-stage tiles from 1,024 on, the others from 256.
// Of the 4-wave tiles the narrow one up to one wide block a compute unit: 1024 x 2048 x 2048 in 256 wide blocks takes
// 19.1 us, in 512 narrow ones 16.0; with 320 wide blocks (1024 x 2560) the wide tile is ahead, 20.9 to 22.3.
#ifndef NNIS_LARGE_TILE_BLOCKS
#define NNIS_LARGE_TILE_BLOCKS 160
#endif
int pick_tile(int m, int columns, int k, int tile_hint) {
  const long long blocks_64_128 = (long long)((m + 63) / 64) * ((columns + 127) / 128);
  int tile = blocks_64_128 > 256 ? 2 : 3;
  struct Candidate { int tile, rows, width, rate[3], stages; };  // rates for a K below 4,096, below 8,192, and beyond
  const int depth = k >= 8192 ? 2 : (k >= 4096 ? 1 : 0);
  long long best = 0;
  for (const Candidate c : {Candidate{4, 256, 256, {110, 103, 97}, 2}, Candidate{5, 256, 192, {108, 93, 93}, 2},
                            Candidate{7, 256, 128, {100, 100, 100}, 3}, Candidate{8, 128, 192, {91, 90, 90}, 3},
                            Candidate{6, 128, 128, {82, 80, 80}, 3}}) {
    const long long row_blocks = (m + c.rows - 1) / c.rows;
    const long long blocks = row_blocks * ((columns + c.width - 1) / c.width);
    const long long rounds = (blocks + 255) / 256;
    if (c.stages == 2) {
      const bool filled = row_blocks >= 4 ? 4LL * m >= 3LL * c.rows * row_blocks : 16LL * m >= 15LL * c.rows * row_blocks;
      if (k < 256 || !filled || blocks < NNIS_LARGE_TILE_BLOCKS) continue;
    } else {
      if (k < 1024 || 4LL * m < 3LL * c.rows * row_blocks) continue;
      if (rounds == 1 ? 8 * blocks < 5 * 256 : (rounds == 2 ? 8 * blocks < 7 * 256 * 2 : 2 * blocks < (2 * rounds - 1) * 256)) continue;
    }
    const long long cost = rounds * c.rows * c.width * 100 / c.rate[depth];
    if (best == 0 || cost < best) {
      best = cost;
      tile = c.tile;
    }
  }
  if (tile_hint >= 2 && tile_hint <= 8) tile = tile_hint;  // for tuning runs
  return tile;
}

// the most parts of a row's sum of squares that a residual epilogue of the tiled kernel writes for these sizes
int tiled_parts(int m, int columns, int k, int tile_hint) {
  const int tile = pick_tile(m, columns, k, tile_hint);
  const int width = tile == 4 ? 256 : (tile == 5 || tile == 8 ? 192 : (tile == 2 || tile == 6 || tile == 7 ? 128 : 64));
  return 2 * ((columns + width - 1) / width);  // with K in parts: one per 64 columns, which is no more
}

// returns the parts of a row's sum of squares written (a residual epilogue)
template <typename OutT>
int dispatch_tiled(const bf16_t* x, const bf16_t* w, OutT y, int m, int n, int k, int tile_hint, Workspace ws, hipStream_t stream,
                   int columns = 0) {
  if (columns <= 0) columns = n;
  const int tile = pick_tile(m, columns, k, tile_hint);
  if (tile == 4) return launch_tiled_large<256, OutT>(x, w, y, m, n, k, columns, stream);
  if (tile == 5) return launch_tiled_large<192, OutT>(x, w, y, m, n, k, columns, stream);
  if (tile == 6) return launch_tiled_medium<128, 128, OutT>(x, w, y, m, n, k, columns, stream);
  if (tile == 7) return launch_tiled_medium<256, 128, OutT>(x, w, y, m, n, k, columns, stream);
  if (tile == 8) return launch_tiled_medium<128, 192, OutT>(x, w, y, m, n, k, columns, stream);
  if (tile == 2) return launch_tiled<64, 128, 64, OutT>(x, w, y, m, n, k, columns, ws, stream);
  return launch_tiled<64, 64, 64, OutT>(x, w, y, m, n, k, columns, ws, stream);
}

// With few strips the waves of a block share a strip's K, so that each wave's
// share is one round of loads (4 steps of 64 for up to 32 tokens, 2 beyond);
// with thousands of strips there are waves enough to hide the latency.
int skinny_split(int m, int n, int k, int split_hint) {
  const int strips = (n + 15) / 16;
  const int chunks = (k + 63) / 64;
  const int depth = skinny_tiles_per_wave(m, n, k) <= 2 ? 4 : 2;
  int split = 1;
  if (strips < 2048) {
    while (split < 8 && chunks > split * depth) split *= 2;
  }
  if (split_hint == 1 || split_hint == 2 || split_hint == 4 || split_hint == 8) split = split_hint;  // for tuning runs
  return split;
}

}  // namespace

// The kernel for few tokens (a wave owns 16 weight rows, no LDS for operands) against the tiled one.
//  * Up to 16 tokens: always.
//  * Up to 64 tokens: unless the weights are large and wide.  A wave of the kernel for few tokens reads all
//    the tokens' activations beside its 16 weight rows -- with 64 tokens four times the bytes of the weights --
//    while a tile shares them among its waves through LDS; the tiled kernel needs enough column blocks to
//    fill the chip, though.  Measured with 64 tokens and K = 2048, microseconds: 11264 rows 34 against 18
//    tiled, 16384 rows 45 against 19, but 2560 rows 12.5 against 14.8.
//  * Beyond, up to kFewTokens: when the weights are small enough to be read once per tile of 16 tokens and
//    its blocks (strips x token tiles) are few enough; measured on products of 32 to 384 tokens with weights
//    of 576 x 576 to 3072 x 576 and 576 x 1536, in microseconds:
//      few tokens: 3 + 0.004 * strips * tiles * K / 576      tiled: 2.6 + 0.0057 * K
bool nnis_gemm_takes_few_tokens(int m, int n, int k) {
  if (m <= 16) return true;
  const bool large = (size_t)n * k * sizeof(bf16_t) > kRereadWeightBytes;
  if (m <= 64) return !(large && (n + 63) / 64 >= 128);
  if (m > kFewTokens || large) return false;
  const double strips = (n + 15) / 16, tiles = (m + 15) / 16;
  return 3.0 + 0.004 * strips * tiles * k / 576.0 <= 2.6 + 0.0057 * k;
}

// The same for a product whose tiled kernel may cut K into parts (it stores, or adds to the stream): large
// weights with few columns still fill the chip then.  Measured with 64 tokens, microseconds: 2048 x 5632
// 28 for few tokens against 15 in 8 parts, 2048 x 8192 39 against 18.
static bool takes_few_tokens_with_parts(int m, int n, int k, bool workspace) {
  if (m <= 16 || m > 64 || !workspace) return nnis_gemm_takes_few_tokens(m, n, k);
  const bool large = (size_t)n * k * sizeof(bf16_t) > kRereadWeightBytes;
  int parts = 1;
  while (parts < 8 && ((k + 63) / 64) / (parts * 2) >= 4) parts *= 2;
  return !(large && (n + 63) / 64 * parts >= 128);
}

int nnis_gemm_scaled_tiled(const bf16_t* scaled, const float* ss_parts, int parts, float eps, const bf16_t* w, int m, int n,
                           int k, int epilogue, bf16_t* y, const RopeTarget& rope, int tile_hint, float* workspace,
                           size_t workspace_bytes, hipStream_t stream) {
  const Workspace ws = {workspace, workspace ? workspace_bytes : 0};
  NNIS_REQUIRE((m + 63) / 64 <= 65535, "gemm_scaled: %d rows exceed the grid limit", m);
  if (epilogue == EPI_STORE) {
    dispatch_tiled<ScaledOut<EPI_STORE>>(scaled, w, {y, ss_parts, parts, eps, rope}, m, n, k, tile_hint, ws, stream);
  } else if (epilogue == EPI_SILU) {
    dispatch_tiled<ScaledOut<EPI_SILU>>(scaled, w, {y, ss_parts, parts, eps, rope}, m, n, k, tile_hint, ws, stream,
                                        32 * ((n / 2 + 15) / 16));
  } else {
    dispatch_tiled<ScaledOut<EPI_ROPE>>(scaled, w, {y, ss_parts, parts, eps, rope}, m, n, k, tile_hint, ws, stream, n);
  }
  NNIS_LAUNCH_CHECK("gemm_scaled");
  return 0;
}

// y_dtype: NNIS_BF16 or NNIS_F32.  Picks the skinny kernel for M <= 64.  split_hint: 0, or the number of
// waves (1, 2, 4, 8) that share a strip's K in the skinny kernel, overriding the choice made here.
extern "C" int nnis_gemm_bf16(const void* x, const void* w, void* y, int y_dtype, int m, int n, int k, int split_hint,
                              float* workspace, size_t workspace_bytes, void* stream_ptr) {
  NNIS_REQUIRE(nnis_dtype_ok(y_dtype), "gemm_bf16: unknown output dtype %d", y_dtype);
  NNIS_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm_bf16: bad sizes m=%d n=%d k=%d", m, n, k);
  NNIS_REQUIRE(k % 8 == 0, "gemm_bf16: K=%d is not a multiple of 8 (16-byte loads); use the ordered kernel", k);
  NNIS_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0) && ((uintptr_t)y % 16 == 0),
               "gemm_bf16: operands must be 16-byte aligned");
  if (m == 0) return 0;
  hipStream_t stream = (hipStream_t)stream_ptr;
  const bf16_t* xp = (const bf16_t*)x;
  const bf16_t* wp = (const bf16_t*)w;
  NNIS_REQUIRE((uintptr_t)workspace % 16 == 0, "gemm_bf16: the workspace must be 16-byte aligned");
  const Workspace ws = {workspace, workspace ? workspace_bytes : 0};
  if (takes_few_tokens_with_parts(m, n, k, workspace != nullptr) && split_hint < 16) {  // a tile hint asks for the tiled kernel
    const int split = skinny_split(m, n, k, split_hint);
    if (y_dtype == NNIS_F32) dispatch_skinny<float*>(xp, wp, (float*)y, m, n, k, split, stream);
    else dispatch_skinny<bf16_t*>(xp, wp, (bf16_t*)y, m, n, k, split, stream);
    NNIS_LAUNCH_CHECK("gemm_skinny");
  } else {
    NNIS_REQUIRE((m + 63) / 64 <= 65535, "gemm_bf16: %d rows exceed the grid limit", m);
    const int tile_hint = split_hint >= 16 ? split_hint / 16 : 0;  // hints of 32, 48, .. 128 pick the tile: 64x128, 64x64, 256x256, 256x192, 128x128, 256x128, 128x192
    if (y_dtype == NNIS_F32) dispatch_tiled<float*>(xp, wp, (float*)y, m, n, k, tile_hint, ws, stream);
    else dispatch_tiled<bf16_t*>(xp, wp, (bf16_t*)y, m, n, k, tile_hint, ws, stream);
    NNIS_LAUNCH_CHECK("gemm_tiled");
  }
  return 0;
}

// The tile that the tiled kernel takes for m rows, `columns` weight rows and a depth of k (2: 64 x 128, 3: 64 x 64,
// 4: 256 x 256, 5: 256 x 192, 6: 128 x 128, 7: 256 x 128, 8: 128 x 192): for tests and tuning.
extern "C" int nnis_gemm_tile(int m, int columns, int k) { return pick_tile(m, columns, k, 0); }

// 1 if nnis_gemm_residual gives these sizes to two blocks a strip (with a workspace of `workspace_bytes` and counts
// behind it), 0 if to another kernel: for callers and tests that have to know which kernel ran.
extern "C" int nnis_gemm_takes_pair(int m, int n, int k, size_t workspace_bytes) {
  static const int some_counts = 0;
  static const float some_workspace = 0.0f;
  return takes_few_tokens_with_parts(m, n, k, true) && takes_paired_blocks(m, n, k, &some_workspace, workspace_bytes, &some_counts) ? 1 : 0;
}

// The projection that ends a part of a pre-norm block: resid += x . w^T in 32-bit, in place, and the norm
// that follows prepared -- scaled = bf16(resid * gain) and parts of each row's sum of squares in ss
// [parts, m].  Returns the number of parts in *parts; ss has ss_rows rows of m floats, of which
// nnis_gemm_residual_parts(m, n) are always enough.
extern "C" int nnis_gemm_residual_parts(int m, int n) {
  (void)m;
  // the kernel for few tokens: a part per strip of 16 columns; the tiled one a part per wave column of its tiles,
  // which is fewer from 17 columns on and two for a single tile
  return n > 16 ? (n + 15) / 16 : 2;
}

extern "C" int nnis_gemm_residual(const void* x, const void* w, float* resid, const void* gain, int gain_dtype, void* scaled,
                                  float* ss, int ss_rows, int m, int n, int k, int* parts, int tile_hint, float* workspace,
                                  size_t workspace_bytes, int* pair_count, void* stream_ptr) {
  NNIS_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm_residual: bad sizes m=%d n=%d k=%d", m, n, k);
  NNIS_REQUIRE(k % 8 == 0, "gemm_residual: K=%d is not a multiple of 8 (16-byte loads)", k);
  NNIS_REQUIRE(nnis_dtype_ok(gain_dtype), "gemm_residual: unknown norm weight dtype %d", gain_dtype);
  NNIS_REQUIRE(resid && gain && scaled && ss && parts, "gemm_residual: missing operand");
  for (const void* p : {x, w, (const void*)resid, gain, (const void*)scaled})
    NNIS_REQUIRE((uintptr_t)p % 16 == 0, "gemm_residual: operands must be 16-byte aligned");
  *parts = 0;
  if (m == 0) return 0;
  hipStream_t stream = (hipStream_t)stream_ptr;
  ResidualOut out = {resid, gain, gain_dtype, (bf16_t*)scaled, ss};
  NNIS_REQUIRE((uintptr_t)workspace % 16 == 0, "gemm_residual: the workspace must be 16-byte aligned");
  NNIS_REQUIRE(tile_hint == 0 || (tile_hint >= 2 && tile_hint <= 8), "gemm_residual: unknown tile %d", tile_hint);
  const bool few = tile_hint == 0 && takes_few_tokens_with_parts(m, n, k, workspace != nullptr);  // a tile hint asks for the tiled kernel
  const int writes = few ? (n + 15) / 16 : tiled_parts(m, n, k, tile_hint);
  NNIS_REQUIRE(writes <= ss_rows, "gemm_residual: ss has %d rows of %d tokens, %d are needed", ss_rows, m, writes);
  if (few) {
    *parts = (n + 15) / 16;
    if (takes_paired_blocks(m, n, k, workspace, workspace_bytes, pair_count))
      launch_skinny_paired((const bf16_t*)x, (const bf16_t*)w, out, m, n, k, workspace, pair_count, stream);
    else
      dispatch_skinny<ResidualOut>((const bf16_t*)x, (const bf16_t*)w, out, m, n, k, skinny_split(m, n, k, 0), stream);
    NNIS_LAUNCH_CHECK("gemm_residual");
  } else {
    NNIS_REQUIRE((m + 63) / 64 <= 65535, "gemm_residual: %d rows exceed the grid limit", m);
    *parts = dispatch_tiled<ResidualOut>((const bf16_t*)x, (const bf16_t*)w, out, m, n, k, tile_hint,
                                         {workspace, workspace ? workspace_bytes : 0}, stream);
    NNIS_LAUNCH_CHECK("gemm_residual");
  }
  return 0;
}

// Whether nnis_gemm_residual_runs takes these sizes: few tokens (the kernel whose blocks each make their
// tokens' activations in LDS), 2 to 8 runs, activations of a block within 64 KB.
extern "C" int nnis_gemm_residual_runs_fits(int m, int n, int heads, int head_dim, int runs) {
  if (m <= 0 || m > 64 || n <= 0 || heads <= 0 || head_dim <= 0 || head_dim % 4 != 0) return 0;
  const long long k = (long long)heads * head_dim;
  if (k % 8 != 0 || k > (1 << 20)) return 0;
  if (runs < 2 || runs > kMostRuns) return 0;
  if (!nnis_gemm_takes_few_tokens(m, n, (int)k)) return 0;
  return skinny_runs_lds(skinny_tiles_per_wave(m, n, (int)k), (int)k) <= 65536 ? 1 : 0;
}

// nnis_gemm_residual on activations that the decode attention left as runs of keys (`partial`: [m, heads,
// runs, head_dim + 4] float32, see RunsIn): the sum over the runs is made inside the projection instead of by
// a kernel between the two.  tok_slot [m]: rows with a negative slot count as zeros.
extern "C" int nnis_gemm_residual_runs(const float* partial, int runs, int heads, int head_dim, const int* tok_slot, const void* w,
                                       float* resid, const void* gain, int gain_dtype, void* scaled, float* ss, int ss_rows,
                                       int m, int n, int* parts, void* stream_ptr) {
  NNIS_REQUIRE(nnis_gemm_residual_runs_fits(m, n, heads, head_dim, runs),
               "gemm_residual_runs: %d tokens x %d rows on %d heads of %d in %d runs are not taken", m, n, heads, head_dim, runs);
  NNIS_REQUIRE(nnis_dtype_ok(gain_dtype), "gemm_residual_runs: unknown norm weight dtype %d", gain_dtype);
  NNIS_REQUIRE(partial && tok_slot && w && resid && gain && scaled && ss && parts, "gemm_residual_runs: missing operand");
  for (const void* p : {(const void*)partial, w, (const void*)resid, gain, (const void*)scaled})
    NNIS_REQUIRE((uintptr_t)p % 16 == 0, "gemm_residual_runs: operands must be 16-byte aligned");
  const int k = heads * head_dim;
  *parts = (n + 15) / 16;
  NNIS_REQUIRE(*parts <= ss_rows, "gemm_residual_runs: ss has %d rows of %d tokens, %d are needed", ss_rows, m, *parts);
  const RunsIn in = {partial, tok_slot, runs, heads, head_dim};
  ResidualOut out = {resid, gain, gain_dtype, (bf16_t*)scaled, ss};
  dispatch_skinny<ResidualOut>(nullptr, (const bf16_t*)w, out, m, n, k, skinny_split(m, n, k, 0), (hipStream_t)stream_ptr, &in);
  NNIS_LAUNCH_CHECK("gemm_residual_runs");
  return 0;
}

// The packed order of a weight [n, k] in the checkpoint's order (common.h has the layout): a thread moves
// the 16 bytes of one lane's load, or writes the padding's zeros.
__global__ __launch_bounds__(256) void pack_weight_kernel(const bf16_t* __restrict__ w, bf16_t* __restrict__ packed, int n, int k,
                                                          size_t pieces) {
  const size_t piece = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (piece >= pieces) return;
  const int stride = nnis_packed_strip_elems(k) / kPackedChunkElems;  // chunks from strip to strip
  const int lane = piece % 64, half = (piece / 64) % 2;
  const size_t block = piece / 128;
  const int chunk = block % stride;
  const int strip = block / stride;
  const int row = strip * 16 + lane % 16, kk = chunk * 64 + (lane / 16) * 16 + half * 8;
  typedef __attribute__((ext_vector_type(4))) unsigned bits128;
  bits128 v = {0u, 0u, 0u, 0u};
  if (row < n && kk + 8 <= k) v = *(const bits128*)(w + (size_t)row * k + kk);  // (a padding chunk's kk is beyond k)
  *(bits128*)(packed + piece * 8) = v;
}

// packed [(n + 15) / 16 strips][nnis_packed_strip_elems(k)] = the weight w [n, k] (bfloat16, K a multiple of 8) in the order the
// matrix-core products read
extern "C" int nnis_pack_weight(const void* w, void* packed, int n, int k, void* stream_ptr) {
  NNIS_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "pack_weight: bad sizes n=%d k=%d (K must be a multiple of 8)", n, k);
  NNIS_REQUIRE(w && packed && (uintptr_t)w % 16 == 0 && (uintptr_t)packed % 16 == 0, "pack_weight: operands must be 16-byte aligned");
  const size_t pieces = nnis_packed_elems(n, k) / 8;
  NNIS_REQUIRE((pieces + 255) / 256 <= 0x7fffffffull, "pack_weight: %d x %d is more than a grid takes", n, k);
  hipLaunchKernelGGL(pack_weight_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, (hipStream_t)stream_ptr, (const bf16_t*)w,
                     (bf16_t*)packed, n, k, pieces);
  NNIS_LAUNCH_CHECK("pack_weight");
  return 0;
}
