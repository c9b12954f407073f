// Causal attention over the paged cache, compiled for one head size
// (-DNNIS_HEAD_DIM=<n>).  A query token at position p of the sequence in
// `slot` reads keys [lo, p] of that slot, lo = 0 or p + 1 - window, whatever
// the step brought: the current step's keys are in the cache before this runs.
//
// Formula (/root/reference/crates/nnis-model/src/kernels.rs:66-125): query
// head h reads KV head h / (heads / kv_heads); score = dot(q, k) * scale, the
// scale applied after the sum; softmax over the visible keys with a running
// maximum; output = sum of weights * values / sum of weights.  All of it in
// 32-bit, whatever the storage type.
//
// Pages: [page][kv_head][64 tokens of one head], keys and values each in the in-page order of common.h
// (keys in chunks of 8 channels, values in tiles of 16 channels with 8 tokens of a channel together).
#include "common.h"

#include <algorithm>

#ifndef NNIS_HEAD_DIM
#error "compile with -DNNIS_HEAD_DIM=<head size>"
#endif
#ifndef NNIS_PREFILL_RING_NARROW
#define NNIS_PREFILL_RING_NARROW 3
#endif
#ifndef NNIS_AHEAD_VALU
#define NNIS_AHEAD_VALU 36  // vector instructions of a unit's exponentials, between which the next unit's score instructions go
#endif
#ifndef NNIS_PREFILL_RING_WIDE
#define NNIS_PREFILL_RING_WIDE 2
#endif

thread_local char g_nnis_error[512] = {0};
extern "C" const char* nnis_last_error() { return g_nnis_error; }
extern "C" int nnis_attention_head_dim() { return NNIS_HEAD_DIM; }

namespace {

constexpr int HD = NNIS_HEAD_DIM;

struct AttnArgs {
  const void* q;  // [tokens, heads, HD]
  int q_dtype;
  void* out;  // [tokens, heads, HD]
  int out_dtype;
  const void* k_pages;
  const void* v_pages;
  int cache_dtype;
  const int* block_table;
  int max_pages;
  const int* tok_slot;
  const int* tok_pos;
  int tokens, heads, kv_heads;
  int window;  // 0: all keys
  float scale;
};

// One wave per (token, query head); lanes take keys lo+lane, lo+lane+64, ...,
// each keeps its own running maximum, sum and output, merged at the end.
template <typename CacheT>
__global__ __launch_bounds__(256) void attention_rows_kernel(AttnArgs a) {
  __shared__ float q_shared[4][HD];
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int item = blockIdx.x * 4 + wave;
  if (item >= a.tokens * a.heads) return;  // no block-wide barrier below
  const int token = item / a.heads;
  const int head = item % a.heads;
  const size_t row = ((size_t)token * a.heads + head) * HD;
  const int slot = a.tok_slot[token];
  if (slot < 0) {  // padding row
    for (int d = lane; d < HD; d += kWave) store_from_f32(a.out, a.out_dtype, row + d, 0.0f);
    return;
  }
  const int pos = a.tok_pos[token];
  const int kv_head = head / (a.heads / a.kv_heads);
  const int kv_len = pos + 1;
  const int lo = (a.window > 0 && kv_len > a.window) ? kv_len - a.window : 0;

  float* qs = q_shared[wave];
  for (int d = lane; d < HD; d += kWave) qs[d] = load_as_f32(a.q, a.q_dtype, row + d);
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_s_waitcnt(0);  // lds writes of this wave are done before its lanes read them

  const CacheT* kp = (const CacheT*)a.k_pages;
  const CacheT* vp = (const CacheT*)a.v_pages;
  const int* pages = a.block_table + (size_t)slot * a.max_pages;

  float m = -INFINITY, l = 0.0f;
  float o[HD];
#pragma unroll
  for (int d = 0; d < HD; ++d) o[d] = 0.0f;

  for (int j = lo + lane; j < kv_len; j += kWave) {
    const int page = pages[j / kPageTokens];
    const int r = j % kPageTokens;
    const CacheT* keys = kp + ((size_t)page * a.kv_heads + kv_head) * nnis_k_page_elems(HD);
    float dot = 0.0f;
#pragma unroll
    for (int d = 0; d < HD; ++d) dot = fmaf(qs[d], to_f32(keys[nnis_k_offset(r, d)]), dot);
    const float s = dot * a.scale;
    const float m_new = fmaxf(m, s);
    const float alpha = expf(m - m_new);  // exp(-inf) = 0 on the first key
    const float p = expf(s - m_new);
    l = l * alpha + p;
    const CacheT* values = vp + ((size_t)page * a.kv_heads + kv_head) * nnis_v_page_elems(HD);
#pragma unroll
    for (int d = 0; d < HD; ++d) o[d] = o[d] * alpha + p * to_f32(values[nnis_v_offset(d, r)]);
    m = m_new;
  }

  const float m_all = wave_max(m);
  const float factor = (m == -INFINITY) ? 0.0f : expf(m - m_all);
  const float l_all = wave_sum(l * factor);
  const float inv = 1.0f / l_all;
  float mine[(HD + kWave - 1) / kWave];
#pragma unroll
  for (int d = 0; d < HD; ++d) {
    const float total = wave_sum(o[d] * factor);
    if (d % kWave == lane) mine[d / kWave] = total * inv;
  }
#pragma unroll
  for (int c = 0; c < (HD + kWave - 1) / kWave; ++c) {
    const int d = c * kWave + lane;
    if (d < HD) store_from_f32(a.out, a.out_dtype, row + d, mine[c]);
  }
}


// =============================================================================
// bfloat16 on the matrix cores (head sizes in steps of 16)
//
// Scores are taken transposed, S^T[key][column] = K[key][:] . Q[column][:], with
// v_mfma_f32_16x16x32_bf16: first operand a tile of 16 keys, second a tile of
// 16 "columns".  A column is one (query token, query head) pair; the columns of
// a wave all read the same key/value head, so a key tile loaded once serves up
// to C column tiles (the heads of a group, or further query positions).  The
// result lies with lane l as S^T[key 4*(l/16)+e][column l%16]: a column's
// softmax state lives in the lanes l%16 == column, its running maximum kept
// equal over the four lane groups.  The output is taken transposed too,
// O^T[d][column] += V^T[d][key] . P^T[key][column]: first operand a tile of 16
// channels from the value page, second the probabilities, which are already in
// the lanes that need them -- the rows of the two score tiles of a block of 32
// keys are dealt so that lane group g ends up with keys 8g .. 8g+7, and the
// value page keeps 8 consecutive keys of a channel together, one 16-byte load
// per lane and tile.  Softmax is in 32-bit (base-2 exponentials of scores
// scaled by log2 e); probabilities are rounded to bfloat16 for the product
// with the bfloat16 values.
// =============================================================================
#if NNIS_HEAD_DIM % 16 == 0

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kFullD = HD / 32;       // steps of 32 channels in a score
constexpr bool kTailD = (HD % 32) != 0;  // plus one of 16
constexpr int kTilesD = HD / 16;      // output tiles of 16 channels
// waves of a block: beyond 64 channels a wave needs more registers than a block of 8 waves leaves it
constexpr int kBlockWaves = HD <= 64 ? 8 : 4;
constexpr int kPartial = HD + 4;  // floats a split leaves per (token, head), rows 16-byte aligned
// key blocks a decoding wave has in flight (its registers hold their operands)
constexpr int kDecodeRing = HD <= 64 ? 4 : (HD <= 128 ? 2 : 1);
// the kernel with keys on lanes: pages in flight, and how far a score may rise above the softmax's
// reference (as a power of two) before the reference moves
constexpr int kKeysRing = HD <= 64 ? 3 : 2;
constexpr int kKeysWaves = 4;  // of a block of that kernel: a wave keeps kKeysRing pages in registers
constexpr int kKeysMaxHD = 128;
constexpr float kLazyRise = 8.0f;
constexpr float kLog2e = 1.4426950408889634f;

struct QFrag {
  bf16x8 full[kFullD > 0 ? kFullD : 1];
  bf16x4 tail;
};

__device__ __forceinline__ bf16x4 zero4() {
  bf16x4 z;
#pragma unroll
  for (int i = 0; i < 4; ++i) z[i] = (__bf16)0.0f;
  return z;
}

// the operand of one row (a key, or a column's query) of HD channels
__device__ __forceinline__ QFrag load_row_operand(const bf16_t* row, int g) {
  QFrag f;
#pragma unroll
  for (int c = 0; c < kFullD; ++c) f.full[c] = *(const bf16x8*)(row + 32 * c + 8 * g);
  f.tail = kTailD ? *(const bf16x4*)(row + 32 * kFullD + 4 * g) : zero4();
  return f;
}

__device__ __forceinline__ f32x4 score_tile(const QFrag& keys, const QFrag& query) {
  f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int c = 0; c < kFullD; ++c) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(keys.full[c], query.full[c], acc, 0, 0, 0);
  if (kTailD) {
    // the 16-channel remainder is a sum of its own, added afterwards: the two
    // instruction shapes never feed each other's accumulator
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    const f32x4 rest = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(keys.tail, query.tail, zero, 0, 0, 0);
    acc = kFullD > 0 ? acc + rest : rest;
  }
  return acc;
}

// Softmax state of C column tiles and their outputs
template <int C>
struct AttnState {
  float m[C];       // reference of the softmax (a base-2 scaled score near the running maximum) of this lane's column, equal over lane groups
  float l[C];       // this lane's part of the running sum
  f32x4 o[C][kTilesD];
};

template <int C>
__device__ __forceinline__ void init_state(AttnState<C>& st) {
#pragma unroll
  for (int c = 0; c < C; ++c) {
    st.m[c] = -INFINITY;
    st.l[c] = 0.0f;
#pragma unroll
    for (int t = 0; t < kTilesD; ++t) st.o[c][t] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
  }
}

// One block of 32 keys (half h of a page): its operands, read in the page's order.  Row i = 4g' + e of
// score tile t is key 8g' + 4t + e of the block, so that a lane's eight probabilities (tile 0, then tile
// 1) are those of keys 8g .. 8g+7, the order in which a value operand holds them.
struct BlockFrags {
  QFrag keys[2];
  bf16x8 values[kTilesD];
};

// k_page, v_page: the page's keys and values of one kv head
__device__ __forceinline__ void load_block(BlockFrags& f, const bf16_t* k_page, const bf16_t* v_page, int h, int r, int g) {
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int key = 32 * h + 8 * (r / 4) + 4 * t + r % 4;
#pragma unroll
    for (int c = 0; c < kFullD; ++c) f.keys[t].full[c] = *(const bf16x8*)(k_page + nnis_k_offset(key, 32 * c + 8 * g));
    f.keys[t].tail = kTailD ? *(const bf16x4*)(k_page + nnis_k_offset(key, 32 * kFullD + 4 * g)) : zero4();
  }
#pragma unroll
  for (int t = 0; t < kTilesD; ++t) f.values[t] = *(const bf16x8*)(v_page + nnis_v_offset(16 * t + r, 32 * h + 8 * g));
}

// Scores, softmax update and output update of one loaded block for C column tiles.
//   lo[c], hi[c]: the column of this lane reads keys lo <= key <= hi
template <int C>
__device__ __forceinline__ void attend_block(AttnState<C>& st, const QFrag (&q)[C], const BlockFrags& f, int key0,
                                             const int (&lo)[C], const int (&hi)[C], float scale_log2, int g) {
#pragma unroll
  for (int c = 0; c < C; ++c) {
    f32x4 s[2];
    float block_max = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t) s[t] = score_tile(f.keys[t], q[c]);
    // most blocks lie wholly inside what every lane's column reads: then no key needs a look at its index
    if (!__all(key0 >= lo[c] && key0 + 31 <= hi[c])) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int key = key0 + 8 * g + 4 * t + e;
          s[t][e] = (key >= lo[c] && key <= hi[c]) ? s[t][e] : -INFINITY;
        }
    }
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) block_max = fmaxf(block_max, s[t][e]);
    block_max *= scale_log2;  // the scale is positive: the largest score stays the largest
    // The column's reference of the softmax (st.m, equal in its four lane groups) moves only when a score
    // rises more than kLazyRise above it -- always for the first keys, whose reference is -inf.  Until then
    // the sums are sums of 2^(score - reference) with terms up to 2^kLazyRise: the result is the same up
    // to rounding, and the block needs no maximum over the lane groups and no scaling of its outputs.
    if (__any(block_max > st.m[c] + kLazyRise)) {
      float moved = fmaxf(st.m[c], block_max);
      moved = fmaxf(moved, __shfl_xor(moved, 16, kWave));
      moved = fmaxf(moved, __shfl_xor(moved, 32, kWave));
      const float shrink = st.m[c] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(st.m[c] - moved);
      st.l[c] *= shrink;
#pragma unroll
      for (int t = 0; t < kTilesD; ++t) st.o[c][t] = st.o[c][t] * shrink;
      st.m[c] = moved;
    }
    const float base = st.m[c] == -INFINITY ? 0.0f : st.m[c];  // a column that has seen no key yet
    bf16x8 p;
    float sum = 0.0f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float w = __builtin_amdgcn_exp2f(fmaf(s[t][e], scale_log2, -base));  // -inf for a masked key: 0
        sum += w;
        p[4 * t + e] = (__bf16)w;
      }
    st.l[c] += sum;
#pragma unroll
    for (int t = 0; t < kTilesD; ++t)
      st.o[c][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.values[t], p, st.o[c][t], 0, 0, 0);
  }
}

// The same work with the matrix unit and the vector unit side by side, for blocks all of whose keys count for
// every column (no key is looked at).  A unit is one block's 32 keys for one column tile: 2 * (HD / 32) matrix
// instructions for its scores, then the softmax's vector work on them (eight exponentials of 16 cycles a wave
// and some thirty other vector instructions of 4: about 250 cycles, where the unit's matrix instructions take
// 16 each), then HD / 16 matrix instructions for the outputs.  A SIMD runs vector instructions while its
// matrix unit works (a matrix instruction with eight independent multiply-adds behind it takes as long as
// the eight alone), but a wave that meets a matrix instruction while the unit is busy stands there: left to
// the compiler the matrix instructions come in runs of six and more and a unit takes about 360 cycles of a
// SIMD with two waves on it.  So every matrix instruction here is one that needs nothing of the vector work
// around it: the scores of the unit that follows (of the next column, or of the next block's first column: `s`
// comes in holding the scores of (f, column 0) and goes out holding those of (`next`, column 0), where AHEAD
// says that `next` holds the block that follows), and the outputs of the unit before, whose probabilities are
// kept for that long; only a block's last column multiplies its own outputs at once (the values' registers are
// asked for again behind the block).  The compiler's scheduler is told the order inside each stretch of
// straight-line code, from behind one unit's test of its maximum to the next unit's: one of those matrix
// instructions, a few vector instructions, and so on.
template <int C, bool AHEAD, int c>
__device__ __forceinline__ void attend_unit_ahead(AttnState<C>& st, const QFrag (&q)[C], const BlockFrags& f, const BlockFrags& next,
                                                  f32x4 (&s)[2], bf16x8& before, float scale_log2, float (&rise)[C]) {
  constexpr int kScores = 2 * (kFullD + (kTailD ? 1 : 0));
  // rise[c]: the raw score (before the scale) above which column c's reference moves, (st.m[c] + kLazyRise) / scale:
  // the test of every unit is then the scores' maximum against a register
  float block_max = -INFINITY;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) block_max = fmaxf(block_max, s[t][e]);
  {
    // the stretch that ends here: the unit before this one (the block before's last column, for column 0)
    constexpr int unit = c == 0 ? C - 1 : c - 1;
    constexpr int free_ones = ((unit + 1 < C || AHEAD) ? kScores : 0) + (unit > 0 ? kTilesD : 0);
    if constexpr (free_ones > 0) {
#pragma unroll
      for (int n = 0; n < free_ones; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, (NNIS_AHEAD_VALU + free_ones - 1) / free_ones, 0);
      }
    }
    if constexpr (unit == C - 1) {
#pragma unroll
      for (int n = 0; n < kTilesD; ++n) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
      }
    }
  }
  if (__any(block_max > rise[c])) {  // (see attend_block)
    float moved = fmaxf(st.m[c], block_max * scale_log2);
    moved = fmaxf(moved, __shfl_xor(moved, 16, kWave));
    moved = fmaxf(moved, __shfl_xor(moved, 32, kWave));
    const float shrink = st.m[c] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(st.m[c] - moved);
    st.l[c] *= shrink;
#pragma unroll
    for (int t = 0; t < kTilesD; ++t) st.o[c][t] = st.o[c][t] * shrink;
    st.m[c] = moved;
    rise[c] = (moved + kLazyRise) / scale_log2;
  }
  f32x4 ahead[2];
  if constexpr (c + 1 < C) {
#pragma unroll
    for (int t = 0; t < 2; ++t) ahead[t] = score_tile(f.keys[t], q[c + 1]);
  } else if constexpr (AHEAD) {
#pragma unroll
    for (int t = 0; t < 2; ++t) ahead[t] = score_tile(next.keys[t], q[0]);
  }
  if constexpr (c > 0) {
#pragma unroll
    for (int t = 0; t < kTilesD; ++t)
      st.o[c - 1][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.values[t], before, st.o[c - 1][t], 0, 0, 0);
  }
  // (No key of these blocks is masked: behind the test above the reference is a score's own size, never -inf.)
  const float base = st.m[c];
  bf16x8 p;
  float w[8];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      w[4 * t + e] = __builtin_amdgcn_exp2f(fmaf(s[t][e], scale_log2, -base));
      p[4 * t + e] = (__bf16)w[4 * t + e];
    }
  st.l[c] += ((w[0] + w[1]) + (w[2] + w[3])) + ((w[4] + w[5]) + (w[6] + w[7]));
  if constexpr (c + 1 < C) {
    before = p;
  } else {
#pragma unroll
    for (int t = 0; t < kTilesD; ++t) st.o[c][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.values[t], p, st.o[c][t], 0, 0, 0);
  }
  if constexpr (c + 1 < C || AHEAD) {
    s[0] = ahead[0];
    s[1] = ahead[1];
  }
  if constexpr (c + 1 < C) attend_unit_ahead<C, AHEAD, c + 1>(st, q, f, next, s, before, scale_log2, rise);
}

template <int C, bool AHEAD>
__device__ __forceinline__ void attend_block_ahead(AttnState<C>& st, const QFrag (&q)[C], const BlockFrags& f, const BlockFrags& next,
                                                   f32x4 (&s)[2], float scale_log2, float (&rise)[C]) {
  bf16x8 before;  // the probabilities of the column before, whose outputs are still to be multiplied
  attend_unit_ahead<C, AHEAD, 0>(st, q, f, next, s, before, scale_log2, rise);
}

// The pages of a run of key blocks, 64 at a time in the lanes of the wave: a
// block's page is a lane broadcast, not a dependent load in front of every block.
struct PageRun {
  const int* pages;
  int max_pages;
  int first, stride;  // lane i holds the page at index first + i * stride of the sequence's block-table row
  int cached;
  __device__ __forceinline__ void fill(int lane) {
    int index = first + lane * stride;
    index = index < max_pages ? index : max_pages - 1;
    cached = pages[index];
  }
  __device__ __forceinline__ int page(int i) const { return __shfl(cached, i, kWave); }
};

struct MfmaArgs {
  const bf16_t* q;  // [tokens, heads, HD]
  bf16_t* out;      // [tokens, heads, HD]
  const bf16_t* k_pages;
  const bf16_t* v_pages;
  const int* block_table;
  int max_pages;
  int rows_by_token;  // decode: block_table holds a row per token of the step (the step's tables), not per slot
  int heads, kv_heads;
  int window;
  float scale_log2;
  // prefill: one work item per (sequence, tile of 16*QT query rows)
  const int* tile_seq;    // [tiles] sequence of the tile
  const int* tile_row0;   // [tiles] first row of the tile within its sequence's new tokens
  const int* seq_slot;    // [batch]
  const int* seq_start;   // [batch + 1] first packed row of each sequence
  const int* seq_pos0;    // [batch] position of a sequence's first new token
  // decode: one token per sequence
  const int* tok_slot;    // [tokens]
  const int* tok_pos;     // [tokens]
  int splits, heads_first;
  float* partial;         // [tokens, heads, splits, kPartial] when splits > 1: HD outputs, maximum, sum
};

__device__ __forceinline__ const bf16_t* k_page_ptr(const MfmaArgs& a, int page, int kv_head) {
  return a.k_pages + ((size_t)page * a.kv_heads + kv_head) * nnis_k_page_elems(HD);
}
__device__ __forceinline__ const bf16_t* v_page_ptr(const MfmaArgs& a, int page, int kv_head) {
  return a.v_pages + ((size_t)page * a.kv_heads + kv_head) * nnis_v_page_elems(HD);
}

// A wave's state in LDS, for another wave to take in: per column the output tiles as 16 bytes a lane
// ([tile][lane][4]: one store or load a tile), then the reference and the sum ([lane] each);
// kStateFloats floats a column.
constexpr int kStateFloats = (kTilesD * 4 + 2) * kWave;

template <int C>
__device__ __forceinline__ void leave_state(const AttnState<C>& st, float* slot, int lane) {
#pragma unroll
  for (int c = 0; c < C; ++c) {
    float* col = slot + (size_t)c * kStateFloats;
#pragma unroll
    for (int t = 0; t < kTilesD; ++t) *(f32x4*)(col + (t * kWave + lane) * 4) = st.o[c][t];
    col[kTilesD * 4 * kWave + lane] = st.m[c];
    col[(kTilesD * 4 + 1) * kWave + lane] = st.l[c];
  }
}

// st becomes the softmax state of its keys and the other wave's together
template <int C>
__device__ __forceinline__ void take_state(AttnState<C>& st, const float* slot, int lane) {
#pragma unroll
  for (int c = 0; c < C; ++c) {
    const float* col = slot + (size_t)c * kStateFloats;
    const float m_other = col[kTilesD * 4 * kWave + lane];
    const float l_other = col[(kTilesD * 4 + 1) * kWave + lane];
    f32x4 theirs[kTilesD];
#pragma unroll
    for (int t = 0; t < kTilesD; ++t) theirs[t] = *(const f32x4*)(col + (t * kWave + lane) * 4);
    const float m_new = fmaxf(st.m[c], m_other);
    const float m_safe = m_new == -INFINITY ? 0.0f : m_new;
    const float mine_w = __builtin_amdgcn_exp2f(st.m[c] - m_safe);
    const float their_w = __builtin_amdgcn_exp2f(m_other - m_safe);
    st.l[c] = st.l[c] * mine_w + l_other * their_w;
    st.m[c] = m_new;
#pragma unroll
    for (int t = 0; t < kTilesD; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) st.o[c][t][e] = st.o[c][t][e] * mine_w + theirs[t][e] * their_w;
  }
}

// Waves of a block (a power of two) that dealt a run of key blocks among themselves fold their states
// into wave 0's, in halving rounds: the upper half of the waves still in play leave their states in LDS,
// the lower half take one each.  Returns false for the waves that are done.  `merge` holds
// [waves / 2][C][kTilesD * 4 + 2][64] floats.
template <int C>
__device__ __forceinline__ bool merge_waves(AttnState<C>& st, float* merge, int wave, int waves, int lane) {
  for (int half = waves >> 1; half >= 1; half >>= 1) {
    if (wave >= half && wave < 2 * half) leave_state<C>(st, merge + (size_t)(wave - half) * C * kStateFloats, lane);
    __syncthreads();
    if (wave < half) take_state<C>(st, merge + (size_t)wave * C * kStateFloats, lane);
    if (half > 1) __syncthreads();  // the next round writes where this one read
  }
  return wave == 0;
}

// The same for a group of `size` waves of the block, of any size, this wave its member `index`: in each round the
// upper half of the members still in play (rounded down) hand their states to the lower ones through `slots`
// (room for size / 2 states).  Every wave of the block runs `rounds` rounds, so that groups of different sizes
// meet at the same barriers; a group that is done early only waits.  Returns true for the member that is left.
template <int C>
__device__ __forceinline__ bool merge_group(AttnState<C>& st, float* slots, int index, int size, int rounds, int lane) {
  int n = size;
  for (int round = 0; round < rounds; ++round) {
    const int keep = (n + 1) / 2;  // members [keep, n) hand over to members [0, n - keep)
    if (index >= keep && index < n) leave_state<C>(st, slots + (size_t)(index - keep) * C * kStateFloats, lane);
    __syncthreads();
    if (index < n - keep) take_state<C>(st, slots + (size_t)index * C * kStateFloats, lane);
    if (round + 1 < rounds) __syncthreads();  // the next round writes where this one read
    n = keep;
  }
  return index == 0;
}

// Runs the pages first, first + stride, ... (`mine` of them) of a sequence through the
// softmax state, each as two blocks of 32 keys one after the other (so both halves of a
// value line are used while it is near).  RING blocks' operands are in flight at a time:
// a block's place is asked for again as soon as it has been worked on.  A load behind a
// branch makes the compiler take it for not issued when it counts what may still be in
// flight at a use, and every block then waits for all the loads asked for after its own.  So
// a run of at least two rounds goes through a loop of whole rounds whose every block has a
// successor RING on, RING blocks in one straight line with nothing behind a branch; what is
// left of it, and a short run, take the loop that looks at every block.  Blocks that start
// beyond `last_key` are left out.
template <int C, int RING>
__device__ __forceinline__ void attend_run(AttnState<C>& st, const QFrag (&q)[C], const MfmaArgs& a, const int* pages,
                                           int kv_head, int first, int stride, int mine, int last_key,
                                           const int (&lo)[C], const int (&hi)[C], int lane) {
  // (The run's bounds are the same in every lane -- they come from sums over the wave -- but the compiler has them
  // in vector registers unless it is told: as scalars the loop's counters, the pages' numbers and the pages'
  // addresses cost no vector instruction, of which the loop has none to spare.)
  first = __builtin_amdgcn_readfirstlane(first);
  stride = __builtin_amdgcn_readfirstlane(stride);
  mine = __builtin_amdgcn_readfirstlane(mine);
  last_key = __builtin_amdgcn_readfirstlane(last_key);
  if (mine <= 0) return;
  const int r = lane % 16, g = lane / 16;
  const bf16_t* k_base = k_page_ptr(a, 0, kv_head);
  const bf16_t* v_base = v_page_ptr(a, 0, kv_head);
  const size_t k_page_stride = (size_t)a.kv_heads * nnis_k_page_elems(HD), v_page_stride = (size_t)a.kv_heads * nnis_v_page_elems(HD);
  PageRun run = {pages, a.max_pages, first, stride, 0};
  run.fill(lane);
  // block b of the run: page index first + (b / 2) * stride, half b % 2
  int blocks = 2 * mine;
  if ((first + (mine - 1) * stride) * kPageTokens + 32 > last_key) --blocks;  // the last page's second half is beyond the keys
  BlockFrags ring[RING];
  // blocks are asked for in rising order, so the 64 cached page ids move on with them
  auto ask = [&](BlockFrags& into, int b) {
    const int n = b >> 1;
    if ((b & 1) == 0 && n > 0 && (n & 63) == 0) {
      run.first = first + n * stride;
      run.fill(lane);
    }
    const int page = __builtin_amdgcn_readfirstlane(run.page(n & 63));
    load_block(into, k_base + page * k_page_stride, v_base + page * v_page_stride, b & 1, r, g);
  };
  auto work = [&](const BlockFrags& f, int b) {
    attend_block<C>(st, q, f, (first + (b >> 1) * stride) * kPageTokens + (b & 1) * 32, lo, hi, a.scale_log2, g);
  };
  int b0 = 0;
  if (blocks >= 2 * RING) {
#pragma unroll
    for (int i = 0; i < RING; ++i) ask(ring[i], i);
  } else {
#pragma unroll
    for (int i = 0; i < RING; ++i)
      if (i < blocks) ask(ring[i], i);
  }
  // The blocks all of whose keys count for every column of every lane lie together in the middle of the run (in
  // a causal step without a window: at its start): pages n of the run with every_lo <= their keys <= every_hi.
  // (A dead column has hi = -1: then there are none.)
  int every_lo = lo[0], every_hi = hi[0];
#pragma unroll
  for (int c = 1; c < C; ++c) {
    every_lo = max(every_lo, lo[c]);
    every_hi = min(every_hi, hi[c]);
  }
#pragma unroll
  for (int offset = kWave / 2; offset > 0; offset >>= 1) {
    every_lo = max(every_lo, __shfl_xor(every_lo, offset, kWave));
    every_hi = min(every_hi, __shfl_xor(every_hi, offset, kWave));
  }
  every_lo = __builtin_amdgcn_readfirstlane(every_lo);
  every_hi = __builtin_amdgcn_readfirstlane(every_hi);
  const int whole_pages = (every_hi + 1) / kPageTokens;  // pages 0 .. whole_pages - 1 of the sequence end at or below every_hi
  const int inner_end = whole_pages > first ? 2 * min(mine, (whole_pages - first + stride - 1) / stride) : 0;  // in blocks of the run
  const int low_page = (every_lo + kPageTokens - 1) / kPageTokens;
  int inner_begin = low_page > first ? 2 * ((low_page - first + stride - 1) / stride) : 0;
  inner_begin = (inner_begin + RING - 1) / RING * RING;  // whole rounds of the ring
  // blocks before them (a window's edge) one by one
  for (; b0 < inner_begin && b0 < blocks; b0 += RING) {
#pragma unroll
    for (int i = 0; i < RING; ++i) {
      const int b = b0 + i;
      if (b < blocks) {
        work(ring[i], b);
        if (b + RING < blocks) ask(ring[i], b + RING);
      }
    }
  }
  // whole rounds of them whose every block has a successor RING on: one straight line, nothing behind a branch
  if (b0 + 2 * RING <= blocks && b0 + RING <= inner_end) {
    constexpr bool kAhead = RING > 1;  // (with one block in flight the next is asked for only when this one is done)
    f32x4 s[2];
    if (kAhead) {
#pragma unroll
      for (int t = 0; t < 2; ++t) s[t] = score_tile(ring[0].keys[t], q[0]);
    }
    float rise[C];
#pragma unroll
    for (int c = 0; c < C; ++c) rise[c] = (st.m[c] + kLazyRise) / a.scale_log2;  // (-inf before a column's first key)
    for (; b0 + 2 * RING <= blocks && b0 + RING <= inner_end; b0 += RING) {
#pragma unroll
      for (int i = 0; i < RING; ++i) {
        if (!kAhead) {
#pragma unroll
          for (int t = 0; t < 2; ++t) s[t] = score_tile(ring[i].keys[t], q[0]);
        }
        attend_block_ahead<C, kAhead>(st, q, ring[i], ring[(i + 1) % RING], s, a.scale_log2, rise);
        ask(ring[i], b0 + i + RING);
      }
    }
  }
  // what is left (the diagonal, a short run) one by one
  for (; b0 < blocks; b0 += RING) {
#pragma unroll
    for (int i = 0; i < RING; ++i) {
      const int b = b0 + i;
      if (b < blocks) {
        work(ring[i], b);
        if (b + RING < blocks) ask(ring[i], b + RING);
      }
    }
  }
}

// key blocks a prefilling wave has in flight: as many as its registers hold beside C columns' states.  Beyond 96
// channels two columns and two blocks need more than 256 registers, which leaves a SIMD one wave: with one block
// in flight two waves fit, and the other wave's work fills the wait (32/8 heads of 128, one wave an item, at 8,192
// tokens 833 -> 687 us a layer, 24/8 heads of 112 922 -> 652; at 80 and 96 channels, where two waves fit either
// way, the second block in flight is worth 5 to 8%).
template <int C>
constexpr int kPrefillRing = HD > 96 ? (C <= 1 ? 2 : 1) : (HD > 64 ? 2 : (C <= 2 ? NNIS_PREFILL_RING_NARROW : NNIS_PREFILL_RING_WIDE));

// ---- prefill: a wave = (query tile, kv head, chunk of GH query heads); C = QT * GH column tiles --------
// An item is a (tile, kv head, chunk of heads); the tiles come longest first, and item i = tile i / per_tile.
// A tile's work grows with its place in its sequence, and a chip with fewer items than twice its compute
// units runs them all at once: its time is the most loaded unit's.  So the grid is folded: block b < singles
// has item b alone, block b >= singles has item b and item items - 1 - (b - singles), a heavy and a light
// one, side by side: the block's waves are dealt to the two in proportion to their pages (an item's time is
// mostly the chain of loads before its first key and the merge after its last, which the two now spend
// together; one after the other a 2,048-token prefill of 9/3 heads took 22 us a layer here, side by side 18).
template <int QT, int GH>
__global__ __launch_bounds__(64 * kBlockWaves) void attention_prefill_kernel(MfmaArgs a, int waves, int items, int singles,
                                                                            int per_tile) {
  extern __shared__ __attribute__((aligned(16))) float merge[];
  constexpr int C = QT * GH;
  const int lane = threadIdx.x % kWave, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), r = lane % 16, g = lane / 16;  // (the wave's number as a scalar)
  const int group = a.heads / a.kv_heads;
  const int chunks = (group + GH - 1) / GH;
  // both items' places in the step, asked for together: each is a chain of dependent loads
  const int count = (int)blockIdx.x < singles ? 1 : 2;
  int item_of[2], seq_of[2], row0_of[2], slot_of[2], start_of[2], rows_of[2], pos0_of[2];
#pragma unroll
  for (int which = 0; which < 2; ++which) {
    item_of[which] = which == 0 ? (int)blockIdx.x : items - 1 - ((int)blockIdx.x - singles);
    const int tile = (which < count ? item_of[which] : item_of[0]) / per_tile;
    seq_of[which] = __builtin_amdgcn_readfirstlane(a.tile_seq[tile]);
    row0_of[which] = __builtin_amdgcn_readfirstlane(a.tile_row0[tile]);
  }
#pragma unroll
  for (int which = 0; which < 2; ++which) {
    slot_of[which] = __builtin_amdgcn_readfirstlane(a.seq_slot[seq_of[which]]);
    start_of[which] = __builtin_amdgcn_readfirstlane(a.seq_start[seq_of[which]]);
    rows_of[which] = __builtin_amdgcn_readfirstlane(a.seq_start[seq_of[which] + 1]) - start_of[which];
    pos0_of[which] = __builtin_amdgcn_readfirstlane(a.seq_pos0[seq_of[which]]);
  }
  // which: the item; this wave is member `index` of the `size` waves that take it; slots: their room for the merge
  auto run_item = [&](int which, int index, int size, float* slots, int rounds) __attribute__((always_inline)) {
    const int part = item_of[which] % per_tile;
    const int kv_head = part / chunks;
    const int head0 = kv_head * group + (part % chunks) * GH;
    const int row0 = row0_of[which], start = start_of[which], rows = rows_of[which], pos0 = pos0_of[which];
    const int* pages = a.block_table + (size_t)slot_of[which] * a.max_pages;

    QFrag q[C];
    int lo[C], hi[C];
    bool live[C];
    int last = -1;
#pragma unroll
    for (int qt = 0; qt < QT; ++qt)
#pragma unroll
      for (int gh = 0; gh < GH; ++gh) {
        const int c = qt * GH + gh;
        const int row = row0 + 16 * qt + r;
        const int head = head0 + gh;
        live[c] = row < rows && head < kv_head * group + group;
        const int safe_row = row < rows ? row : rows - 1;
        const int safe_head = head < a.heads ? head : a.heads - 1;
        q[c] = load_row_operand(a.q + ((size_t)(start + safe_row) * a.heads + safe_head) * HD, g);
        hi[c] = live[c] ? pos0 + row : -1;
        lo[c] = (a.window > 0 && hi[c] + 1 > a.window) ? hi[c] + 1 - a.window : 0;
        last = hi[c] > last ? hi[c] : last;
      }
    // the wave runs to the farthest key any of its columns reads, from the nearest
    int first = 0x7fffffff;
#pragma unroll
    for (int c = 0; c < C; ++c) first = (live[c] && lo[c] < first) ? lo[c] : first;
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) {
      last = max(last, __shfl_xor(last, offset, kWave));
      first = min(first, __shfl_xor(first, offset, kWave));
    }
    AttnState<C> st;
    init_state(st);
    if (last >= 0) {
      const int first_page = first / kPageTokens, page_count = last / kPageTokens + 1 - first_page;
      const int mine = page_count > index ? (page_count - index + size - 1) / size : 0;  // pages of this wave
      attend_run<C, kPrefillRing<C>>(st, q, a, pages, kv_head, first_page + index, size, mine, last, lo, hi, lane);
    }
    if (!merge_group<C>(st, slots, index, size, rounds, lane)) return;
#pragma unroll
    for (int qt = 0; qt < QT; ++qt)
#pragma unroll
      for (int gh = 0; gh < GH; ++gh) {
        const int c = qt * GH + gh;
        float total = st.l[c];
        total += __shfl_xor(total, 16, kWave);
        total += __shfl_xor(total, 32, kWave);
        if (!live[c]) continue;
        const float inv = 1.0f / total;
        bf16_t* dst = a.out + ((size_t)(start + row0 + 16 * qt + r) * a.heads + head0 + gh) * HD;
#pragma unroll
        for (int t = 0; t < kTilesD; ++t) {
          bf16x4 packed;
#pragma unroll
          for (int e = 0; e < 4; ++e) packed[e] = (__bf16)(st.o[c][t][e] * inv);
          *(bf16x4*)(dst + 16 * t + 4 * g) = packed;
        }
      }
  };
  int rounds = 0;
  while ((1 << rounds) < waves) ++rounds;
  if (count == 1) {
    run_item(0, wave, waves, merge, rounds);
  } else if (waves == 1) {
    run_item(0, 0, 1, merge, 0);
    run_item(1, 0, 1, merge, 0);
  } else {
    // pages of the two (up to the last row's position; a window's lower end does not matter for the shares)
    int pages_of[2];
#pragma unroll
    for (int which = 0; which < 2; ++which) {
      const int rows_here = min(row0_of[which] + 16 * QT, rows_of[which]);
      pages_of[which] = (pos0_of[which] + rows_here - 1) / kPageTokens + 1;
    }
    // shares in proportion to the pages, at least one wave each (a group of n waves needs n / 2 states of room, rounded
    // down, for its merge: the two groups' rooms lie behind one another and come to at most waves / 2 together).  With
    // even shares only, four waves went 2 + 2 whatever the pages: 30 pages beside 3 were 15 a wave where 3 + 1 give 10.
    // The shares that leave the busiest wave the fewest pages (in proportion to the pages, 21 beside 12 went 3 + 1:
    // 12 pages on the light item's one wave where 2 + 2 give 11 and 6).
    int first_share = 1, fewest = 0x7fffffff;
    for (int share = 1; share < waves; ++share) {
      const int most = max((pages_of[0] + share - 1) / share, (pages_of[1] + waves - share - 1) / (waves - share));
      if (most < fewest) {
        fewest = most;
        first_share = share;
      }
    }
    if (wave < first_share) run_item(0, wave, first_share, merge, rounds);
    else run_item(1, wave - first_share, waves - first_share, merge + (size_t)(first_share / 2) * C * kStateFloats, rounds);
  }
}

// The end of a decode block: the waves' states merge in LDS; the wave that is left writes the output
// (one split) or leaves its state in `partial` for the combine kernel.
template <int C>
__device__ __forceinline__ void finish_decode(AttnState<C>& st, const bool (&live)[C], const MfmaArgs& a, float* merge,
                                              int token, int kv_head, int split, int wave, int waves, int lane) {
  const int r = lane % 16, g = lane / 16;
  const int group = a.heads / a.kv_heads;
  if (!merge_waves<C>(st, merge, wave, waves, lane)) return;  // one wave is left
  float total[C];
#pragma unroll
  for (int c = 0; c < C; ++c) {
    total[c] = st.l[c];
    total[c] += __shfl_xor(total[c], 16, kWave);
    total[c] += __shfl_xor(total[c], 32, kWave);
  }
  if (a.splits == 1) {
#pragma unroll
    for (int c = 0; c < C; ++c) {
      if (!live[c]) continue;
      const float inv = 1.0f / total[c];
      bf16_t* dst = a.out + ((size_t)token * a.heads + kv_head * group + 16 * c + r) * HD;
#pragma unroll
      for (int t = 0; t < kTilesD; ++t) {
        bf16x4 packed;
#pragma unroll
        for (int e = 0; e < 4; ++e) packed[e] = (__bf16)(st.o[c][t][e] * inv);
        *(bf16x4*)(dst + 16 * t + 4 * g) = packed;
      }
    }
    return;
  }
#pragma unroll
  for (int c = 0; c < C; ++c) {
    if (!live[c]) continue;
    float* dst = a.partial + (((size_t)token * a.heads + kv_head * group + 16 * c + r) * a.splits + split) * kPartial;
#pragma unroll
    for (int t = 0; t < kTilesD; ++t) *(f32x4*)(dst + 16 * t + 4 * g) = st.o[c][t];
    if (g == 0) {
      dst[HD] = st.m[c];
      dst[HD + 1] = total[c];
    }
  }
}

// ---- decode: a block = (token, kv head, split of the keys); columns are the heads of the group; ------
// the block's waves deal the split's pages among themselves and merge their states through LDS.  With
// more than one split every block leaves its state in `partial` for the combine kernel.
template <int C>
__global__ __launch_bounds__(64 * kBlockWaves) void attention_decode_kernel(MfmaArgs a, int waves) {
  extern __shared__ __attribute__((aligned(16))) float merge[];  // [waves / 2][C][kTilesD * 4 + 2][64]
  const int lane = threadIdx.x % kWave, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), r = lane % 16, g = lane / 16;  // (the wave's number as a scalar)
  const int token = a.heads_first ? blockIdx.y : blockIdx.x, kv_head = a.heads_first ? blockIdx.x : blockIdx.y, split = blockIdx.z;
  // With the step's tables a token's pages are a row of its own and nothing is asked of its slot: the first
  // pages' numbers are one round trip away, not two.  (A padding row then reads the page its row names, 0,
  // and leaves a result that nobody reads.)
  int slot = 0;
  if (!a.rows_by_token) {
    slot = a.tok_slot[token];
    if (slot < 0) return;  // a padding row (the whole block leaves): its output is never read
  }
  const int group = a.heads / a.kv_heads;
  const int pos = a.tok_pos[token];
  const int first_key = (a.window > 0 && pos + 1 > a.window) ? pos + 1 - a.window : 0;
  const int* pages = a.block_table + (size_t)(a.rows_by_token ? token : slot) * a.max_pages;

  QFrag q[C];
  int lo[C], hi[C];
  bool live[C];
#pragma unroll
  for (int c = 0; c < C; ++c) {
    const int member = 16 * c + r;
    live[c] = member < group;
    const int head = kv_head * group + (live[c] ? member : 0);
    q[c] = load_row_operand(a.q + ((size_t)token * a.heads + head) * HD, g);
    lo[c] = first_key;
    hi[c] = live[c] ? pos : -1;
  }
  // pages are dealt to the splits in contiguous runs, and within a split to the waves in turn
  const int page_first = first_key / kPageTokens, page_count = pos / kPageTokens + 1 - page_first;
  const int per_split = (page_count + a.splits - 1) / a.splits;
  const int begin = page_first + split * per_split;
  const int end = min(begin + per_split, page_first + page_count);
  AttnState<C> st;
  init_state(st);
  const int mine = end > begin + wave ? (end - begin - wave + waves - 1) / waves : 0;  // pages of this wave
  attend_run<C, (kDecodeRing / C >= 2 ? kDecodeRing / C : 2)>(st, q, a, pages, kv_head, begin + wave, waves, mine, pos, lo, hi, lane);
  finish_decode<C>(st, live, a, merge, token, kv_head, split, wave, waves, lane);
}

// ---- decode with keys on lanes, for groups of up to 4 query heads ------------------------------------
// The kernel above spends a lane on every (key, column) pair of a 16-column tile, of which a small
// group fills a few.  Here scores are taken with v_mfma_f32_4x4x4_16B_bf16, sixteen products of 4x4
// at a time: block b of the instruction multiplies keys 4b .. 4b+3 of a page (first operand: lane l
// holds 4 channels of key l) by the group's heads (second operand: lane 4b+j holds the same channels
// of head j), so lane 4b+j ends up with the scores of its head for its four keys and the softmax
// arithmetic of a page of 64 keys x 4 heads is four values a lane.  The probabilities go through LDS
// into the columns operand of the 16x16x32 product with the value page, whose outputs and end are
// those of the kernel above (heads in columns 0..3).  All lanes of a head share one reference of the
// softmax, which moves only when a score rises more than kLazyRise above it (then every lane's
// sums are scaled, as in the running maximum; until then they are sums of 2^(score - reference) with
// terms up to 2^kLazyRise, which changes no result beyond rounding).
#if NNIS_HEAD_DIM <= 128
struct KeysPage {
  bf16x8 k[HD / 8];        // this lane's key, all channels
  bf16x8 v[2][kTilesD];    // value operands of the two halves of the page
};

__device__ __forceinline__ void load_keys_page(KeysPage& f, const bf16_t* k_page, const bf16_t* v_page, int lane) {
  const int r = lane % 16, g = lane / 16;
#pragma unroll
  for (int c = 0; c < HD / 8; ++c) f.k[c] = *(const bf16x8*)(k_page + nnis_k_offset(lane, 8 * c));
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int t = 0; t < kTilesD; ++t) f.v[h][t] = *(const bf16x8*)(v_page + nnis_v_offset(16 * t + r, 32 * h + 8 * g));
}

__device__ __forceinline__ bf16x4 low4(bf16x8 v) { return __builtin_shufflevector(v, v, 0, 1, 2, 3); }
__device__ __forceinline__ bf16x4 high4(bf16x8 v) { return __builtin_shufflevector(v, v, 4, 5, 6, 7); }

__global__ __launch_bounds__(64 * kKeysWaves) void attention_decode_keys_kernel(MfmaArgs a, int waves) {
  extern __shared__ __attribute__((aligned(16))) float merge[];  // [waves / 2][kTilesD * 4 + 2][64]
  constexpr int kStageRow = kPageTokens + 8;  // bfloat16 per head: a page's probabilities, rows apart in the banks
  __shared__ __attribute__((aligned(16))) bf16_t stage[kKeysWaves][4][kStageRow];
  const int lane = threadIdx.x % kWave, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), r = lane % 16, g = lane / 16;  // (the wave's number as a scalar)
  const int blk = lane / 4, j = lane % 4;  // the scores' layout: keys 4 blk .. 4 blk + 3 of a page, head j of the group
  const int token = a.heads_first ? blockIdx.y : blockIdx.x, kv_head = a.heads_first ? blockIdx.x : blockIdx.y, split = blockIdx.z;
  int slot = 0;
  if (!a.rows_by_token) {  // (see attention_decode_kernel)
    slot = a.tok_slot[token];
    if (slot < 0) return;  // a padding row (the whole block leaves): its output is never read
  }
  const int group = a.heads / a.kv_heads;
  const int pos = a.tok_pos[token];
  const int first_key = (a.window > 0 && pos + 1 > a.window) ? pos + 1 - a.window : 0;
  const int* pages = a.block_table + (size_t)(a.rows_by_token ? token : slot) * a.max_pages;

  // the query of head j, all channels (heads beyond the group: zeros, their columns are never written)
  bf16x8 q[HD / 8];
  {
    const bf16_t* row = a.q + ((size_t)token * a.heads + kv_head * group + (j < group ? j : 0)) * HD;
#pragma unroll
    for (int c = 0; c < HD / 8; ++c) {
      q[c] = *(const bf16x8*)(row + 8 * c);
      if (j >= group) {
#pragma unroll
        for (int e = 0; e < 8; ++e) q[c][e] = (__bf16)0.0f;
      }
    }
  }
  const int page_first = first_key / kPageTokens, page_count = pos / kPageTokens + 1 - page_first;
  const int per_split = (page_count + a.splits - 1) / a.splits;
  const int begin = page_first + split * per_split;
  const int end = min(begin + per_split, page_first + page_count);
  const int mine = end > begin + wave ? (end - begin - wave + waves - 1) / waves : 0;  // pages of this wave
  const int first = begin + wave, stride = waves;

  AttnState<1> st;
  init_state(st);
  float reference = -INFINITY;  // of head j; equal in all lanes of the head
  float sum = 0.0f;             // this lane's part of the head's sum
  if (mine > 0) {
    const bf16_t* k_base = k_page_ptr(a, 0, kv_head);
    const bf16_t* v_base = v_page_ptr(a, 0, kv_head);
    const size_t k_page_stride = (size_t)a.kv_heads * nnis_k_page_elems(HD), v_page_stride = (size_t)a.kv_heads * nnis_v_page_elems(HD);
    PageRun run = {pages, a.max_pages, first, stride, 0};
    run.fill(lane);
    KeysPage ring[kKeysRing];
    auto ask = [&](KeysPage& into, int n) {
      if (n > 0 && (n & 63) == 0) {
        run.first = first + n * stride;
        run.fill(lane);
      }
      const int page = __builtin_amdgcn_readfirstlane(run.page(n & 63));
      load_keys_page(into, k_base + page * k_page_stride, v_base + page * v_page_stride, lane);
    };
    bf16_t* mine_stage = &stage[wave][0][0];
    // page n of this wave's run, whose operands are in f, through the softmax state
    auto work = [&](const KeysPage& f, int n) {
      const int key0 = (first + n * stride) * kPageTokens;
      // scores of this lane's head for keys key0 + 4 blk + (0..3): two chains of products, added
      f32x4 s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int c = 0; c < HD / 8; ++c) {
        s0 = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(low4(f.k[c]), low4(q[c]), s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(high4(f.k[c]), high4(q[c]), s1, 0, 0, 0);
      }
      f32x4 s = s0 + s1;
      const bool inside = key0 >= first_key && key0 + kPageTokens - 1 <= pos;  // every key of the page is read
      float top = -INFINITY;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int key = key0 + 4 * blk + e;
        s[e] = (inside || (key >= first_key && key <= pos)) ? s[e] * a.scale_log2 : -INFINITY;
        top = fmaxf(top, s[e]);
      }
      if (__any(top > reference + kLazyRise)) {  // also the first page, whose reference is -inf
        float moved = fmaxf(reference, top);
#pragma unroll
        for (int offset = 4; offset < kWave; offset <<= 1) moved = fmaxf(moved, __shfl_xor(moved, offset, kWave));
        // the lanes 16 g + r with r < 4 hold head r in both layouts: the outputs are scaled by the same factor
        const float shrink = reference == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(reference - moved);
        sum *= shrink;
#pragma unroll
        for (int t = 0; t < kTilesD; ++t) st.o[0][t] = st.o[0][t] * shrink;
        reference = moved;
      }
      const float base = reference == -INFINITY ? 0.0f : reference;
      bf16x4 p;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float w = __builtin_amdgcn_exp2f(s[e] - base);
        sum += w;
        p[e] = (__bf16)w;
      }
      // through LDS into the columns operand: column = head, 8 consecutive keys a lane
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();  // the reads of the page before are done
      *(bf16x4*)(mine_stage + j * kStageRow + 4 * blk) = p;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        bf16x8 columns = *(const bf16x8*)(mine_stage + (r < 4 ? r : 0) * kStageRow + 32 * h + 8 * g);
        if (r >= 4) {
#pragma unroll
          for (int e = 0; e < 8; ++e) columns[e] = (__bf16)0.0f;
        }
#pragma unroll
        for (int t = 0; t < kTilesD; ++t)
          st.o[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.v[h][t], columns, st.o[0][t], 0, 0, 0);
      }
    };
    // A run of at least two rounds: whole rounds whose every page has a successor kKeysRing on, in one straight
    // line with no load behind a branch (see attend_run); the rest, and a short run, page by page.
    int n0 = 0;
    if (mine >= 2 * kKeysRing) {
#pragma unroll
      for (int i = 0; i < kKeysRing; ++i) ask(ring[i], i);
      for (; n0 + 2 * kKeysRing <= mine; n0 += kKeysRing) {
#pragma unroll
        for (int i = 0; i < kKeysRing; ++i) {
          work(ring[i], n0 + i);
          ask(ring[i], n0 + i + kKeysRing);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < kKeysRing; ++i)
        if (i < mine) ask(ring[i], i);
    }
    for (; n0 < mine; n0 += kKeysRing) {
#pragma unroll
      for (int i = 0; i < kKeysRing; ++i) {
        const int n = n0 + i;
        if (n >= mine) continue;
        work(ring[i], n);
        if (n + kKeysRing < mine) ask(ring[i], n + kKeysRing);
      }
    }
  }
  // into the state the end works on: a column's maximum in its lanes, and parts of its sum that add up over
  // the lane groups g -- the lanes 16 g + r, r < 4, take the sums of the blocks 4 g .. 4 g + 3 of head r
  sum += __shfl_xor(sum, 4, kWave);
  sum += __shfl_xor(sum, 8, kWave);
  st.m[0] = reference;
  st.l[0] = sum;
  bool live[1] = {r < group && r < 4};
  if (r >= 4) {  // columns that hold no head
    st.m[0] = -INFINITY;
    st.l[0] = 0.0f;
  }
  finish_decode<1>(st, live, a, merge, token, kv_head, split, wave, waves, lane);
}
#endif  // NNIS_HEAD_DIM <= 128

// sums the splits of one (token, head): out = sum_s O_s 2^(m_s - M) / sum_s l_s 2^(m_s - M).
// A kernel of its own: letting the last block of a (token, kv head) do it needs a device-wide fence in
// every block, which was measured several times dearer than this launch.
__global__ void attention_combine_kernel(const float* __restrict__ partial, bf16_t* __restrict__ out,
                                         const int* __restrict__ tok_slot, int heads, int splits) {
  const int token = blockIdx.x, head = blockIdx.y;
  const float* base = partial + ((size_t)token * heads + head) * splits * kPartial;
  constexpr int kAtOnce = 8;  // runs whose references, sums and outputs a thread asks for together: one round trip
  if (splits <= kAtOnce) {
    // a padding row's runs hold whatever the scratch held: they are read like any (the slot is asked for in the
    // same round trip, not before it) and nothing is stored for them
    const int slot = tok_slot[token];
    for (int d = threadIdx.x; d < HD; d += blockDim.x) {
      float m[kAtOnce], l[kAtOnce], o[kAtOnce];
#pragma unroll
      for (int s = 0; s < kAtOnce; ++s) {
        const float* p = base + (size_t)(s < splits ? s : splits - 1) * kPartial;  // (beyond the last: the last again, not counted)
        m[s] = p[HD];
        l[s] = p[HD + 1];
        o[s] = p[d];
      }
      float m_all = -INFINITY;
#pragma unroll
      for (int s = 0; s < kAtOnce; ++s) m_all = s < splits ? fmaxf(m_all, m[s]) : m_all;
      float num = 0.0f, den = 0.0f;
#pragma unroll
      for (int s = 0; s < kAtOnce; ++s) {
        if (s < splits) {
          const float w = m[s] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m[s] - m_all);
          num += o[s] * w;
          den += l[s] * w;
        }
      }
      if (slot >= 0) out[((size_t)token * heads + head) * HD + d] = (bf16_t)(num / den);
    }
    return;
  }
  if (tok_slot[token] < 0) return;
  float m_all = -INFINITY;
  for (int s = 0; s < splits; ++s) m_all = fmaxf(m_all, base[(size_t)s * kPartial + HD]);
  for (int d = threadIdx.x; d < HD; d += blockDim.x) {
    float num = 0.0f, den = 0.0f;
    for (int s = 0; s < splits; ++s) {
      const float* p = base + (size_t)s * kPartial;
      const float m = p[HD];
      const float w = m == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m - m_all);
      num += p[d] * w;
      den += p[HD + 1] * w;
    }
    out[((size_t)token * heads + head) * HD + d] = (bf16_t)(num / den);
  }
}

#endif  // NNIS_HEAD_DIM % 16 == 0

}  // namespace

extern "C" int nnis_attention_rows(const void* q, int q_dtype, void* out, int out_dtype, const void* k_pages,
                                   const void* v_pages, int cache_dtype, const int* block_table, int max_pages,
                                   const int* tok_slot, const int* tok_pos, int tokens, int heads, int kv_heads,
                                   int head_dim, int window, float scale, void* stream) {
  NNIS_REQUIRE(head_dim == HD, "attention: this module is compiled for head_dim %d, got %d", HD, head_dim);
  NNIS_REQUIRE(nnis_dtype_ok(q_dtype) && nnis_dtype_ok(out_dtype) && nnis_dtype_ok(cache_dtype),
               "attention: unknown dtype (q %d, out %d, cache %d)", q_dtype, out_dtype, cache_dtype);
  NNIS_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "attention: %d heads do not divide into %d kv heads",
               heads, kv_heads);
  NNIS_REQUIRE(window >= 0 && max_pages > 0, "attention: bad window %d or block table width %d", window, max_pages);
  if (tokens <= 0) return 0;
  AttnArgs a;
  a.q = q; a.q_dtype = q_dtype; a.out = out; a.out_dtype = out_dtype;
  a.k_pages = k_pages; a.v_pages = v_pages; a.cache_dtype = cache_dtype;
  a.block_table = block_table; a.max_pages = max_pages; a.tok_slot = tok_slot; a.tok_pos = tok_pos;
  a.tokens = tokens; a.heads = heads; a.kv_heads = kv_heads; a.window = window; a.scale = scale;
  const long long items = (long long)tokens * heads;
  const unsigned blocks = (unsigned)((items + 3) / 4);
  if (cache_dtype == NNIS_F32) {
    hipLaunchKernelGGL(attention_rows_kernel<float>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, a);
  } else {
    hipLaunchKernelGGL(attention_rows_kernel<bf16_t>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, a);
  }
  NNIS_LAUNCH_CHECK("attention_rows");
  return 0;
}


#if NNIS_HEAD_DIM % 16 == 0
namespace {
constexpr int kMaxColumns = HD <= 64 ? 4 : (HD <= 128 ? 2 : 1);  // column tiles a wave carries (registers)

int fill_common(MfmaArgs& a, const void* q, void* out, const void* k_pages, const void* v_pages, const int* block_table,
                int max_pages, int heads, int kv_heads, int head_dim, int window, float scale) {
  NNIS_REQUIRE(head_dim == HD, "attention: this module is compiled for head_dim %d, got %d", HD, head_dim);
  NNIS_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "attention: %d heads do not divide into %d kv heads",
               heads, kv_heads);
  NNIS_REQUIRE(window >= 0 && max_pages > 0, "attention: bad window %d or block table width %d", window, max_pages);
  NNIS_REQUIRE(scale > 0.0f, "attention: the scale of the scores must be positive");
  NNIS_REQUIRE(((uintptr_t)q % 16 == 0) && ((uintptr_t)out % 16 == 0) && ((uintptr_t)k_pages % 16 == 0) &&
                   ((uintptr_t)v_pages % 16 == 0),
               "attention: operands must be 16-byte aligned");
  a.q = (const bf16_t*)q; a.out = (bf16_t*)out; a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages;
  a.block_table = block_table; a.max_pages = max_pages; a.heads = heads; a.kv_heads = kv_heads; a.window = window;
  a.scale_log2 = scale * kLog2e;
  a.tile_seq = a.tile_row0 = a.seq_slot = a.seq_start = a.seq_pos0 = a.tok_slot = a.tok_pos = nullptr;
  a.splits = 1; a.heads_first = 0; a.partial = nullptr; a.rows_by_token = 0;
  return 0;
}
}  // namespace

// compute units of the device in use (the library serves one device a process)
static int compute_units() {
  static const int units = [] {
    int device = 0, n = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || n <= 0)
      n = 256;
    return n;
  }();
  return units;
}

// rows of 16*QT queries per tile, as the host must cut them
// `columns`: the most column tiles a wave carries, 1 .. kMaxColumns (0: as many as the head size allows).
// Fewer columns mean more, lighter blocks and more waves to deal a tile's keys to.
static void prefill_shape(int heads, int kv_heads, int columns, int* qt, int* gh) {
  const int group = heads / (kv_heads > 0 ? kv_heads : 1);
  const int most = (columns >= 1 && columns < kMaxColumns) ? columns : kMaxColumns;
  *gh = group < most ? group : most;
  if (*gh < 1) *gh = 1;
  *qt = most / *gh;
  if (*qt == 3) *qt = 2;  // query tiles come in 1, 2 or 4
}

extern "C" int nnis_attention_prefill_tile_rows(int heads, int kv_heads, int columns) {
  int qt, gh;
  prefill_shape(heads, kv_heads, columns, &qt, &gh);
  return 16 * qt;
}

// the most LDS a block's merge takes: half its waves leave a state at a time (eight waves of four columns at 64
// channels: 72 KB)
constexpr size_t kMergeLdsMost = 96 * 1024;

// waves a block of the prefill kernel may have for these sizes (LDS of the merge)
extern "C" int nnis_attention_prefill_max_waves(int heads, int kv_heads, int columns) {
  int qt, gh;
  prefill_shape(heads, kv_heads, columns, &qt, &gh);
  const size_t per_wave = (size_t)qt * gh * (kTilesD * 4 + 2) * kWave * sizeof(float);
  int waves = 1;  // a power of two; half of them leave a state in LDS at a time
  while (waves * 2 <= kBlockWaves && waves * per_wave <= kMergeLdsMost) waves *= 2;
  return waves;
}

extern "C" int nnis_attention_prefill_bf16(const void* q, void* out, const void* k_pages, const void* v_pages,
                                           const int* block_table, int max_pages, const int* tile_seq,
                                           const int* tile_row0, int tiles, const int* seq_slot, const int* seq_start,
                                           const int* seq_pos0, int heads, int kv_heads, int head_dim, int window,
                                           float scale, int waves, int columns, void* stream) {
  MfmaArgs a;
  if (fill_common(a, q, out, k_pages, v_pages, block_table, max_pages, heads, kv_heads, head_dim, window, scale)) return 1;
  if (tiles <= 0) return 0;
  a.tile_seq = tile_seq; a.tile_row0 = tile_row0; a.seq_slot = seq_slot; a.seq_start = seq_start; a.seq_pos0 = seq_pos0;
  const int group = heads / kv_heads;
  int qt, gh;
  prefill_shape(heads, kv_heads, columns, &qt, &gh);
  const int chunks = (group + gh - 1) / gh;
  const int per_tile = kv_heads * chunks;
  NNIS_REQUIRE((long long)tiles * per_tile <= 0x7fffffff, "attention: %d tiles x %d head chunks exceed the grid limit", tiles, per_tile);
  const int items = tiles * per_tile;
  // blocks: one per item while each compute unit gets at most one; beyond that two items a block, until
  // every block has two
  const int units = compute_units();
  const int blocks = std::max((items + 1) / 2, std::min(items, units));
  const int singles = 2 * blocks - items;
  const dim3 grid(blocks);
  const size_t per_wave = (size_t)qt * gh * (kTilesD * 4 + 2) * kWave * sizeof(float);
  NNIS_REQUIRE(waves >= 1 && waves <= kBlockWaves && (waves & (waves - 1)) == 0 && (waves / 2) * per_wave <= kMergeLdsMost,
               "attention: %d waves a block: a power of two that fits this head size (LDS) is needed", waves);
  const size_t lds = (waves / 2) * per_wave;
  const dim3 block(kWave * waves);
  hipStream_t s = (hipStream_t)stream;
  // (beyond 64 KB a kernel has to be told once; a refusal shows as the launch's failure)
#define NNIS_PREFILL(QT_, GH_)                                                                                          \
  do {                                                                                                                  \
    static const hipError_t allowed = hipFuncSetAttribute((const void*)attention_prefill_kernel<QT_, GH_>,              \
                                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMergeLdsMost); \
    (void)allowed;                                                                                                      \
    hipLaunchKernelGGL((attention_prefill_kernel<QT_, GH_>), grid, block, lds, s, a, waves, items, singles, per_tile); \
  } while (0)
  bool launched = true;
  if constexpr (kMaxColumns >= 4) {
    if (qt == 4 && gh == 1) NNIS_PREFILL(4, 1);
    else if (qt == 2 && gh == 2) NNIS_PREFILL(2, 2);
    else if (qt == 1 && gh == 3) NNIS_PREFILL(1, 3);
    else if (qt == 1 && gh == 4) NNIS_PREFILL(1, 4);
    else launched = false;
  } else {
    launched = false;
  }
  if (!launched) {
    launched = true;
    if constexpr (kMaxColumns >= 2) {
      if (qt == 2 && gh == 1) NNIS_PREFILL(2, 1);
      else if (qt == 1 && gh == 2) NNIS_PREFILL(1, 2);
      else launched = false;
    } else {
      launched = false;
    }
  }
  if (!launched) {
    if (qt == 1 && gh == 1) NNIS_PREFILL(1, 1);
    else return nnis_fail("attention: no kernel for %d query tiles x %d heads", qt, gh);
  }
#undef NNIS_PREFILL
  NNIS_LAUNCH_CHECK("attention_prefill");
  return 0;
}

extern "C" int nnis_attention_decode_max_waves(int heads, int kv_heads) {
  const int group = heads / (kv_heads > 0 ? kv_heads : 1);
  const int tiles = (group + 15) / 16;
  const int per_wave = tiles * (kTilesD * 4 + 2) * kWave * 4;  // bytes of LDS a wave's state takes in the merge
  const int most = (group <= 4 && HD <= kKeysMaxHD && kKeysWaves < kBlockWaves) ? kKeysWaves : kBlockWaves;
  int waves = 1;
  while (waves * 2 <= most && waves * per_wave <= 65536) waves *= 2;
  return waves;
}

// With splits > 1 the call needs scratch memory: `partial`, float32 of at least tokens * heads * splits *
// (head_dim + 4), contents of no matter.  Two calls that run at the same time must not share it.
// kind: 0 picks the kernel (keys on lanes for groups of up to 4 heads, else heads in columns); 1 and 2 ask
// for columns or keys on lanes and fail where that kernel does not take the sizes.  combine: 0 leaves the
// runs in `partial` ([tokens, heads, splits, head_dim + 4]: outputs, reference, sum) and writes no output: the
// projection that follows, or nnis_attention_combine, adds them up.
extern "C" int nnis_attention_decode_bf16(const void* q, void* out, const void* k_pages, const void* v_pages,
                                          const int* block_table, int max_pages, const int* tok_slot, const int* tok_pos,
                                          int tokens, int heads, int kv_heads, int head_dim, int window, float scale,
                                          int splits, int waves, float* partial, int kind, int combine, int rows_by_token,
                                          void* stream) {
  MfmaArgs a;
  if (fill_common(a, q, out, k_pages, v_pages, block_table, max_pages, heads, kv_heads, head_dim, window, scale)) return 1;
  a.rows_by_token = rows_by_token ? 1 : 0;
  NNIS_REQUIRE(splits >= 1 && splits <= 65535, "attention: bad number of splits %d", splits);
  NNIS_REQUIRE(splits == 1 || partial != nullptr, "attention: splits need scratch memory");
  NNIS_REQUIRE((uintptr_t)partial % 16 == 0, "attention: scratch memory must be 16-byte aligned");
  NNIS_REQUIRE(kv_heads <= 65535, "attention: %d kv heads exceed the grid limit", kv_heads);
  NNIS_REQUIRE(waves >= 1 && waves <= nnis_attention_decode_max_waves(heads, kv_heads) && (waves & (waves - 1)) == 0,
               "attention: %d waves a block; this head size and group take a power of two up to %d", waves,
               nnis_attention_decode_max_waves(heads, kv_heads));
  if (tokens <= 0) return 0;
  const int group = heads / kv_heads;
  NNIS_REQUIRE(group <= 16 * kMaxColumns, "attention: a group of %d query heads is more than this head size's decode kernel carries (%d)",
               group, 16 * kMaxColumns);
  NNIS_REQUIRE(kind >= 0 && kind <= 2, "attention: unknown decode kernel %d", kind);
  const bool keys_fit = group <= 4 && HD <= kKeysMaxHD;
  NNIS_REQUIRE(kind != 2 || keys_fit, "attention: the kernel with keys on lanes takes groups of up to 4 heads of up to %d channels",
               kKeysMaxHD);
  a.tok_slot = tok_slot; a.tok_pos = tok_pos; a.splits = splits; a.partial = partial;
  // Blocks go to the chip's 8 dies in turn.  With the tokens as the grid's fastest index a die runs all heads of its
  // tokens: its L2 holds a token's query, pages' numbers and tables once (8 tokens on 9/3 heads: 9,470 tokens/s
  // against 9,200 with a token's blocks spread), but a long sequence's keys all come through one die.  Where the
  // key/value heads deal evenly to the dies (a multiple of 8) they are the fastest index: every die then reads an
  // eighth of every sequence (32/32 heads of 64, unequal lengths up to 2k keys: 64 tokens 15,330 -> 16,860 tokens/s in
  // whole steps, 8 tokens 5,430 -> 5,515; 32/8 heads of 128: 60,700 -> 62,150 and 11,950 -> 12,020).
  // (4 and 3 key/value heads as the fastest index at 16 to 64 tokens: 0.3% slower in whole steps.)
  a.heads_first = kv_heads % 8 == 0 && tokens <= 65535;
  const dim3 grid(a.heads_first ? kv_heads : tokens, a.heads_first ? tokens : kv_heads, splits);
  hipStream_t s = (hipStream_t)stream;
  const int tiles = (group + 15) / 16;
  const size_t lds = (size_t)(waves / 2) * tiles * (kTilesD * 4 + 2) * kWave * sizeof(float);
#if NNIS_HEAD_DIM <= 128
  {
    if (kind == 2 || (kind == 0 && keys_fit)) {
      hipLaunchKernelGGL(attention_decode_keys_kernel, grid, dim3(kWave * waves), lds, s, a, waves);
      NNIS_LAUNCH_CHECK("attention_decode");
      if (splits > 1 && combine) {
        hipLaunchKernelGGL(attention_combine_kernel, dim3(tokens, heads), dim3(HD < 64 ? 64 : (HD > 256 ? 256 : HD)), 0, s,
                           partial, (bf16_t*)out, tok_slot, heads, splits);
        NNIS_LAUNCH_CHECK("attention_combine");
      }
      return 0;
    }
  }
#endif
  if (tiles == 1) hipLaunchKernelGGL((attention_decode_kernel<1>), grid, dim3(kWave * waves), lds, s, a, waves);
  else if (tiles == 2) hipLaunchKernelGGL((attention_decode_kernel<(kMaxColumns >= 2 ? 2 : 1)>), grid, dim3(kWave * waves), lds, s, a, waves);
  else hipLaunchKernelGGL((attention_decode_kernel<kMaxColumns>), grid, dim3(kWave * waves), lds, s, a, waves);  // 3 or 4 tiles
  NNIS_LAUNCH_CHECK("attention_decode");
  if (splits > 1 && combine) {
    hipLaunchKernelGGL(attention_combine_kernel, dim3(tokens, heads), dim3(HD < 64 ? 64 : (HD > 256 ? 256 : HD)), 0, s, partial,
                       (bf16_t*)out, tok_slot, heads, splits);
    NNIS_LAUNCH_CHECK("attention_combine");
  }
  return 0;
}

// The sum over the key runs that a call with combine = 0 left in `partial`, for a consumer that does not
// take the runs as they are.
extern "C" int nnis_attention_combine(const float* partial, void* out, const int* tok_slot, int tokens, int heads, int head_dim,
                                      int splits, void* stream) {
  NNIS_REQUIRE(head_dim == HD, "attention: this module is compiled for head_dim %d, got %d", HD, head_dim);
  NNIS_REQUIRE(partial && out && tok_slot && splits >= 1 && heads > 0, "attention_combine: missing operand");
  if (tokens <= 0) return 0;
  hipLaunchKernelGGL(attention_combine_kernel, dim3(tokens, heads), dim3(HD < 64 ? 64 : (HD > 256 ? 256 : HD)), 0,
                     (hipStream_t)stream, partial, (bf16_t*)out, tok_slot, heads, splits);
  NNIS_LAUNCH_CHECK("attention_combine");
  return 0;
}
#else
extern "C" int nnis_attention_prefill_tile_rows(int, int, int) { return 0; }
extern "C" int nnis_attention_prefill_max_waves(int, int, int) { return 1; }
extern "C" int nnis_attention_prefill_bf16(const void*, void*, const void*, const void*, const int*, int, const int*, const int*,
                                           int, const int*, const int*, const int*, int, int, int, int, float, int, int, void*) {
  return nnis_fail("attention: the matrix-core kernels need a head size in steps of 16; this module has %d", NNIS_HEAD_DIM);
}
extern "C" int nnis_attention_decode_max_waves(int, int) { return 1; }
extern "C" int nnis_attention_combine(const float*, void*, const int*, int, int, int, int, void*) {
  return nnis_fail("attention: the matrix-core kernels need a head size in steps of 16; this module has %d", NNIS_HEAD_DIM);
}
extern "C" int nnis_attention_decode_bf16(const void*, void*, const void*, const void*, const int*, int, const int*, const int*,
                                          int, int, int, int, int, float, int, int, float*, int, int, int, void*) {
  return nnis_fail("attention: the matrix-core kernels need a head size in steps of 16; this module has %d", NNIS_HEAD_DIM);
}
#endif
