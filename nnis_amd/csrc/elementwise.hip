// Row-wise kernels of the decoder: embedding gather, RMSNorm (optionally fused
// with the residual sum and a row gather), rotate-half RoPE fused with the
// write of keys and values into cache pages, SiLU-multiply and argmax.
// Storage types are chosen at run time (32-bit float or bfloat16); every sum,
// statistic and rotation is computed in 32-bit.
#include "common.h"
#include "nnis_noalloc.h"

#include <mutex>

thread_local char g_nnis_error[512] = {0};

extern "C" const char* nnis_last_error() { return g_nnis_error; }

// -----------------------------------------------------------------------------
// embedding: out[t, :] = table[ids[t], :]   (a row copy, no scaling;
// /root/reference/crates/nnis-kernels/src/gather.rs:17-33)
// -----------------------------------------------------------------------------
__global__ void embed_kernel(const int* __restrict__ ids, const void* __restrict__ table, int table_dtype,
                             float* __restrict__ out, int width, int vocab) {
  const int token = blockIdx.x;
  const int id = ids[token];
  float* dst = out + (size_t)token * width;
  if (id < 0 || id >= vocab) {  // padding rows carry -1; never read outside the table
    for (int c = threadIdx.x; c < width; c += blockDim.x) dst[c] = 0.0f;
    return;
  }
  const size_t base = (size_t)id * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) dst[c] = load_as_f32(table, table_dtype, base + c);
}

extern "C" int nnis_embed(const int* ids, const void* table, int table_dtype, float* out, int tokens, int width,
                          int vocab, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(table_dtype), "embed: unknown table dtype %d", table_dtype);
  NNIS_REQUIRE(tokens >= 0 && width > 0 && vocab > 0, "embed: bad sizes tokens=%d width=%d vocab=%d", tokens, width, vocab);
  if (tokens == 0) return 0;
  hipLaunchKernelGGL(embed_kernel, dim3(tokens), dim3(256), 0, (hipStream_t)stream, ids, table, table_dtype, out,
                     width, vocab);
  NNIS_LAUNCH_CHECK("embed");
  return 0;
}

// The same row copy out of a table kept in the packed order of the matrix-core products (common.h): a head
// that shares the table needs that order, and the table is then kept once.  8 consecutive channels of a row lie
// together (16 bytes); a thread copies one such piece.
__global__ void embed_packed_kernel(const int* __restrict__ ids, const bf16_t* __restrict__ packed,
                                    float* __restrict__ out, int width, int vocab) {
  const int token = blockIdx.x;
  const int id = ids[token];
  float* dst = out + (size_t)token * width;
  const bool inside = id >= 0 && id < vocab;
  const size_t strip = inside ? (size_t)(id >> 4) * nnis_packed_strip_elems(width) : 0;
  for (int k = threadIdx.x * 8; k < width; k += blockDim.x * 8) {
    uint4 piece = make_uint4(0, 0, 0, 0);
    if (inside) {
      const size_t at = strip + (size_t)(k / 64) * kPackedChunkElems + (size_t)((k % 16) / 8) * kPackedHalfElems +
                        (size_t)(16 * ((k % 64) / 16) + (id & 15)) * 8;
      piece = *(const uint4*)(packed + at);
    }
    const uint32_t words[4] = {piece.x, piece.y, piece.z, piece.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {  // bfloat16 widens by a shift
      dst[k + 2 * i] = __uint_as_float(words[i] << 16);
      dst[k + 2 * i + 1] = __uint_as_float(words[i] & 0xffff0000u);
    }
  }
}

extern "C" int nnis_embed_packed(const int* ids, const void* packed, float* out, int tokens, int width, int vocab,
                                 void* stream) {
  NNIS_REQUIRE(tokens >= 0 && width > 0 && vocab > 0, "embed: bad sizes tokens=%d width=%d vocab=%d", tokens, width, vocab);
  NNIS_REQUIRE(width % 8 == 0, "embed: a packed table has a width that is a multiple of 8, got %d", width);
  if (tokens == 0) return 0;
  hipLaunchKernelGGL(embed_packed_kernel, dim3(tokens), dim3(64 * ((width / 8 + 63) / 64 > 4 ? 4 : (width / 8 + 63) / 64)), 0,
                     (hipStream_t)stream, ids, (const bf16_t*)packed, out, width, vocab);
  NNIS_LAUNCH_CHECK("embed_packed");
  return 0;
}

// -----------------------------------------------------------------------------
// The step's tables: what every layer's kernels would otherwise look up again through each token's slot and
// position, gathered once per step by token: its rows of the rotation tables, the cache page that takes its
// key and value, and (for a step of single tokens) the pages of its sequence.  A kernel that reads them has
// nothing to wait for before it can ask for its data.  A padding row (negative slot) gets the identity
// rotation, page -1 and, as its sequence's only page, page 0 (read by nobody who stores a result).
// -----------------------------------------------------------------------------
__global__ __launch_bounds__(64) void step_tables_kernel(const int* __restrict__ tok_slot, const int* __restrict__ tok_pos,
                                                         const float* __restrict__ cos_table, const float* __restrict__ sin_table,
                                                         int half, int table_positions, const int* __restrict__ block_table,
                                                         int max_pages, float* __restrict__ tok_cos, float* __restrict__ tok_sin,
                                                         int* __restrict__ tok_page, int* __restrict__ tok_pages) {
  const int token = blockIdx.x;
  const int slot = tok_slot[token];
  int pos = tok_pos[token];
  const bool live = slot >= 0 && pos >= 0;
  if (cos_table) {
    const int row = live && pos < table_positions ? pos : 0;
    for (int c = threadIdx.x; c < half; c += blockDim.x) {
      tok_cos[(size_t)token * half + c] = live ? cos_table[(size_t)row * half + c] : 1.0f;
      tok_sin[(size_t)token * half + c] = live ? sin_table[(size_t)row * half + c] : 0.0f;
    }
  }
  if (block_table) {
    const int* row = block_table + (size_t)(live ? slot : 0) * max_pages;
    int last = live ? pos / kPageTokens : 0;
    last = last < max_pages ? last : max_pages - 1;
    if (threadIdx.x == 0) tok_page[token] = live ? row[last] : -1;
    if (tok_pages)
      for (int i = threadIdx.x; i <= last; i += blockDim.x) tok_pages[(size_t)token * max_pages + i] = live ? row[i] : 0;
  }
}

// tok_cos / tok_sin: [tokens, half] (with cos_table); tok_page: [tokens] and tok_pages: [tokens, max_pages] or
// null (with block_table).  Either half of the work may be left out (null tables).
extern "C" int nnis_step_tables(const int* tok_slot, const int* tok_pos, int tokens, const float* cos_table,
                                const float* sin_table, int half, int table_positions, const int* block_table, int max_pages,
                                float* tok_cos, float* tok_sin, int* tok_page, int* tok_pages, void* stream) {
  NNIS_REQUIRE(tokens >= 0 && tok_slot && tok_pos, "step_tables: the tokens' slots and positions are missing");
  NNIS_REQUIRE((cos_table == nullptr) == (sin_table == nullptr), "step_tables: cos and sin tables come together");
  NNIS_REQUIRE(cos_table == nullptr || (half > 0 && table_positions > 0 && tok_cos && tok_sin), "step_tables: rotation rows need a place and sizes");
  NNIS_REQUIRE(block_table == nullptr || (max_pages > 0 && tok_page), "step_tables: pages need a place and the table's width");
  if (tokens == 0 || (cos_table == nullptr && block_table == nullptr)) return 0;
  hipLaunchKernelGGL(step_tables_kernel, dim3(tokens), dim3(64), 0, (hipStream_t)stream, tok_slot, tok_pos, cos_table, sin_table,
                     half, table_positions, block_table, max_pages, tok_cos, tok_sin, tok_page, tok_pages);
  NNIS_LAUNCH_CHECK("step_tables");
  return 0;
}

// -----------------------------------------------------------------------------
// RMSNorm: y[c] = (x[c] * (1/sqrt(mean(x^2) + eps))) * w[c]
// (/root/reference/crates/nnis-model/src/kernels.rs:15-48: eps inside the
// root, mean over the row, x*scale*weight in that order).
//   delta != null : the row normalised is x + delta (sum in 32-bit); without
//                   `rows` the sum is written back to x, which must be 32-bit.
//   rows  != null : output row r reads input row rows[r]; nothing is written back.
// -----------------------------------------------------------------------------
__global__ void rmsnorm_kernel(void* __restrict__ x, int x_dtype, const void* __restrict__ delta, int delta_dtype,
                               const void* __restrict__ weight, int weight_dtype, void* __restrict__ out,
                               int out_dtype, const int* __restrict__ rows, int width, float inv_width, float eps) {
  __shared__ float scratch[16];
  const int out_row = blockIdx.x;
  const int in_row = rows ? rows[out_row] : out_row;
  const size_t in_base = (size_t)in_row * width;
  const size_t out_base = (size_t)out_row * width;
  const bool write_back = delta != nullptr && rows == nullptr;

  float sumsq = 0.0f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float v = load_as_f32(x, x_dtype, in_base + c);
    if (delta) {
      v += load_as_f32(delta, delta_dtype, in_base + c);
      if (write_back) ((float*)x)[in_base + c] = v;
    }
    sumsq = fmaf(v, v, sumsq);
  }
  const float total = block_sum(sumsq, scratch);
  const float scale = 1.0f / sqrtf(total * inv_width + eps);
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float v = load_as_f32(x, x_dtype, in_base + c);  // holds the sum already when written back
    if (delta && !write_back) v += load_as_f32(delta, delta_dtype, in_base + c);
    store_from_f32(out, out_dtype, out_base + c, (v * scale) * load_as_f32(weight, weight_dtype, c));
  }
}

// One wave per row, the row held in registers: a single pass over memory and no
// block barrier.  Needs width % 4 == 0 (16-byte accesses) and width <= 256 * CH.
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;

__device__ __forceinline__ f32x4_t load4_as_f32(const void* base, int dtype, size_t index) {
  if (dtype == NNIS_F32) return *(const f32x4_t*)((const float*)base + index);
  const bf16x4_t v = *(const bf16x4_t*)((const bf16_t*)base + index);
  return (f32x4_t){(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}

__device__ __forceinline__ void store4_from_f32(void* base, int dtype, size_t index, f32x4_t v) {
  if (dtype == NNIS_F32) {
    *(f32x4_t*)((float*)base + index) = v;
  } else {
    bf16x4_t packed;
#pragma unroll
    for (int e = 0; e < 4; ++e) packed[e] = (__bf16)v[e];
    *(bf16x4_t*)((bf16_t*)base + index) = packed;
  }
}

template <int CH>
__global__ __launch_bounds__(256) void rmsnorm_wave_kernel(void* __restrict__ x, int x_dtype, const void* __restrict__ delta,
                                                           int delta_dtype, const void* __restrict__ weight, int weight_dtype,
                                                           void* __restrict__ out, int out_dtype, const int* __restrict__ rows,
                                                           int out_rows, int width, float inv_width, float eps) {
  const int lane = threadIdx.x % kWave;
  const int out_row = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (out_row >= out_rows) return;
  const int in_row = rows ? rows[out_row] : out_row;
  const size_t in_base = (size_t)in_row * width;
  const size_t out_base = (size_t)out_row * width;
  const bool write_back = delta != nullptr && rows == nullptr;
  f32x4_t v[CH];
  float sumsq = 0.0f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int col = 4 * (lane + kWave * c);
    if (col < width) {
      v[c] = load4_as_f32(x, x_dtype, in_base + col);
      if (delta) {
        v[c] += load4_as_f32(delta, delta_dtype, in_base + col);
        if (write_back) *(f32x4_t*)((float*)x + in_base + col) = v[c];
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) sumsq = fmaf(v[c][e], v[c][e], sumsq);
    }
  }
  const float scale = 1.0f / sqrtf(wave_sum(sumsq) * inv_width + eps);
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int col = 4 * (lane + kWave * c);
    if (col < width) {
      const f32x4_t w = load4_as_f32(weight, weight_dtype, col);
      store4_from_f32(out, out_dtype, out_base + col, (v[c] * scale) * w);
    }
  }
}

template <int CH>
static void launch_rmsnorm_wave(void* x, int x_dtype, const void* delta, int delta_dtype, const void* weight, int weight_dtype,
                                void* out, int out_dtype, const int* rows, int out_rows, int width, float eps,
                                hipStream_t stream) {
  const int waves = out_rows >= 1024 ? 4 : 1;  // few rows: one wave a block, spread over the chip
  hipLaunchKernelGGL(rmsnorm_wave_kernel<CH>, dim3((out_rows + waves - 1) / waves), dim3(waves * kWave), 0, stream, x,
                     x_dtype, delta, delta_dtype, weight, weight_dtype, out, out_dtype, rows, out_rows, width,
                     1.0f / (float)width, eps);
}

extern "C" int nnis_rmsnorm(void* x, int x_dtype, const void* delta, int delta_dtype, const void* weight,
                            int weight_dtype, void* out, int out_dtype, const int* rows, int out_rows, int width,
                            float eps, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(x_dtype) && nnis_dtype_ok(weight_dtype) && nnis_dtype_ok(out_dtype),
               "rmsnorm: unknown dtype (x %d, weight %d, out %d)", x_dtype, weight_dtype, out_dtype);
  NNIS_REQUIRE(delta == nullptr || nnis_dtype_ok(delta_dtype), "rmsnorm: unknown delta dtype %d", delta_dtype);
  NNIS_REQUIRE(!(delta != nullptr && rows == nullptr && x_dtype != NNIS_F32),
               "rmsnorm: the residual sum is kept in 32-bit; x must be float32 when delta is added in place");
  NNIS_REQUIRE(out_rows >= 0 && width > 0, "rmsnorm: bad sizes rows=%d width=%d", out_rows, width);
  NNIS_REQUIRE(eps > 0.0f, "rmsnorm: eps must be positive, got %g", (double)eps);
  if (out_rows == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const bool aligned = ((uintptr_t)x % 16 == 0) && ((uintptr_t)out % 16 == 0) && ((uintptr_t)weight % 16 == 0) &&
                       (delta == nullptr || (uintptr_t)delta % 16 == 0);
  if (width % 4 == 0 && aligned && width <= 256 * 32) {
    const int chunks = (width + 255) / 256;
#define NNIS_NORM_CASE(CH)                                                                                          \
  launch_rmsnorm_wave<CH>(x, x_dtype, delta, delta_dtype, weight, weight_dtype, out, out_dtype, rows, out_rows, width, \
                          eps, s)
    if (chunks <= 1) NNIS_NORM_CASE(1);
    else if (chunks <= 2) NNIS_NORM_CASE(2);
    else if (chunks <= 3) NNIS_NORM_CASE(3);
    else if (chunks <= 4) NNIS_NORM_CASE(4);
    else if (chunks <= 8) NNIS_NORM_CASE(8);
    else if (chunks <= 16) NNIS_NORM_CASE(16);
    else NNIS_NORM_CASE(32);
#undef NNIS_NORM_CASE
    NNIS_LAUNCH_CHECK("rmsnorm_wave");
    return 0;
  }
  const int threads = width >= 1024 ? 256 : (width >= 256 ? 128 : 64);
  hipLaunchKernelGGL(rmsnorm_kernel, dim3(out_rows), dim3(threads), 0, s, x, x_dtype, delta,
                     delta_dtype, weight, weight_dtype, out, out_dtype, rows, width, 1.0f / (float)width, eps);
  NNIS_LAUNCH_CHECK("rmsnorm");
  return 0;
}

// -----------------------------------------------------------------------------
// rotate-half RoPE on queries and keys, fused with the cache write.
//   qkv   [tokens, (heads + 2*kv_heads) * head_dim] : q heads, then k heads, then v heads
//   q_out [tokens, heads * head_dim]
//   K page layout  [page][kv_head][token in page][head_dim]
//   V page layout  [page][kv_head][head_dim][token in page]   (keys contiguous)
// pair j < rot_dim/2 of a head:  out[j] = x[j]*c - x[j+half]*s,
//                                out[j+half] = x[j+half]*c + x[j]*s
// with (c, s) = table[pos][j]  (/root/reference/crates/nnis-model/src/runtime_kernels.rs:38-66);
// elements at and beyond rot_dim pass through.  V is not rotated
// (/root/reference/crates/nnis-model/src/runtime.rs:997-1016).
// A token whose slot is negative is padding: nothing is written for it.
// -----------------------------------------------------------------------------
struct RopeWriteArgs {
  const void* qkv;
  int qkv_dtype;
  void* q_out;
  int q_dtype;
  const float* cos_table;  // [positions][rot_dim/2] or null (no rotation)
  const float* sin_table;
  int table_positions;
  int rot_dim;
  const int* tok_slot;
  const int* tok_pos;
  void* k_pages;  // null: this run keeps no cache of its own
  void* v_pages;
  int cache_dtype;
  const int* block_table;  // [slots][max_pages]
  int max_pages;
  int heads, kv_heads, head_dim;
};

__global__ void rope_kv_write_kernel(RopeWriteArgs a) {
  const int token = blockIdx.x;
  const int slot = a.tok_slot[token];
  if (slot < 0) return;
  const int pos = a.tok_pos[token];
  const int hd = a.head_dim;
  const int half = a.rot_dim / 2;
  const int row_width = (a.heads + 2 * a.kv_heads) * hd;
  const size_t in_base = (size_t)token * row_width;
  const bool rotate = a.cos_table != nullptr && pos < a.table_positions;
  const float* cos_row = rotate ? a.cos_table + (size_t)pos * half : nullptr;
  const float* sin_row = rotate ? a.sin_table + (size_t)pos * half : nullptr;

  int page = -1;
  if (a.k_pages) page = a.block_table[(size_t)slot * a.max_pages + pos / kPageTokens];
  const int in_page = pos % kPageTokens;

  // queries and keys: one work item per (head, element below head_dim/2 or pass-through element)
  const int rot_heads = a.heads + a.kv_heads;
  const int items_per_head = hd - half;  // `half` rotated pairs + (hd - rot_dim) pass-through elements
  for (int item = threadIdx.x; item < rot_heads * items_per_head; item += blockDim.x) {
    const int head = item / items_per_head;
    const int e = item % items_per_head;
    const size_t src = in_base + (size_t)head * hd;
    float lo, hi = 0.0f;
    int lo_index, hi_index = -1;
    if (e < half) {
      const float x0 = load_as_f32(a.qkv, a.qkv_dtype, src + e);
      const float x1 = load_as_f32(a.qkv, a.qkv_dtype, src + e + half);
      float c = 1.0f, s = 0.0f;
      if (rotate) {
        c = cos_row[e];
        s = sin_row[e];
      }
      lo = x0 * c - x1 * s;
      hi = x1 * c + x0 * s;
      lo_index = e;
      hi_index = e + half;
    } else {
      lo_index = e + half;  // element index in [rot_dim, head_dim)
      lo = load_as_f32(a.qkv, a.qkv_dtype, src + lo_index);
    }
    if (head < a.heads) {
      const size_t dst = ((size_t)token * a.heads + head) * hd;
      store_from_f32(a.q_out, a.q_dtype, dst + lo_index, lo);
      if (hi_index >= 0) store_from_f32(a.q_out, a.q_dtype, dst + hi_index, hi);
    } else if (page >= 0) {
      const int kv_head = head - a.heads;
      const size_t dst = ((size_t)page * a.kv_heads + kv_head) * nnis_k_page_elems(hd);
      store_from_f32(a.k_pages, a.cache_dtype, dst + nnis_k_offset(in_page, lo_index), lo);
      if (hi_index >= 0) store_from_f32(a.k_pages, a.cache_dtype, dst + nnis_k_offset(in_page, hi_index), hi);
    }
  }
  // values: copied into the page's order
  if (page >= 0) {
    const size_t v_src = in_base + (size_t)(a.heads + a.kv_heads) * hd;
    for (int item = threadIdx.x; item < a.kv_heads * hd; item += blockDim.x) {
      const int kv_head = item / hd;
      const int d = item % hd;
      const float v = load_as_f32(a.qkv, a.qkv_dtype, v_src + item);
      const size_t dst = ((size_t)page * a.kv_heads + kv_head) * nnis_v_page_elems(hd) + nnis_v_offset(d, in_page);
      store_from_f32(a.v_pages, a.cache_dtype, dst, v);
    }
  }
}

// The same for bfloat16 throughout with rot_dim / 2 and head_dim - rot_dim multiples of 4: a
// thread takes 4 consecutive pairs (or 4 pass-through or value channels), 8- and 16-byte accesses.
__global__ void rope_kv_write_bf16_kernel(RopeWriteArgs a) {
  const int token = blockIdx.x;
  const int slot = a.tok_slot[token];
  if (slot < 0) return;
  const int pos = a.tok_pos[token];
  const int hd = a.head_dim;
  const int half = a.rot_dim / 2;
  const int row_width = (a.heads + 2 * a.kv_heads) * hd;
  const bf16_t* src = (const bf16_t*)a.qkv + (size_t)token * row_width;
  const bool rotate = a.cos_table != nullptr && pos < a.table_positions;
  int page = -1;
  if (a.k_pages) page = a.block_table[(size_t)slot * a.max_pages + pos / kPageTokens];
  const int in_page = pos % kPageTokens;
  const int rot_heads = a.heads + a.kv_heads;
  const int groups_per_head = (hd - half) / 4;  // half/4 groups of pairs, then (hd - rot_dim)/4 pass-through groups
  const int rot_items = rot_heads * groups_per_head;
  const int v_items = page >= 0 ? a.kv_heads * (hd / 4) : 0;
  for (int item = threadIdx.x; item < rot_items + v_items; item += blockDim.x) {
    if (item < rot_items) {
      const int head = item / groups_per_head;
      const int e = (item % groups_per_head) * 4;
      // where 4 channels from channel `ch` on go: a query row, or the key page (4 channels lie within a chunk of 8)
      bf16_t* q_row = nullptr;
      bf16_t* k_page = nullptr;
      if (head < a.heads) {
        q_row = (bf16_t*)a.q_out + ((size_t)token * a.heads + head) * hd;
      } else {
        if (page < 0) continue;
        k_page = (bf16_t*)a.k_pages + ((size_t)page * a.kv_heads + (head - a.heads)) * nnis_k_page_elems(hd);
      }
      auto place = [&](int ch) { return q_row ? q_row + ch : k_page + nnis_k_offset(in_page, ch); };
      const bf16_t* x = src + (size_t)head * hd;
      if (e < half) {
        const bf16x4_t x0 = *(const bf16x4_t*)(x + e), x1 = *(const bf16x4_t*)(x + e + half);
        f32x4_t c = {1.0f, 1.0f, 1.0f, 1.0f}, sn = {0.0f, 0.0f, 0.0f, 0.0f};
        if (rotate) {
          c = *(const f32x4_t*)(a.cos_table + (size_t)pos * half + e);
          sn = *(const f32x4_t*)(a.sin_table + (size_t)pos * half + e);
        }
        bf16x4_t lo, hi;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float f0 = (float)x0[j], f1 = (float)x1[j];
          lo[j] = (__bf16)(f0 * c[j] - f1 * sn[j]);
          hi[j] = (__bf16)(f1 * c[j] + f0 * sn[j]);
        }
        *(bf16x4_t*)place(e) = lo;
        *(bf16x4_t*)place(e + half) = hi;
      } else {
        *(bf16x4_t*)place(e + half) = *(const bf16x4_t*)(x + e + half);  // channels at and beyond rot_dim
      }
    } else {
      const int v_item = item - rot_items;
      const int kv_head = v_item / (hd / 4);
      const int d = (v_item % (hd / 4)) * 4;
      const bf16x4_t v = *(const bf16x4_t*)(src + (size_t)(a.heads + a.kv_heads + kv_head) * hd + d);
      bf16_t* dst = (bf16_t*)a.v_pages + ((size_t)page * a.kv_heads + kv_head) * nnis_v_page_elems(hd);
#pragma unroll
      for (int j = 0; j < 4; ++j) dst[nnis_v_offset(d + j, in_page)] = v[j];
    }
  }
}

extern "C" int nnis_rope_kv_write(const void* qkv, int qkv_dtype, void* q_out, int q_dtype, const float* cos_table,
                                  const float* sin_table, int table_positions, int rot_dim, const int* tok_slot,
                                  const int* tok_pos, void* k_pages, void* v_pages, int cache_dtype,
                                  const int* block_table, int max_pages, int tokens, int heads, int kv_heads,
                                  int head_dim, void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(qkv_dtype) && nnis_dtype_ok(q_dtype), "rope_kv_write: unknown dtype");
  NNIS_REQUIRE(k_pages == nullptr || nnis_dtype_ok(cache_dtype), "rope_kv_write: unknown cache dtype %d", cache_dtype);
  NNIS_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "rope_kv_write: key and value pages must come together");
  NNIS_REQUIRE(k_pages == nullptr || (block_table != nullptr && max_pages > 0), "rope_kv_write: cache without a block table");
  NNIS_REQUIRE(heads > 0 && kv_heads > 0 && head_dim > 0, "rope_kv_write: bad head sizes %d/%d/%d", heads, kv_heads, head_dim);
  NNIS_REQUIRE(rot_dim >= 0 && rot_dim <= head_dim && rot_dim % 2 == 0,
               "rope_kv_write: rot_dim %d must be even and at most head_dim %d", rot_dim, head_dim);
  NNIS_REQUIRE((cos_table == nullptr) == (sin_table == nullptr), "rope_kv_write: cos and sin tables must come together");
  if (tokens <= 0) return 0;
  RopeWriteArgs a;
  a.qkv = qkv; a.qkv_dtype = qkv_dtype; a.q_out = q_out; a.q_dtype = q_dtype;
  a.cos_table = cos_table; a.sin_table = sin_table; a.table_positions = table_positions;
  a.rot_dim = cos_table ? rot_dim : 0;
  a.tok_slot = tok_slot; a.tok_pos = tok_pos; a.k_pages = k_pages; a.v_pages = v_pages;
  a.cache_dtype = cache_dtype; a.block_table = block_table; a.max_pages = max_pages;
  a.heads = heads; a.kv_heads = kv_heads; a.head_dim = head_dim;
  const bool all_bf16 = qkv_dtype == NNIS_BF16 && q_dtype == NNIS_BF16 && (k_pages == nullptr || cache_dtype == NNIS_BF16);
  const bool aligned = ((uintptr_t)qkv % 16 == 0) && ((uintptr_t)q_out % 16 == 0) && ((uintptr_t)k_pages % 16 == 0) &&
                       ((uintptr_t)v_pages % 16 == 0) && ((uintptr_t)cos_table % 16 == 0) && ((uintptr_t)sin_table % 16 == 0);
  if (all_bf16 && aligned && head_dim % 4 == 0 && (a.rot_dim / 2) % 4 == 0) {
    const int items = (heads + kv_heads) * (head_dim - a.rot_dim / 2) / 4 + kv_heads * head_dim / 4;
    const int threads = items > 128 ? 256 : (items > 64 ? 128 : 64);
    hipLaunchKernelGGL(rope_kv_write_bf16_kernel, dim3(tokens), dim3(threads), 0, (hipStream_t)stream, a);
    NNIS_LAUNCH_CHECK("rope_kv_write_bf16");
    return 0;
  }
  const int work = (heads + 2 * kv_heads) * head_dim / 2;
  const int threads = work >= 512 ? 256 : (work >= 128 ? 128 : 64);
  hipLaunchKernelGGL(rope_kv_write_kernel, dim3(tokens), dim3(threads), 0, (hipStream_t)stream, a);
  NNIS_LAUNCH_CHECK("rope_kv_write");
  return 0;
}

// -----------------------------------------------------------------------------
// SiLU-multiply on a fused [tokens, 2*inner] projection (gate columns first):
// out = gate / (1 + exp(-gate)) * up
// (/root/reference/crates/nnis-model/src/fused_swiglu.rs:14-28)
// -----------------------------------------------------------------------------
__global__ void silu_mul_kernel(const void* __restrict__ gate_up, int in_dtype, void* __restrict__ out, int out_dtype,
                                int inner, size_t total) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const size_t row = i / inner;
    const size_t col = i % inner;
    const float g = load_as_f32(gate_up, in_dtype, row * 2 * inner + col);
    const float u = load_as_f32(gate_up, in_dtype, row * 2 * inner + inner + col);
    const float act = g / (1.0f + expf(-g));
    store_from_f32(out, out_dtype, i, act * u);
  }
}

// the same on bfloat16 rows whose width is a multiple of 8: 16-byte accesses, 8 channels a thread
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;

__global__ void silu_mul_bf16_kernel(const bf16_t* __restrict__ gate_up, bf16_t* __restrict__ out, int inner, size_t groups) {
  const int per_row = inner / 8;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < groups; i += (size_t)gridDim.x * blockDim.x) {
    const size_t row = i / per_row;
    const int col = (int)(i % per_row) * 8;
    const bf16x8_t g = *(const bf16x8_t*)(gate_up + row * 2 * inner + col);
    const bf16x8_t u = *(const bf16x8_t*)(gate_up + row * 2 * inner + inner + col);
    bf16x8_t y;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float gate = (float)g[e];
      y[e] = (__bf16)(gate / (1.0f + expf(-gate)) * (float)u[e]);
    }
    *(bf16x8_t*)(out + row * inner + col) = y;
  }
}

extern "C" int nnis_silu_mul(const void* gate_up, int in_dtype, void* out, int out_dtype, int tokens, int inner,
                             void* stream) {
  NNIS_REQUIRE(nnis_dtype_ok(in_dtype) && nnis_dtype_ok(out_dtype), "silu_mul: unknown dtype");
  NNIS_REQUIRE(tokens >= 0 && inner > 0, "silu_mul: bad sizes tokens=%d inner=%d", tokens, inner);
  if (tokens == 0) return 0;
  if (in_dtype == NNIS_BF16 && out_dtype == NNIS_BF16 && inner % 8 == 0 && (uintptr_t)gate_up % 16 == 0 &&
      (uintptr_t)out % 16 == 0) {
    const size_t groups = (size_t)tokens * (inner / 8);
    size_t blocks = (groups + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(silu_mul_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const bf16_t*)gate_up, (bf16_t*)out, inner, groups);
    NNIS_LAUNCH_CHECK("silu_mul_bf16");
    return 0;
  }
  const size_t total = (size_t)tokens * inner;
  size_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, gate_up, in_dtype,
                     out, out_dtype, inner, total);
  NNIS_LAUNCH_CHECK("silu_mul");
  return 0;
}

// -----------------------------------------------------------------------------
// argmax per row, lowest index on ties
// (/root/reference/crates/nnis-kernels/src/top_k.rs:41-92: value descending,
// then lower index).  NaN never wins.
// -----------------------------------------------------------------------------
__device__ __forceinline__ bool better(float v, int i, float best_v, int best_i) {
  return v > best_v || (v == best_v && i < best_i);
}

constexpr int kArgmaxChunk = 4096;  // columns a block of the first pass takes: 16 a thread, all asked for at once

__device__ __forceinline__ void wave_best(float& best_v, int& best_i) {
#pragma unroll
  for (int offset = kWave / 2; offset > 0; offset >>= 1) {
    const float ov = __shfl_xor(best_v, offset, kWave);
    const int oi = __shfl_xor(best_i, offset, kWave);
    if (better(ov, oi, best_v, best_i)) {
      best_v = ov;
      best_i = oi;
    }
  }
}

// first pass: block (chunk, row) leaves the best of its chunk of the row in part_v / part_i [rows, chunks]
__global__ __launch_bounds__(256) void argmax_chunk_kernel(const float* __restrict__ logits, float* __restrict__ part_v,
                                                           int* __restrict__ part_i, int vocab, int chunks) {
  __shared__ float s_val[4];
  __shared__ int s_idx[4];
  const int chunk = blockIdx.x, row_index = blockIdx.y;
  const float* row = logits + (size_t)row_index * vocab;
  const int c0 = chunk * kArgmaxChunk;
  float v[16];
  if (vocab % 4 == 0) {  // rows are 16-byte aligned: four loads of four a thread
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = c0 + (j * 256 + threadIdx.x) * 4;
      f32x4_t four = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
      if (c + 4 <= vocab) four = *(const f32x4_t*)(row + c);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[4 * j + e] = four[e];
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int c = c0 + (j * 256 + threadIdx.x) * 4 + e;
        v[4 * j + e] = c < vocab ? row[c] : -INFINITY;
      }
  }
  float best_v = -INFINITY;
  int best_i = 0x7fffffff;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int c = c0 + (j * 256 + threadIdx.x) * 4 + e;
      if (c < vocab && better(v[4 * j + e], c, best_v, best_i)) {
        best_v = v[4 * j + e];
        best_i = c;
      }
    }
  wave_best(best_v, best_i);
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  if (lane == 0) {
    s_val[wave] = best_v;
    s_idx[wave] = best_i;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) {
      if (better(s_val[w], s_idx[w], best_v, best_i)) {
        best_v = s_val[w];
        best_i = s_idx[w];
      }
    }
    part_v[(size_t)row_index * chunks + chunk] = best_v;
    part_i[(size_t)row_index * chunks + chunk] = best_i;
  }
}

// second pass: a wave per row over the chunks' bests
__global__ __launch_bounds__(64) void argmax_rows_kernel(const float* __restrict__ part_v, const int* __restrict__ part_i,
                                                         int* __restrict__ out, int chunks) {
  const int row_index = blockIdx.x;
  float best_v = -INFINITY;
  int best_i = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += kWave) {
    const float v = part_v[(size_t)row_index * chunks + c];
    const int i = part_i[(size_t)row_index * chunks + c];
    if (better(v, i, best_v, best_i)) {
      best_v = v;
      best_i = i;
    }
  }
  wave_best(best_v, best_i);
  if (threadIdx.x == 0) out[row_index] = best_i == 0x7fffffff ? 0 : best_i;
}

// scratch: at least nnis_argmax_scratch(rows, vocab) 4-byte words, 16-byte aligned
extern "C" int nnis_argmax_scratch(int rows, int vocab) {
  const int chunks = (vocab + kArgmaxChunk - 1) / kArgmaxChunk;
  return 2 * rows * chunks;
}

extern "C" int nnis_argmax(const float* logits, int* out, int rows, int vocab, void* scratch, void* stream) {
  NNIS_REQUIRE(rows >= 0 && vocab > 0, "argmax: bad sizes rows=%d vocab=%d", rows, vocab);
  if (rows == 0) return 0;
  NNIS_REQUIRE(scratch != nullptr, "argmax: needs scratch memory");
  NNIS_REQUIRE(rows <= 65535, "argmax: %d rows exceed the grid limit", rows);
  const int chunks = (vocab + kArgmaxChunk - 1) / kArgmaxChunk;
  float* part_v = (float*)scratch;
  int* part_i = (int*)(part_v + (size_t)rows * chunks);
  hipLaunchKernelGGL(argmax_chunk_kernel, dim3(chunks, rows), dim3(256), 0, (hipStream_t)stream, logits, part_v, part_i, vocab,
                     chunks);
  NNIS_LAUNCH_CHECK("argmax");
  hipLaunchKernelGGL(argmax_rows_kernel, dim3(rows), dim3(64), 0, (hipStream_t)stream, part_v, part_i, out, chunks);
  NNIS_LAUNCH_CHECK("argmax");
  return 0;
}

// -----------------------------------------------------------------------------
// The same argmax from a fixed array in device memory (nnis_noalloc.h): no allocation anywhere on the way.
// Host code never uses the array's name for its memory: the name is a host-side stand-in, and each GPU has a
// copy of the array at an address of its own, asked for once per device with that device current.
// -----------------------------------------------------------------------------
static __device__ __align__(256) unsigned int nnis_static_scratch[NNIS_STATIC_SCRATCH_WORDS];

constexpr int kStaticScratchDevices = 64;
static void* g_static_scratch_ptr[kStaticScratchDevices] = {nullptr};
static std::mutex g_static_scratch_mutex;

// the current device's copy of the array (nullptr with a message left on failure)
static void* nnis_static_scratch_address() {
  int device = -1;
  hipError_t status = hipGetDevice(&device);
  if (status != hipSuccess || device < 0 || device >= kStaticScratchDevices) {
    nnis_fail("argmax_static: no current device (%s)", status != hipSuccess ? hipGetErrorString(status) : "index out of range");
    return nullptr;
  }
  std::lock_guard<std::mutex> guard(g_static_scratch_mutex);
  if (g_static_scratch_ptr[device] == nullptr) {
    void* address = nullptr;
    status = hipGetSymbolAddress(&address, HIP_SYMBOL(nnis_static_scratch));
    if (status != hipSuccess || address == nullptr) {
      nnis_fail("argmax_static: the fixed array has no address on device %d (%s)", device, hipGetErrorString(status));
      return nullptr;
    }
    g_static_scratch_ptr[device] = address;
  }
  return g_static_scratch_ptr[device];
}

extern "C" int nnis_argmax_static(const float* logits, int* out, int rows, int vocab, void* stream) {
  NNIS_REQUIRE(rows >= 0 && vocab > 0, "argmax_static: bad sizes rows=%d vocab=%d", rows, vocab);
  if (rows == 0) return 0;
  NNIS_REQUIRE(logits != nullptr && out != nullptr, "argmax_static: logits and out must be given");
  NNIS_REQUIRE(rows <= 65535, "argmax_static: %d rows exceed the grid limit", rows);
  const long long chunks = ((long long)vocab + kArgmaxChunk - 1) / kArgmaxChunk;
  const long long words = 2LL * rows * chunks;
  NNIS_REQUIRE(words <= NNIS_STATIC_SCRATCH_WORDS,
               "argmax_static: %d rows of %d columns need %lld words of scratch; the fixed array holds %d "
               "(use nnis_argmax with scratch of the caller's)", rows, vocab, words, NNIS_STATIC_SCRATCH_WORDS);
  void* scratch = nnis_static_scratch_address();
  if (scratch == nullptr) return 1;
  float* part_v = (float*)scratch;
  int* part_i = (int*)(part_v + (size_t)rows * chunks);
  hipLaunchKernelGGL(argmax_chunk_kernel, dim3((int)chunks, rows), dim3(256), 0, (hipStream_t)stream, logits, part_v, part_i,
                     vocab, (int)chunks);
  NNIS_LAUNCH_CHECK("argmax_static");
  hipLaunchKernelGGL(argmax_rows_kernel, dim3(rows), dim3(64), 0, (hipStream_t)stream, part_v, part_i, out, (int)chunks);
  NNIS_LAUNCH_CHECK("argmax_static");
  return 0;
}
