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
// Page layouts:  K [page][kv_head][token in page][head_dim]
//                V [page][kv_head][head_dim][token in page]
#include "common.h"

#ifndef NNIS_HEAD_DIM
#error "compile with -DNNIS_HEAD_DIM=<head size>"
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
    const CacheT* krow = kp + (((size_t)page * a.kv_heads + kv_head) * kPageTokens + r) * HD;
    float dot = 0.0f;
#pragma unroll
    for (int d = 0; d < HD; ++d) dot = fmaf(qs[d], to_f32(krow[d]), dot);
    const float s = dot * a.scale;
    const float m_new = fmaxf(m, s);
    const float alpha = expf(m - m_new);  // exp(-inf) = 0 on the first key
    const float p = expf(s - m_new);
    l = l * alpha + p;
    const CacheT* vcol = vp + ((size_t)page * a.kv_heads + kv_head) * HD * kPageTokens + r;
#pragma unroll
    for (int d = 0; d < HD; ++d) o[d] = o[d] * alpha + p * to_f32(vcol[(size_t)d * kPageTokens]);
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
