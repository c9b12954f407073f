// What the fused projections do with a finished product besides storing it: the gated
// activation of a feed-forward, and the rotation of queries and keys with the write of keys
// and values into the cache.  Shared by the kernel for few tokens (gemm_fused.hip) and the
// tiled one (gemm_mfma.hip); in both a lane ends up with four consecutive features of one
// token from each of two strips of 16 weight rows that belong together.
#pragma once

#include "common.h"

enum : int { EPI_STORE = 0, EPI_SILU = 1, EPI_ROPE = 2 };

typedef __attribute__((ext_vector_type(4))) __bf16 epi_bf16x4;
typedef __attribute__((ext_vector_type(4))) float epi_f32x4;

// SiLU(gate) * up as /root/reference/crates/nnis-model/src/fused_swiglu.rs:14-28: gate / (1 + exp(-gate)) * up,
// with the hardware's base-2 exponential and reciprocal (each within an ulp of 32-bit; the result is
// rounded to bfloat16).  The 32-bit path of the model has a kernel of its own with the library's exp.
__device__ __forceinline__ float silu_times(float gate, float up) {
  const float e = __builtin_amdgcn_exp2f(gate * -1.4426950408889634f);
  return gate * __builtin_amdgcn_rcpf(1.0f + e) * up;
}

// column: the first of the lane's four channels; inner: channels of the feed-forward
__device__ __forceinline__ void epilogue_silu(bf16_t* y, int token, int inner, int column, const float (&gate)[4],
                                              const float (&up)[4]) {
  if (column + 4 <= inner && inner % 4 == 0) {
    epi_bf16x4 packed;
#pragma unroll
    for (int e = 0; e < 4; ++e) packed[e] = (__bf16)silu_times(gate[e], up[e]);
    *(epi_bf16x4*)(y + (size_t)token * inner + column) = packed;
  } else {
    for (int e = 0; e < 4; ++e)
      if (column + e < inner) y[(size_t)token * inner + column + e] = (bf16_t)silu_times(gate[e], up[e]);
  }
}

struct RopeTarget {
  bf16_t* q_out;  // [tokens, heads, head_dim]
  const float* cos_table;  // [positions, head_dim / 2]
  const float* sin_table;
  const int* tok_slot;
  const int* tok_pos;
  bf16_t* k_pages;  // null: this run keeps no cache of its own
  bf16_t* v_pages;
  const int* block_table;
  int max_pages;
  int heads, kv_heads, head_dim;
  // The step's tables, where the caller brings them (all three, or none): each token's rows of the rotation
  // tables [tokens, head_dim / 2] and the cache page of its position [tokens] (< 0: a padding row).  With them
  // nothing the epilogue needs hangs on a value that has to be loaded first.
  const float* tok_cos;
  const float* tok_sin;
  const int* tok_page;
};

__device__ __forceinline__ const float* rope_cos_row(const RopeTarget& a, int token, int pos) {
  return a.tok_cos ? a.tok_cos + (size_t)token * (a.head_dim / 2) : a.cos_table + (size_t)pos * (a.head_dim / 2);
}
__device__ __forceinline__ const float* rope_sin_row(const RopeTarget& a, int token, int pos) {
  return a.tok_sin ? a.tok_sin + (size_t)token * (a.head_dim / 2) : a.sin_table + (size_t)pos * (a.head_dim / 2);
}
// the cache page that takes the token's key and value, or < 0 (a padding row, or a run that keeps no cache)
__device__ __forceinline__ int rope_page(const RopeTarget& a, int token, int slot, int pos) {
  if (!a.k_pages) return -1;
  if (a.tok_page) return a.tok_page[token];
  return slot >= 0 ? a.block_table[(size_t)slot * a.max_pages + pos / kPageTokens] : -1;
}

// Rotate-half RoPE as /root/reference/crates/nnis-model/src/runtime_kernels.rs:38-66; keys stored rotated,
// values as they are (runtime.rs:997-1016).  head: index among queries, then keys, then values; f0: the
// first of the lane's four features in the lower half of the head (lo), whose partners f0 + head_dim / 2
// are in hi; c, s: cos and sin of features f0 .. f0+3 at the token's position; page: the cache page of the
// token's position, or < 0 (padding row, or no cache).
__device__ __forceinline__ void epilogue_rope(const RopeTarget& a, int token, int pos, int page, int head, int f0,
                                              const float (&lo)[4], const float (&hi)[4], epi_f32x4 c, epi_f32x4 s) {
  const int hd = a.head_dim, half = hd / 2;
  if (head < a.heads + a.kv_heads) {  // queries and keys rotate
    epi_bf16x4 out_lo, out_hi;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      out_lo[e] = (__bf16)(lo[e] * c[e] - hi[e] * s[e]);
      out_hi[e] = (__bf16)(hi[e] * c[e] + lo[e] * s[e]);
    }
    if (head < a.heads) {
      bf16_t* dst = a.q_out + ((size_t)token * a.heads + head) * hd;
      *(epi_bf16x4*)(dst + f0) = out_lo;
      *(epi_bf16x4*)(dst + f0 + half) = out_hi;
    } else if (page >= 0) {
      bf16_t* dst = a.k_pages + ((size_t)page * a.kv_heads + (head - a.heads)) * nnis_k_page_elems(hd);
      *(epi_bf16x4*)(dst + nnis_k_offset(pos % kPageTokens, f0)) = out_lo;  // 4 channels lie within a chunk of 8
      *(epi_bf16x4*)(dst + nnis_k_offset(pos % kPageTokens, f0 + half)) = out_hi;
    }
  } else if (page >= 0) {  // values are stored as they are
    bf16_t* dst = a.v_pages + ((size_t)page * a.kv_heads + (head - a.heads - a.kv_heads)) * nnis_v_page_elems(hd);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      dst[nnis_v_offset(f0 + e, pos % kPageTokens)] = (bf16_t)lo[e];
      dst[nnis_v_offset(f0 + half + e, pos % kPageTokens)] = (bf16_t)hi[e];
    }
  }
}

// which of the two families of kernels a product of these sizes takes (gemm_mfma.hip)
bool nnis_gemm_takes_few_tokens(int m, int n, int k);

// the tiled kernel on an operand that a residual epilogue prepared (gemm_mfma.hip)
int nnis_gemm_scaled_tiled(const bf16_t* scaled, const float* ss_parts, int parts, float eps, const bf16_t* w, int m, int n,
                           int k, int epilogue, bf16_t* y, const RopeTarget& rope, int tile_hint, float* workspace,
                           size_t workspace_bytes, hipStream_t stream);
