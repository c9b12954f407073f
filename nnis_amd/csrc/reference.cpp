// Plain host references of the kernels' operations: scalar C++, one loop nest an operation, no vendor library,
// no threads, 32-bit arithmetic in a fixed order (the role of the reference's CPU executor,
// /root/reference/crates/nnis-cpu/src/numerical.rs:13-15: "finite-f32-le-ordered-fma-v1").  They are what the
// device kernels are compared with (tests/test_cpp_reference.py, tests/test_gpu_kernels.py), and are themselves
// compared with the tests' plain Python model; the product never calls them.  Built by the host compiler with
// floating-point contraction off, so that a multiply-add is fused only where the source says fmaf.
//
// Every function returns 0, or 1 with a message for nnis_last_error().
#include <cmath>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <vector>

namespace {
thread_local char g_error[512] = {0};
int fail(const char* fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, args);
  va_end(args);
  return 1;
}
}  // namespace

extern "C" const char* nnis_last_error() { return g_error; }

// x[t, :] = table[ids[t], :], a row copy without scaling; an id outside the table gives a row of zeros (as the
// device kernel; the engine refuses such ids before it launches anything)
// (/root/reference/crates/nnis-kernels/src/gather.rs:17-33).
extern "C" int nnis_ref_embed(const int* ids, const float* table, float* out, int tokens, int width, int vocab) {
  if (tokens < 0 || width <= 0 || vocab <= 0) return fail("ref_embed: bad sizes");
  for (int t = 0; t < tokens; ++t)
    for (int c = 0; c < width; ++c)
      out[(size_t)t * width + c] = (ids[t] >= 0 && ids[t] < vocab) ? table[(size_t)ids[t] * width + c] : 0.0f;
  return 0;
}

// y[c] = x[c] * (1 / sqrt(sum(x^2) * (1 / cols) + eps)) * w[c]: the sum a chain of fused multiply-adds over the
// row, eps inside the root, a multiplicative weight without "+1"
// (/root/reference/crates/nnis-model/src/kernels.rs:15-48).
extern "C" int nnis_ref_rmsnorm(const float* x, const float* weight, float* y, int rows, int cols, float eps) {
  if (rows < 0 || cols <= 0) return fail("ref_rmsnorm: bad sizes");
  const float inv_cols = 1.0f / (float)cols;
  for (int r = 0; r < rows; ++r) {
    const float* in = x + (size_t)r * cols;
    float sumsq = 0.0f;
    for (int c = 0; c < cols; ++c) sumsq = fmaf(in[c], in[c], sumsq);
    const float scale = 1.0f / sqrtf(sumsq * inv_cols + eps);
    for (int c = 0; c < cols; ++c) y[(size_t)r * cols + c] = in[c] * scale * weight[c];
  }
  return 0;
}

// cos / sin [positions, rot_dim / 2] in 32-bit: exponent = (2 * pair) / rot_dim, inverse frequency = 1 / theta ^
// exponent, angle = position * inverse frequency, each step rounded to 32-bit; powf, cosf and sinf are taken as
// correctly rounded (evaluated in 64-bit on the 32-bit argument and rounded once)
// (/root/reference/crates/nnis-model/src/runtime.rs:1166-1184).
extern "C" int nnis_ref_rope_tables(float* cos_out, float* sin_out, int positions, int rot_dim, float theta) {
  if (positions < 0 || rot_dim <= 0 || rot_dim % 2 != 0) return fail("ref_rope_tables: bad sizes");
  const int half = rot_dim / 2;
  for (int pair = 0; pair < half; ++pair) {
    const float exponent = (2.0f * (float)pair) / (float)rot_dim;
    const float power = (float)pow((double)theta, (double)exponent);
    const float inv_freq = 1.0f / power;
    for (int p = 0; p < positions; ++p) {
      const float angle = (float)p * inv_freq;
      cos_out[(size_t)p * half + pair] = (float)cos((double)angle);
      sin_out[(size_t)p * half + pair] = (float)sin((double)angle);
    }
  }
  return 0;
}

// Rotate-half on x [tokens, heads, head_dim], the first rot_dim channels of a head: with j < rot_dim / 2,
// out[j] = x[j] * c - x[j + half] * s and out[j + half] = x[j + half] * c + x[j] * s, (c, s) the table's row of the
// token's position, the same for both halves; channels beyond rot_dim pass through
// (/root/reference/crates/nnis-model/src/runtime_kernels.rs:38-66).
extern "C" int nnis_ref_rope_rotate_half(const float* x, float* out, const float* cos_table, const float* sin_table,
                                         const int* positions, int tokens, int heads, int head_dim, int rot_dim,
                                         int table_positions) {
  if (tokens < 0 || heads <= 0 || head_dim <= 0 || rot_dim < 0 || rot_dim > head_dim || rot_dim % 2 != 0)
    return fail("ref_rope: bad sizes");
  const int half = rot_dim / 2;
  for (int t = 0; t < tokens; ++t) {
    if (positions[t] < 0 || positions[t] >= table_positions) return fail("ref_rope: position %d is beyond the tables", positions[t]);
    const float* c = cos_table + (size_t)positions[t] * half;
    const float* s = sin_table + (size_t)positions[t] * half;
    for (int h = 0; h < heads; ++h) {
      const float* in = x + ((size_t)t * heads + h) * head_dim;
      float* to = out + ((size_t)t * heads + h) * head_dim;
      for (int j = 0; j < half; ++j) {
        const float left = in[j], right = in[j + half];
        to[j] = left * c[j] - right * s[j];
        to[j + half] = right * c[j] + left * s[j];
      }
      for (int j = rot_dim; j < head_dim; ++j) to[j] = in[j];
    }
  }
  return 0;
}

// Causal attention of one whole sequence with grouped key/value heads.  q [tokens, heads, head_dim]; k, v
// [first + tokens, kv_heads, head_dim]: the sequence's keys and values from position 0, the queries being those
// of positions first .. first + tokens - 1.  Query head h reads key/value head h / (heads / kv_heads)
// (/root/reference/crates/nnis-model/src/kernels.rs:84-85); a score is the dot product, a chain of fused
// multiply-adds over the channels, times `scale` after the sum (kernels.rs:103-106); key p counts for the query
// at position i iff p <= i (/root/reference/crates/nnis-kernels/src/attention.rs:99-100) and, with a window,
// p > i - window; softmax over the keys that count, then the weighted sum of their values (kernels.rs:97-124:
// there with a running maximum, here in two passes over the row, which is the same function).
extern "C" int nnis_ref_attention(const float* q, const float* k, const float* v, float* out, int tokens, int first,
                                  int heads, int kv_heads, int head_dim, float scale, int window) {
  if (tokens < 0 || first < 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || head_dim <= 0)
    return fail("ref_attention: bad sizes");
  const int group = heads / kv_heads;
  std::vector<float> scores((size_t)first + tokens);
  for (int t = 0; t < tokens; ++t) {
    const int position = first + t;
    const int low = (window > 0 && position + 1 > window) ? position + 1 - window : 0;
    for (int h = 0; h < heads; ++h) {
      const int kv_head = h / group;
      const float* query = q + ((size_t)t * heads + h) * head_dim;
      float best = -INFINITY;
      for (int p = low; p <= position; ++p) {
        const float* key = k + ((size_t)p * kv_heads + kv_head) * head_dim;
        float dot = 0.0f;
        for (int c = 0; c < head_dim; ++c) dot = fmaf(query[c], key[c], dot);
        scores[p] = dot * scale;
        best = fmaxf(best, scores[p]);
      }
      float total = 0.0f;
      for (int p = low; p <= position; ++p) {
        scores[p] = expf(scores[p] - best);
        total += scores[p];
      }
      float* to = out + ((size_t)t * heads + h) * head_dim;
      for (int c = 0; c < head_dim; ++c) {
        float sum = 0.0f;
        for (int p = low; p <= position; ++p) sum = fmaf(scores[p], v[((size_t)p * kv_heads + kv_head) * head_dim + c], sum);
        to[c] = sum / total;
      }
    }
  }
  return 0;
}

// out = silu(gate) * up with silu(x) = x / (1 + exp(-x)): SiLU on the gate branch
// (/root/reference/crates/nnis-kernels/src/lib.rs:111-122; /root/reference/crates/nnis-model/src/fused_swiglu.rs:14-28).
extern "C" int nnis_ref_silu_mul(const float* gate, const float* up, float* out, size_t elements) {
  for (size_t i = 0; i < elements; ++i) out[i] = (gate[i] / (1.0f + expf(-gate[i]))) * up[i];
  return 0;
}

// y[m, n] = x[m, k] w[n, k]^T with the checkpoint's [out, in] weight and no bias: every output one chain of
// fused multiply-adds over ascending k that starts at +0
// (/root/reference/crates/nnis-kernels/src/gemm.rs:16-64, gemv.rs:45-62).
extern "C" int nnis_ref_gemm(const float* x, const float* w, float* y, int m, int n, int k) {
  if (m < 0 || n <= 0 || k <= 0) return fail("ref_gemm: bad sizes");
  for (int i = 0; i < m; ++i)
    for (int j = 0; j < n; ++j) {
      float sum = 0.0f;
      for (int kk = 0; kk < k; ++kk) sum = fmaf(x[(size_t)i * k + kk], w[(size_t)j * k + kk], sum);
      y[(size_t)i * n + j] = sum;
    }
  return 0;
}

// residual[i] += delta[i] in 32-bit (/root/reference/crates/nnis-model/src/runtime.rs:1030-1044,1088-1093)
extern "C" int nnis_ref_residual_add(float* residual, const float* delta, size_t elements) {
  for (size_t i = 0; i < elements; ++i) residual[i] += delta[i];
  return 0;
}

// out[r] = the index of the row's largest logit, the lowest index on ties
// (/root/reference/crates/nnis-kernels/src/top_k.rs:41-92).
extern "C" int nnis_ref_argmax(const float* logits, int* out, int rows, int vocab) {
  if (rows < 0 || vocab <= 0) return fail("ref_argmax: bad sizes");
  for (int r = 0; r < rows; ++r) {
    int best = 0;
    for (int i = 1; i < vocab; ++i)
      if (logits[(size_t)r * vocab + i] > logits[(size_t)r * vocab + best]) best = i;
    out[r] = best;
  }
  return 0;
}

// SplitMix64 (/root/reference/crates/nnis-model/src/sampling.rs:261-284): the state moves on by the golden
// ratio's odd constant, the output is mixed by two multiply-xorshifts; a unit draw is the top 53 bits over 2^53.
static uint64_t splitmix_next(uint64_t* state) {
  *state += 0x9E3779B97F4A7C15ull;
  uint64_t z = *state;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

extern "C" int nnis_ref_splitmix64(uint64_t* state, uint64_t* out, int draws) {
  for (int i = 0; i < draws; ++i) out[i] = splitmix_next(state);
  return 0;
}

// One seeded draw from a row of logits, step by step as the reference's sampler
// (/root/reference/crates/nnis-model/src/sampling.rs:113-202): candidates in the order of their logits, the
// largest first and the lower id first among equals; the top_k first of them (0: all); weights exp((logit -
// largest) / temperature) in 64-bit, summed in that order; top_p (0: off) keeps the candidates up to and with the
// one at which the running sum reaches top_p * total; then the first candidate whose running sum exceeds u * total,
// u one unit draw of the sequence's generator (the last candidate if none does).  Returns the token in *token and
// leaves the generator's state moved on by one draw; a logit that is not finite is refused.
extern "C" int nnis_ref_sample(const float* logits, int vocab, float temperature, int top_k, float top_p, uint64_t* rng_state,
                               int* token) {
  if (vocab <= 0 || !(temperature > 0.0f)) return fail("ref_sample: bad sizes or temperature");
  for (int i = 0; i < vocab; ++i)
    if (!std::isfinite(logits[i])) return fail("ref_sample: logit %d is not finite", i);
  std::vector<int> order(vocab);
  for (int i = 0; i < vocab; ++i) order[i] = i;
  // an insertion-free, stable order: by logit descending, then by id ascending (a plain merge sort)
  std::vector<int> scratch(vocab);
  for (int width = 1; width < vocab; width *= 2) {
    for (int lo = 0; lo < vocab; lo += 2 * width) {
      const int mid = lo + width < vocab ? lo + width : vocab, hi = lo + 2 * width < vocab ? lo + 2 * width : vocab;
      int a = lo, b = mid, at = lo;
      while (a < mid && b < hi) {
        const bool take_b = logits[order[b]] > logits[order[a]];  // equal logits: the left run holds the lower ids
        scratch[at++] = take_b ? order[b++] : order[a++];
      }
      while (a < mid) scratch[at++] = order[a++];
      while (b < hi) scratch[at++] = order[b++];
    }
    order.swap(scratch);
  }
  int count = (top_k > 0 && top_k < vocab) ? top_k : vocab;
  const double inv_t = 1.0 / (double)temperature;
  const double largest = (double)logits[order[0]] * inv_t;
  std::vector<double> weights(count);
  double total = 0.0;
  for (int i = 0; i < count; ++i) {
    weights[i] = exp((double)logits[order[i]] * inv_t - largest);
    total += weights[i];
  }
  if (top_p > 0.0f) {
    const double threshold = (double)top_p * total;
    double running = 0.0;
    int kept = count;
    for (int i = 0; i < count; ++i) {
      running += weights[i];
      if (running >= threshold) {
        kept = i + 1;
        break;
      }
    }
    count = kept > 1 ? kept : 1;
    total = 0.0;
    for (int i = 0; i < count; ++i) total += weights[i];
  }
  const double unit = (double)(splitmix_next(rng_state) >> 11) * (1.0 / 9007199254740992.0);
  const double draw = unit * total;
  double running = 0.0;
  for (int i = 0; i < count; ++i) {
    running += weights[i];
    if (draw < running) {
      *token = order[i];
      return 0;
    }
  }
  *token = order[count - 1];
  return 0;
}
