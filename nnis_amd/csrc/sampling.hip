// Seeded temperature / top-k / top-p sampling on the device, one block per row.
//
// Semantics are the reference's host sampler
// (/root/reference/crates/nnis-model/src/sampling.rs:113-202): candidates in
// order of logit descending, ties by lower id; top-k keeps the first k;
// weights exp((l - l_max) / T) in 64-bit; top-p keeps the shortest prefix
// whose weight reaches p * total (the crossing candidate stays); one
// SplitMix64 draw u in [0,1) per token (sampling.rs:261-284); the result is
// the first candidate whose cumulative weight exceeds u * total.
//
// No sort: a prefix of the sorted order is described by a cut (key, ties): all
// tokens whose key is above `key`, and the first `ties` tokens (by id) whose key
// equals it.  Each cut is found by a bitwise search over the 32-bit ordered
// key with a block-wide sum per probe; sums are taken in a fixed order, so a
// seed always gives the same token.  Sums differ from the reference's running
// sum in the last bits only.
#include "common.h"

namespace {

constexpr int kSampleThreads = 512;  // 8 waves: a thread may keep up to 128 keys of its row in registers

__device__ __forceinline__ unsigned ordered_key(float v) {
  if (v == 0.0f) v = 0.0f;  // -0 and +0 compare equal
  const unsigned bits = __float_as_uint(v);
  return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}

template <typename T>
__device__ __forceinline__ T block_total(T v, T* scratch) {
#pragma unroll
  for (int offset = kWave / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, kWave);
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  T total = 0;
  for (int w = 0; w < kSampleThreads / kWave; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ unsigned long long splitmix64_next(unsigned long long* state) {
  *state += 0x9E3779B97F4A7C15ull;
  unsigned long long z = *state;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

struct RowView {
  const float* logits;
  const double* weights;
  int vocab;
};

// A thread's elements are threadIdx.x + i * kSampleThreads.  With PER > 0 it keeps their ordered keys in
// registers (vocab <= PER * kSampleThreads; 0 for an element beyond the row, which is below every finite
// value's key) and a pass over the row reads the weights only, every load asked for before the first is used;
// PER == 0 reads keys and weights from memory, for rows of any length.  The sums are the same term by term
// either way: an element that does not count adds 0.
template <int PER>
struct Keys {
  unsigned held[PER > 0 ? PER : 1];
};

// Returns whether one of this thread's logits is not finite.
template <int PER>
__device__ __forceinline__ int load_keys(Keys<PER>& keys, const RowView& r) {
  int bad = 0;
  if constexpr (PER > 0) {
#pragma clang loop unroll(full)
    for (int i = 0; i < PER; ++i) {
      const int c = threadIdx.x + i * kSampleThreads;
      const float v = c < r.vocab ? r.logits[c] : 0.0f;
      bad |= isfinite(v) ? 0 : 1;
      keys.held[i] = c < r.vocab ? ordered_key(v) : 0u;
    }
  } else {
    for (int c = threadIdx.x; c < r.vocab; c += kSampleThreads) bad |= isfinite(r.logits[c]) ? 0 : 1;
  }
  return bad;
}

// The weights exp((l - l_max) / T) of every row that samples, 64-bit, with all of the chip (a row's own block
// would take 49,152 of them 40 us and more).  `best` holds an index of each row's maximum.
constexpr int kWeightThreads = 256, kWeightsEach = 8;
__global__ __launch_bounds__(kWeightThreads) void sample_weights_kernel(
    const float* __restrict__ logits, double* __restrict__ weights, int vocab, const int* __restrict__ row_slot,
    const float* __restrict__ temperature, int by_slot, const int* __restrict__ best) {
  const int row = blockIdx.y;
  const int slot = row_slot[row];
  if (slot < 0) return;
  const float* l = logits + (size_t)row * vocab;
  double* w = weights + (size_t)row * vocab;
  const double inv_t = 1.0 / (double)temperature[by_slot ? slot : row];
  const int best_at = best[row];
  float top = l[best_at < 0 ? 0 : (best_at < vocab ? best_at : vocab - 1)];  // (in range for a row of finite logits; never read outside)
  if (top == 0.0f) top = 0.0f;
  const double max_scaled = (double)top * inv_t;
  const int c0 = blockIdx.x * (kWeightThreads * kWeightsEach) + threadIdx.x;
  float v[kWeightsEach];
#pragma unroll
  for (int j = 0; j < kWeightsEach; ++j) {
    const int c = c0 + j * kWeightThreads;
    v[j] = l[c < vocab ? c : vocab - 1];
  }
#pragma unroll
  for (int j = 0; j < kWeightsEach; ++j) {
    const int c = c0 + j * kWeightThreads;
    if (c < vocab) w[c] = exp((double)v[j] * inv_t - max_scaled);
  }
}

// weight of all tokens whose key is >= t
template <int PER>
__device__ __forceinline__ double mass_at_least(const RowView& r, const Keys<PER>& keys, unsigned t, double* scratch) {
  double sum = 0.0;
  if constexpr (PER > 0) {
    constexpr int kBatch = 8;
    const unsigned from = t > 1u ? t : 1u;  // an element beyond the row has key 0 and never counts
    int first = threadIdx.x;
    asm volatile("" : "+v"(first));  // each pass works out its addresses again: kept from pass to pass they would take the keys' registers
#pragma clang loop unroll(full)
    for (int i0 = 0; i0 < PER; i0 += kBatch) {
      double w[kBatch];
#pragma clang loop unroll(full)
      for (int j = 0; j < kBatch; ++j) {
        const int c = first + (i0 + j) * kSampleThreads;
        w[j] = i0 + j < PER ? r.weights[c < r.vocab ? c : r.vocab - 1] : 0.0;  // (beyond the row: the last again, not counted)
      }
#pragma clang loop unroll(full)
      for (int j = 0; j < kBatch; ++j)
        if (i0 + j < PER) sum += keys.held[i0 + j] >= from ? w[j] : 0.0;
      __builtin_amdgcn_sched_barrier(0);  // a batch's loads at a time: the registers hold the keys
    }
  } else {
    for (int c = threadIdx.x; c < r.vocab; c += kSampleThreads)
      if (ordered_key(r.logits[c]) >= t) sum += r.weights[c];
  }
  return block_total(sum, scratch);
}

// number of tokens whose key is >= t
template <int PER>
__device__ __forceinline__ int count_at_least(const RowView& r, const Keys<PER>& keys, unsigned t, int* scratch) {
  if constexpr (PER > 0) {
    // a comparison and an add with carry an element (counting the lanes' bits with the scalar unit instead was
    // slower at 96 keys a thread: 239 against 182 us for a whole draw)
    const unsigned from = t > 1u ? t : 1u;  // an element beyond the row has key 0 and never counts
    int count = 0;
#pragma clang loop unroll(full)
    for (int i = 0; i < PER; ++i) count += keys.held[i] >= from ? 1 : 0;
    return block_total(count, scratch);
  } else {
    int count = 0;
    for (int c = threadIdx.x; c < r.vocab; c += kSampleThreads)
      if (ordered_key(r.logits[c]) >= t) ++count;
    return block_total(count, scratch);
  }
}

template <int PER>
__global__ __launch_bounds__(kSampleThreads) void sample_kernel(
    const float* __restrict__ logits, double* __restrict__ weights, int vocab, const int* __restrict__ row_slot,
    unsigned long long* __restrict__ rng, const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, int by_slot, const int* best, int* out) {  // (`best` may be `out`)
  __shared__ double scratch_d[kSampleThreads / kWave];
  __shared__ int scratch_i[kSampleThreads / kWave];
  __shared__ int found;
  const int row = blockIdx.x;
  const int slot = row_slot[row];
  if (slot < 0) return;  // padding row (uniform over the block)
  RowView r;
  r.logits = logits + (size_t)row * vocab;
  double* w = weights + (size_t)row * vocab;
  r.weights = w;
  r.vocab = vocab;
  Keys<PER> keys;
  // a check that every logit is finite, on the way
  if (block_total(load_keys<PER>(keys, r), scratch_i)) {
    if (threadIdx.x == 0) out[row] = -1;  // the host raises: a non-finite logit is refused
    return;
  }
  const int at = by_slot ? slot : row;  // where the row's options lie: per sequence (kept with its slot) or per row
  const double inv_t = 1.0 / (double)temperature[at];
  const int best_at = best[row];
  float top = r.logits[best_at < 0 ? 0 : (best_at < vocab ? best_at : vocab - 1)];  // (as sample_weights_kernel took it)
  if (top == 0.0f) top = 0.0f;
  const double max_scaled = (double)top * inv_t;

  // the kept prefix: everything with key > cut_key plus `cut_ties` tokens at cut_key
  unsigned cut_key = 0;
  int cut_ties = 0;          // meaningful only when limited
  bool limited = false;
  // The largest key t at which `holds(weight of all kept tokens with key >= t)` is still true, by bits from the
  // top.  With the keys in registers a probe first counts (no memory): a probe that holds the same tokens as
  // the bound above it (which failed) or as the bound below (which held) needs no sum -- among 49,152 keys that
  // is about half of the 32 probes, the upper bits that all keys share and the lower ones between neighbours.
  // And once the kept tokens between the two bounds are few (kNear), their keys and weights are put into LDS, in
  // a fixed order, and a probe sums those on top of the upper bound's weight: a sum over the row's weights in
  // memory takes 6 to 8 us, one over the near ones under 1.
  constexpr int kNear = 2048;
  __shared__ unsigned near_key[kNear];
  __shared__ int near_at[kNear];
  __shared__ double near_weight[kNear];
  __shared__ int wave_near[kSampleThreads / kWave];
  bool near = false;         // the search's state, for `mass_from` after it too
  int near_count = 0;
  double mass_above = 0.0;   // weight of the tokens at and above the lowest probe that failed before the near ones were taken

  auto gather_near = [&](unsigned lower, unsigned upper, bool has_upper) __attribute__((always_inline)) {
    const unsigned from = lower > 1u ? lower : 1u;
    int mine = 0;
    if constexpr (PER > 0) {
#pragma clang loop unroll(full)
      for (int i = 0; i < PER; ++i) mine += (keys.held[i] >= from && (!has_upper || keys.held[i] < upper)) ? 1 : 0;
    }
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    int upto = mine;  // with this thread's
#pragma unroll
    for (int offset = 1; offset < kWave; offset <<= 1) {
      const int other = __shfl_up(upto, offset, kWave);
      upto += lane >= offset ? other : 0;
    }
    __syncthreads();
    if (lane == kWave - 1) wave_near[wave] = upto;
    __syncthreads();
    int place = upto - mine, all = 0;
    for (int w = 0; w < kSampleThreads / kWave; ++w) {
      place += w < wave ? wave_near[w] : 0;
      all += wave_near[w];
    }
    if constexpr (PER > 0) {
#pragma clang loop unroll(full)
      for (int i = 0; i < PER; ++i) {
        if (keys.held[i] >= from && (!has_upper || keys.held[i] < upper)) {
          near_key[place] = keys.held[i];
          near_at[place] = threadIdx.x + i * kSampleThreads;
          ++place;
        }
      }
    }
    __syncthreads();
    for (int j = threadIdx.x; j < all; j += kSampleThreads) near_weight[j] = r.weights[near_at[j]];
    __syncthreads();
    near = true;
    near_count = all;
  };
  // weight of the kept tokens with key >= probe (above the limit, if there is one)
  auto mass_from = [&](unsigned probe) __attribute__((always_inline)) -> double {
    if (!near) return mass_at_least<PER>(r, keys, probe, scratch_d);
    double sum = 0.0;
    for (int j = threadIdx.x; j < near_count; j += kSampleThreads) sum += near_key[j] >= probe ? near_weight[j] : 0.0;
    return mass_above + block_total(sum, scratch_d);
  };

  auto find_cut = [&](auto holds) __attribute__((always_inline)) -> unsigned {
    unsigned t = 0;
    int count_below = -1;  // tokens with key >= t, where known (not at the start: with a limit `total` is not all tokens' weight)
    int count_above = 0;   // tokens at and above the lowest probe that failed; at first none, whose weight 0 never holds
    unsigned upper = 0;    // the lowest probe that failed, if one has
    bool has_upper = false;
    near = false;
    mass_above = 0.0;
    for (int bit = 31; bit >= 0; --bit) {
      const unsigned probe = t | (1u << bit);
      if (limited && probe <= cut_key) {  // everything kept lies at or above the limit: the whole kept weight, which holds
        t = probe;
        count_below = -1;
        continue;
      }
      if (near) {  // the sums decide by themselves: over the same tokens they are the same sums
        if (holds(mass_from(probe))) t = probe;
        continue;
      }
      int count = -2;
      if constexpr (PER > 0) {
        count = count_at_least<PER>(r, keys, probe, scratch_i);
        if (count == count_above) continue;
        if (count == count_below) {
          t = probe;
          continue;
        }
        if (!near) {
          const unsigned lower = (limited && t <= cut_key) ? cut_key + 1u : t;  // (cut_key < probe <= 2^32 - 1)
          const int between = (count_below >= 0 && lower == t ? count_below : count_at_least<PER>(r, keys, lower, scratch_i)) - count_above;
          if (between <= kNear) gather_near(lower, upper, has_upper);
        }
      }
      const double mass = mass_from(probe);
      if (holds(mass)) {
        t = probe;
        count_below = count;
      } else {
        count_above = count;
        if (!near) {  // (the near tokens were taken below the bound of that moment: its weight stays their base)
          mass_above = mass;
          upper = probe;
          has_upper = true;
        }
      }
    }
    return t;
  };

  // top-k: the k-th largest key by a search over counts; once the tokens between its bounds are few, over those
  const int k = top_k[at];
  double total;
  if (k > 0 && k < vocab) {
    unsigned t = 0, upper = 0;
    bool has_upper = false;
    int above = 0, below = vocab;  // tokens at and above `upper`, at and above t (while the search counts the whole row)
    for (int bit = 31; bit >= 0; --bit) {
      const unsigned probe = t | (1u << bit);
      int count;
      if (near) {
        int some = 0;
        for (int j = threadIdx.x; j < near_count; j += kSampleThreads) some += near_key[j] >= probe ? 1 : 0;
        count = above + block_total(some, scratch_i);
      } else {
        count = count_at_least<PER>(r, keys, probe, scratch_i);
      }
      if (count >= k) {
        t = probe;
        if (!near) below = count;
      } else if (!near) {
        above = count;
        upper = probe;
        has_upper = true;
      }
      if constexpr (PER > 0) {
        if (!near && below - above <= kNear) gather_near(t, upper, has_upper);
      }
    }
    near = false;
    const int over = count_at_least<PER>(r, keys, t + 1u, scratch_i);
    cut_key = t;
    cut_ties = k - over;
    limited = true;
    const double weight_at = exp((double)__uint_as_float((t & 0x80000000u) ? (t & 0x7fffffffu) : ~t) * inv_t - max_scaled);
    total = mass_at_least<PER>(r, keys, t + 1u, scratch_d) + (double)cut_ties * weight_at;
  } else {
    total = mass_at_least<PER>(r, keys, 0u, scratch_d);
  }

  const float p = top_p[at];
  // (A top_p of 1 keeps every candidate: the running sum reaches the whole weight at the last one that adds to it,
  // and what lies behind that one has no weight to be drawn with.  It must not go through the search: sums of the
  // same weights in another order may stay a rounding below the whole, and the search then finds no cut at all.)
  if (p > 0.0f && p < 1.0f) {
    const double threshold = (double)p * total;
    const unsigned t = find_cut([&](double mass) { return mass >= threshold; });
    // t >= cut_key when limited, because the whole kept mass reaches the threshold
    const double base = mass_from(t + 1u);
    const double weight_at = exp((double)__uint_as_float((t & 0x80000000u) ? (t & 0x7fffffffu) : ~t) * inv_t - max_scaled);
    int available = (limited && t == cut_key) ? cut_ties
                                              : count_at_least<PER>(r, keys, t, scratch_i) - count_at_least<PER>(r, keys, t + 1u, scratch_i);
    int need = 1;
    double reached = base + weight_at;
    while (need < available && reached < threshold) {
      ++need;
      reached += weight_at;
    }
    cut_key = t;
    cut_ties = need;
    limited = true;
    total = base + (double)need * weight_at;
  }

  unsigned long long state = rng[slot];
  const unsigned long long raw = splitmix64_next(&state);
  const double unit = (double)(raw >> 11) * (1.0 / 9007199254740992.0);
  const double draw = unit * total;

  const unsigned t = find_cut([&](double mass) { return mass > draw; });
  const double base = mass_from(t + 1u);
  const double weight_at = exp((double)__uint_as_float((t & 0x80000000u) ? (t & 0x7fffffffu) : ~t) * inv_t - max_scaled);
  int same = -1;  // tokens whose key equals t, where it is known or cheap to know
  if (PER > 0 || !(limited && t == cut_key)) same = count_at_least<PER>(r, keys, t, scratch_i) - count_at_least<PER>(r, keys, t + 1u, scratch_i);
  const int available = (limited && t == cut_key) ? cut_ties : same;
  int index = 0;
  double reached = base + weight_at;
  while (index + 1 < available && !(draw < reached)) {
    ++index;
    reached += weight_at;
  }

  if constexpr (PER > 0) {
    if (same == 1) {  // the usual case, no ties at t: the thread that holds the key names the token
#pragma clang loop unroll(full)
      for (int i = 0; i < PER; ++i)
        if (keys.held[i] == t) out[row] = threadIdx.x + i * kSampleThreads;
      if (threadIdx.x == 0) rng[slot] = state;
      return;
    }
  }
  // the index-th token (by id) whose key equals t: contiguous chunks per thread, then a scan
  const int chunk = (vocab + kSampleThreads - 1) / kSampleThreads;
  const int begin = threadIdx.x * chunk;
  const int end = begin + chunk < vocab ? begin + chunk : vocab;
  int mine = 0;
  for (int c = begin; c < end; ++c)
    if (ordered_key(r.logits[c]) == t) ++mine;
  __shared__ int counts[kSampleThreads];
  counts[threadIdx.x] = mine;
  if (threadIdx.x == 0) found = -1;
  __syncthreads();
  if (threadIdx.x == 0) {
    int before = 0;
    for (int i = 0; i < kSampleThreads; ++i) {
      if (index < before + counts[i]) {
        found = (i << 16) | (index - before);  // thread and its local index; chunk counts fit in 16 bits
        break;
      }
      before += counts[i];
    }
  }
  __syncthreads();
  if (found >= 0 && threadIdx.x == (found >> 16)) {
    int local = found & 0xffff;
    for (int c = begin; c < end; ++c) {
      if (ordered_key(r.logits[c]) == t) {
        if (local == 0) {
          out[row] = c;
          break;
        }
        --local;
      }
    }
  }
  if (threadIdx.x == 0) {
    rng[slot] = state;
    if (found < 0) out[row] = -2;  // cannot happen for finite logits; reported rather than hidden
  }
}

}  // namespace

extern "C" int nnis_sample(const float* logits, double* weights, int rows, int vocab, const int* row_slot,
                           unsigned long long* rng, const float* temperature, const int* top_k, const float* top_p,
                           int by_slot, const int* best, int* out, void* stream) {
  NNIS_REQUIRE(rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", rows, vocab);
  NNIS_REQUIRE(best != nullptr, "sample: needs an index of each row's maximum");
  NNIS_REQUIRE(rows <= 65535, "sample: %d rows are more than a launch takes", rows);
  NNIS_REQUIRE((long long)vocab <= 65535LL * kSampleThreads, "sample: vocabulary %d is too large for this kernel", vocab);
  if (rows == 0) return 0;
  const dim3 grid(rows), block(kSampleThreads);
  hipStream_t s = (hipStream_t)stream;
  hipLaunchKernelGGL(sample_weights_kernel, dim3((vocab + kWeightThreads * kWeightsEach - 1) / (kWeightThreads * kWeightsEach), rows),
                     dim3(kWeightThreads), 0, s, logits, weights, vocab, row_slot, temperature, by_slot, best);
#define NNIS_SAMPLE(PER) hipLaunchKernelGGL(sample_kernel<PER>, grid, block, 0, s, logits, weights, vocab, row_slot, rng, temperature, top_k, top_p, by_slot, best, out)
  // elements a thread keeps in registers: the least that covers the row
  if (vocab <= 8 * kSampleThreads) NNIS_SAMPLE(8);
  else if (vocab <= 16 * kSampleThreads) NNIS_SAMPLE(16);
  else if (vocab <= 32 * kSampleThreads) NNIS_SAMPLE(32);
  else if (vocab <= 64 * kSampleThreads) NNIS_SAMPLE(64);
  else if (vocab <= 96 * kSampleThreads) NNIS_SAMPLE(96);
  else if (vocab <= 128 * kSampleThreads) NNIS_SAMPLE(128);
  else NNIS_SAMPLE(0);
#undef NNIS_SAMPLE
  NNIS_LAUNCH_CHECK("sample");
  return 0;
}
