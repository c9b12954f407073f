// Decode-sized projections (M <= 64 tokens) fused with what stands before and
// after them in a pre-norm block, so that a layer is five kernels, not eleven:
//
//   prologue   v = x + delta            residual sum in 32-bit, written once to x_out
//              operand = bf16(v * g)    g: the norm's weight
//              ss += v * v              while K streams by anyway
//   product    acc = W . operand        v_mfma_f32_16x16x32_bf16, weights streamed once
//   epilogue   y = acc / sqrt(ss / K + eps)   the row's scale commutes with the product
//              then one of: store | SiLU(gate) * up | rotate-half RoPE and cache write
//
// When the projection before (nnis_gemm_residual) has taken the sum and left bf16(v * g) and parts of ss
// behind, the prologue is a plain operand load and a sum of those parts (PREP).
//
// RMSNorm as in /root/reference/crates/nnis-model/src/kernels.rs:15-48 (eps inside
// the root, mean over the row); SiLU-multiply as fused_swiglu.rs:14-28; RoPE as
// runtime_kernels.rs:38-66; keys stored rotated, values as they are
// (runtime.rs:997-1016).  Statistics, the scale, the activation and the rotation
// are 32-bit; the only rounding before the product is that of its bfloat16 operand.
//
// A wave owns one unit of output: a strip of 16 weight rows, or a pair of strips
// that the epilogue needs together (gate and up rows of the same channels; the
// two halves of a head that rotate into each other).  KSPLIT waves share a
// unit's K and add their parts, and their partial sums of squares, through LDS.
#include "common.h"
#include "epilogue.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr size_t kRereadWeightBytes = 8u << 20;  // as in gemm_mfma.hip

struct FusedArgs {
  // prepared by the projection before: the operand and parts of each row's sum of squares
  const bf16_t* scaled;  // [m, k]
  const float* ss_parts;  // [parts, m]
  int parts;
  // or taken here:
  const float* x_in;    // [m, k]
  const bf16_t* delta;  // [m, k] or null
  float* x_out;         // [m, k], written when delta != null
  const void* norm_w;   // [k]
  int norm_w_dtype;
  float eps;
  const bf16_t* w;  // [n, k], packed (nnis_pack_weight)
  int stream_weights;  // large weights, read once: loaded past the caches' keeping (as in gemm_mfma.hip)
  int m, n, k;
  bf16_t* y;  // store: [m, n]; silu: [m, n / 2]; rope: queries [m, heads * head_dim] (= rope.q_out)
  RopeTarget rope;
};

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

constexpr size_t kStreamWeightBytes = 16u << 20;  // as in gemm_mfma.hip

__device__ __forceinline__ bf16x8 load_weight(const bf16_t* p, int stream) {
  return stream ? __builtin_nontemporal_load((const bf16x8*)p) : *(const bf16x8*)p;
}

// eight consecutive floats of the norm weight, whatever its storage type
__device__ __forceinline__ void load_gain8(const void* base, int dtype, int index, float (&out)[8]) {
  if (dtype == NNIS_F32) {
    const f32x4 a = *(const f32x4*)((const float*)base + index);
    const f32x4 b = *(const f32x4*)((const float*)base + index + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      out[e] = a[e];
      out[4 + e] = b[e];
    }
  } else {
    const bf16x8 v = *(const bf16x8*)((const bf16_t*)base + index);
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = (float)v[e];
  }
}

template <int MT, int KSPLIT, int EPI, bool PREP, bool DEAL = false>
__global__ __launch_bounds__(KSPLIT > 4 ? 64 * KSPLIT : 256) void gemm_fused_kernel(FusedArgs a, int tiles) {
  constexpr bool PAIR = EPI != EPI_STORE;
  constexpr int NACC = PAIR ? 2 : 1;
  constexpr int kWaves = KSPLIT > 4 ? KSPLIT : 4;
  constexpr int kUnits = kWaves / KSPLIT;  // units per block
  // steps of 64 k whose loads are in flight together
  constexpr int DEPTH = PREP ? (MT <= 2 ? 4 : 2) : (MT == 1 ? 2 : 1);
  __shared__ float part_acc[KSPLIT > 1 ? kWaves : 1][NACC][MT][kWave][4];
  __shared__ float part_ss[KSPLIT > 1 ? kWaves : 1][MT][kWave];

  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  int unit_block, tile;
  nnis_deal_tiles(blockIdx.x, tiles, unit_block, tile);
  const int unit = unit_block * kUnits + wave / KSPLIT;
  const int token0 = tile * 16 * MT;  // this block's tokens: token0 + (0 .. 16 * MT - 1)
  const int part = wave % KSPLIT;
  const int r = lane % 16, g = lane / 16;
  const int k = a.k, m = a.m, n = a.n;

  // rows of the weight this unit multiplies
  int units, row0, row1 = 0;
  if (EPI == EPI_STORE) {
    units = (n + 15) / 16;
    row0 = unit * 16;
  } else if (EPI == EPI_SILU) {
    units = (n / 2 + 15) / 16;
    row0 = unit * 16;
    row1 = n / 2 + unit * 16;
  } else {
    const int per_head = a.rope.head_dim / 32;
    units = (a.rope.heads + 2 * a.rope.kv_heads) * per_head;
    row0 = (unit / per_head) * a.rope.head_dim + (unit % per_head) * 16;
    row1 = row0 + a.rope.head_dim / 2;
  }
  const bool active = unit < units;
  const int row_limit = EPI == EPI_SILU ? n / 2 : n;  // rows0 beyond this are padding of the last strip

  // What the rotating epilogue needs of each token hangs on the token's position and slot, which are
  // asked for here; the loads that depend on them (`dependent` below) are issued after the first
  // round of weight loads, so that the wave that ends the unit does not wait for them before it
  // has asked for its weights.  The same goes for the parts of a prepared norm's sums of squares.
  int tok_slot[MT], tok_pos[MT], tok_page[MT];
  f32x4 tok_cos[MT], tok_sin[MT];
  constexpr int kPartRegs = 8;  // parts of a row's sum of squares a lane keeps in flight (4 lane groups share a row)
  float ss_held[MT][kPartRegs];
  const bool ends_unit = active && part == 0;
  // The parts of a prepared row's sum of squares: a narrow row's few (up to 64) are all asked for by the lane
  // groups of the wave that ends the unit, eight in flight each.  DEAL: a wide row's (a hundred and more) are
  // dealt to the lane groups of all the waves that share the unit's K, so that they are one round trip too and
  // not a chain of them (2048 columns, 8 tokens: the gate/up product 24.9 -> 16 us, the QKV product 14.2 -> 9).
  // The waves' sums meet in LDS with the products' (part_ss), the lane groups' in the shuffles below.  A
  // variant of its own: on narrow rows the dealing, and even its code beside the other, was measured slower
  // (576 columns: a decode step of 30 layers 0.896 and 0.882 against 0.859 ms).
  static_assert(!DEAL || (PREP && KSPLIT > 1), "parts are dealt among the waves that share a prepared operand's K");
  const bool takes_parts = DEAL ? active : ends_unit;
  const int part_first = g + (DEAL ? 4 * part : 0);
  constexpr int part_stride = DEAL ? 4 * KSPLIT : 4;
  const bool tables = EPI == EPI_ROPE && a.rope.tok_cos != nullptr;  // the step's tables: nothing hangs on a loaded value
  if (EPI == EPI_ROPE && ends_unit) {
    const int head = row0 / a.rope.head_dim;
    const int f0 = row0 % a.rope.head_dim + g * 4;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      int token = token0 + t * 16 + r;
      token = token < m ? token : m - 1;
      tok_slot[t] = tables ? 0 : a.rope.tok_slot[token];
      tok_pos[t] = a.rope.tok_pos[token];
      tok_page[t] = -1;
      if (tables) {
        if (head < a.rope.heads + a.rope.kv_heads) {
          tok_cos[t] = *(const f32x4*)(a.rope.tok_cos + (size_t)token * (a.rope.head_dim / 2) + f0);
          tok_sin[t] = *(const f32x4*)(a.rope.tok_sin + (size_t)token * (a.rope.head_dim / 2) + f0);
        }
        if (head >= a.rope.heads && a.rope.k_pages) tok_page[t] = a.rope.tok_page[token];
      }
    }
  }
  auto dependent = [&]() {
    if (EPI == EPI_ROPE && ends_unit && !tables) {
      const int head = row0 / a.rope.head_dim;
      const int f0 = row0 % a.rope.head_dim + g * 4;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        if (head < a.rope.heads + a.rope.kv_heads) {
          tok_cos[t] = *(const f32x4*)(a.rope.cos_table + (size_t)tok_pos[t] * (a.rope.head_dim / 2) + f0);
          tok_sin[t] = *(const f32x4*)(a.rope.sin_table + (size_t)tok_pos[t] * (a.rope.head_dim / 2) + f0);
        }
        if (head >= a.rope.heads && tok_slot[t] >= 0 && a.rope.k_pages)
          tok_page[t] = a.rope.block_table[(size_t)tok_slot[t] * a.rope.max_pages + tok_pos[t] / kPageTokens];
      }
    }
    if (PREP && takes_parts) {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int token = token0 + t * 16 + r;
#pragma unroll
        for (int i = 0; i < kPartRegs; ++i) {
          const int p = part_first + part_stride * i;
          ss_held[t][i] = (token < m && p < a.parts) ? a.ss_parts[(size_t)p * m + token] : 0.0f;
        }
      }
    }
  };

  f32x4 acc[NACC][MT];
  float ss[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    ss[t] = 0.0f;
#pragma unroll
    for (int j = 0; j < NACC; ++j) acc[j][t] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
  }
  if (active) {
    int wr0 = row0 + r, wr1 = row1 + r;
    wr0 = wr0 < row_limit ? wr0 : row_limit - 1;
    wr1 = wr1 < n ? wr1 : n - 1;
    const int chunks = nnis_packed_chunks(k);
    const bf16_t* w0 = a.w + nnis_packed_lane(wr0, g, k);  // packed weights: chunk c at + c * 1024, the second half at + 512
    const bf16_t* w1 = a.w + nnis_packed_lane(wr1, g, k);
    size_t x_row[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      int token = token0 + t * 16 + r;
      token = token < m ? token : m - 1;
      x_row[t] = (size_t)token * k;
    }
    const bool writes_x = !PREP && a.delta != nullptr && unit == 0;  // the first unit's waves cover every k once
    const bool gain_f32 = a.norm_w_dtype == NNIS_F32;
    if (DEAL && part >= chunks) dependent();  // a wave without a share of K still takes its share of the parts
    if constexpr (PREP) {
      for (int base = part; base < chunks; base += KSPLIT * DEPTH) {
        bf16x8 wa[DEPTH][2], wb[DEPTH][2], xs[DEPTH][2][MT];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d)
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const int c = base + d * KSPLIT;
            const int kk = c * 64 + g * 16 + half * 8;
            const bool in = kk + 8 <= k;
            const size_t at = (size_t)c * kPackedChunkElems + half * kPackedHalfElems;
            wa[d][half] = in ? load_weight(w0 + at, a.stream_weights) : zero8();
            wb[d][half] = (PAIR && in) ? load_weight(w1 + at, a.stream_weights) : zero8();
#pragma unroll
            for (int t = 0; t < MT; ++t) xs[d][half][t] = in ? *(const bf16x8*)(a.scaled + x_row[t] + kk) : zero8();
          }
        if (base == part) dependent();
#pragma unroll
        for (int d = 0; d < DEPTH; ++d)
#pragma unroll
          for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int t = 0; t < MT; ++t) {
              acc[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[d][half], xs[d][half][t], acc[0][t], 0, 0, 0);
              if (PAIR) acc[1][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[d][half], xs[d][half][t], acc[1][t], 0, 0, 0);
            }
      }
    } else
    // The product is bound by memory latency: a wave asks for everything its next
    // DEPTH steps of 64 k need (weights, residual, pending sum, gain) before it
    // touches any of it, so its share of K is one round trip, not one per step.
    // A matrix instruction runs for the whole wave whatever lanes a branch has
    // switched off: a lane whose 8 k lie beyond K feeds it zeros, it never skips
    // it.  K is a multiple of 8: a group of 8 is whole or absent.
    for (int base = part; base < chunks; base += KSPLIT * DEPTH) {
      bf16x8 wa[DEPTH][2], wb[DEPTH][2], dl[DEPTH][2][MT];
      f32x4 xr[DEPTH][2][MT][2], gr[DEPTH][2][2];
#pragma unroll
      for (int d = 0; d < DEPTH; ++d)
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const int c = base + d * KSPLIT;
          const int kk = c * 64 + g * 16 + half * 8;
          const bool in = kk + 8 <= k;
          const size_t at = (size_t)c * kPackedChunkElems + half * kPackedHalfElems;
          wa[d][half] = in ? load_weight(w0 + at, a.stream_weights) : zero8();
          wb[d][half] = (PAIR && in) ? load_weight(w1 + at, a.stream_weights) : zero8();
          if (in) {
            if (gain_f32) {
              gr[d][half][0] = *(const f32x4*)((const float*)a.norm_w + kk);
              gr[d][half][1] = *(const f32x4*)((const float*)a.norm_w + kk + 4);
            } else {
              gr[d][half][0] = *(const f32x4*)((const bf16_t*)a.norm_w + kk);  // 8 bfloat16, unpacked below
            }
#pragma unroll
            for (int t = 0; t < MT; ++t) {
              xr[d][half][t][0] = *(const f32x4*)(a.x_in + x_row[t] + kk);
              xr[d][half][t][1] = *(const f32x4*)(a.x_in + x_row[t] + kk + 4);
              if (a.delta) dl[d][half][t] = *(const bf16x8*)(a.delta + x_row[t] + kk);
            }
          }
        }
      if (base == part) dependent();
#pragma unroll
      for (int d = 0; d < DEPTH; ++d)
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const int kk = (base + d * KSPLIT) * 64 + g * 16 + half * 8;
          const bool in = kk + 8 <= k;
          float gain[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) gain[e] = 0.0f;
          if (in) {
            if (gain_f32) {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                gain[e] = gr[d][half][0][e];
                gain[4 + e] = gr[d][half][1][e];
              }
            } else {
              const bf16x8 packed = __builtin_bit_cast(bf16x8, gr[d][half][0]);
#pragma unroll
              for (int e = 0; e < 8; ++e) gain[e] = (float)packed[e];
            }
          }
#pragma unroll
          for (int t = 0; t < MT; ++t) {
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = 0.0f;
            if (in) {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                v[e] = xr[d][half][t][0][e];
                v[4 + e] = xr[d][half][t][1][e];
              }
              if (a.delta) {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] += (float)dl[d][half][t][e];
                if (writes_x && token0 + t * 16 + r < m) {
                  *(f32x4*)(a.x_out + x_row[t] + kk) = (f32x4){v[0], v[1], v[2], v[3]};
                  *(f32x4*)(a.x_out + x_row[t] + kk + 4) = (f32x4){v[4], v[5], v[6], v[7]};
                }
              }
            }
            bf16x8 operand;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              ss[t] = fmaf(v[e], v[e], ss[t]);
              operand[e] = (__bf16)(v[e] * gain[e]);
            }
            acc[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[d][half], operand, acc[0][t], 0, 0, 0);
            if (PAIR) acc[1][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wb[d][half], operand, acc[1][t], 0, 0, 0);
          }
        }
    }
  }
  if (PREP && takes_parts) {
#pragma unroll
    for (int t = 0; t < MT; ++t) {
#pragma unroll
      for (int i = 0; i < kPartRegs; ++i) ss[t] += ss_held[t][i];
      const int token = token0 + t * 16 + r;
      if (token < m) {  // more parts than the lanes that take them hold at once
        if constexpr (DEAL) {  // eight more at a time
          for (int p0 = part_first + part_stride * kPartRegs; p0 < a.parts; p0 += part_stride * kPartRegs) {
            float more[kPartRegs];
#pragma unroll
            for (int i = 0; i < kPartRegs; ++i) {
              const int p = p0 + part_stride * i;
              more[i] = p < a.parts ? a.ss_parts[(size_t)p * m + token] : 0.0f;
            }
#pragma unroll
            for (int i = 0; i < kPartRegs; ++i) ss[t] += more[i];
          }
        } else {
          for (int p = g + 4 * kPartRegs; p < a.parts; p += 4) ss[t] += a.ss_parts[(size_t)p * m + token];
        }
      }
    }
  }
  // a token's sum of squares: over the four lane groups of this wave, then over the waves that share K
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    ss[t] += __shfl_xor(ss[t], 16, kWave);
    ss[t] += __shfl_xor(ss[t], 32, kWave);
  }
  if constexpr (KSPLIT > 1) {
    if (part != 0) {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        part_ss[wave][t][lane] = ss[t];
#pragma unroll
        for (int j = 0; j < NACC; ++j)
#pragma unroll
          for (int e = 0; e < 4; ++e) part_acc[wave][j][t][lane][e] = acc[j][t][e];
      }
    }
    __syncthreads();
    if (part != 0) return;
#pragma unroll
    for (int other = 1; other < KSPLIT; ++other)
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        ss[t] += part_ss[wave + other][t][lane];
#pragma unroll
        for (int j = 0; j < NACC; ++j)
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[j][t][e] += part_acc[wave + other][j][t][lane][e];
      }
  }
  if (!active) return;

  // lane holds D[row 4g + e][token r] of each strip
  const float inv_k = 1.0f / (float)k;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int token = token0 + t * 16 + r;
    if (token >= m) continue;
    const float scale = 1.0f / sqrtf(ss[t] * inv_k + a.eps);
    if (EPI == EPI_STORE) {
      const int n0 = row0 + g * 4;
      for (int e = 0; e < 4; ++e)
        if (n0 + e < n) a.y[(size_t)token * n + n0 + e] = (bf16_t)(acc[0][t][e] * scale);
    } else {
      float lo[4], hi[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo[e] = acc[0][t][e] * scale;
        hi[e] = acc[1][t][e] * scale;
      }
      if (EPI == EPI_SILU) {
        epilogue_silu(a.y, token, n / 2, row0 + g * 4, lo, hi);
      } else {
        const int hd = a.rope.head_dim;
        epilogue_rope(a.rope, token, tok_pos[t], tok_page[t], row0 / hd, row0 % hd + g * 4, lo, hi, tok_cos[t], tok_sin[t]);
      }
    }
  }
}

constexpr int kDealPartsFrom = 64;  // rows of more parts than this take the variant that deals them to all waves

template <int MT, int KSPLIT, int EPI>
void launch_fused(const FusedArgs& a, int units, hipStream_t stream) {
  constexpr int kWaves = KSPLIT > 4 ? KSPLIT : 4;
  constexpr int kUnits = kWaves / KSPLIT;
  const int unit_blocks = (units + kUnits - 1) / kUnits;
  const int tiles = (a.m + 16 * MT - 1) / (16 * MT);
  const dim3 grid(tiles == 1 ? unit_blocks : (unit_blocks + 7) / 8 * 8 * tiles), block(64 * kWaves);
  if constexpr (KSPLIT > 1) {
    if (a.scaled && a.parts > kDealPartsFrom) {
      hipLaunchKernelGGL((gemm_fused_kernel<MT, KSPLIT, EPI, true, true>), grid, block, 0, stream, a, tiles);
      return;
    }
  }
  if (a.scaled) hipLaunchKernelGGL((gemm_fused_kernel<MT, KSPLIT, EPI, true>), grid, block, 0, stream, a, tiles);
  else hipLaunchKernelGGL((gemm_fused_kernel<MT, KSPLIT, EPI, false>), grid, block, 0, stream, a, tiles);
}

template <int MT, int EPI>
void dispatch_fused_split(const FusedArgs& a, int units, int split, hipStream_t stream) {
  if (split == 8 && MT <= 2) launch_fused<MT, (MT <= 2 ? 8 : 4), EPI>(a, units, stream);
  else if (split >= 4) launch_fused<MT, 4, EPI>(a, units, stream);
  else if (split == 2) launch_fused<MT, 2, EPI>(a, units, stream);
  else launch_fused<MT, 1, EPI>(a, units, stream);
}

// Weights that the dies' L2 keep (a few MB) are cheaper to read again than a wave is to load with the work of
// several token tiles: then a block takes one tile of 16 tokens and the grid the rest.  Large weights are
// read once, by waves that take all tiles (up to 4).
template <int EPI>
void dispatch_fused(const FusedArgs& a, int units, int split, hipStream_t stream) {
  int tiles = (a.m + 15) / 16;
  if ((size_t)a.n * a.k * sizeof(bf16_t) <= kRereadWeightBytes) tiles = 1;
  if (tiles == 1) dispatch_fused_split<1, EPI>(a, units, split, stream);
  else if (tiles == 2) dispatch_fused_split<2, EPI>(a, units, split, stream);
  else if (tiles == 3) dispatch_fused_split<3, EPI>(a, units, split, stream);
  else dispatch_fused_split<4, EPI>(a, units, split, stream);
}

// checks what the epilogue needs, picks the split of K and launches; a.scaled tells the prologue
int run_fused(FusedArgs& a, int epilogue, int table_positions, int split_hint, float* workspace, size_t workspace_bytes,
              hipStream_t stream) {
  const int n = a.n, k = a.k;
  a.stream_weights = (size_t)n * k * sizeof(bf16_t) > kStreamWeightBytes;
  int units;
  if (epilogue == EPI_STORE) {
    units = (n + 15) / 16;
  } else if (epilogue == EPI_SILU) {
    NNIS_REQUIRE(n % 2 == 0, "gemm_fused: gate and up rows must be as many (n=%d)", n);
    units = (n / 2 + 15) / 16;
  } else if (epilogue == EPI_ROPE) {
    NNIS_REQUIRE(a.rope.heads > 0 && a.rope.kv_heads > 0 && a.rope.head_dim > 0 && a.rope.head_dim % 32 == 0,
                 "gemm_fused: the rotating epilogue needs a head size in steps of 32, got %d", a.rope.head_dim);
    NNIS_REQUIRE(n == (a.rope.heads + 2 * a.rope.kv_heads) * a.rope.head_dim, "gemm_fused: %d weight rows for %d+2*%d heads of %d", n, a.rope.heads,
                 a.rope.kv_heads, a.rope.head_dim);
    NNIS_REQUIRE(a.rope.cos_table && a.rope.sin_table && a.rope.tok_slot && a.rope.tok_pos, "gemm_fused: the rotating epilogue needs tables and positions");
    NNIS_REQUIRE((a.rope.k_pages == nullptr) == (a.rope.v_pages == nullptr), "gemm_fused: key and value pages must come together");
    NNIS_REQUIRE(a.rope.k_pages == nullptr || (a.rope.block_table && a.rope.max_pages > 0), "gemm_fused: cache without a block table");
    NNIS_REQUIRE(table_positions > 0, "gemm_fused: empty rotation tables");
    NNIS_REQUIRE((a.rope.tok_cos != nullptr) == (a.rope.tok_sin != nullptr) && (a.rope.tok_cos != nullptr) == (a.rope.tok_page != nullptr),
                 "gemm_fused: the step's tables (rotation rows and pages of the tokens) come together or not at all");
    NNIS_REQUIRE((uintptr_t)a.rope.tok_cos % 16 == 0 && (uintptr_t)a.rope.tok_sin % 16 == 0, "gemm_fused: the step's tables must be 16-byte aligned");
    units = (a.rope.heads + 2 * a.rope.kv_heads) * (a.rope.head_dim / 32);
  } else {
    return nnis_fail("gemm_fused: unknown epilogue %d", epilogue);
  }
  // With pairs of rows a unit is 32 weight rows and there are half as many waves: beyond 32 tokens on large
  // weights the tiled kernel is faster on a prepared operand whatever the width (64 tokens, K = 2048,
  // microseconds: 2560 rows 25.5 against 18.1, 6144 rows 33 against 20; at 32 tokens 15.8 against 16.7).
  const bool many = a.scaled != nullptr && a.m > 32 && (size_t)n * k * sizeof(bf16_t) > kRereadWeightBytes;
  if (!nnis_gemm_takes_few_tokens(a.m, n, k) || many || (split_hint >= 16 && a.scaled != nullptr)) {  // a tile hint asks for the tiled kernel
    NNIS_REQUIRE(a.scaled != nullptr, "gemm_fused: %d tokens are too many for a weight of %d x %d", a.m, n, k);
    const int tile_hint = split_hint >= 16 ? split_hint / 16 : 0;
    return nnis_gemm_scaled_tiled(a.scaled, a.ss_parts, a.parts, a.eps, a.w, a.m, n, k, epilogue, a.y, a.rope, tile_hint, workspace,
                                  workspace_bytes, stream);
  }
  // few units: their waves share K so that each wave's share is one round of loads
  const int chunks = (k + 63) / 64;
  const int per_wave = (size_t)n * k * sizeof(bf16_t) <= kRereadWeightBytes ? 1 : (a.m + 15) / 16;  // token tiles a wave takes
  const int depth = a.scaled ? (per_wave <= 2 ? 4 : 2) : (per_wave == 1 ? 2 : 1);  // the kernel's steps in flight
  // On a prepared operand no more waves than take 4,096 strips of 16 weight rows between them (two waves a SIMD at
  // pairs of strips): every wave begins with the row's scale, and beyond that number the beginnings cost more than
  // the shorter shares save.  Measured at 1 and 8 tokens over cold weights, microseconds with 8 / 4 / 2 waves a unit:
  // gate/up of 2 x 5632 x 2048 14.1 / 12.5 / 13.3, 2 x 8192 x 2048 16.2 / 15.3 / 15.5, 2 x 14336 x 4096 49.0 / 46.1 /
  // 45.3; plain rows 11264 x 2048 14.2 / 11.7 / 14.5, 28672 x 2048 30.5 / 25.6 / 25.9; up to 512 strips 8 waves
  // are the fastest (8192 x 2048 9.4 / 9.9 / 11.3).
  const int strips = epilogue == EPI_STORE ? units : (epilogue == EPI_SILU ? 2 * units : 0);  // (the rotating epilogue gains nothing: 96 x 128 x 4096 25.1 / 25.7 / 26.0)
  int split = 1;
  if (units < 2048) {
    while (split < 8 && chunks > split * depth && (!a.scaled || strips * split * 2 <= 4096)) split *= 2;
  }
  if (split_hint == 1 || split_hint == 2 || split_hint == 4 || split_hint == 8) split = split_hint;  // for tuning runs
  if (epilogue == EPI_STORE) dispatch_fused<EPI_STORE>(a, units, split, stream);
  else if (epilogue == EPI_SILU) dispatch_fused<EPI_SILU>(a, units, split, stream);
  else dispatch_fused<EPI_ROPE>(a, units, split, stream);
  NNIS_LAUNCH_CHECK("gemm_fused");
  return 0;
}

}  // namespace

// epilogue: 0 store [m, n]; 1 SiLU(gate) * up -> [m, n / 2] (gate rows first); 2 RoPE + cache write,
// queries -> y [m, heads * head_dim].  delta may be null (then x_out is not written).  split_hint: 0, or the
// number of waves (1, 2, 4, 8) that share a unit's K, overriding the choice made here.
extern "C" int nnis_gemm_fused(const float* x_in, const void* delta, float* x_out, const void* norm_w, int norm_w_dtype,
                               float eps, const void* w, int m, int n, int k, int epilogue, void* y, const float* cos_table,
                               const float* sin_table, int table_positions, const int* tok_slot, const int* tok_pos,
                               void* k_pages, void* v_pages, const int* block_table, int max_pages, int heads, int kv_heads,
                               int head_dim, const float* tok_cos, const float* tok_sin, const int* tok_page, int split_hint,
                               void* stream_ptr) {
  NNIS_REQUIRE(m > 0 && nnis_gemm_takes_few_tokens(m, n, k), "gemm_fused: %d tokens are too many for a weight of %d x %d", m, n, k);
  NNIS_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_fused: bad sizes n=%d k=%d (K must be a multiple of 8)", n, k);
  NNIS_REQUIRE(nnis_dtype_ok(norm_w_dtype), "gemm_fused: unknown norm weight dtype %d", norm_w_dtype);
  NNIS_REQUIRE(eps > 0.0f, "gemm_fused: eps must be positive");
  NNIS_REQUIRE(delta == nullptr || x_out != nullptr, "gemm_fused: a pending sum needs a place for the new residual");
  NNIS_REQUIRE(x_out != x_in, "gemm_fused: the new residual must not overwrite the one being read");
  for (const void* p : {(const void*)x_in, delta, (const void*)x_out, norm_w, w, (const void*)y})
    NNIS_REQUIRE((uintptr_t)p % 16 == 0, "gemm_fused: operands must be 16-byte aligned");
  FusedArgs a;
  a.scaled = nullptr; a.ss_parts = nullptr; a.parts = 0;
  a.x_in = x_in; a.delta = (const bf16_t*)delta; a.x_out = x_out; a.norm_w = norm_w; a.norm_w_dtype = norm_w_dtype;
  a.eps = eps; a.w = (const bf16_t*)w; a.m = m; a.n = n; a.k = k; a.y = (bf16_t*)y;
  a.rope.q_out = (bf16_t*)y; a.rope.cos_table = cos_table; a.rope.sin_table = sin_table; a.rope.tok_slot = tok_slot; a.rope.tok_pos = tok_pos;
  a.rope.k_pages = (bf16_t*)k_pages; a.rope.v_pages = (bf16_t*)v_pages; a.rope.block_table = block_table; a.rope.max_pages = max_pages;
  a.rope.heads = heads; a.rope.kv_heads = kv_heads; a.rope.head_dim = head_dim;
  a.rope.tok_cos = tok_cos; a.rope.tok_sin = tok_sin; a.rope.tok_page = tok_page;
  return run_fused(a, epilogue, table_positions, split_hint, nullptr, 0, (hipStream_t)stream_ptr);
}

// The same product and epilogues on an operand that nnis_gemm_residual prepared: scaled = bf16(v * g)
// [m, k] and ss_parts [parts, m], whose sum over the parts is a row's sum of squares.
extern "C" int nnis_gemm_scaled(const void* scaled, const float* ss_parts, int parts, float eps, const void* w, int m, int n,
                                int k, int epilogue, void* y, const float* cos_table, const float* sin_table,
                                int table_positions, const int* tok_slot, const int* tok_pos, void* k_pages, void* v_pages,
                                const int* block_table, int max_pages, int heads, int kv_heads, int head_dim,
                                const float* tok_cos, const float* tok_sin, const int* tok_page, int split_hint,
                                float* workspace, size_t workspace_bytes, void* stream_ptr) {
  NNIS_REQUIRE(m > 0, "gemm_scaled: no tokens");
  NNIS_REQUIRE((uintptr_t)workspace % 16 == 0, "gemm_scaled: the workspace must be 16-byte aligned");
  NNIS_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_scaled: bad sizes n=%d k=%d (K must be a multiple of 8)", n, k);
  NNIS_REQUIRE(scaled && ss_parts && parts > 0, "gemm_scaled: the prepared operand is missing");
  NNIS_REQUIRE(eps > 0.0f, "gemm_scaled: eps must be positive");
  for (const void* p : {scaled, w, (const void*)y})
    NNIS_REQUIRE((uintptr_t)p % 16 == 0, "gemm_scaled: operands must be 16-byte aligned");
  FusedArgs a;
  a.scaled = (const bf16_t*)scaled; a.ss_parts = ss_parts; a.parts = parts;
  a.x_in = nullptr; a.delta = nullptr; a.x_out = nullptr; a.norm_w = nullptr; a.norm_w_dtype = NNIS_F32;
  a.eps = eps; a.w = (const bf16_t*)w; a.m = m; a.n = n; a.k = k; a.y = (bf16_t*)y;
  a.rope.q_out = (bf16_t*)y; a.rope.cos_table = cos_table; a.rope.sin_table = sin_table; a.rope.tok_slot = tok_slot; a.rope.tok_pos = tok_pos;
  a.rope.k_pages = (bf16_t*)k_pages; a.rope.v_pages = (bf16_t*)v_pages; a.rope.block_table = block_table; a.rope.max_pages = max_pages;
  a.rope.heads = heads; a.rope.kv_heads = kv_heads; a.rope.head_dim = head_dim;
  a.rope.tok_cos = tok_cos; a.rope.tok_sin = tok_sin; a.rope.tok_page = tok_page;
  return run_fused(a, epilogue, table_positions, split_hint, workspace, workspace_bytes, (hipStream_t)stream_ptr);
}
