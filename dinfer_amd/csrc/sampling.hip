// Token selection on float logits: argmax, and the chain penalties -> temperature ->
// min_p -> top-k / top-p -> inverse-CDF draw with a counter-based random number.
// The chain exists in two forms that follow the same rule: one kernel with one
// workgroup of 1024 threads per row (first half of this file), and five launches
// that spread a row over many workgroups (second half; what the sampler uses, a
// tenth of the time at a vocabulary of 152k). Penalties come from a list of the
// row's tokens, or from a per-request history kept on the device.
//
//   greedy (temperature <= 1e-5): largest logit, ties to the lowest index.
//   otherwise: z = logit / temperature; min_p drops z with
//     softmax(z) < min_p * max softmax(z); top-k keeps the k largest; top-p
//     keeps, of what is left, the most probable tokens up to and including
//     the one that crosses p; then p_i = exp(z_i - max z),
//     u = Philox4x32-10(key = seed, counter = (offset, 0, 0)) -> (c0 >> 8) * 2^-24,
//     target = u * sum p, and the first index in vocabulary order whose
//     running sum reaches target (with p_i > 0) is chosen; if rounding leaves
//     none, the last index with a finite logit.
// The (seed, offset) pair alone fixes the random number, so a request's draw
// does not depend on its row in the batch or on the other rows.
//
// Reference behaviour: crates/kernels/cuda/sampling.cu:13-56 (argmax),
// :85-133 (top-k / top-p by threshold search), :137-157 (Philox), :159-263
// (draw), :266-283 (fused order), :318-349 (penalties), :352-364 (min_p),
// :290-316 (logit_bias), :380-430 (log-probabilities of the chosen and the most probable tokens).
#include "common.cuh"

using namespace dinfer;

namespace {

constexpr int BLOCK = 1024;
constexpr int NWAVE = BLOCK / 64;

struct Red {
  float f[NWAVE];
  int i[NWAVE];
};

__device__ __forceinline__ void better(float& v, int& i, float ov, int oi) {
  if (ov > v || (ov == v && oi < i)) {
    v = ov;
    i = oi;
  }
}

// (value, index) argmax over the workgroup; every thread gets the result.
__device__ int block_argmax(float v, int i, Red& red, float* best_out) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, 64);
    const int oi = __shfl_xor(i, o, 64);
    better(v, i, ov, oi);
  }
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) {
    red.f[w] = v;
    red.i[w] = i;
  }
  __syncthreads();
  float bv = red.f[0];
  int bi = red.i[0];
  for (int k = 1; k < NWAVE; ++k) better(bv, bi, red.f[k], red.i[k]);
  if (best_out) *best_out = bv;
  return bi;
}

__device__ int row_argmax(const float* row, int vocab, Red& red) {
  float best = -INFINITY;
  int besti = 0x7fffffff;
  int i0 = 0;
  if (((uintptr_t)row & 15) == 0) {
    // 16-byte loads, four in flight per thread; a thread's indices still grow, so ties keep the lowest
    const f32x4* r4 = (const f32x4*)row;
    const int n4 = vocab >> 2;
    int j = threadIdx.x;
    for (; j + 3 * BLOCK < n4; j += 4 * BLOCK) {
      const f32x4 a = r4[j], b = r4[j + BLOCK], c = r4[j + 2 * BLOCK], d = r4[j + 3 * BLOCK];
#pragma unroll
      for (int e = 0; e < 4; ++e) better(best, besti, a[e], 4 * j + e);
#pragma unroll
      for (int e = 0; e < 4; ++e) better(best, besti, b[e], 4 * (j + BLOCK) + e);
#pragma unroll
      for (int e = 0; e < 4; ++e) better(best, besti, c[e], 4 * (j + 2 * BLOCK) + e);
#pragma unroll
      for (int e = 0; e < 4; ++e) better(best, besti, d[e], 4 * (j + 3 * BLOCK) + e);
    }
    for (; j < n4; j += BLOCK) {
      const f32x4 a = r4[j];
#pragma unroll
      for (int e = 0; e < 4; ++e) better(best, besti, a[e], 4 * j + e);
    }
    i0 = n4 << 2;
  }
  for (int i = i0 + threadIdx.x; i < vocab; i += BLOCK) better(best, besti, row[i], i);
  const int r = block_argmax(best, besti, red, nullptr);
  return r == 0x7fffffff ? 0 : r;
}

__device__ float row_max(const float* row, int vocab, float* red) {
  float m = -INFINITY;
  for (int i = threadIdx.x; i < vocab; i += BLOCK) m = fmaxf(m, row[i]);
  return block_max(m, red);
}

__device__ float row_expsum_ge(const float* row, int vocab, float m, float t, float* red) {
  float s = 0.f;
  for (int i = threadIdx.x; i < vocab; i += BLOCK) {
    const float v = row[i];
    if (v >= t && v > -INFINITY) s += expf(v - m);
  }
  return block_sum(s, red);
}

__device__ void row_min_p(float* row, int vocab, float mp, float* red) {
  if (mp <= 0.f) return;
  const float m = row_max(row, vocab, red);
  // p_i / p_max = exp(z_i - m) < min_p  <=>  dropped
  __syncthreads();
  for (int i = threadIdx.x; i < vocab; i += BLOCK) {
    const float v = row[i];
    if (v > -INFINITY && expf(v - m) < mp) row[i] = -INFINITY;
  }
  __syncthreads();
}

// Floats as unsigned keys of the same order (a larger float has a larger key; -0 counts as +0, -inf is the lowest
// key a row holds): thresholds can then be found digit by digit, exactly, instead of by halving an interval.
__device__ __forceinline__ uint32_t order_key(float v) {
  const uint32_t u = __float_as_uint(v + 0.f);
  return (u >> 31) ? ~u : (u | 0x80000000u);
}

// The key of the k-th largest entry of the row (1 <= k <= vocab): a radix selection, eight bits a pass. Each pass
// counts, among the entries that share the digits fixed so far, how many hold each value of the next digit
// (integer counters in LDS: the counts do not depend on the order of arrival), then walks the 256 counters from
// the top until the k-th entry is reached.
__device__ uint32_t row_kth_key(const float* row, int vocab, int k) {
  __shared__ int digit_count[256];
  __shared__ uint32_t chosen[2];   // the digit found, and how many entries are still to be skipped inside it
  uint32_t prefix = 0;
  int skip = k;                    // the entry looked for is the skip-th largest among those that match the prefix
  for (int shift = 24; shift >= 0; shift -= 8) {
    __syncthreads();
    if (threadIdx.x < 256) digit_count[threadIdx.x] = 0;
    __syncthreads();
    const uint32_t fixed = shift == 24 ? 0u : 0xffffffffu << (shift + 8);
    for (int i = threadIdx.x; i < vocab; i += BLOCK) {
      const uint32_t key = order_key(row[i]);
      if ((key & fixed) == prefix) atomicAdd(&digit_count[(key >> shift) & 255u], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      int d = 255, left = skip;
      while (d > 0 && digit_count[d] < left) left -= digit_count[d--];
      chosen[0] = (uint32_t)d;
      chosen[1] = (uint32_t)left;
    }
    __syncthreads();
    prefix |= chosen[0] << shift;
    skip = (int)chosen[1];
  }
  return prefix;
}

// Sum of exp(v - m) over the entries whose key is at least `least`.
__device__ float row_mass_from_key(const float* row, int vocab, float m, uint32_t least, float* red) {
  float s = 0.f;
  for (int i = threadIdx.x; i < vocab; i += BLOCK) {
    const float v = row[i];
    if (order_key(v) >= least && v > -INFINITY) s += expf(v - m);
  }
  return block_sum(s, red);
}

// top-k, then top-p on what it left: entries below the k-th largest value go, then entries below the largest value t
// for which the entries from t up still hold the share p of the remaining mass (entries equal to a threshold stay).
// The second threshold is built bit by bit from the top: a bit stays set if the mass from the key so formed up
// still reaches the share.
__device__ void row_topk_topp(float* row, int vocab, int k, float p, float* red) {
  const bool cut_count = k > 0 && k < vocab, cut_mass = p > 0.f && p < 1.f;
  if (!cut_count && !cut_mass) return;
  uint32_t least = cut_count ? row_kth_key(row, vocab, k) : 0u;
  if (cut_mass) {
    const float m = row_max(row, vocab, red);
    const float share = p * row_mass_from_key(row, vocab, m, least, red);
    uint32_t t = 0;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t with_bit = t | (1u << bit);
      if (row_mass_from_key(row, vocab, m, with_bit > least ? with_bit : least, red) >= share) t = with_bit;
    }
    if (t > least) least = t;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < vocab; i += BLOCK)
    if (order_key(row[i]) < least) row[i] = -INFINITY;
  __syncthreads();
}

// Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3", SC'11): ten rounds, each
// of which multiplies words 0 and 2 of the counter by the two round constants to 64 bits, crosses the halves over
// and mixes in the key, which grows by the two Weyl constants from round to round. The uniform number of a draw is
// made of (seed, offset) alone, as the reference makes it (crates/kernels/cuda/sampling.cu:137-157): key = seed,
// counter = (offset, 0, 0), the top 24 bits of the first output word.
struct Philox {
  static constexpr uint64_t MUL_A = 0xD2511F53u, MUL_B = 0xCD9E8D57u;
  static constexpr uint32_t WEYL_A = 0x9E3779B9u, WEYL_B = 0xBB67AE85u;
  uint32_t x0, x1, x2, x3, ka, kb;

  __device__ void round() {
    const uint64_t pa = MUL_A * x0, pb = MUL_B * x2;
    const uint32_t y0 = (uint32_t)(pb >> 32) ^ x1 ^ ka, y2 = (uint32_t)(pa >> 32) ^ x3 ^ kb;
    x1 = (uint32_t)pb;
    x3 = (uint32_t)pa;
    x0 = y0;
    x2 = y2;
    ka += WEYL_A;
    kb += WEYL_B;
  }
};

__device__ float philox_uniform(uint64_t seed, uint64_t offset) {
  Philox g{(uint32_t)offset, (uint32_t)(offset >> 32), 0u, 0u, (uint32_t)seed, (uint32_t)(seed >> 32)};
#pragma unroll
  for (int r = 0; r < 10; ++r) g.round();
  return (float)(g.x0 >> 8) * 0x1p-24f;
}

struct DrawShared {
  float wave_tot[NWAVE];
  float carry;
  int choice;
};

// row holds z (already divided by the temperature, masked entries -inf).
__device__ int row_draw(const float* row, int vocab, uint64_t seed, uint64_t offset, float* red, DrawShared& sh) {
  const float m = row_max(row, vocab, red);
  const float denom = row_expsum_ge(row, vocab, m, -INFINITY, red);
  const float target = philox_uniform(seed, offset) * denom;
  if (threadIdx.x == 0) {
    sh.carry = 0.f;
    sh.choice = 0x7fffffff;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  for (int base = 0; base < vocab; base += BLOCK) {
    const int i = base + threadIdx.x;
    float p = 0.f;
    if (i < vocab) {
      const float v = row[i];
      p = v > -INFINITY ? expf(v - m) : 0.f;
    }
    // inclusive scan inside the wave, then over the 16 wave totals in index order
    float incl = p;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const float up = __shfl_up(incl, o, 64);
      if (lane >= o) incl += up;
    }
    if (lane == 63) sh.wave_tot[w] = incl;
    __syncthreads();
    float before = sh.carry;
    for (int k = 0; k < w; ++k) before += sh.wave_tot[k];
    const float cum = before + incl;
    const float prev = cum - p;
    if (i < vocab && p > 0.f && prev < target && cum >= target) atomicMin(&sh.choice, i);
    __syncthreads();
    if (threadIdx.x == BLOCK - 1) sh.carry = cum;
    __syncthreads();
    if (sh.choice != 0x7fffffff) break;  // uniform: read after the barrier
  }
  int c = sh.choice;
  if (c == 0x7fffffff) {
    // target above the rounded total: the last index with a finite logit
    int last = -1;
    for (int i = threadIdx.x; i < vocab; i += BLOCK)
      if (row[i] > -INFINITY) last = i;
    float lv = (float)last;  // indices < 2^24 are exact in float
    lv = block_max(lv, red);
    c = lv < 0.f ? 0 : (int)lv;
  }
  return c;
}

// logits [R, ld] are read only; work [R, vocab] is scratch for non-greedy rows.
__global__ void __launch_bounds__(BLOCK) sample_kernel(const float* __restrict__ logits, int64_t ld,
                                                       float* __restrict__ work, const float* __restrict__ temperature,
                                                       const int32_t* __restrict__ top_k,
                                                       const float* __restrict__ top_p, const float* __restrict__ min_p,
                                                       const uint64_t* __restrict__ seeds,
                                                       const uint64_t* __restrict__ offsets,
                                                       int32_t* __restrict__ out, int vocab) {
  __shared__ Red red;
  __shared__ float fred[NWAVE];
  __shared__ DrawShared sh;
  const int b = blockIdx.x;
  const float* row = logits + (int64_t)b * ld;
  const float temp = temperature ? temperature[b] : 0.f;
  if (temp <= 1e-5f) {
    const int c = row_argmax(row, vocab, red);
    if (threadIdx.x == 0) out[b] = c;
    return;
  }
  float* z = work + (int64_t)b * vocab;
  const float inv_t = 1.f / temp;
  for (int i = threadIdx.x; i < vocab; i += BLOCK) z[i] = row[i] * inv_t;
  __syncthreads();
  row_min_p(z, vocab, min_p ? min_p[b] : 0.f, fred);
  row_topk_topp(z, vocab, top_k ? top_k[b] : -1, top_p ? top_p[b] : 1.f, fred);
  const int c = row_draw(z, vocab, seeds[b], offsets[b], fred, sh);
  if (threadIdx.x == 0) out[b] = c;
}

__global__ void __launch_bounds__(BLOCK) argmax_kernel(const float* __restrict__ logits, int64_t ld,
                                                       int32_t* __restrict__ out, int vocab) {
  __shared__ Red red;
  const int c = row_argmax(logits + (int64_t)blockIdx.x * ld, vocab, red);
  if (threadIdx.x == 0) out[blockIdx.x] = c;
}

// The same argmax with a row spread over many workgroups (a row of 152k entries is 600 KB: one workgroup needs
// 16 us for it, whatever the batch): every workgroup names the best of ARG_SEG entries, a second launch picks among
// the names. Both compare like row_argmax, so the result is the same index.
constexpr int ARG_SEG = 4096;
constexpr int ARG_THREADS = 256;

__global__ void __launch_bounds__(ARG_THREADS) argmax_parts_kernel(const float* __restrict__ logits, int64_t ld,
                                                                   float* __restrict__ part_val,
                                                                   int32_t* __restrict__ part_idx, int vocab, int segs) {
  __shared__ float sv[ARG_THREADS / 64];
  __shared__ int si[ARG_THREADS / 64];
  const int r = blockIdx.y, s = blockIdx.x;
  const float* row = logits + (int64_t)r * ld;
  const int lo = s * ARG_SEG, hi = min(vocab, lo + ARG_SEG);
  float best = -INFINITY;
  int besti = 0x7fffffff;
  if (((uintptr_t)(row + lo) & 15) == 0) {
    const f32x4* r4 = (const f32x4*)(row + lo);
    const int n4 = (hi - lo) >> 2;
    for (int j = threadIdx.x; j < n4; j += ARG_THREADS) {  // (ARG_SEG / 4 / ARG_THREADS = 4 loads a thread, unrolled)
      const f32x4 v = r4[j];
#pragma unroll
      for (int e = 0; e < 4; ++e) better(best, besti, v[e], lo + 4 * j + e);
    }
    for (int i = lo + 4 * n4 + threadIdx.x; i < hi; i += ARG_THREADS) better(best, besti, row[i], i);
  } else {
    for (int i = lo + threadIdx.x; i < hi; i += ARG_THREADS) better(best, besti, row[i], i);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(besti, o, 64);
    better(best, besti, ov, oi);
  }
  if ((threadIdx.x & 63) == 0) {
    sv[threadIdx.x >> 6] = best;
    si[threadIdx.x >> 6] = besti;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < ARG_THREADS / 64; ++w) better(best, besti, sv[w], si[w]);
    part_val[(int64_t)r * segs + s] = best;
    part_idx[(int64_t)r * segs + s] = besti;
  }
}

__global__ void __launch_bounds__(64) argmax_join_kernel(const float* __restrict__ part_val,
                                                         const int32_t* __restrict__ part_idx,
                                                         int32_t* __restrict__ out, int segs) {
  const int r = blockIdx.x;
  float best = -INFINITY;
  int besti = 0x7fffffff;
  for (int s = threadIdx.x; s < segs; s += 64) better(best, besti, part_val[(int64_t)r * segs + s], part_idx[(int64_t)r * segs + s]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(besti, o, 64);
    better(best, besti, ov, oi);
  }
  if (threadIdx.x == 0) out[r] = besti == 0x7fffffff ? 0 : besti;
}

// ---- the same rule in a few passes over many workgroups -----------------------------------------
// One workgroup per row needs about a hundred passes over the row for top-k and top-p (two
// bisections) and walks the running sum 1024 entries at a time: 0.25 to 2.7 ms at a vocabulary of
// 152k, however few the rows. Here a row is cut into segments of 2048 entries, one workgroup each:
//   1. max:      the segment's largest z                          -> the row's maximum M
//   2. hist:     per segment the mass sum exp(z - M) of the entries that survive min_p; for rows with
//                top-k / top-p a histogram of (M - z) in bins of 1/64: count and mass (fixed point,
//                integer atomics: the sums do not depend on the order of arrival)
//   3. cut, extract: from the histogram, the bin that must hold the k-th largest entry, or the entry at
//                which the mass reaches p; every entry of that bin and of the bins above goes to a list
//   4. final:    one workgroup per row sorts the list (a few dozen to a few thousand entries), finds
//                both thresholds exactly as the definitions say, and draws among what is left in
//                vocabulary order; rows without top-k / top-p draw through the segment masses.
// A row whose list would not fit (a flat distribution with a wide nucleus), or whose list turns out
// too short for p, takes the one-workgroup path above inside step 4: slower, same rule.
struct SampleRow {
  float temperature;
  int32_t top_k;
  float top_p, min_p;
  uint64_t seed, offset;
};
static_assert(sizeof(SampleRow) == 32, "rows are packed by the caller");

constexpr int SEG = 2048;          // entries per segment
constexpr int SEG_THREADS = 256;
constexpr int NB = 2048;           // bins below the maximum
constexpr float BINS_PER_UNIT = 64.f;
constexpr int CAP = 4096;          // most entries of a row's list
constexpr float MASS_ONE = 1099511627776.f;  // 2^40: fixed-point unit of the histogram's mass

struct Plan {
  bool active, do_k, do_p;
  float inv_t, min_p, top_p;
  int top_k;
};
__device__ __forceinline__ Plan plan_of(const SampleRow& r, int vocab) {
  Plan p;
  p.active = r.temperature > 1e-5f;
  p.inv_t = p.active ? 1.f / r.temperature : 0.f;
  p.min_p = r.min_p;
  p.top_p = r.top_p;
  p.top_k = r.top_k;
  p.do_k = r.top_k > 0 && r.top_k < vocab;
  p.do_p = r.top_p < 1.f && r.top_p > 0.f;
  return p;
}
__device__ __forceinline__ bool survives(float z, float M, float min_p) {
  return z > -INFINITY && !(min_p > 0.f && expf(z - M) < min_p);
}
__device__ __forceinline__ int bin_of(float z, float M) {
  const float d = (M - z) * BINS_PER_UNIT;
  return d < (float)(NB - 1) ? (int)d : NB - 1;
}
// ascending keys = descending z, ties by ascending index
__device__ __forceinline__ uint32_t ordered_bits(float z) {
  const uint32_t b = __float_as_uint(z);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float from_ordered_bits(uint32_t o) {
  return __uint_as_float((o & 0x80000000u) ? (o & 0x7fffffffu) : ~o);
}
__device__ __forceinline__ uint64_t key_of(float z, int i) { return ((uint64_t)(~ordered_bits(z)) << 32) | (uint32_t)i; }
__device__ __forceinline__ float key_value(uint64_t k) { return from_ordered_bits(~(uint32_t)(k >> 32)); }

struct Scratch {
  float* seg_max;                  // [rows][segs]
  float* seg_mass;                 // [rows][segs]
  unsigned long long* hist_mass;   // [rows][NB]
  uint32_t* hist_count;            // [rows][NB]
  unsigned long long* cand;        // [rows][CAP]
  uint32_t* n_cand;                // [rows]
  uint32_t* generic;               // [rows]: 1 = the list would not fit
  int32_t* cut;                    // [rows]: the lowest bin on the list
};
inline size_t scratch_bytes(int64_t rows, int64_t segs) {
  return (size_t)rows * ((size_t)segs * 8 + (size_t)NB * 12 + (size_t)CAP * 8 + 12);
}
inline Scratch carve(void* base, int64_t rows, int64_t segs) {
  Scratch s;
  char* p = (char*)base;
  s.hist_mass = (unsigned long long*)p; p += (size_t)rows * NB * 8;
  s.cand = (unsigned long long*)p;      p += (size_t)rows * CAP * 8;
  s.hist_count = (uint32_t*)p;          p += (size_t)rows * NB * 4;
  s.seg_max = (float*)p;                p += (size_t)rows * segs * 4;
  s.seg_mass = (float*)p;               p += (size_t)rows * segs * 4;
  s.n_cand = (uint32_t*)p;              p += (size_t)rows * 4;
  s.generic = (uint32_t*)p;             p += (size_t)rows * 4;
  s.cut = (int32_t*)p;
  return s;
}

__device__ float row_max_of_segments(const float* seg_max, int segs, float* red) {
  float m = -INFINITY;
  for (int s = threadIdx.x; s < segs; s += blockDim.x) m = fmaxf(m, seg_max[s]);
  return block_max(m, red);
}

__global__ void __launch_bounds__(SEG_THREADS) sample_max_kernel(const float* __restrict__ logits, int64_t ld,
                                                                 const SampleRow* __restrict__ rows, Scratch sc,
                                                                 int vocab, int segs) {
  __shared__ float red[16];
  const int r = blockIdx.y, s = blockIdx.x;
  const Plan pl = plan_of(rows[r], vocab);
  if (!pl.active) return;
  if (pl.do_k || pl.do_p)
    for (int b = s * SEG_THREADS + threadIdx.x; b < NB; b += segs * SEG_THREADS) {
      sc.hist_count[(int64_t)r * NB + b] = 0u;
      sc.hist_mass[(int64_t)r * NB + b] = 0ull;
    }
  if (s == 0 && threadIdx.x == 0) {
    sc.n_cand[r] = 0u;
    sc.generic[r] = 0u;
  }
  const float* row = logits + (int64_t)r * ld;
  float m = -INFINITY;
  for (int i = s * SEG + threadIdx.x; i < min(vocab, (s + 1) * SEG); i += SEG_THREADS) m = fmaxf(m, row[i] * pl.inv_t);
  m = block_max(m, red);
  if (threadIdx.x == 0) sc.seg_max[(int64_t)r * segs + s] = m;
}

__global__ void __launch_bounds__(SEG_THREADS) sample_hist_kernel(const float* __restrict__ logits, int64_t ld,
                                                                  const SampleRow* __restrict__ rows, Scratch sc,
                                                                  int vocab, int segs) {
  __shared__ float red[16];
  __shared__ uint32_t count[NB];
  __shared__ unsigned long long mass[NB];
  const int r = blockIdx.y, s = blockIdx.x;
  const Plan pl = plan_of(rows[r], vocab);
  if (!pl.active) return;
  const bool filtered = pl.do_k || pl.do_p;
  const float M = row_max_of_segments(sc.seg_max + (int64_t)r * segs, segs, red);
  if (filtered) {
    for (int b = threadIdx.x; b < NB; b += SEG_THREADS) {
      count[b] = 0u;
      mass[b] = 0ull;
    }
    __syncthreads();
  }
  const float* row = logits + (int64_t)r * ld;
  float local = 0.f;
  for (int i = s * SEG + threadIdx.x; i < min(vocab, (s + 1) * SEG); i += SEG_THREADS) {
    const float z = row[i] * pl.inv_t;
    if (!survives(z, M, pl.min_p)) continue;
    const float e = expf(z - M);
    local += e;
    if (filtered) {
      const int b = bin_of(z, M);
      atomicAdd(&count[b], 1u);
      atomicAdd(&mass[b], (unsigned long long)(e * MASS_ONE));
    }
  }
  local = block_sum(local, red);
  if (threadIdx.x == 0) sc.seg_mass[(int64_t)r * segs + s] = local;
  if (filtered) {
    __syncthreads();
    for (int b = threadIdx.x; b < NB; b += SEG_THREADS)
      if (count[b]) {
        atomicAdd(&sc.hist_count[(int64_t)r * NB + b], count[b]);
        atomicAdd(&sc.hist_mass[(int64_t)r * NB + b], mass[b]);
      }
  }
}

// Step 3a, one workgroup per row: the lowest bin whose entries must be on the list, and how many entries
// that makes (more than CAP: the row takes the one-workgroup path).
__global__ void __launch_bounds__(SEG_THREADS) sample_cut_kernel(const SampleRow* __restrict__ rows, Scratch sc, int vocab) {
  constexpr int PER = NB / SEG_THREADS;  // consecutive bins per thread
  __shared__ uint32_t tc[SEG_THREADS];
  __shared__ unsigned long long tm[SEG_THREADS];
  __shared__ int cut_bin;
  const int r = blockIdx.x;
  const Plan pl = plan_of(rows[r], vocab);
  if (!pl.active || !(pl.do_k || pl.do_p)) return;
  // running count and mass from the top bin down
  uint32_t c[PER];
  unsigned long long m[PER];
  uint32_t csum = 0;
  unsigned long long msum = 0;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    c[e] = sc.hist_count[(int64_t)r * NB + threadIdx.x * PER + e];
    m[e] = sc.hist_mass[(int64_t)r * NB + threadIdx.x * PER + e];
    csum += c[e];
    msum += m[e];
  }
  tc[threadIdx.x] = csum;
  tm[threadIdx.x] = msum;
  if (threadIdx.x == 0) cut_bin = NB - 1;
  __syncthreads();
  uint32_t cbefore = 0, ctotal = 0;
  unsigned long long mbefore = 0, mtotal = 0;
  for (int t = 0; t < SEG_THREADS; ++t) {
    if (t == (int)threadIdx.x) {
      cbefore = ctotal;
      mbefore = mtotal;
    }
    ctotal += tc[t];
    mtotal += tm[t];
  }
  // the first bin at which the count reaches k, or else (top-p alone) the one after the bin at which
  // the mass reaches p of all of it: one bin of margin for the rounding of the sums in step 4
  const double want_mass = (double)pl.top_p * (double)mtotal;
  int found = NB;
  {
    uint32_t cc = cbefore;
    unsigned long long mm = mbefore;
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      cc += c[e];
      mm += m[e];
      const bool hit = pl.do_k ? cc >= (uint32_t)pl.top_k : (double)mm >= want_mass;
      if (hit && found == NB) found = threadIdx.x * PER + e;
    }
  }
  if (found < NB) atomicMin(&cut_bin, pl.do_k ? found : min(found + 1, NB - 1));
  __syncthreads();
  const int cut = cut_bin;
  uint32_t cc = cbefore;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    cc += c[e];
    if ((int)threadIdx.x * PER + e == cut) {
      sc.cut[r] = cut;
      sc.generic[r] = cc > (uint32_t)CAP ? 1u : 0u;
    }
  }
}

// Step 3b: every surviving entry of the bins down to the cut goes to the row's list.
__global__ void __launch_bounds__(SEG_THREADS) sample_extract_kernel(const float* __restrict__ logits, int64_t ld,
                                                                     const SampleRow* __restrict__ rows, Scratch sc,
                                                                     int vocab, int segs) {
  __shared__ float red[16];
  const int r = blockIdx.y, s = blockIdx.x;
  const Plan pl = plan_of(rows[r], vocab);
  if (!pl.active || !(pl.do_k || pl.do_p) || sc.generic[r]) return;
  const float M = row_max_of_segments(sc.seg_max + (int64_t)r * segs, segs, red);
  const int cut = sc.cut[r];
  const float* row = logits + (int64_t)r * ld;
  for (int i = s * SEG + threadIdx.x; i < min(vocab, (s + 1) * SEG); i += SEG_THREADS) {
    const float z = row[i] * pl.inv_t;
    if (!survives(z, M, pl.min_p) || bin_of(z, M) > cut) continue;
    const uint32_t slot = atomicAdd(&sc.n_cand[r], 1u);
    if (slot < (uint32_t)CAP) sc.cand[(int64_t)r * CAP + slot] = key_of(z, i);
  }
}

// Inclusive running sum over the workgroup's threads in thread order; every thread gets its own.
__device__ float block_scan(float v, float* wave_tot) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  float incl = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float up = __shfl_up(incl, o, 64);
    if (lane >= o) incl += up;
  }
  __syncthreads();
  if (lane == 63) wave_tot[w] = incl;
  __syncthreads();
  float before = 0.f;
  for (int k = 0; k < w; ++k) before += wave_tot[k];
  return before + incl;
}

// ascending bitonic sort of n_pow2 keys in LDS
__device__ void sort_keys(unsigned long long* keys, int n_pow2) {
  for (int k = 2; k <= n_pow2; k <<= 1)
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int t = threadIdx.x; t < n_pow2 / 2; t += BLOCK) {
        const int i = (t / j) * 2 * j + (t % j), l = i + j;
        const bool asc = (i & k) == 0;
        const unsigned long long a = keys[i], b = keys[l];
        if ((a > b) == asc) {
          keys[i] = b;
          keys[l] = a;
        }
      }
      __syncthreads();
    }
}

struct FinalShared {
  Red red;
  float fred[NWAVE];
  float wave_tot[NWAVE];
  DrawShared draw;
  int pick;
  int edge;
  float carry, before;
};

// The one-workgroup form of the whole chain for this row (its z goes to `z`).
__device__ int generic_row(const float* row, float* z, int vocab, const Plan& pl, uint64_t seed, uint64_t offset,
                           FinalShared& sh) {
  for (int i = threadIdx.x; i < vocab; i += BLOCK) z[i] = row[i] * pl.inv_t;
  __syncthreads();
  row_min_p(z, vocab, pl.min_p, sh.fred);
  row_topk_topp(z, vocab, pl.top_k, pl.top_p, sh.fred);
  return row_draw(z, vocab, seed, offset, sh.fred, sh.draw);
}

// Number of leading keys (sorted by descending value) whose value is >= t.
__device__ int count_at_least(const unsigned long long* keys, int n, float t, FinalShared& sh) {
  __syncthreads();
  if (threadIdx.x == 0) sh.edge = 0;
  __syncthreads();
  for (int j = threadIdx.x; j < n; j += BLOCK)
    if (key_value(keys[j]) >= t && (j + 1 == n || key_value(keys[j + 1]) < t)) sh.edge = j + 1;
  __syncthreads();
  return sh.edge;
}

__global__ void __launch_bounds__(BLOCK) sample_final_kernel(const float* __restrict__ logits, int64_t ld,
                                                             float* __restrict__ work,
                                                             const SampleRow* __restrict__ rows, Scratch sc,
                                                             int32_t* __restrict__ out, int vocab, int segs,
                                                             int force_generic) {
  __shared__ FinalShared sh;
  __shared__ unsigned long long keys[CAP];
  __shared__ float cum[CAP];
  const int r = blockIdx.x;
  const SampleRow sr = rows[r];
  const Plan pl = plan_of(sr, vocab);
  const float* row = logits + (int64_t)r * ld;
  if (!pl.active) {
    const int c = row_argmax(row, vocab, sh.red);
    if (threadIdx.x == 0) out[r] = c;
    return;
  }
  const bool filtered = pl.do_k || pl.do_p;
  if (force_generic || (filtered && sc.generic[r])) {
    const int c = generic_row(row, work + (int64_t)r * vocab, vocab, pl, sr.seed, sr.offset, sh);
    if (threadIdx.x == 0) out[r] = c;
    return;
  }
  const float M = row_max_of_segments(sc.seg_max + (int64_t)r * segs, segs, sh.fred);
  const float u = philox_uniform(sr.seed, sr.offset);
  const float* seg_mass = sc.seg_mass + (int64_t)r * segs;

  if (!filtered) {
    // the segment in which the running sum of the survivors' mass reaches u * total, then the entry in it
    float total = 0.f;
    for (int base = 0; base < segs; base += BLOCK) {
      const int s = base + threadIdx.x;
      const float c = total + block_scan(s < segs ? seg_mass[s] : 0.f, sh.wave_tot);
      __syncthreads();
      if (threadIdx.x == BLOCK - 1) sh.carry = c;
      __syncthreads();
      total = sh.carry;
    }
    // the first segment with survivors at which the running sum reaches the target
    const float target = u * total;
    if (threadIdx.x == 0) sh.pick = 0x7fffffff;
    __syncthreads();
    float before_all = 0.f;
    for (int base = 0; base < segs; base += BLOCK) {
      const int s = base + threadIdx.x;
      const float mine = s < segs ? seg_mass[s] : 0.f;
      const float c = before_all + block_scan(mine, sh.wave_tot);
      if (mine > 0.f && c >= target) atomicMin(&sh.pick, s);
      __syncthreads();
      if (threadIdx.x == BLOCK - 1) sh.carry = c;
      if (s == sh.pick) sh.before = c - mine;
      __syncthreads();
      before_all = sh.carry;
      if (sh.pick != 0x7fffffff) break;
    }
    const int seg = sh.pick;
    if (seg == 0x7fffffff) {  // no survivor at all: every logit is -inf (or the total is no number)
      if (threadIdx.x == 0) out[r] = 0;
      return;
    }
    const float local_target = target - sh.before;
    __syncthreads();
    if (threadIdx.x == 0) {
      sh.pick = 0x7fffffff;
      sh.edge = -1;
    }
    __syncthreads();
    float run = 0.f;
    for (int base = seg * SEG; base < min(vocab, (seg + 1) * SEG); base += BLOCK) {
      const int i = base + threadIdx.x;
      float e = 0.f;
      if (i < min(vocab, (seg + 1) * SEG)) {
        const float z = row[i] * pl.inv_t;
        if (survives(z, M, pl.min_p)) e = expf(z - M);
      }
      const float c = run + block_scan(e, sh.wave_tot);
      if (e > 0.f) {
        atomicMax(&sh.edge, i);  // the last survivor, should rounding leave the target above the segment's sum
        if (c >= local_target) atomicMin(&sh.pick, i);
      }
      __syncthreads();
      if (threadIdx.x == BLOCK - 1) sh.carry = c;
      __syncthreads();
      run = sh.carry;
    }
    if (threadIdx.x == 0) out[r] = sh.pick != 0x7fffffff ? sh.pick : (sh.edge >= 0 ? sh.edge : 0);
    return;
  }

  // the list, sorted by descending value
  const int n = (int)min(sc.n_cand[r], (uint32_t)CAP);
  int n2 = 64;
  while (n2 < n) n2 <<= 1;
  for (int j = threadIdx.x; j < n2; j += BLOCK) keys[j] = j < n ? sc.cand[(int64_t)r * CAP + j] : ~0ull;
  __syncthreads();
  sort_keys(keys, n2);
  int kept = n;
  if (pl.do_k && n > pl.top_k) kept = count_at_least(keys, n, key_value(keys[pl.top_k - 1]), sh);
  if (pl.do_p) {
    // running mass in sorted order; the denominator is the mass of what top-k left
    float run = 0.f;
    for (int base = 0; base < kept; base += BLOCK) {
      const int j = base + threadIdx.x;
      const float c = run + block_scan(j < kept ? expf(key_value(keys[j]) - M) : 0.f, sh.wave_tot);
      if (j < kept) cum[j] = c;
      __syncthreads();
      if (threadIdx.x == BLOCK - 1) sh.carry = c;
      __syncthreads();
      run = sh.carry;
    }
    float denom = run;
    if (!pl.do_k) {  // nothing was cut before: all survivors count, the list holds only the largest of them
      float t = 0.f;
      for (int s = threadIdx.x; s < segs; s += BLOCK) t += seg_mass[s];
      denom = block_sum(t, sh.fred);
    }
    if (threadIdx.x == 0) sh.pick = 0x7fffffff;
    __syncthreads();
    const float want = pl.top_p * denom;
    for (int j = threadIdx.x; j < kept; j += BLOCK)
      if (cum[j] >= want) atomicMin(&sh.pick, j);
    __syncthreads();
    const int cross = sh.pick;
    __syncthreads();
    if (cross == 0x7fffffff) {
      if (!pl.do_k) {  // the list is too short for p after all
        const int c = generic_row(row, work + (int64_t)r * vocab, vocab, pl, sr.seed, sr.offset, sh);
        if (threadIdx.x == 0) out[r] = c;
        return;
      }
    } else {
      kept = count_at_least(keys, kept, key_value(keys[cross]), sh);
    }
  }
  // what is left, in vocabulary order
  __syncthreads();
  int k2 = 64;
  while (k2 < kept) k2 <<= 1;
  for (int j = threadIdx.x; j < max(k2, n2); j += BLOCK) {
    const unsigned long long k = keys[j];
    const unsigned long long v = j < kept ? ((k & 0xffffffffull) << 32) | (uint32_t)__float_as_uint(key_value(k)) : ~0ull;
    if (j < k2) keys[j] = v;
  }
  __syncthreads();
  sort_keys(keys, k2);
  float run = 0.f;
  for (int base = 0; base < kept; base += BLOCK) {
    const int j = base + threadIdx.x;
    const float c = run + block_scan(j < kept ? expf(__uint_as_float((uint32_t)keys[j]) - M) : 0.f, sh.wave_tot);
    if (j < kept) cum[j] = c;
    __syncthreads();
    if (threadIdx.x == BLOCK - 1) sh.carry = c;
    __syncthreads();
    run = sh.carry;
  }
  const float target = u * run;
  if (threadIdx.x == 0) sh.pick = 0x7fffffff;
  __syncthreads();
  for (int j = threadIdx.x; j < kept; j += BLOCK)
    if (cum[j] >= target && expf(__uint_as_float((uint32_t)keys[j]) - M) > 0.f) atomicMin(&sh.pick, j);
  __syncthreads();
  if (threadIdx.x == 0) {
    const int j = sh.pick != 0x7fffffff ? sh.pick : kept - 1;
    out[r] = kept > 0 ? (int)(keys[j] >> 32) : 0;
  }
}


// ---- penalties from a history kept on the device ---------------------------------------------------
// history [slots, vocab] int32: bit 30 = the token occurs in the request's prompt, the low bits count
// its occurrences among the request's outputs. The host sends only what is new (a prompt once, then
// the token of each step), so a step costs no pass over the request's tokens on the host.
constexpr int32_t IN_PROMPT = 1 << 30;

struct PenaltyRow {
  int32_t slot;  // < 0: the row has no penalties
  float repetition, frequency, presence;
};
static_assert(sizeof(PenaltyRow) == 16, "rows are packed by the caller");

// entries [n][3] = (slot, token, kind): kind 0 marks a prompt token, kind 1 counts one more output
__global__ void __launch_bounds__(256) history_add_kernel(int32_t* __restrict__ history, int64_t vocab,
                                                          const int32_t* __restrict__ entries, int n, int slots) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= n) return;
  const int slot = entries[3 * e], tok = entries[3 * e + 1], kind = entries[3 * e + 2];
  if (slot < 0 || slot >= slots || tok < 0 || tok >= vocab) return;
  int32_t* cell = history + (int64_t)slot * vocab + tok;
  if (kind == 0) atomicOr(cell, IN_PROMPT);
  else atomicAdd(cell, 1);
}

__global__ void __launch_bounds__(256) penalties_dense_kernel(float* __restrict__ logits, int64_t ld,
                                                              const int32_t* __restrict__ history,
                                                              const PenaltyRow* __restrict__ rows, int vocab) {
  const PenaltyRow pr = rows[blockIdx.y];
  if (pr.slot < 0) return;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= vocab) return;
  const int32_t st = history[(int64_t)pr.slot * vocab + i];
  if (st == 0) return;
  float v = logits[(int64_t)blockIdx.y * ld + i];
  if (pr.repetition != 1.f) v = v > 0.f ? v / pr.repetition : v * pr.repetition;
  const int c = st & (IN_PROMPT - 1);
  if (c > 0) v -= pr.frequency * (float)c + pr.presence;
  logits[(int64_t)blockIdx.y * ld + i] = v;
}

// ---- what a request may add to its logits, and what it may ask about the token that was chosen -------
// entries [n][2] int32 = (row, token), vals [n]: logits[row][token] += val. A token occurs once a row.
__global__ void __launch_bounds__(256) logit_bias_kernel(float* __restrict__ logits, int64_t ld,
                                                         const int32_t* __restrict__ entries,
                                                         const float* __restrict__ vals, int n, int rows, int vocab) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= n) return;
  const int row = entries[2 * e], tok = entries[2 * e + 1];
  if (row < 0 || row >= rows || tok < 0 || tok >= vocab) return;
  logits[(int64_t)row * ld + tok] += vals[e];
}

constexpr int MAX_TOP = 32;

// (value, index) pairs in falling order of value, rising index among equals: is (v, i) behind (pv, pi)?
__device__ __forceinline__ bool behind(float v, int i, float pv, int pi) { return v < pv || (v == pv && i > pi); }

// A row cut into pieces that threads own in turn: where the row is 16-byte aligned the first vocab / 4 pieces are
// four entries each (one load), the rest (and every entry of an unaligned row) single entries. Piece p belongs to
// thread p % BLOCK.
struct Pieces {
  const float* row;
  int n4, total;  // pieces of four; all pieces
  __device__ Pieces(const float* r, int vocab) : row(r) {
    n4 = ((uintptr_t)r & 15) == 0 ? vocab >> 2 : 0;
    total = n4 + (vocab - 4 * n4);
  }
  __device__ int piece_of(int i) const { return i < 4 * n4 ? i >> 2 : n4 + (i - 4 * n4); }
  template <class F>
  __device__ void visit(int p, F&& f) const {  // f(value, index), indices rising
    if (p < n4) {
      const f32x4 v = ((const f32x4*)row)[p];
#pragma unroll
      for (int e = 0; e < 4; ++e) f(v[e], 4 * p + e);
    } else {
      const int i = 4 * n4 + (p - n4);
      f(row[i], i);
    }
  }
};

// One workgroup a row; k_of[row] < 0: nothing is asked about the row. log-softmax of the row as it is given:
// column 0 of out_ids / out_lp [rows][stride] takes the chosen token and its log-probability, columns 1..k the k
// most probable tokens in falling order (equal values: lower index first), rank[row] the number of tokens
// whose logit is larger than the chosen one's. One pass over the row gives every thread the best of its own
// entries, its count of entries larger than the chosen one and its share of the sum (kept relative to its own
// running maximum). The k best then come from a tournament: the workgroup picks among the 1024 names, and the
// wave of the thread whose entry won looks through that thread's entries for its next one, a piece a lane.
__global__ void __launch_bounds__(BLOCK) logprobs_kernel(const float* __restrict__ logits, int64_t ld,
                                                         const int32_t* __restrict__ chosen,
                                                         const int32_t* __restrict__ k_of, int stride,
                                                         int32_t* __restrict__ out_ids, float* __restrict__ out_lp,
                                                         int32_t* __restrict__ rank, int vocab) {
  __shared__ Red red;
  __shared__ float fred[NWAVE];
  const int b = blockIdx.x;
  const int k = k_of[b] < stride - 1 ? k_of[b] : stride - 1;
  if (k < 0) return;
  const Pieces pc(logits + (int64_t)b * ld, vocab);
  int c = chosen[b];
  c = c < 0 ? 0 : (c >= vocab ? vocab - 1 : c);
  const float cv = pc.row[c];
  float best = -INFINITY, sum = 0.f;  // (best is also the maximum that sum is relative to)
  int besti = 0x7fffffff, larger = 0;
  auto take = [&](f32x4 v, int p) {
    const float pm = fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3]));
    if (pm > best) sum = best == -INFINITY ? 0.f : sum * expf(best - pm);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      better(best, besti, v[e], 4 * p + e);
      larger += v[e] > cv;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) sum += expf(v[e] - best);
  };
  int p = threadIdx.x;
  for (; p + 3 * BLOCK < pc.n4; p += 4 * BLOCK) {  // four loads in flight
    const f32x4* r4 = (const f32x4*)pc.row;
    const f32x4 v0 = r4[p], v1 = r4[p + BLOCK], v2 = r4[p + 2 * BLOCK], v3 = r4[p + 3 * BLOCK];
    take(v0, p);
    take(v1, p + BLOCK);
    take(v2, p + 2 * BLOCK);
    take(v3, p + 3 * BLOCK);
  }
  for (; p < pc.total; p += BLOCK)
    pc.visit(p, [&](float v, int i) {
      if (v > best) sum = best == -INFINITY ? 0.f : sum * expf(best - v);
      better(best, besti, v, i);
      larger += v > cv;
      sum += expf(v - best);
    });
  const float own_top = best;
  float top = 0.f;
  int wi = block_argmax(best, besti, red, &top);
  sum = block_sum(own_top == -INFINITY ? 0.f : sum * expf(own_top - top), fred);
  const float lse = top + logf(sum);
  const float n_larger = block_sum((float)larger, fred);  // (a count below 2^24 is exact in a float)
  int32_t* ids = out_ids + (int64_t)b * stride;
  float* lps = out_lp + (int64_t)b * stride;
  if (threadIdx.x == 0) {
    ids[0] = c;
    lps[0] = cv - lse;
    rank[b] = (int)n_larger;
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float wv = top;
  for (int j = 0; j < k; ++j) {
    if (j > 0) wi = block_argmax(best, besti, red, &wv);
    const bool none = wi == 0x7fffffff;  // fewer tokens than k
    if (threadIdx.x == 0) {
      ids[1 + j] = none ? -1 : wi;
      lps[1 + j] = none ? -INFINITY : wv - lse;
    }
    if (none) continue;
    const int owner = pc.piece_of(wi) % BLOCK;
    if ((owner >> 6) != wave) continue;  // (the same for the whole wave)
    float nv = -INFINITY;
    int ni = 0x7fffffff;
    for (int q = owner + BLOCK * lane; q < pc.total; q += BLOCK * 64)
      pc.visit(q, [&](float v, int i) {
        if (behind(v, i, wv, wi)) better(nv, ni, v, i);
      });
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(nv, o, 64);
      const int oi = __shfl_xor(ni, o, 64);
      better(nv, ni, ov, oi);
    }
    if (lane == (owner & 63)) {
      best = nv;
      besti = ni;
    }
  }
}

}  // namespace

// Bytes of scratch with which dinfer_argmax spreads a row over many workgroups.
extern "C" int dinfer_argmax_scratch_bytes(int64_t rows, int64_t vocab, int64_t* bytes) {
  if (rows <= 0 || vocab <= 0 || !bytes) return ERR_BAD_SHAPE;
  *bytes = rows * ((vocab + ARG_SEG - 1) / ARG_SEG) * 8;
  return OK;
}

// out[r] = index of the largest entry of row r (the lowest such index). scratch (device memory, 4-byte aligned, may
// be null): with dinfer_argmax_scratch_bytes of it a long row is spread over many workgroups in two launches;
// without it, or for short rows, one workgroup takes a row.
extern "C" int dinfer_argmax(const float* logits, int64_t ld, int32_t* out, int64_t rows, int64_t vocab,
                             void* scratch, int64_t scratch_bytes, hipStream_t stream) {
  if (rows <= 0) return OK;
  if (vocab <= 0 || vocab > (1 << 24) || ld < vocab || rows > 0x7fffffff) return ERR_BAD_SHAPE;
  const int64_t segs = (vocab + ARG_SEG - 1) / ARG_SEG;
  if (scratch && segs >= 4 && rows <= 65535 && scratch_bytes >= rows * segs * 8 && ((uintptr_t)scratch & 3) == 0) {
    float* val = (float*)scratch;
    int32_t* idx = (int32_t*)(val + rows * segs);
    argmax_parts_kernel<<<dim3((unsigned)segs, (unsigned)rows), ARG_THREADS, 0, stream>>>(logits, ld, val, idx, (int)vocab,
                                                                                         (int)segs);
    argmax_join_kernel<<<(unsigned)rows, 64, 0, stream>>>(val, idx, out, (int)segs);
    return launch_status();
  }
  argmax_kernel<<<(unsigned)rows, BLOCK, 0, stream>>>(logits, ld, out, (int)vocab);
  return launch_status();
}

// temperature/top_k/top_p/min_p may be null (greedy / disabled). seeds and offsets
// are needed when any row has temperature > 1e-5.
extern "C" int dinfer_sample(const float* logits, int64_t ld, float* work, const float* temperature,
                             const int32_t* top_k, const float* top_p, const float* min_p, const uint64_t* seeds,
                             const uint64_t* offsets, int32_t* out, int64_t rows, int64_t vocab, hipStream_t stream) {
  if (rows <= 0) return OK;
  if (vocab <= 0 || vocab > (1 << 24) || ld < vocab || rows > 0x7fffffff) return ERR_BAD_SHAPE;
  if (temperature && (!work || !seeds || !offsets)) return ERR_BAD_SHAPE;
  sample_kernel<<<(unsigned)rows, BLOCK, 0, stream>>>(logits, ld, work, temperature, top_k, top_p, min_p, seeds,
                                                      offsets, out, (int)vocab);
  return launch_status();
}

// Bytes of scratch that dinfer_sample_rows needs for this many rows and this vocabulary.
extern "C" int dinfer_sample_scratch_bytes(int64_t rows, int64_t vocab, int64_t* bytes) {
  if (rows <= 0 || vocab <= 0 || !bytes) return ERR_BAD_SHAPE;
  *bytes = (int64_t)scratch_bytes(rows, (vocab + SEG - 1) / SEG);
  return OK;
}

// The same rule as dinfer_sample, rows packed as {float temperature; int32 top_k; float top_p; float min_p;
// uint64 seed; uint64 offset} (32 bytes each), in five launches that spread a row over many workgroups.
// work [rows, vocab] floats and scratch (dinfer_sample_scratch_bytes, 8-byte aligned) are device memory;
// what they hold before and after does not matter. any_filter = 0 promises that no row has top-k or top-p (two
// launches fewer); force_generic != 0: every row takes the one-workgroup path.
extern "C" int dinfer_sample_rows(const float* logits, int64_t ld, float* work, void* scratch, int64_t scratch_size,
                                  const void* rows_packed, int32_t* out, int64_t rows, int64_t vocab,
                                  int any_filter, int force_generic, hipStream_t stream) {
  if (rows <= 0) return OK;
  if (vocab <= 0 || vocab > (1 << 24) || ld < vocab || rows > 65535) return ERR_BAD_SHAPE;
  if (!work || !scratch || !rows_packed || ((uintptr_t)scratch & 7) || ((uintptr_t)rows_packed & 7)) return ERR_BAD_SHAPE;
  const int64_t segs = (vocab + SEG - 1) / SEG;
  if ((size_t)scratch_size < scratch_bytes(rows, segs)) return ERR_WORKSPACE;
  const Scratch sc = carve(scratch, rows, segs);
  const SampleRow* sr = (const SampleRow*)rows_packed;
  if (!force_generic) {
    const dim3 grid((unsigned)segs, (unsigned)rows);
    sample_max_kernel<<<grid, SEG_THREADS, 0, stream>>>(logits, ld, sr, sc, (int)vocab, (int)segs);
    sample_hist_kernel<<<grid, SEG_THREADS, 0, stream>>>(logits, ld, sr, sc, (int)vocab, (int)segs);
    if (any_filter) {
      sample_cut_kernel<<<(unsigned)rows, SEG_THREADS, 0, stream>>>(sr, sc, (int)vocab);
      sample_extract_kernel<<<grid, SEG_THREADS, 0, stream>>>(logits, ld, sr, sc, (int)vocab, (int)segs);
    }
  }
  sample_final_kernel<<<(unsigned)rows, BLOCK, 0, stream>>>(logits, ld, work, sr, sc, out, (int)vocab, (int)segs,
                                                            force_generic);
  return launch_status();
}


// history [slots, vocab] int32 (zero = a request without tokens yet); entries [n][3] int32 = (slot, token,
// kind 0: the token occurs in the prompt, kind 1: one more occurrence among the outputs).
extern "C" int dinfer_history_add(int32_t* history, int64_t slots, int64_t vocab, const int32_t* entries, int64_t n,
                                  hipStream_t stream) {
  if (n <= 0) return OK;
  if (!history || !entries || slots <= 0 || vocab <= 0 || n > 0x7fffffff || slots > 0x7fffffff) return ERR_BAD_SHAPE;
  history_add_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(history, vocab, entries, (int)n, (int)slots);
  return launch_status();
}

// In place on logits [rows, ld]: rows packed as {int32 slot; float repetition, frequency, presence} (slot < 0:
// untouched) take their penalties from history[slot]: a token seen in the prompt or among the outputs has a positive
// logit divided by `repetition` and a negative one multiplied by it; one seen c > 0 times among the outputs loses
// frequency * c + presence on top (crates/kernels/cuda/sampling.cu:318-349).
extern "C" int dinfer_penalties_dense(float* logits, int64_t ld, const int32_t* history, int64_t slots,
                                      const void* rows_packed, int64_t rows, int64_t vocab, hipStream_t stream) {
  if (rows <= 0) return OK;
  if (!history || !rows_packed || vocab <= 0 || ld < vocab || rows > 65535 || vocab > 0x7fffffff || slots <= 0)
    return ERR_BAD_SHAPE;
  const dim3 grid((unsigned)((vocab + 255) / 256), (unsigned)rows);
  penalties_dense_kernel<<<grid, 256, 0, stream>>>(logits, ld, history, (const PenaltyRow*)rows_packed, (int)vocab);
  return launch_status();
}


// logits[row][token] += val for n entries (row, token) [n][2] int32 with vals [n] float (a request's logit_bias,
// crates/kernels/cuda/sampling.cu:290-316 without the grammar mask). Tokens outside the vocabulary and rows
// outside [0, rows) are ignored; a (row, token) pair must not occur twice.
extern "C" int dinfer_logit_bias(float* logits, int64_t ld, const int32_t* entries, const float* vals, int64_t n,
                                 int64_t rows, int64_t vocab, hipStream_t stream) {
  if (n <= 0 || rows <= 0) return OK;
  if (!logits || !entries || !vals || vocab <= 0 || ld < vocab || n > 0x7fffffff || rows > 0x7fffffff ||
      vocab > 0x7fffffff)
    return ERR_BAD_SHAPE;
  logit_bias_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(logits, ld, entries, vals, (int)n, (int)rows,
                                                                     (int)vocab);
  return launch_status();
}

// Log-probabilities of the chosen tokens and of the k most probable ones per row (k_of[row], < 0: none asked,
// at most stride - 1 <= 32), from the log-softmax of logits as given (the caller passes the logits the model
// produced, before penalties and temperature): out_ids / out_lp [rows][stride], rank [rows]
// (crates/kernels/cuda/sampling.cu:380-430).
extern "C" int dinfer_logprobs(const float* logits, int64_t ld, const int32_t* chosen, const int32_t* k_of,
                               int64_t stride, int32_t* out_ids, float* out_lp, int32_t* rank, int64_t rows,
                               int64_t vocab, hipStream_t stream) {
  if (rows <= 0) return OK;
  if (!logits || !chosen || !k_of || !out_ids || !out_lp || !rank) return ERR_BAD_SHAPE;
  if (vocab <= 0 || vocab > (1 << 24) || ld < vocab || rows > 0x7fffffff) return ERR_BAD_SHAPE;
  if (stride < 1 || stride > MAX_TOP + 1) return ERR_UNSUPPORTED;
  logprobs_kernel<<<(unsigned)rows, BLOCK, 0, stream>>>(logits, ld, chosen, k_of, (int)stride, out_ids, out_lp, rank,
                                                        (int)vocab);
  return launch_status();
}
