// Token selection on float logits, one workgroup of 1024 threads per row:
// argmax, and the chain penalties -> temperature -> min_p -> top-k / top-p ->
// inverse-CDF draw with a counter-based random number, fused in one kernel.
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
// (draw), :266-283 (fused order), :318-349 (penalties), :352-364 (min_p).
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

__device__ int row_count_ge(const float* row, int vocab, float t, float* red) {
  float c = 0.f;
  for (int i = threadIdx.x; i < vocab; i += BLOCK) c += row[i] >= t ? 1.f : 0.f;
  return (int)block_sum(c, red);
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

// Keeps the k largest, then of those the smallest set of most probable tokens whose
// mass reaches p. Both thresholds are found by bisection on the value axis.
__device__ void row_topk_topp(float* row, int vocab, int k, float p, float* red) {
  const bool do_k = k > 0 && k < vocab;
  const bool do_p = p < 1.f && p > 0.f;
  if (!do_k && !do_p) return;
  const float m = row_max(row, vocab, red);
  float lo_local = INFINITY;
  for (int i = threadIdx.x; i < vocab; i += BLOCK) {
    const float v = row[i];
    if (v > -INFINITY) lo_local = fminf(lo_local, v);
  }
  const float lo = -block_max(-lo_local, red);
  float floor_ = -INFINITY;
  if (do_k) {
    float a = lo, b = m;  // invariant: count(v >= a) >= k
    for (int it = 0; it < 48 && b > a; ++it) {
      const float mid = 0.5f * (a + b);
      if (mid <= a || mid >= b) break;
      if (row_count_ge(row, vocab, mid, red) >= k) a = mid; else b = mid;
    }
    floor_ = row_count_ge(row, vocab, b, red) >= k ? b : a;
  }
  float thresh = floor_;
  if (do_p) {
    const float denom = row_expsum_ge(row, vocab, m, floor_, red);
    float a = fmaxf(lo, floor_), b = m;  // invariant: mass(v >= a) >= p
    for (int it = 0; it < 48 && b > a; ++it) {
      const float mid = 0.5f * (a + b);
      if (mid <= a || mid >= b) break;
      if (row_expsum_ge(row, vocab, m, fmaxf(mid, floor_), red) >= p * denom) a = mid; else b = mid;
    }
    if (row_expsum_ge(row, vocab, m, fmaxf(b, floor_), red) >= p * denom) a = b;
    thresh = fmaxf(thresh, a);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < vocab; i += BLOCK)
    if (row[i] < thresh) row[i] = -INFINITY;
  __syncthreads();
}

__device__ __forceinline__ uint32_t mulhilo(uint32_t a, uint32_t b, uint32_t* hi) {
  const uint64_t p = (uint64_t)a * b;
  *hi = (uint32_t)(p >> 32);
  return (uint32_t)p;
}

__device__ void philox4x32_10(uint32_t c[4], uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    uint32_t hi0, hi1;
    const uint32_t lo0 = mulhilo(0xD2511F53u, c[0], &hi0);
    const uint32_t lo1 = mulhilo(0xCD9E8D57u, c[2], &hi1);
    const uint32_t n0 = hi1 ^ c[1] ^ k0, n1 = lo1, n2 = hi0 ^ c[3] ^ k1, n3 = lo0;
    c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
}

__device__ float philox_uniform(uint64_t seed, uint64_t offset) {
  uint32_t c[4] = {(uint32_t)offset, (uint32_t)(offset >> 32), 0u, 0u};
  philox4x32_10(c, (uint32_t)seed, (uint32_t)(seed >> 32));
  return (float)(c[0] >> 8) * (1.f / 16777216.f);
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

// One entry per distinct token of a row's history: ids[e], count among the
// outputs cnt[e] (0 if it occurs in the prompt only). Row b owns the entries
// offsets[b] .. offsets[b+1].
__global__ void __launch_bounds__(256) penalties_kernel(float* __restrict__ logits, int64_t ld,
                                                        const int32_t* __restrict__ ids,
                                                        const int32_t* __restrict__ cnt,
                                                        const int32_t* __restrict__ offsets,
                                                        const float* __restrict__ rep, const float* __restrict__ freq,
                                                        const float* __restrict__ pres, int vocab) {
  const int b = blockIdx.x;
  const float r = rep[b], f = freq[b], pr = pres[b];
  if (r == 1.f && f == 0.f && pr == 0.f) return;
  float* row = logits + (int64_t)b * ld;
  for (int e = offsets[b] + threadIdx.x; e < offsets[b + 1]; e += blockDim.x) {
    const int t = ids[e];
    if (t < 0 || t >= vocab) continue;
    float v = row[t];
    if (r != 1.f) v = v > 0.f ? v / r : v * r;
    const int c = cnt[e];
    if (c > 0) v -= f * (float)c + pr;
    row[t] = v;
  }
}

}  // namespace

extern "C" int dinfer_argmax(const float* logits, int64_t ld, int32_t* out, int64_t rows, int64_t vocab,
                             hipStream_t stream) {
  if (rows <= 0) return OK;
  if (vocab <= 0 || vocab > (1 << 24) || ld < vocab || rows > 0x7fffffff) return ERR_BAD_SHAPE;
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

extern "C" int dinfer_penalties(float* logits, int64_t ld, const int32_t* ids, const int32_t* counts,
                                const int32_t* offsets, const float* repetition, const float* frequency,
                                const float* presence, int64_t rows, int64_t vocab, hipStream_t stream) {
  if (rows <= 0) return OK;
  if (vocab <= 0 || ld < vocab || rows > 0x7fffffff) return ERR_BAD_SHAPE;
  penalties_kernel<<<(unsigned)rows, 256, 0, stream>>>(logits, ld, ids, counts, offsets, repetition, frequency,
                                                       presence, (int)vocab);
  return launch_status();
}
