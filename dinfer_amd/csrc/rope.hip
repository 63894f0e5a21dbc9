// Per-head q/k RMSNorm, rotary position encoding and the K/V cache write in
// one pass over a step's fused projection output.
//
//   qkv [T, ld]:  q heads at column q_off (H x D), k heads at k_off (Hkv x D),
//                 v heads at v_off (Hkv x D).
//   q, k:  y = x * rsqrt(mean(x^2) + eps) * (w + w_offset)   (skipped when the
//          gain pointer is null), then rotation of the first `rot` dims by the
//          angles of the token's position, all in float, one rounding.
//          q is written back in place; k goes to the cache only.
//   v:     copied to the cache unchanged.
//
// Cache pages (chosen for MFMA operand loads on gfx950: both operands of
// Q.K^T and P.V want 8 consecutive elements of the contraction dimension):
//   K page  [Hkv][page][D]   a key's head is one contiguous row of D
//   V page  [Hkv][D][page]   transposed: for one d, the page's keys are contiguous
// A token's slot is block * page + offset; a negative slot writes nothing.
//
// The table row of position p is [cos(p f_0..f_{rot/2-1}) | sin(...)], float.
// style 0 pairs (i, i + rot/2) ("neox"), style 1 pairs (2i, 2i+1).
//
// Reference behaviour: crates/kernels/cuda/qkv_post.cu:26-91 (order norm ->
// rotation -> one rounding; v untouched; k written after norm and rotation),
// crates/layers/src/nn.rs:152-185 (table layout).
#include "common.cuh"

using namespace dinfer;

namespace {

constexpr int MAX_D = 512;
constexpr int WAVES = 4;

template <class S>
__global__ void __launch_bounds__(WAVES * 64) qkv_post_kernel(
    S* __restrict__ qkv, int64_t ld, int64_t q_off, int64_t k_off, int64_t v_off, const void* __restrict__ wq,
    const void* __restrict__ wk, int wf32, float eps, float w_offset, const int32_t* __restrict__ pos,
    const float* __restrict__ cos_sin, int rot, int style, S* __restrict__ k_cache, S* __restrict__ v_cache,
    const int64_t* __restrict__ slots, int H, int Hkv, int D, int page) {
  __shared__ float xs[WAVES][MAX_D];
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int item = blockIdx.y * WAVES + wave;
  const bool live = item < H + 2 * Hkv;
  const bool is_v = live && item >= H + Hkv;
  const bool is_qk = live && !is_v;
  const bool is_q = live && item < H;
  S* row = qkv + t * ld;
  const int64_t slot = slots ? slots[t] : -1;
  const int64_t blk = slot >= 0 ? slot / page : 0;
  const int off = slot >= 0 ? (int)(slot % page) : 0;

  if (is_v && slot >= 0) {  // a v head: cache copy only
    const int hk = item - H - Hkv;
    const S* vs = row + v_off + (int64_t)hk * D;
    S* vd = v_cache + ((blk * Hkv + hk) * (int64_t)D) * page + off;
    for (int d = lane; d < D; d += 64) vd[(int64_t)d * page] = vs[d];
  }

  const int hk = item - H;
  S* base = is_q ? row + q_off + (int64_t)item * D : row + k_off + (int64_t)hk * D;
  const void* w = is_q ? wq : wk;
  float* x = xs[wave];

  if (is_qk) {
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) {
      const float v = to_f32(base[d]);
      x[d] = v;
      ss += v * v;
    }
    if (w) {
      ss = wave_sum(ss);
      const float inv = 1.f / sqrtf(ss / (float)D + eps);
      // each lane rescales only the entries it wrote itself
      for (int d = lane; d < D; d += 64) x[d] = x[d] * inv * (ld_param<S>(w, d, wf32) + w_offset);
    }
  }
  __syncthreads();  // the rotation reads partners that other lanes wrote
  if (!is_qk) return;

  S* kd = (!is_q && slot >= 0) ? k_cache + ((blk * Hkv + hk) * (int64_t)page + off) * D : nullptr;
  const float* cs = cos_sin ? cos_sin + (int64_t)pos[t] * rot : nullptr;
  const int half = rot / 2;
  for (int d = lane; d < D; d += 64) {
    float y = x[d];
    if (cs && d < rot) {
      int i;         // index of the frequency
      float other;   // the partner in the pair
      bool first;    // whether d is the first element of its pair
      if (style == 0) {
        first = d < half;
        i = first ? d : d - half;
        other = x[first ? d + half : d - half];
      } else {
        first = (d & 1) == 0;
        i = d >> 1;
        other = x[d ^ 1];
      }
      const float c = cs[i], s = cs[half + i];
      y = first ? y * c - other * s : y * c + other * s;
    }
    const S r = from_f32<S>(y);
    if (is_q) base[d] = r;
    if (kd) kd[d] = r;
  }
}

// The common case (pairs (i, i + D/2), the whole head rotated): both elements of a pair live in one
// lane, so there is no exchange through LDS and no barrier, and every load of a head (values, gains,
// angles) is issued before the first use. NP pairs per lane cover D <= 128 * NP.
template <class S, int NP>
__global__ void __launch_bounds__(WAVES * 64) qkv_post_neox_kernel(
    S* __restrict__ qkv, int64_t ld, int64_t q_off, int64_t k_off, int64_t v_off, const void* __restrict__ wq,
    const void* __restrict__ wk, int wf32, float eps, float w_offset, const int32_t* __restrict__ pos,
    const float* __restrict__ cos_sin, S* __restrict__ k_cache, S* __restrict__ v_cache,
    const int64_t* __restrict__ slots, int H, int Hkv, int D, int page) {
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int item = blockIdx.y * WAVES + wave;
  if (item >= H + 2 * Hkv) return;
  S* row = qkv + t * ld;
  const int64_t slot = slots ? slots[t] : -1;
  const int64_t blk = slot >= 0 ? slot / page : 0;
  const int off = slot >= 0 ? (int)(slot % page) : 0;
  if (item >= H + Hkv) {
    if (slot < 0) return;
    const int hk = item - H - Hkv;
    const S* vs = row + v_off + (int64_t)hk * D;
    S* vd = v_cache + ((blk * Hkv + hk) * (int64_t)D) * page + off;
    for (int d = lane; d < D; d += 64) vd[(int64_t)d * page] = vs[d];
    return;
  }
  const bool is_q = item < H;
  const int hk = item - H;
  S* base = is_q ? row + q_off + (int64_t)item * D : row + k_off + (int64_t)hk * D;
  const void* w = is_q ? wq : wk;
  const int half = D / 2;
  const float* cs = cos_sin ? cos_sin + (int64_t)pos[t] * D : nullptr;
  float x1[NP], x2[NP], g1[NP], g2[NP], c[NP], sn[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int i = lane + 64 * p;
    const bool ok = i < half;
    x1[p] = ok ? to_f32(base[i]) : 0.f;
    x2[p] = ok ? to_f32(base[i + half]) : 0.f;
    g1[p] = (ok && w) ? ld_param<S>(w, i, wf32) + w_offset : 1.f;
    g2[p] = (ok && w) ? ld_param<S>(w, i + half, wf32) + w_offset : 1.f;
    c[p] = (ok && cs) ? cs[i] : 1.f;
    sn[p] = (ok && cs) ? cs[half + i] : 0.f;
  }
  float inv = 1.f;
  if (w) {
    float ss = 0.f;
#pragma unroll
    for (int p = 0; p < NP; ++p) ss += x1[p] * x1[p] + x2[p] * x2[p];
    ss = wave_sum(ss);
    inv = 1.f / sqrtf(ss / (float)D + eps);
  }
  S* kd = (!is_q && slot >= 0) ? k_cache + ((blk * Hkv + hk) * (int64_t)page + off) * D : nullptr;
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int i = lane + 64 * p;
    if (i < half) {
      const float y1 = w ? x1[p] * inv * g1[p] : x1[p], y2 = w ? x2[p] * inv * g2[p] : x2[p];
      const S r1 = from_f32<S>(y1 * c[p] - y2 * sn[p]), r2 = from_f32<S>(y2 * c[p] + y1 * sn[p]);
      if (is_q) {
        base[i] = r1;
        base[i + half] = r2;
      }
      if (kd) {
        kd[i] = r1;
        kd[i + half] = r2;
      }
    }
  }
}

}  // namespace

extern "C" int dinfer_qkv_post(int dtype, void* qkv, int64_t tokens, int64_t ld, int64_t q_off, int64_t k_off,
                               int64_t v_off, const void* q_gain, const void* k_gain, int w_f32, float eps,
                               float w_offset, const int32_t* positions, const float* cos_sin, int rotary_dim,
                               int style, void* k_cache, void* v_cache, const int64_t* slot_mapping, int heads,
                               int kv_heads, int head_dim, int page_size, hipStream_t stream) {
  if (tokens <= 0) return OK;
  if (heads <= 0 || kv_heads <= 0 || head_dim <= 0 || page_size <= 0 || tokens > 0x7fffffff) return ERR_BAD_SHAPE;
  if (head_dim > MAX_D) return ERR_UNSUPPORTED;
  if (cos_sin && (rotary_dim <= 0 || rotary_dim > head_dim || rotary_dim % 2 != 0)) return ERR_BAD_SHAPE;
  if (style != 0 && style != 1) return ERR_UNSUPPORTED;
  if ((q_gain == nullptr) != (k_gain == nullptr)) return ERR_BAD_SHAPE;
  const int items = heads + 2 * kv_heads;
  const dim3 grid((unsigned)tokens, (unsigned)((items + WAVES - 1) / WAVES));
  const bool whole_head_neox = style == 0 && head_dim % 2 == 0 && (!cos_sin || rotary_dim == head_dim);
  if (whole_head_neox) {
    DINFER_DISPATCH_DTYPE(dtype, {
      if (head_dim <= 128)
        qkv_post_neox_kernel<S, 1><<<grid, WAVES * 64, 0, stream>>>(
            (S*)qkv, ld, q_off, k_off, v_off, q_gain, k_gain, w_f32, eps, w_offset, positions, cos_sin, (S*)k_cache,
            (S*)v_cache, slot_mapping, heads, kv_heads, head_dim, page_size);
      else if (head_dim <= 256)
        qkv_post_neox_kernel<S, 2><<<grid, WAVES * 64, 0, stream>>>(
            (S*)qkv, ld, q_off, k_off, v_off, q_gain, k_gain, w_f32, eps, w_offset, positions, cos_sin, (S*)k_cache,
            (S*)v_cache, slot_mapping, heads, kv_heads, head_dim, page_size);
      else
        qkv_post_neox_kernel<S, 4><<<grid, WAVES * 64, 0, stream>>>(
            (S*)qkv, ld, q_off, k_off, v_off, q_gain, k_gain, w_f32, eps, w_offset, positions, cos_sin, (S*)k_cache,
            (S*)v_cache, slot_mapping, heads, kv_heads, head_dim, page_size);
    });
    return launch_status();
  }
  DINFER_DISPATCH_DTYPE(dtype, {
    qkv_post_kernel<S><<<grid, WAVES * 64, 0, stream>>>((S*)qkv, ld, q_off, k_off, v_off, q_gain, k_gain, w_f32, eps,
                                                        w_offset, positions, cos_sin, rotary_dim, style, (S*)k_cache,
                                                        (S*)v_cache, slot_mapping, heads, kv_heads, head_dim,
                                                        page_size);
  });
  return launch_status();
}
