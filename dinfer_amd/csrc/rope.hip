// Per-head q/k RMSNorm, rotary position encoding and the K/V cache write in
// one pass over a step's fused projection output.
//
//   qkv [T, ld]:  q heads at column q_off (H x D), k heads at k_off (Hkv x D),
//                 v heads at v_off (Hkv x D).
//   q, k:  y = x * rsqrt(mean(x^2) + eps) * (w + w_offset)   (skipped when the
//          gain pointer is null), then rotation of the first `rot` dims by the
//          angles of the token's position, all in float, one rounding.
//          q is written back in place; k goes to the cache only, or, where no
//          slot mapping is given (nothing is cached), back in place like q.
//   v:     copied to the cache unchanged.
//
// Cache pages (chosen for MFMA operand loads on gfx950: both operands of
// Q.K^T and P.V want 8 consecutive elements of the contraction dimension):
//   K page  [Hkv][D / 8][page][8]   the 8-element pieces of consecutive keys are contiguous
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

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
  return z;
}

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

  S* kd = (!is_q && slot >= 0) ? k_cache + (blk * Hkv + hk) * (int64_t)page * D : nullptr;  // the head's page
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
    if (is_q || !slots) base[d] = r;  // without a slot mapping nothing goes to the cache and k is written back like q
    if (kd) kd[k_page_offset((int)off, d, page)] = r;
  }
}

// The common case (pairs (i, i + D/2), the whole head rotated): both elements of a pair live in one
// lane, so there is no exchange through LDS and no barrier. A wave takes IPW heads of one token and
// issues every load of all of them (values, gains, angles) before the first use; fewer, fatter waves
// also keep the kernel off the wave-launch limit. NP pairs per lane cover D <= 128 * NP.
constexpr int IPW = 4;  // head items per wave

template <class S, int NP>
__global__ void __launch_bounds__(WAVES * 64) qkv_post_neox_kernel(
    S* __restrict__ qkv, int64_t ld, int64_t q_off, int64_t k_off, int64_t v_off, const void* __restrict__ wq,
    const void* __restrict__ wk, int wf32, float eps, float w_offset, const int32_t* __restrict__ pos,
    const float* __restrict__ cos_sin, S* __restrict__ k_cache, S* __restrict__ v_cache,
    const int64_t* __restrict__ slots, int H, int Hkv, int D, int page) {
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int item0 = (blockIdx.y * WAVES + wave) * IPW;
  const int items = H + 2 * Hkv;
  if (item0 >= items) return;
  S* row = qkv + t * ld;
  const int64_t slot = slots ? slots[t] : -1;
  const int64_t blk = slot >= 0 ? slot / page : 0;
  const int off = slot >= 0 ? (int)(slot % page) : 0;
  const int half = D / 2;
  const float* cs = cos_sin ? cos_sin + (int64_t)pos[t] * D : nullptr;

  float x1[IPW][NP], x2[IPW][NP];
  float g1q[NP], g2q[NP], g1k[NP], g2k[NP], c[NP], sn[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int i = lane + 64 * p;
    const bool ok = i < half;
    g1q[p] = (ok && wq) ? ld_param<S>(wq, i, wf32) + w_offset : 1.f;
    g2q[p] = (ok && wq) ? ld_param<S>(wq, i + half, wf32) + w_offset : 1.f;
    g1k[p] = (ok && wk) ? ld_param<S>(wk, i, wf32) + w_offset : 1.f;
    g2k[p] = (ok && wk) ? ld_param<S>(wk, i + half, wf32) + w_offset : 1.f;
    c[p] = (ok && cs) ? cs[i] : 1.f;
    sn[p] = (ok && cs) ? cs[half + i] : 0.f;
  }
#pragma unroll
  for (int u = 0; u < IPW; ++u) {
    const int item = item0 + u;
    // q heads, then k heads, then v heads lie one after the other in the row when the offsets say so;
    // in general each kind has its own offset
    const S* src = item < H ? row + q_off + (int64_t)item * D
                 : item < H + Hkv ? row + k_off + (int64_t)(item - H) * D
                                  : row + v_off + (int64_t)(item - H - Hkv) * D;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int i = lane + 64 * p;
      const bool ok = i < half && item < items;
      x1[u][p] = ok ? to_f32(src[i]) : 0.f;
      x2[u][p] = ok ? to_f32(src[i + half]) : 0.f;
    }
  }
#pragma unroll
  for (int u = 0; u < IPW; ++u) {
    const int item = item0 + u;
    if (item >= items) break;
    if (item >= H + Hkv) {  // a v head: cache copy only
      if (slot < 0) continue;
      const int hk = item - H - Hkv;
      S* vd = v_cache + ((blk * Hkv + hk) * (int64_t)D) * page + off;
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        const int i = lane + 64 * p;
        if (i < half) {
          vd[(int64_t)i * page] = from_f32<S>(x1[u][p]);  // the value came from S: the round trip is exact
          vd[(int64_t)(i + half) * page] = from_f32<S>(x2[u][p]);
        }
      }
      continue;
    }
    const bool is_q = item < H;
    const bool normed = is_q ? wq != nullptr : wk != nullptr;
    float inv = 1.f;
    if (normed) {
      float ss = 0.f;
#pragma unroll
      for (int p = 0; p < NP; ++p) ss += x1[u][p] * x1[u][p] + x2[u][p] * x2[u][p];
      ss = wave_sum(ss);
      inv = 1.f / sqrtf(ss / (float)D + eps);
    }
    const int hk = item - H;
    S* base = is_q ? row + q_off + (int64_t)item * D : slots ? nullptr : row + k_off + (int64_t)hk * D;
    S* kd = (!is_q && slot >= 0) ? k_cache + (blk * Hkv + hk) * (int64_t)page * D : nullptr;  // the head's page
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int i = lane + 64 * p;
      if (i < half) {
        const float y1 = normed ? x1[u][p] * inv * (is_q ? g1q[p] : g1k[p]) : x1[u][p];
        const float y2 = normed ? x2[u][p] * inv * (is_q ? g2q[p] : g2k[p]) : x2[u][p];
        const S r1 = from_f32<S>(y1 * c[p] - y2 * sn[p]), r2 = from_f32<S>(y2 * c[p] + y1 * sn[p]);
        if (base) {
          base[i] = r1;
          base[i + half] = r2;
        }
        if (kd) {
          kd[k_page_offset((int)off, i, page)] = r1;
          kd[k_page_offset((int)off, i + half, page)] = r2;
        }
      }
    }
  }
}

// V into its transposed pages for many tokens: one wave takes 8 consecutive tokens of one kv head.
// When their slots are 8 consecutive slots starting at a multiple of 8 (a prompt portion that starts
// on such a boundary), a lane gathers two dims of the 8 tokens and stores them as two 16-byte rows
// of V^T; otherwise it falls back to one 2-byte store per element.
// (group: which run of 8 * WAVES tokens the workgroup takes.)
__device__ __forceinline__ void v_write_transposed(const bf16* __restrict__ qkv, int64_t ld, int64_t v_off,
                                                   bf16* __restrict__ v_cache, const int64_t* __restrict__ slots, int T,
                                                   int Hkv, int D, int page, int group, int hk) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t0 = (group * WAVES + wave) * 8;
  if (t0 >= T) return;
  const int n = T - t0 < 8 ? T - t0 : 8;
  const int64_t s0 = slots[t0];
  bool aligned = n == 8 && s0 >= 0 && (s0 & 7) == 0;
  for (int j = 1; j < n && aligned; ++j) aligned = slots[t0 + j] == s0 + j;
  const bf16* src = qkv + (int64_t)t0 * ld + v_off + (int64_t)hk * D;
  for (int d2 = lane; d2 < D / 2; d2 += 64) {
    bf16x2 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (j < n) v[j] = *(const bf16x2*)(src + (int64_t)j * ld + 2 * d2);
    if (aligned) {
      const int64_t blk = s0 / page;
      const int off = (int)(s0 % page);
      bf16* vd = v_cache + ((blk * Hkv + hk) * (int64_t)D + 2 * d2) * page + off;
      bf16x8 a, b;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        a[j] = v[j][0];
        b[j] = v[j][1];
      }
      *(bf16x8*)vd = a;
      *(bf16x8*)(vd + page) = b;
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (j >= n) break;
        const int64_t sl = slots[t0 + j];
        if (sl < 0) continue;
        bf16* vd = v_cache + (((sl / page) * Hkv + hk) * (int64_t)D + 2 * d2) * page + sl % page;
        vd[0] = v[j][0];
        vd[page] = v[j][1];
      }
    }
  }
}

// bf16, whole-head neox rotation, D in {64, 128, 256}: LPH = D / 8 lanes share a head, each with 8
// consecutive dims in one 16-byte load; the partner of a pair sits LPH / 2 lanes away and comes by a
// cross-lane read. A wave covers 64 / LPH heads of one token per instruction, an order of magnitude
// fewer memory instructions than 2-byte accesses.
// gather_v > 0: V is not written by the heads' lanes; the workgroups from blockIdx.x = `tokens` on (gather_v of them,
// one per kv head and run of 8 * WAVES tokens) gather it into its transposed pages, in the same launch (a kernel of
// its own for that cost a prefill layer 5.7 us, a step of prompt portions beside decoding requests 7.8).
template <int LPH>
__global__ void __launch_bounds__(WAVES * 64) qkv_post_vec_kernel(
    bf16* __restrict__ qkv, int64_t ld, int64_t q_off, int64_t k_off, int64_t v_off, const void* __restrict__ wq,
    const void* __restrict__ wk, int wf32, float eps, float w_offset, const int32_t* __restrict__ pos,
    const float* __restrict__ cos_sin, bf16* __restrict__ k_cache, bf16* __restrict__ v_cache,
    const int64_t* __restrict__ slots, int H, int Hkv, int page, int tokens, int gather_v) {
  constexpr int D = LPH * 8, HALF = D / 2, HPW = 64 / LPH;  // heads per wave
  if ((int)blockIdx.x >= tokens) {
    const int j = (int)blockIdx.x - tokens;
    if (blockIdx.y == 0) v_write_transposed(qkv, ld, v_off, v_cache, slots, tokens, Hkv, D, page, j / Hkv, j % Hkv);
    return;
  }
  const bool skip_v = gather_v > 0;
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int sub = lane / LPH, l = lane % LPH;  // which head of the wave, which 8 dims of it
  const int items = H + 2 * Hkv;
  // The workgroups of a token (gridDim.y of them) take its heads in rounds of gridDim.y * WAVES * HPW; a lane keeps
  // its 8 dims from round to round, so the angles of those dims are fetched once (with one workgroup a token, which
  // is how many tokens are launched, a lane serves three heads of the 8B sizes with one fetch: the angles are four
  // times the bytes of the head's own 8 values).
  const int per_round = gridDim.y * WAVES * HPW;
  const int first_item = (blockIdx.y * WAVES + wave) * HPW + sub;
  bf16* row = qkv + t * ld;
  const int64_t slot = slots ? slots[t] : -1;
  const int64_t blk = slot >= 0 ? slot / page : 0;
  const int off = slot >= 0 ? (int)(slot % page) : 0;
  const int d0 = 8 * l;
  auto source = [&](int item) {
    return item < H ? row + q_off + (int64_t)item * D
                    : item < H + Hkv ? row + k_off + (int64_t)(item - H) * D : row + v_off + (int64_t)(item - H - Hkv) * D;
  };
  // angles of this lane's dims: the pair index of dim d is d mod D/2
  float c[8], sn[8];
  const int pi = d0 % HALF;
  if (cos_sin) {
    const float* cs = cos_sin + (int64_t)pos[t] * D;
    const f32x4 c0 = *(const f32x4*)(cs + pi), c1 = *(const f32x4*)(cs + pi + 4);
    const f32x4 s0 = *(const f32x4*)(cs + HALF + pi), s1 = *(const f32x4*)(cs + HALF + pi + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) { c[e] = c0[e]; c[4 + e] = c1[e]; sn[e] = s0[e]; sn[4 + e] = s1[e]; }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) { c[e] = 1.f; sn[e] = 0.f; }
  }
  // (a wave's lanes leave the loop together: the cross-lane steps below need all of them)
  const int wave_first = (blockIdx.y * WAVES + wave) * HPW;
  bf16x8 xv = zero8();
  if (first_item < items) xv = *(const bf16x8*)(source(first_item) + d0);
  for (int base = 0; wave_first + base < items; base += per_round) {
    const int item = first_item + base;
    const bool live = item < items;
    const bool is_v = live && item >= H + Hkv, is_q = live && item < H, is_k = live && !is_q && !is_v;
    bf16* src = live ? source(item) : row;
    const bf16x8 xc = xv;
    // the next round's values are on their way while this round is computed
    xv = zero8();
    if (item + per_round < items) xv = *(const bf16x8*)(source(item + per_round) + d0);
    if (is_v) {
      if (slot >= 0 && !skip_v) {
        bf16* vd = v_cache + ((blk * Hkv + (item - H - Hkv)) * (int64_t)D + d0) * page + off;
#pragma unroll
        for (int e = 0; e < 8; ++e) vd[(int64_t)e * page] = xc[e];
      }
    }
    const bool qk = is_q || is_k;
    const void* w = is_q ? wq : wk;
    float g[8];
    if (qk && w) {
      if (wf32) {
        const f32x4 a = *(const f32x4*)((const float*)w + d0), b = *(const f32x4*)((const float*)w + d0 + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) { g[e] = a[e] + w_offset; g[4 + e] = b[e] + w_offset; }
      } else {
        const bf16x8 gv = *(const bf16x8*)((const bf16*)w + d0);
#pragma unroll
        for (int e = 0; e < 8; ++e) g[e] = (float)gv[e] + w_offset;
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] = 1.f;
    }
    float x[8], ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      x[e] = (float)xc[e];
      ss = add_square(ss, x[e]);
    }
    // every lane takes part in the cross-lane steps, whatever its head is
#pragma unroll
    for (int o = LPH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    const float inv = (qk && w) ? 1.f / sqrtf(ss / (float)D + eps) : 1.f;
    float y[8], other[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = (qk && w) ? x[e] * inv * g[e] : x[e];
#pragma unroll
    for (int e = 0; e < 8; ++e) other[e] = __shfl_xor(y[e], LPH / 2, 64);
    if (!qk) continue;
    const bool first = l < LPH / 2;  // this lane holds the first elements of its pairs
    bf16x8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e)
      r[e] = (bf16)(first ? rotated_first(y[e], other[e], c[e], sn[e]) : rotated_second(other[e], y[e], c[e], sn[e]));
    if (is_q || !slots) {
      *(bf16x8*)(src + d0) = r;
    } else if (slot >= 0) {
      *(bf16x8*)(k_cache + (blk * Hkv + (item - H)) * (int64_t)page * D + k_page_offset((int)off, d0, page)) = r;
    }
  }
}

}  // namespace

extern "C" int dinfer_qkv_post(int dtype, void* qkv, int64_t tokens, int64_t ld, int64_t q_off, int64_t k_off,
                               int64_t v_off, const void* q_gain, const void* k_gain, int w_f32, float eps,
                               float w_offset, const int32_t* positions, const float* cos_sin, int rotary_dim,
                               int style, void* k_cache, void* v_cache, const int64_t* slot_mapping, int heads,
                               int kv_heads, int head_dim, int page_size, int token_runs, hipStream_t stream) {
  // token_runs: the tokens come in runs of consecutive positions of a request (prompt portions), so
  // that gathering 8 tokens' values into 16-byte rows of the transposed V pages pays
  if (tokens <= 0) return OK;
  if (heads <= 0 || kv_heads <= 0 || head_dim <= 0 || page_size <= 0 || tokens > 0x7fffffff) return ERR_BAD_SHAPE;
  if (head_dim > MAX_D) return ERR_UNSUPPORTED;
  if (cos_sin && (rotary_dim <= 0 || rotary_dim > head_dim || rotary_dim % 2 != 0)) return ERR_BAD_SHAPE;
  if (style != 0 && style != 1) return ERR_UNSUPPORTED;
  if ((q_gain == nullptr) != (k_gain == nullptr)) return ERR_BAD_SHAPE;
  const int items = heads + 2 * kv_heads;
  const dim3 grid((unsigned)tokens, (unsigned)((items + WAVES - 1) / WAVES));
  const bool whole_head_neox = style == 0 && head_dim % 2 == 0 && (!cos_sin || rotary_dim == head_dim);
  const bool vec_ok = dtype == DT_BF16 && (head_dim == 64 || head_dim == 128 || head_dim == 256) && ld % 8 == 0 &&
                      q_off % 8 == 0 && k_off % 8 == 0 && v_off % 8 == 0 && ((uintptr_t)qkv % 16) == 0 &&
                      ((uintptr_t)q_gain % 16) == 0 && ((uintptr_t)k_gain % 16) == 0 && ((uintptr_t)cos_sin % 16) == 0 &&
                      ((uintptr_t)k_cache % 16) == 0;
  if (whole_head_neox && vec_ok) {
    const int lph = head_dim / 8, hpw = 64 / lph;
    // many tokens fill the chip with one workgroup each; few tokens spread their heads over several
    // many tokens: V goes to its transposed pages through workgroups that gather it (16-byte stores)
    const bool gather = slot_mapping && token_runs && tokens >= 64 && page_size % 8 == 0 && ((uintptr_t)v_cache % 16) == 0;
    const int64_t gather_v = gather ? (tokens + 8 * WAVES - 1) / (8 * WAVES) * kv_heads : 0;
    if (tokens + gather_v > 0x7fffffff) return ERR_BAD_SHAPE;
    const dim3 vgrid((unsigned)(tokens + gather_v),
                     tokens >= 512 ? 1u : (unsigned)((items + WAVES * hpw - 1) / (WAVES * hpw)));
#define DINFER_QKV_VEC(LPH_)                                                                                          \
  qkv_post_vec_kernel<LPH_><<<vgrid, WAVES * 64, 0, stream>>>(                                                         \
      (bf16*)qkv, ld, q_off, k_off, v_off, q_gain, k_gain, w_f32, eps, w_offset, positions, cos_sin, (bf16*)k_cache, \
      (bf16*)v_cache, slot_mapping, heads, kv_heads, page_size, (int)tokens, (int)gather_v)
    if (lph == 8) DINFER_QKV_VEC(8);
    else if (lph == 16) DINFER_QKV_VEC(16);
    else DINFER_QKV_VEC(32);
#undef DINFER_QKV_VEC
    return launch_status();
  }
  if (whole_head_neox) {
    const dim3 grid((unsigned)tokens, (unsigned)((items + WAVES * IPW - 1) / (WAVES * IPW)));
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
