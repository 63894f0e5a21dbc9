// Plain paged attention for any head size, group size, page size and storage
// type: the kernel of the 32-bit path and the reference beside the MFMA
// kernels. One wave per (token, query head); keys are visited in ascending
// order in tiles of 64, so a row's arithmetic depends only on its own position
// and never on how the step was cut or batched.
//
//   row i of request b has position p = seq_len[b] - q_len[b] + i and sees the
//   keys j in [max(0, p - window + 1), p]  (window 0: all keys up to p);
//   s_j = scale * <q, k_j>;  P = softmax(s);  o = sum_j P_j v_j   (all float)
//
// K and V are read from the cache pages through the request's block table
// (K page [Hkv][D / 8][page][8], V page [Hkv][D][page]); the step's own tokens were
// written there before this kernel runs.
//
// Reference behaviour: crates/kernels/cuda/gqa.cu:1037-1118 (plain paged
// kernel: causal inclusive, query head h reads kv head h / G, online softmax,
// 0 when nothing was summed).
#include "common.cuh"

using namespace dinfer;

namespace {

constexpr int MAX_D = 512;
constexpr int WAVES = 4;

template <class S>
__global__ void __launch_bounds__(WAVES * 64) attn_paged_ref_kernel(
    const S* __restrict__ q, int64_t ld_q, S* __restrict__ out, int64_t ld_out, const S* __restrict__ k_cache,
    const S* __restrict__ v_cache, const int32_t* __restrict__ block_table, int64_t max_blocks,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_lens, int num_reqs, float scale,
    int window, int H, int Hkv, int D, int page) {
  __shared__ float qs[WAVES][MAX_D];
  __shared__ float ps[WAVES][64];
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y * WAVES + wave;
  const bool live = h < H;

  // the request of token t: cu[b] <= t < cu[b+1]
  int lo_b = 0, hi_b = num_reqs - 1;
  while (lo_b < hi_b) {
    const int mid = (lo_b + hi_b + 1) >> 1;
    if (cu_seqlens[mid] <= t) lo_b = mid; else hi_b = mid - 1;
  }
  const int b = lo_b;
  const int q_len = cu_seqlens[b + 1] - cu_seqlens[b];
  const int p = seq_lens[b] - q_len + (t - cu_seqlens[b]);
  const int first_key = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
  const int32_t* bt = block_table + (int64_t)b * max_blocks;
  const int hk = live ? h / (H / Hkv) : 0;

  if (live) {
    const S* qr = q + (int64_t)t * ld_q + (int64_t)h * D;
    for (int d = lane; d < D; d += 64) qs[wave][d] = to_f32(qr[d]);
  }
  __syncthreads();

  constexpr int NC = MAX_D / 64;
  float o[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) o[c] = 0.f;
  float m = -INFINITY, l = 0.f;

  for (int j0 = first_key; j0 <= p; j0 += 64) {
    const int j = j0 + lane;
    float s = -INFINITY;
    if (live && j <= p) {
      const int blk = bt[j / page];
      const S* kr = k_cache + ((int64_t)blk * Hkv + hk) * page * D;  // the head's page
      const int off = j % page;
      float acc = 0.f;
      for (int d = 0; d < D; ++d) acc += qs[wave][d] * to_f32(kr[k_page_offset(off, d, page)]);
      s = acc * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float pj = (live && j <= p) ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);  // m = -inf on the first tile: alpha = 0
    l = l * alpha + wave_sum(pj);
    m = m_new;
    __syncthreads();  // the previous tile's ps[] has been consumed
    ps[wave][lane] = pj;
    __syncthreads();
    if (live) {
      const int n = p - j0 + 1 < 64 ? p - j0 + 1 : 64;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int d = lane + 64 * c;
        if (d < D) {
          float acc = o[c] * alpha;
          for (int jj = 0; jj < n; ++jj) {
            const int key = j0 + jj;
            const int blk = bt[key / page];
            const S* vr = v_cache + (((int64_t)blk * Hkv + hk) * D + d) * page + (key % page);
            acc += ps[wave][jj] * to_f32(*vr);
          }
          o[c] = acc;
        }
      }
    }
  }
  if (live) {
    S* orow = out + (int64_t)t * ld_out + (int64_t)h * D;
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d = lane + 64 * c;
      if (d < D) orow[d] = from_f32<S>(o[c] * inv);
    }
  }
}

}  // namespace

// q [T, ld_q] (head h at column h*D), out [T, ld_out]; block_table [num_reqs, max_blocks];
// cu_seqlens [num_reqs+1] prefix sums of the rows per request; seq_lens [num_reqs]
// lengths after this step.
extern "C" int dinfer_attn_paged_ref(int dtype, const void* q, int64_t ld_q, void* out, int64_t ld_out,
                                     const void* k_cache, const void* v_cache, const int32_t* block_table,
                                     int64_t max_blocks, const int32_t* cu_seqlens, const int32_t* seq_lens,
                                     int num_reqs, int64_t tokens, float scale, int window, int heads, int kv_heads,
                                     int head_dim, int page_size, hipStream_t stream) {
  if (tokens <= 0 || num_reqs <= 0) return OK;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || head_dim <= 0 || page_size <= 0 || max_blocks <= 0 ||
      window < 0 || tokens > 0x7fffffff)
    return ERR_BAD_SHAPE;
  if (head_dim > MAX_D) return ERR_UNSUPPORTED;
  const dim3 grid((unsigned)tokens, (unsigned)((heads + WAVES - 1) / WAVES));
  DINFER_DISPATCH_DTYPE(dtype, {
    attn_paged_ref_kernel<S><<<grid, WAVES * 64, 0, stream>>>(
        (const S*)q, ld_q, (S*)out, ld_out, (const S*)k_cache, (const S*)v_cache, block_table, max_blocks, cu_seqlens,
        seq_lens, num_reqs, scale, window, heads, kv_heads, head_dim, page_size);
  });
  return launch_status();
}
