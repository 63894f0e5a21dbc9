// MFMA attention over the paged cache for bf16, gfx950.
//
// Both kernels compute S^T = K . Q^T and O^T = V^T . P with
// v_mfma_f32_16x16x32_bf16, whose operands want, per lane, 8 consecutive
// elements of the contraction dimension:
//   A (16 x 32): lane l holds A[l % 16][8 * (l / 16) .. + 8]
//   B (32 x 16): lane l holds B[8 * (l / 16) .. + 8][l % 16]
//   D (16 x 16): lane l holds D[4 * (l / 16) + r][l % 16], r = 0..3
// K pages [Hkv][D / 8][page][8] give A = 8-element pieces of K rows straight from
// memory (contraction over d; the pieces of consecutive keys are contiguous, so
// a quad of lanes reads 64 contiguous bytes); V pages [Hkv][D][page] (transposed)
// give A = V^T rows straight from memory (contraction over keys). K and V are
// not staged through LDS.
//
// A block of 32 keys is scored by two MFMA chains (a = 0, 1). Row i of chain a
// is key  kb + 8 * (i / 4) + 4 * a + (i % 4),  so lane group g = l / 16 ends up
// with the scores of keys kb + 8 g .. kb + 8 g + 7 in its eight result
// registers: exactly the B operand of the P.V product, with no shuffle.
// A query (a column, l % 16) keeps its running maximum, sum and output column in
// the same lanes through both products.
//
//   flash:  query rows with or without history, causal, optional window; a
//           workgroup owns QT x 16 query rows of one head, its four waves walk a
//           quarter of the keys each in blocks of 32 (online softmax in base 2)
//           and combine their results in LDS.
//   decode: all requests bring one row; the G query heads of a kv head are the
//           16 columns, so K and V are read once per group; the keys are split
//           over workgroups, each writing (m, l, o) partials; a merge kernel
//           combines them.
//
// Sizes: head_dim a multiple of 16 from the instantiated list, page size a
// multiple of 8, G <= 16 for decode. Anything else is refused (the caller then
// uses the plain kernel).
//
// Reference behaviour: crates/kernels/cuda/gqa.cu:167-369 (flash prefill and
// paged: 64-key tiles, base-2 online softmax, P rounded to bf16 before P.V),
// gqa_decode_v3_core.cuh:72-242 and gqa.cu:1423-1461 (split-K decode, merge of
// (m, l, o) partials).
#include <cmath>

#include "common.cuh"

using namespace dinfer;

namespace {

constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
  return z;
}

__device__ __forceinline__ int lane_of() { return threadIdx.x & 63; }

// 2^x by the hardware instruction alone: results below 2^-126 become 0, which a softmax weight may
__device__ __forceinline__ float exp2_raw(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// Block-table entries of 64 consecutive pages of one request, one per lane; a lane gets the
// entry it needs by a cross-lane read, so no key block waits for a table load of its own.
// P2: the page size is a power of two (shifts and masks instead of divisions).
template <bool P2>
struct Pages {
  const int32_t* bt;
  int max_blocks, base, reg, ps, ps_shift;

  __device__ __forceinline__ void init(const int32_t* table, int max_blocks_, int page_size, int first_key) {
    bt = table;
    max_blocks = max_blocks_;
    ps = page_size;
    ps_shift = P2 ? __builtin_ctz(page_size) : 0;
    fetch(page_of(first_key));
  }
  __device__ __forceinline__ int page_of(int key) const { return P2 ? key >> ps_shift : key / ps; }
  __device__ __forceinline__ int offset_of(int key) const { return P2 ? key & (ps - 1) : key % ps; }
  __device__ __forceinline__ void fetch(int first_page) {
    base = first_page;
    const int i = base + (int)(threadIdx.x & 63);
    reg = i < max_blocks ? bt[i] : 0;
  }
  // kb is wave-uniform and only grows; afterwards the pages of keys [kb, kb + 32) are on board
  __device__ __forceinline__ void ensure(int kb) {
    if (page_of(kb + 31) - base >= 64) fetch(page_of(kb));
  }
  // every lane of the wave must call this (it is a cross-lane operation)
  __device__ __forceinline__ int get(int page) const { return __shfl(reg, page - base, 64); }
};

// 16 bytes of cache pages; stream: past the caches (the bytes are used once)
template <bool STREAM>
__device__ __forceinline__ bf16x8 ld16(const bf16* p) {
  if constexpr (STREAM)
    return __builtin_nontemporal_load((const bf16x8*)p);
  else
    return *(const bf16x8*)p;
}

template <int DT>
struct Frags {
  static constexpr int KS = (DT + 1) / 2;
  bf16x8 k[2][KS];
  bf16x8 v[DT];
};

// NT column tiles (queries, or the heads of a group) against the keys of one request, 32 at a time.
//   qf[t][ks]   B operands of the score product, the whole head in registers
//   col_lo/hi   per column tile and lane: the column's visible keys are [col_lo, col_hi)
//   k_lo, k_hi  the keys this wave may touch at all (held pages, written slots)
// load() issues the loads of one block, compute() consumes them; walk() keeps the next block's
// loads in flight while the current one is computed.
template <int DT, int NT, bool P2>
struct Tile {
  static constexpr int KS = (DT + 1) / 2;  // 32-wide steps over the head dimension
  static constexpr float LAZY = 6.f;       // weights up to 2^6 before the reference follows the maximum
  f32x4 o[NT][DT];
  float m[NT], l[NT];
  Pages<P2> pages;
  const bf16* kc;
  const bf16* vc;
  int hk, Hkv, k_lo, k_hi;
  int page_stride, head_off;  // elements from page to page, and from the page's start to this kv head
  float scale_log2e;

  __device__ __forceinline__ void init(const bf16* kc_, const bf16* vc_, const int32_t* bt, int max_blocks, int hk_,
                                       int Hkv_, int ps, int k_lo_, int k_hi_, float scale_log2e_) {
    kc = kc_; vc = vc_; hk = hk_; Hkv = Hkv_; k_lo = k_lo_; k_hi = k_hi_; scale_log2e = scale_log2e_;
    page_stride = Hkv_ * ps * DT * 16;  // the host checks that this fits 31 bits
    head_off = hk_ * ps * DT * 16;
    pages.init(bt, max_blocks, ps, k_lo_ & ~31);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      m[t] = -INFINITY;
      l[t] = 0.f;
#pragma unroll
      for (int d = 0; d < DT; ++d) o[t][d] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  }

  // Loads are unconditional: a key outside [k_lo, k_hi) is replaced by the nearest key inside, which
  // lies in a page the request holds, so straight-line code with all loads in flight at once. What
  // was loaded for such a key never counts: its score is masked, and accumulate() zeroes its value.
  // CLAMP = false: the block lies wholly inside [k_lo, k_hi), so no key needs replacing.
  // STREAM: K and V are read with non-temporal loads (a step's keys exceed the caches and each byte is used once).
  template <bool CLAMP, bool STREAM>
  __device__ __forceinline__ void load_k(Frags<DT>& f, int kb) {
    constexpr int D = DT * 16;
    const int lane = threadIdx.x & 63, i16 = lane & 15, g4 = lane >> 4;
    const int last = k_hi - 1;
    // K rows of this lane: keys kg_row + (i16 & 3) and + 4: one aligned group of 8, so one page (page size % 8 == 0)
    int key0 = kb + 8 * (i16 >> 2) + (i16 & 3), key1 = key0 + 4;
    if (CLAMP) {
      key0 = key0 < k_lo ? k_lo : (key0 > last ? last : key0);
      key1 = key1 < k_lo ? k_lo : (key1 > last ? last : key1);
    }
    const int pg0 = pages.get(pages.page_of(key0));
    const int pg1 = CLAMP ? pages.get(pages.page_of(key1)) : pg0;  // clamping may move the two into different pages
    // K pages are [Hkv][D / 8][page][8]: the 16-byte pieces of consecutive keys lie next to each other,
    // so the four lanes of a quad (four consecutive keys, one piece index) read 64 contiguous bytes
    const bf16* kr0 = kc + ((int64_t)pg0 * page_stride + (head_off + pages.offset_of(key0) * 8));
    const bf16* kr1 = CLAMP ? kc + ((int64_t)pg1 * page_stride + (head_off + pages.offset_of(key1) * 8)) : kr0 + 32;
    const int piece = pages.ps * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      int c = ks * 4 + g4;
      const bool dv = c * 8 < D;  // D % 32 == 16: the upper half of the last step is padding
      if (!dv) c = 0;
      f.k[0][ks] = ld16<STREAM>(kr0 + c * piece);
      f.k[1][ks] = ld16<STREAM>(kr1 + c * piece);
      if (DT % 2 == 1 && ks == KS - 1 && !dv) f.k[0][ks] = f.k[1][ks] = zero8();
    }
  }

  template <bool CLAMP, bool STREAM>
  __device__ __forceinline__ void load_v(Frags<DT>& f, int kb) {
    const int lane = threadIdx.x & 63, i16 = lane & 15, g4 = lane >> 4;
    const int ps = pages.ps;
    // V^T rows of this lane: d = 16 dt + i16, keys kg .. kg + 7 (one page)
    int kg = kb + 8 * g4;
    if (CLAMP) {
      const int g_lo = k_lo & ~7, g_hi = (k_hi - 1) & ~7;
      kg = kg < g_lo ? g_lo : (kg > g_hi ? g_hi : kg);
    }
    const int pgv = pages.get(pages.page_of(kg));
    const bf16* vrow = vc + ((int64_t)pgv * page_stride + (head_off + i16 * ps + pages.offset_of(kg)));
#pragma unroll
    for (int d = 0; d < DT; ++d) f.v[d] = ld16<STREAM>(vrow + d * 16 * ps);
  }

  template <bool CLAMP, bool STREAM>
  __device__ __forceinline__ void load(Frags<DT>& f, int kb) {
    pages.ensure(kb);
    load_k<CLAMP, STREAM>(f, kb);
    load_v<CLAMP, STREAM>(f, kb);
  }

  // S^T of one block: s[t][a] holds, for column i16 of tile t, the keys kb + 8 g4 + 4 a + {0..3}
  __device__ __forceinline__ void scores(const Frags<DT>& f, const bf16x8 (&qf)[NT][KS], f32x4 (&s)[NT][2]) {
#pragma unroll
    for (int t = 0; t < NT; ++t) s[t][0] = s[t][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        s[t][0] = mfma16(f.k[0][ks], qf[t][ks], s[t][0]);
        s[t][1] = mfma16(f.k[1][ks], qf[t][ks], s[t][1]);
      }
  }

  // Online softmax per column; this lane holds keys kb + 8 g4 + {0..7} of column i16. Returns the
  // weights as the B operand of the second product.
  // MASK: some key of the block is invisible to some column, or lies outside [k_lo, k_hi)
  template <bool MASK>
  __device__ __forceinline__ void softmax(const f32x4 (&s)[NT][2], bf16x8 (&pf)[NT], int kb, const int (&col_lo)[NT],
                                          const int (&col_hi)[NT]) {
    const int kg = kb + 8 * ((threadIdx.x & 63) >> 4);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      // raw scores; the running maximum m is kept in raw units too, and the scale is folded into
      // one fused multiply-add per score: p = 2^(c s - c m), c = scale * log2(e) > 0
      float x[8];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        x[r] = s[t][0][r];
        x[4 + r] = s[t][1][r];
      }
      if (MASK) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (kg + e < col_lo[t] || kg + e >= col_hi[t]) x[e] = -INFINITY;
      }
      float mx = x[0];
#pragma unroll
      for (int e = 1; e < 8; ++e) mx = fmaxf(mx, x[e]);
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      // m is the reference the weights are taken against, not the maximum itself: it follows the maximum only
      // when that has risen by more than LAZY (in base-2 units) for some column of the wave (a uniform branch),
      // so weights stay below 2^LAZY and the output is rescaled rarely. Counted on random scores: among the
      // columns of a tile some maximum rises in most blocks, and every rise used to cost a multiplication of
      // the whole output tile. The sums and the final division use the same reference: the result is the same.
      if (__any((mx - m[t]) * scale_log2e > LAZY)) {  // m = -inf: any visible key moves it
        const float m_new = fmaxf(m[t], mx);
        const float alpha = m_new == m[t] ? 1.f : exp2_raw((m[t] - m_new) * scale_log2e);  // m = -inf: 0
        l[t] *= alpha;
#pragma unroll
        for (int d = 0; d < DT; ++d) o[t][d] *= alpha;
        m[t] = m_new;
      }
      const float mc = (m[t] == -INFINITY ? 0.f : m[t]) * scale_log2e;  // nothing visible yet: everything stays zero
      float ps_ = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float p = exp2_raw(fmaf(x[e], scale_log2e, -mc));
        ps_ += p;
        pf[t][e] = (bf16)p;
      }
      l[t] += ps_;  // partial over this lane's keys; lane groups are summed at the end
    }
  }

  // O^T += V^T . P
  template <bool MASK>
  __device__ __forceinline__ void accumulate(const Frags<DT>& f, const bf16x8 (&pf)[NT], int kb) {
    const int kg = kb + 8 * ((threadIdx.x & 63) >> 4);
#pragma unroll
    for (int d = 0; d < DT; ++d) {
      bf16x8 vf = f.v[d];
      if (MASK) {
        // a stale slot may hold anything; its weight is 0, but 0 * inf would poison the sum
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (kg + e < k_lo || kg + e >= k_hi) vf[e] = (bf16)0.f;
      }
#pragma unroll
      for (int t = 0; t < NT; ++t) o[t][d] = mfma16(vf, pf[t], o[t][d]);
    }
  }

  template <bool MASK>
  __device__ __forceinline__ void compute(const Frags<DT>& f, const bf16x8 (&qf)[NT][KS], int kb,
                                          const int (&col_lo)[NT], const int (&col_hi)[NT]) {
    f32x4 s[NT][2];
    bf16x8 pf[NT];
    scores(f, qf, s);
    softmax<MASK>(s, pf, kb, col_lo, col_hi);
    accumulate<MASK>(f, pf, kb);
  }

  // All key blocks of [k_lo, k_hi); mask(kb) says whether block kb needs per-key masking.
  // TWO_BODIES: blocks that need no masking run a body without it (more code, fewer instructions
  // per block); otherwise every block runs the masking body.
  // A block's loads are issued right before its use and other waves hide the latency: reading a
  // block ahead was measured and does not pay (neither with a second set of registers nor by
  // refilling each fragment as soon as its last reader has issued; the split-K kernel with a second set at 8 to 64
  // requests of 2k and 4k keys, one wave a SIMD: within 1 % either way, 5.6 to 5.9 TB/s with it and without).
  // hook(kb, last): called before block kb's loads are issued; `last` says that kb is the wave's last block. The wave
  // that brings the row's own key issues that key's loads a block early there and stores it before the last block.
  template <bool TWO_BODIES, bool STREAM, class MaskFn, class Hook>
  __device__ __forceinline__ void walk(const bf16x8 (&qf)[NT][KS], const int (&col_lo)[NT], const int (&col_hi)[NT],
                                       MaskFn mask, Hook hook) {
    Frags<DT> f;
#pragma nounroll
    for (int kb = k_lo & ~31; kb < k_hi; kb += 32) {
      hook(kb, kb + 32 >= k_hi);
      if (!TWO_BODIES || mask(kb)) {
        load<true, STREAM>(f, kb);
        compute<true>(f, qf, kb, col_lo, col_hi);
      } else {
        load<false, STREAM>(f, kb);
        compute<false>(f, qf, kb, col_lo, col_hi);
      }
    }
  }
  template <bool TWO_BODIES, class MaskFn>
  __device__ __forceinline__ void walk(const bf16x8 (&qf)[NT][KS], const int (&col_lo)[NT], const int (&col_hi)[NT],
                                       MaskFn mask) {
    walk<TWO_BODIES, false>(qf, col_lo, col_hi, mask, [](int, bool) {});
  }

  // total of l over the four lane groups of a column
  __device__ __forceinline__ float sum_l(int t) const {
    float v = l[t];
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
  }
};

// Flash kernel. A workgroup owns QT x 16 query rows of one head; its four waves share the rows and
// deal the key blocks among themselves in four contiguous runs, each wave keeping its own running
// (maximum, sum, output); at the end waves 1..3 hand theirs to wave 0 through LDS, which combines
// them and stores the rows. So every key block is read by one wave only, and a long row tile (many
// keys under a causal mask) is four short pieces of work instead of one long one: with a few
// thousand workgroups of unequal length issued longest first, the chip stays evenly busy.
// Measured on MI355X at head size 128 (one 2,048-token prompt, 32 heads): 122 us for the former
// one-wave-per-tile kernel, where the longest tile set the time.
template <int DT, int QT, bool P2>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 8))) attn_flash_kernel(
    const bf16* __restrict__ q, int64_t ld_q, bf16* __restrict__ out, int64_t ld_out, const bf16* __restrict__ kc,
    const bf16* __restrict__ vc, const int32_t* __restrict__ block_table, int64_t max_blocks,
    const int32_t* __restrict__ cu_seqlens, const int32_t* __restrict__ seq_lens, int tiles_x, float scale_log2e,
    int window, int H, int Hkv, int ps, int skip_single) {
  constexpr int D = DT * 16;
  constexpr int KS = (DT + 1) / 2;
  constexpr int QW = 16 * QT;  // query rows per workgroup
  // what waves 1..3 hand to wave 0 (dynamic: three row tiles of head size 128 need more than the 64 KB a kernel
  // may declare): part_o[3][QT][DT][64] of f32x4, then part_m and part_l [3][QT][64] of float
  extern __shared__ __attribute__((aligned(16))) char flash_smem[];
  f32x4* const part_o_ = (f32x4*)flash_smem;
  float* const part_m_ = (float*)(flash_smem + sizeof(f32x4) * 3 * QT * DT * 64);
  float* const part_l_ = part_m_ + 3 * QT * 64;
  auto part_o = [&](int r, int t, int d) -> f32x4& { return part_o_[((r * QT + t) * DT + d) * 64 + lane_of()]; };
  auto part_m = [&](int r, int t) -> float& { return part_m_[(r * QT + t) * 64 + lane_of()]; };
  auto part_l = [&](int r, int t) -> float& { return part_l_[(r * QT + t) * 64 + lane_of()]; };
  // Block order: the head index runs fastest and visits kv heads round-robin, so that the
  // workgroups an XCD receives (linear id modulo 8) share kv heads, and with them the L2 lines
  // of K and V. Late query tiles (most keys) are issued first.
  const int L = blockIdx.x;
  const int e = L % H, rest = L / H;
  const int tile = tiles_x - 1 - rest % tiles_x, b = rest / tiles_x;
  const int G = H / Hkv;
  const int hk = e % Hkv, h = hk * G + e / Hkv;
  const int q_begin = cu_seqlens[b];
  const int q_len = cu_seqlens[b + 1] - q_begin;
  const int hist = seq_lens[b] - q_len;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, i16 = lane & 15, g4 = lane >> 4;
  const int q0 = tile * QW;
  if (q0 >= q_len) return;                // the whole workgroup: nobody is left waiting at the barrier below
  if (skip_single && q_len == 1) return;  // single rows go to the split-K kernel
  const int32_t* bt = block_table + (int64_t)b * max_blocks;

  bf16x8 qf[QT][KS];
  int col_lo[QT], col_hi[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const int row = q0 + t * 16 + i16;
    const int rc = row < q_len ? row : q_len - 1;  // rows past the end compute something harmless, never stored
    const bf16* qp = q + (int64_t)(q_begin + rc) * ld_q + (int64_t)h * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + g4 * 8;
      qf[t][ks] = d < D ? *(const bf16x8*)(qp + d) : zero8();
    }
    const int pos = hist + rc;
    col_hi[t] = pos + 1;
    col_lo[t] = window > 0 ? (pos - window + 1 > 0 ? pos - window + 1 : 0) : 0;
  }
  // the keys any row of the tile sees, and this wave's run of 32-key blocks among them
  const int p_first = hist + q0;
  const int p_last = hist + (q0 + QW < q_len ? q0 + QW : q_len) - 1;
  const int all_hi = p_last + 1;
  const int all_lo = window > 0 ? (p_first - window + 1 > 0 ? p_first - window + 1 : 0) : 0;
  const int blk_first = all_lo >> 5, blk_end = (all_hi + 31) >> 5;
  const int per = (blk_end - blk_first + 3) >> 2;
  const int blk0 = blk_first + wave * per;
  const int blk1 = blk0 + per < blk_end ? blk0 + per : blk_end;
  const int k_lo = blk0 * 32 > all_lo ? blk0 * 32 : all_lo;
  const int k_hi = blk1 * 32 < all_hi ? blk1 * 32 : all_hi;

  Tile<DT, QT, P2> tl;
  tl.init(kc, vc, bt, (int)max_blocks, hk, Hkv, ps, k_lo, k_hi, scale_log2e);
  tl.template walk<true>(qf, col_lo, col_hi, [&](int kb) {
    return kb + 31 > p_first || kb < all_lo || (window > 0 && kb < p_last - window + 1);
  });

  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      part_m(wave - 1, t) = tl.m[t];
      part_l(wave - 1, t) = tl.l[t];
#pragma unroll
      for (int d = 0; d < DT; ++d) part_o(wave - 1, t, d) = tl.o[t][d];
    }
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    // every wave keeps a lane's share in the same places, so the parts combine lane by lane:
    // o = sum_r 2^(c (m_r - M)) o_r, likewise l (still a partial over the lane's keys)
    float mr[3], M = tl.m[t];
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      mr[r] = part_m(r, t);
      M = fmaxf(M, mr[r]);
    }
    const float mc = (M == -INFINITY ? 0.f : M) * scale_log2e;
    const float a0 = exp2_raw(fmaf(tl.m[t], scale_log2e, -mc));  // an empty part has m = -inf: weight 0
    float lsum = tl.l[t] * a0;
#pragma unroll
    for (int d = 0; d < DT; ++d) tl.o[t][d] *= a0;
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      const float ar = exp2_raw(fmaf(mr[r], scale_log2e, -mc));
      lsum += part_l(r, t) * ar;
#pragma unroll
      for (int d = 0; d < DT; ++d) tl.o[t][d] += part_o(r, t, d) * ar;
    }
    tl.l[t] = lsum;
    const float lt = tl.sum_l(t);
    const float inv = lt > 0.f ? 1.f / lt : 0.f;
    const int row = q0 + t * 16 + i16;
    if (row < q_len) {
      bf16* op = out + (int64_t)(q_begin + row) * ld_out + (int64_t)h * D + 4 * g4;
#pragma unroll
      for (int d = 0; d < DT; ++d) {
        bf16x4 r;
#pragma unroll
        for (int k = 0; k < 4; ++k) r[k] = (bf16)(tl.o[t][d][k] * inv);
        *(bf16x4*)(op + d * 16) = r;
      }
    }
  }
}

// What the decode kernel does itself in a step of single rows only, so that no kernel runs between the q|k|v product
// and the attention: the per-head norm of q and k, the rotation (pairs (i, i + D/2), whole head, angles of the row's
// position), and the new key and value into their pages. Same arithmetic, in the same order, as qkv_post_vec_kernel.
struct DecodePost {
  const bf16* wq;        // gains of the q and k norms (null: no norm)
  const bf16* wk;
  float eps, w_offset;
  const int32_t* pos;    // [rows] position of each row
  const float* cos_sin;  // [positions][D]: cos of the D/2 angles, then sin (null: no rotation)
  const int64_t* slots;  // [rows] block * page + offset of the new key; negative or null: nothing is written
  const bf16* k_new;     // the rows' new keys and values, [rows, ld_q] like q
  const bf16* v_new;
  bf16* k_cache;         // the same pages the kernel reads
  bf16* v_cache;
};

// One head of D = 16 DT dims (DT % 4 == 0) in MFMA operand order: a lane holds the pieces d = 32 ks + 8 g4 .. + 8,
// ks < KS, of the head its lane group of 16 selects; the partner of a pair lies KS / 2 pieces further in the same lane.
// In three steps, so that the kernel can issue every load whose address it knows before it waits for any: load (the
// head and the gains: addresses known at once), Angles::load (needs the position), finish (arithmetic only).
template <int DT>
struct HeadPost {
  static constexpr int KS = DT / 2, D = DT * 16, HALF = D / 2;
  struct Angles {
    f32x4 c[KS / 2][2], s[KS / 2][2];
    __device__ __forceinline__ void load(const float* cs) {
      const int g4 = (threadIdx.x & 63) >> 4;
#pragma unroll
      for (int ks = 0; ks < KS / 2; ++ks) {
        const int pi = ks * 32 + g4 * 8;
        c[ks][0] = *(const f32x4*)(cs + pi);
        c[ks][1] = *(const f32x4*)(cs + pi + 4);
        s[ks][0] = *(const f32x4*)(cs + HALF + pi);
        s[ks][1] = *(const f32x4*)(cs + HALF + pi + 4);
      }
    }
  };
  bf16x8 x[KS];
  bf16x8 g[KS];  // the gains (bf16)

  __device__ __forceinline__ void load(const bf16* src, bool active) {
    const int g4 = (threadIdx.x & 63) >> 4;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) x[ks] = active ? *(const bf16x8*)(src + ks * 32 + g4 * 8) : zero8();
  }
  __device__ __forceinline__ void load_gains(const bf16* w) {
    const int g4 = (threadIdx.x & 63) >> 4;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) g[ks] = *(const bf16x8*)(w + ks * 32 + g4 * 8);
  }

  // normed: gains were loaded; rotate: a holds the angles of the row's position
  __device__ __forceinline__ void finish(const Angles& a, bool normed, float eps, float w_offset, bool rotate,
                                         bf16x8 (&r)[KS]) const {
    float inv = 1.f;
    if (normed) {
      float s[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        s[ks] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) s[ks] = add_square(s[ks], (float)x[ks][e]);
      }
      // the sum of squares over the head's D / 8 pieces as a butterfly over the piece index, highest bit first
#pragma unroll
      for (int o = KS / 2; o > 0; o >>= 1)
#pragma unroll
        for (int ks = 0; ks < o; ++ks) s[ks] = s[ks] + s[ks + o];
      float ss = s[0];
      ss += __shfl_xor(ss, 32, 64);
      ss += __shfl_xor(ss, 16, 64);
      inv = 1.f / sqrtf(ss / (float)D + eps);
    }
#pragma unroll
    for (int ks = 0; ks < KS / 2; ++ks) {
      const int k2 = ks + KS / 2;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float y1 = (float)x[ks][e], y2 = (float)x[k2][e];
        if (normed) {
          y1 = y1 * inv * ((float)g[ks][e] + w_offset);
          y2 = y2 * inv * ((float)g[k2][e] + w_offset);
        }
        const float c = rotate ? a.c[ks][e >> 2][e & 3] : 1.f, sn = rotate ? a.s[ks][e >> 2][e & 3] : 0.f;
        r[ks][e] = (bf16)rotated_first(y1, y2, c, sn);
        r[k2][e] = (bf16)rotated_second(y1, y2, c, sn);
      }
    }
  }
};

// The keys a request's row sees, [first, seq), are cut into `splits` equal parts of a multiple of
// 32 keys; short requests leave the last parts empty. Computed alike by the decode and merge kernels.
__device__ __forceinline__ void split_range(int seq, int window, int splits, int sp, int* k_lo, int* k_hi, int* kps) {
  const int first = window > 0 ? (seq - window > 0 ? seq - window : 0) : 0;  // the row's position is seq - 1
  const int base = first & ~31;
  const int per = (((seq - base) + splits - 1) / splits + 31) & ~31;
  const int lo = base + sp * per, hi = lo + per;
  *k_lo = lo > first ? lo : first;
  *k_hi = hi < seq ? hi : seq;
  *kps = per;
}

// One wave per (split, kv head, request). part: [B, H, splits, D + 4] float = (m in base-2 units, l, -, -, o[D]).
// JOIN (up to JOIN_SPLITS parts: many requests): the parts of a (kv head, request) are the waves of one workgroup,
// meet in LDS and are combined there as attn_decode_merge_kernel combines them, so that kernel does not run.
constexpr int JOIN_SPLITS = 4;
constexpr int64_t STREAM_FROM_BYTES = 100 * 1000 * 1000;
constexpr int64_t STREAM_FROM_BYTES_FEW = 170 * 1000 * 1000;  // for one or two requests

// POST: q arrives as the product left it; the kernel norms and rotates it on the way into its registers (every part
// for itself: the head is 2 D bytes), and the wave whose part ends with the row's own position norms and rotates the
// new key and stores it and the new value into their pages before it reads its last block.
// (The pages are written through post.k_cache / v_cache and read through kc / vc: no __restrict__ on those.)
// LATE (POST only): the new key is dealt with inside the walk instead of before it (see there).
// stream_from: from this many bytes of keys and values in a step on (the request's own visible keys times the number
// of requests: a wave knows no more) they are read with non-temporal loads.
template <int DT, bool P2, bool LATE, bool JOIN = false, bool POST = false>
// (These launches aim at about one wave a SIMD, and JOIN runs where a CU holds 4 to 8 of its waves: registers are no
// limit; POST holds a head, gains and angles at once in its prologue.)
__global__ void __launch_bounds__(JOIN ? 64 * JOIN_SPLITS : 64)
__attribute__((amdgpu_waves_per_eu(2, 8)))
attn_decode_kernel(
    const bf16* __restrict__ q, int64_t ld_q, float* __restrict__ part, const bf16* kc, const bf16* vc,
    const int32_t* __restrict__ block_table, int64_t max_blocks, const int32_t* __restrict__ cu_seqlens,
    const int32_t* __restrict__ seq_lens, int splits, float scale_log2e, int window, int H, int Hkv, int ps,
    int64_t stream_from, bf16* __restrict__ out = nullptr, int64_t ld_out = 0, DecodePost post = DecodePost{}) {
  constexpr int D = DT * 16;
  constexpr int KS = (DT + 1) / 2;
  static_assert(!POST || DT % 4 == 0, "the fused norm and rotation keep both elements of a pair in one lane");
  const int sp = JOIN ? (int)(threadIdx.x >> 6) : (int)blockIdx.x, hk = blockIdx.y, b = blockIdx.z;
  const int G = H / Hkv;
  int row = b;  // without cu_seqlens every request has exactly one row
  if (cu_seqlens) {
    row = cu_seqlens[b];
    if (cu_seqlens[b + 1] - row != 1) return;  // a longer run of rows belongs to the flash kernel
  }
  const int lane = threadIdx.x & 63, i16 = lane & 15, g4 = lane >> 4;
  const int32_t* bt = block_table + (int64_t)b * max_blocks;
  const bf16* qp = q + (int64_t)row * ld_q + (int64_t)(hk * G + (i16 < G ? i16 : 0)) * D;
  int k_lo, k_hi, kps;
  bf16x8 qf[1][KS];
  Tile<DT, 1, P2> tl;
  int seq;
  bool writer = false;
  int w_pos = 0;
  int64_t w_slot = -1;
  if constexpr (POST) {
    // in the order of what is known when: the head, its gains, the row's position and slot at once; ...
    HeadPost<DT> qh;
    qh.load(qp, i16 < G);
    if (post.wq) qh.load_gains(post.wq);
    const int pos_row = post.cos_sin ? post.pos[row] : 0;
    const int64_t slot = post.slots ? post.slots[row] : -1;
    seq = seq_lens[b];
    split_range(seq, window, splits, sp, &k_lo, &k_hi, &kps);
    if (!JOIN && k_lo >= k_hi) return;
    // ... with the length the block table, with the position the angles; the part that ends with the row's own
    // position (wave-uniform) also takes the new key and value
    tl.init(kc, vc, bt, (int)max_blocks, hk, Hkv, ps, k_lo, k_hi, scale_log2e);
    typename HeadPost<DT>::Angles ang;
    if (post.cos_sin) ang.load(post.cos_sin + (int64_t)pos_row * D);
    writer = slot >= 0 && k_lo < k_hi && k_hi == seq;
    qh.finish(ang, post.wq != nullptr, post.eps, post.w_offset, post.cos_sin != nullptr, qf[0]);
    if (i16 >= G) {  // columns beyond the group stay zero whatever the norm made of nothing
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) qf[0][ks] = zero8();
    }
    w_pos = pos_row;
    w_slot = slot;
    if (!LATE && writer) {
      // few requests, short parts: the new key and value are dealt with here, at once (the loads are asked for only now,
      // when the registers of q's head are free); see below for the launches of many requests
      const int64_t blk = slot / ps;
      const int off = (int)(slot - blk * ps);
      const int64_t head = (blk * Hkv + hk) * (int64_t)ps * D;
      HeadPost<DT> kh;
      bf16x8 vv;
      kh.load(post.k_new + (int64_t)row * ld_q + (int64_t)hk * D, i16 == 0);
      if (post.wk) kh.load_gains(post.wk);
      if (lane < D / 8) vv = *(const bf16x8*)(post.v_new + (int64_t)row * ld_q + (int64_t)hk * D + lane * 8);
      bf16x8 kr[KS];
      kh.finish(ang, post.wk != nullptr, post.eps, post.w_offset, post.cos_sin != nullptr, kr);
      if (i16 == 0) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          *(bf16x8*)(post.k_cache + head + k_page_offset(off, ks * 32 + g4 * 8, ps)) = kr[ks];
      }
      if (lane < D / 8) {  // V pages are transposed: the 8 dims of a piece go to 8 rows of keys
        bf16* vd = post.v_cache + head + (int64_t)(lane * 8) * ps + off;
#pragma unroll
        for (int e = 0; e < 8; ++e) vd[(int64_t)e * ps] = vv[e];
      }
    }
  } else {
    seq = seq_lens[b];
    split_range(seq, window, splits, sp, &k_lo, &k_hi, &kps);
    // an empty part writes nothing; the merge kernel skips it by the same rule. (JOIN: it walks no block and
    // leaves m = -inf, which weighs nothing; its wave must reach the barrier below.)
    if (!JOIN && k_lo >= k_hi) return;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + g4 * 8;
      qf[0][ks] = (d < D && i16 < G) ? *(const bf16x8*)(qp + d) : zero8();
    }
    tl.init(kc, vc, bt, (int)max_blocks, hk, Hkv, ps, k_lo, k_hi, scale_log2e);
  }
  const int col_lo[1] = {k_lo}, col_hi[1] = {k_hi};
  // (reading the first block before q is normed, or two blocks ahead, was measured at 1 and 8 requests: no gain)
  const auto partial = [&](int kb) { return kb < k_lo || kb + 32 > k_hi; };
  // Where a step's keys and values exceed the caches they are read past them (every layer has keys of its own, so
  // none is read twice anyway): 8 kv heads of 128, 8 requests of 32k keys 193 -> 175 us, 16 of 2k 33.7 -> 31.7,
  // 8 of 4k 33.6 -> 31.7; below about 100 MB a step the plain loads are faster (one request of 8k keys 19.0 against
  // 21.6 us, 4 of 2k 16.1 against 17.6; one or two requests up to 170 MB: one of 32k 39.7 against 42.1, of 48k 51.5
  // against 48.9). Both walks are in the kernel, the choice is uniform over the wave.
  const int seen = window > 0 && window < seq ? window : seq;
  const auto walk = [&](auto hook) {
    // (LATE is for many requests, whose keys exceed the caches at any length worth a thought)
    if (LATE || (int64_t)gridDim.z * seen * (Hkv * D * 4) >= stream_from)
      tl.template walk<false, true>(qf, col_lo, col_hi, partial, hook);
    else
      tl.template walk<false, false>(qf, col_lo, col_hi, partial, hook);
  };
  if constexpr (POST && !LATE) {
    // the key was stored in the prologue; the fence lets the wave's own loads of its last block see it
    walk([&](int, bool last) {
      if (writer && last) __threadfence_block();
    });
  } else if constexpr (POST) {
    // Many requests (parts of dozens of blocks, every workgroup waiting for the wave that writes):
    // The wave whose part ends with the row's own position brings the new key and value: their loads (the head, the
    // value) go out three blocks before the end, a block later the key is normed (gains and angles asked for there:
    // kept through a block they would cost the walk a hundred registers), rotated and stored with the value, and
    // before the last block a fence lets the wave's own loads of that block see them: the latencies lie under the
    // blocks' work instead of on the path of the wave that ends its workgroup (64 requests of 2,064 keys: 96.9 ->
    // 92.3 us, of 4,080 keys 181 -> 174.5; at 8 requests, where a part is five blocks, the larger kernel loses 1.5 us,
    // hence the two forms). A part of fewer blocks does the steps as early as it can.
    HeadPost<DT> kh;   // only its head is kept from one block to the next: the gains and angles are asked for where
    bf16x8 vv;         // they are used (they come from L2), or the walk would hold a hundred registers for them
    bool fetched = false;
    const auto fetch_key = [&]() {
      kh.load(post.k_new + (int64_t)row * ld_q + (int64_t)hk * D, i16 == 0);
      if (lane < D / 8) vv = *(const bf16x8*)(post.v_new + (int64_t)row * ld_q + (int64_t)hk * D + lane * 8);
      fetched = true;
    };
    const auto store_key = [&]() {
      const int64_t blk = w_slot / ps;
      const int off = (int)(w_slot - blk * ps);
      const int64_t head = (blk * Hkv + hk) * (int64_t)ps * D;
      typename HeadPost<DT>::Angles kang;
      if (post.wk) kh.load_gains(post.wk);
      if (post.cos_sin) kang.load(post.cos_sin + (int64_t)w_pos * D);
      bf16x8 kr[KS];
      kh.finish(kang, post.wk != nullptr, post.eps, post.w_offset, post.cos_sin != nullptr, kr);
      if (i16 == 0) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          *(bf16x8*)(post.k_cache + head + k_page_offset(off, ks * 32 + g4 * 8, ps)) = kr[ks];
      }
      if (lane < D / 8) {  // V pages are transposed: the 8 dims of a piece go to 8 rows of keys
        bf16* vd = post.v_cache + head + (int64_t)(lane * 8) * ps + off;
#pragma unroll
        for (int e = 0; e < 8; ++e) vd[(int64_t)e * ps] = vv[e];
      }
    };
    bool stored = false;
    walk([&](int kb, bool last) {
      if (!writer) return;
      if (fetched && !stored) store_key(), stored = true;   // (the loads went out a block ago)
      if (!fetched && kb + 96 >= k_hi) fetch_key();
      if (last) {
        if (!stored) store_key(), stored = true;
        __threadfence_block();
      }
    });
  } else {
    walk([](int, bool) {});
  }
  const float lt = tl.sum_l(0);
  if constexpr (JOIN) {
    __shared__ __attribute__((aligned(16))) float joined[JOIN_SPLITS][16][D + 4];
    if (i16 < G) {
      float* pp = &joined[sp][i16][0];
      if (g4 == 0) {
        pp[0] = tl.m[0] * scale_log2e;  // -inf for an empty part
        pp[1] = lt;
      }
#pragma unroll
      for (int d = 0; d < DT; ++d) *(f32x4*)(pp + 4 + d * 16 + 4 * g4) = tl.o[0][d];
    }
    __syncthreads();
    // out[head, d] = sum_s 2^(m_s - M) o_s / sum_s 2^(m_s - M) l_s, parts in ascending order
    for (int idx = threadIdx.x; idx < G * D; idx += blockDim.x) {
      const int i = idx / D, d = idx - i * D;
      float M = -INFINITY;
      for (int s = 0; s < splits; ++s) M = fmaxf(M, joined[s][i][0]);
      float L = 0.f, acc = 0.f;
      for (int s = 0; s < splits; ++s) {
        const float m = joined[s][i][0];
        const float a = m == -INFINITY ? 0.f : exp2f(m - M);
        if (a > 0.f) {
          L += a * joined[s][i][1];
          acc += a * joined[s][i][4 + d];
        }
      }
      const float inv = L > 0.f ? 1.f / L : 0.f;
      out[(int64_t)row * ld_out + (int64_t)(hk * G + i) * D + d] = (bf16)(acc * inv);
    }
  } else if (i16 < G) {
    float* pp = part + (((int64_t)b * H + hk * G + i16) * splits + sp) * (D + 4);
    if (g4 == 0) {
      pp[0] = tl.m[0] * scale_log2e;  // the tile keeps raw maxima; partials carry base-2 units
      pp[1] = lt;
    }
#pragma unroll
    for (int d = 0; d < DT; ++d) *(f32x4*)(pp + 4 + d * 16 + 4 * g4) = tl.o[0][d];
  }
}

constexpr int MAX_SPLITS = 256;

// out[b, h, :] = sum_s 2^(m_s - M) o_s / sum_s 2^(m_s - M) l_s over the non-empty parts. One wave per (head, request).
// The kernel is a chain of memory round trips and little else, so everything whose address is known at the start
// is asked for at the start: the length, every part's (m, l), and the outputs of the first MERGE_AHEAD parts; which
// parts are empty (they hold anything) is settled afterwards. Head sizes up to 256, up to MAX_SPLITS parts.
constexpr int MERGE_AHEAD = 8;
__global__ void __launch_bounds__(64) attn_decode_merge_kernel(const float* __restrict__ part, bf16* __restrict__ out,
                                                               int64_t ld_out, const int32_t* __restrict__ cu_seqlens,
                                                               const int32_t* __restrict__ seq_lens, int splits,
                                                               int window, int H, int D) {
  __shared__ float wgt[MAX_SPLITS];
  const int h = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
  int row = b;
  if (cu_seqlens) {
    row = cu_seqlens[b];
    if (cu_seqlens[b + 1] - row != 1) return;
  }
  const float* pp = part + ((int64_t)b * H + h) * splits * (D + 4);
  f32x2 ml[MAX_SPLITS / 64];
#pragma unroll
  for (int j = 0; j < MAX_SPLITS / 64; ++j) {
    const int s = lane + 64 * j < splits ? lane + 64 * j : splits - 1;  // clamped, not skipped: no branch around a load
    ml[j] = *(const f32x2*)(pp + (int64_t)s * (D + 4));
  }
  float ahead[MERGE_AHEAD][4];
#pragma unroll
  for (int s = 0; s < MERGE_AHEAD; ++s)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int sc = s < splits ? s : splits - 1, d = lane + 64 * j < D ? lane + 64 * j : D - 1;
      ahead[s][j] = pp[(int64_t)sc * (D + 4) + 4 + d];
    }
  const int seq = seq_lens[b];
  float mloc = -INFINITY;
#pragma unroll
  for (int j = 0; j < MAX_SPLITS / 64; ++j) {
    const int s = lane + 64 * j;
    int k_lo, k_hi, kps;
    split_range(seq, window, splits, s, &k_lo, &k_hi, &kps);
    const float m = s < splits && k_lo < k_hi ? ml[j][0] : -INFINITY;
    ml[j][0] = m;
    mloc = fmaxf(mloc, m);
  }
  const float M = wave_max(mloc);
  float lloc = 0.f;
#pragma unroll
  for (int j = 0; j < MAX_SPLITS / 64; ++j) {
    const int s = lane + 64 * j;
    const float m = ml[j][0];
    const float a = m == -INFINITY ? 0.f : exp2f(m - M);
    if (s < splits) wgt[s] = a;
    lloc += a > 0.f ? a * ml[j][1] : 0.f;
  }
  const float L = wave_sum(lloc);
  __syncthreads();
  const float inv = L > 0.f ? 1.f / L : 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int d = lane + 64 * j;
    if (d >= D) break;
    float acc = 0.f;
#pragma unroll
    for (int s = 0; s < MERGE_AHEAD; ++s) {
      const float a = s < splits ? wgt[s] : 0.f;
      acc += a > 0.f ? a * ahead[s][j] : 0.f;
    }
#pragma unroll 8
    for (int s = MERGE_AHEAD; s < splits; ++s) {
      const float a = wgt[s];
      const float v = pp[(int64_t)s * (D + 4) + 4 + d];  // loads do not wait for the weights
      acc += a > 0.f ? a * v : 0.f;
    }
    out[(int64_t)row * ld_out + (int64_t)h * D + d] = (bf16)(acc * inv);
  }
}

inline bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

template <int DT>
int launch_flash(const bf16* q, int64_t ld_q, bf16* out, int64_t ld_out, const bf16* kc, const bf16* vc,
                 const int32_t* bt, int64_t max_blocks, const int32_t* cu, const int32_t* sl, int num_reqs,
                 int max_q_len, float scale, int window, int H, int Hkv, int ps, int skip_single, hipStream_t stream) {
  const float sl2 = scale * LOG2E;
  const bool p2 = (ps & (ps - 1)) == 0;
  // 32 rows per workgroup where the head size leaves room for two row tiles (registers, and the LDS the
  // waves meet in), and the portions are longer than one tile; otherwise 16
  auto lds_of = [](int qt) { return (size_t)3 * qt * 64 * (sizeof(f32x4) * DT + 2 * sizeof(float)); };
  // 48 rows per workgroup at head size 128: every K and V fragment a wave loads serves three row tiles instead of two
  // (the path on which loads return is what this kernel fills first), at 256 registers, still two waves a SIMD.
  // It pays where the rows still make several rounds of workgroups over the chip (measured, 32 heads: 3,072 rows
  // 135 -> 121 us, 8,192 rows 783 -> 642 us = 34 % of the MFMA peak, 32,768 rows 37 %; 2,048 rows, 1,376 workgroups, level; a portion
  // of 512 rows behind 30,000 keys, 352 workgroups instead of 512, loses 17 %). Head size 64 gains nothing.
  constexpr bool WIDE_OK = DT == 8;
  const int64_t wide_blocks = (int64_t)((max_q_len + 47) / 48) * H * num_reqs;
  if (WIDE_OK && wide_blocks >= 2000) {
    constexpr int QT = WIDE_OK ? 3 : 1;
    const int tiles = (max_q_len + 16 * QT - 1) / (16 * QT);
    if (wide_blocks > 0x7fffffff) return ERR_UNSUPPORTED;
    auto kernel = p2 ? attn_flash_kernel<DT, QT, true> : attn_flash_kernel<DT, QT, false>;
    // (more than the 64 KB of LDS a launch may ask for without saying so)
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_of(QT)) != hipSuccess)
      return ERR_LAUNCH;
    kernel<<<(unsigned)wide_blocks, 256, lds_of(QT), stream>>>(q, ld_q, out, ld_out, kc, vc, bt, max_blocks, cu, sl, tiles,
                                                              sl2, window, H, Hkv, ps, skip_single);
  } else if (DT <= 8 && max_q_len > 16) {
    constexpr int QT = DT <= 8 ? 2 : 1;
    const int tiles = (max_q_len + 16 * QT - 1) / (16 * QT);
    const int64_t blocks = (int64_t)tiles * H * num_reqs;
    if (blocks > 0x7fffffff) return ERR_UNSUPPORTED;
    auto kernel = p2 ? attn_flash_kernel<DT, QT, true> : attn_flash_kernel<DT, QT, false>;
    kernel<<<(unsigned)blocks, 256, lds_of(QT), stream>>>(q, ld_q, out, ld_out, kc, vc, bt, max_blocks, cu, sl, tiles, sl2,
                                                         window, H, Hkv, ps, skip_single);
  } else {
    const int tiles = (max_q_len + 15) / 16;
    const int64_t blocks = (int64_t)tiles * H * num_reqs;
    if (blocks > 0x7fffffff) return ERR_UNSUPPORTED;
    auto kernel = p2 ? attn_flash_kernel<DT, 1, true> : attn_flash_kernel<DT, 1, false>;
    kernel<<<(unsigned)blocks, 256, lds_of(1), stream>>>(q, ld_q, out, ld_out, kc, vc, bt, max_blocks, cu, sl, tiles, sl2,
                                                        window, H, Hkv, ps, skip_single);
  }
  return launch_status();
}

// CUs of the current device (asked once per device).
inline int compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (!cached[dev]) {
    int n = 0;
    cached[dev] = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0 ? n : 256;
  }
  return cached[dev];
}

// The form of the decode kernel for a launch. LATE exists where the new key is the kernel's business and its
// registers allow it (head size 256 would spill).
template <int DT, bool P2, bool JOIN, bool POST>
auto decode_kernel_for(bool late) {
  if constexpr (POST && DT <= 8) {
    if (late) return attn_decode_kernel<DT, P2, true, JOIN, POST>;
  }
  return attn_decode_kernel<DT, P2, false, JOIN, POST>;
}

template <int DT, bool POST>
int launch_decode(const bf16* q, int64_t ld_q, bf16* out, int64_t ld_out, float* part, const bf16* kc, const bf16* vc,
                  const int32_t* bt, int64_t max_blocks, const int32_t* cu, const int32_t* sl, int num_reqs,
                  int splits, float scale, int window, int H, int Hkv, int ps, const DecodePost& post,
                  hipStream_t stream) {
  // many requests (parts of dozens of blocks): the new key is dealt with inside the walk
  const bool p2 = (ps & (ps - 1)) == 0, late = num_reqs >= 32;
  // (one or two requests: measured level at 134 MB a step or behind by 6 %, ahead by 5 to 8 % from 200 MB on)
  const int64_t stream_from = num_reqs <= 2 ? STREAM_FROM_BYTES_FEW : STREAM_FROM_BYTES;
  if constexpr (DT <= 8) {  // (the parts of head size 256 do not fit the LDS of a workgroup)
    // Workgroups of `splits` waves are placed whole: where their number leaves the last round over the CUs thin
    // (320 workgroups on 256 CUs: some CUs get two, most one) single waves spread better and the merge kernel is the
    // lesser cost. Measured at 8 kv heads: 32, 56 and 64 requests gain 0.12 to 0.17 ms a step, 40 and 48 lose.
    const double per_cu = (double)Hkv * num_reqs / compute_units();
    if (splits <= JOIN_SPLITS && (per_cu <= 1. || ceil(per_cu) <= 1.15 * per_cu)) {
      auto kernel = p2 ? decode_kernel_for<DT, true, true, POST>(late) : decode_kernel_for<DT, false, true, POST>(late);
      kernel<<<dim3(1, (unsigned)Hkv, (unsigned)num_reqs), 64 * splits, 0, stream>>>(
          q, ld_q, part, kc, vc, bt, max_blocks, cu, sl, splits, scale * LOG2E, window, H, Hkv, ps, stream_from, out, ld_out,
          post);
      return launch_status();
    }
  }
  auto kernel = p2 ? decode_kernel_for<DT, true, false, POST>(late) : decode_kernel_for<DT, false, false, POST>(late);
  kernel<<<dim3((unsigned)splits, (unsigned)Hkv, (unsigned)num_reqs), 64, 0, stream>>>(
      q, ld_q, part, kc, vc, bt, max_blocks, cu, sl, splits, scale * LOG2E, window, H, Hkv, ps, stream_from,
      (bf16*)nullptr, (int64_t)0, post);
  const int D = DT * 16;
  attn_decode_merge_kernel<<<dim3((unsigned)H, (unsigned)num_reqs), 64, 0, stream>>>(part, out, ld_out, cu, sl, splits,
                                                                                     window, H, D);
  return launch_status();
}

#define DINFER_DISPATCH_HEAD_DIM(head_dim, CALL) \
  switch (head_dim) {                            \
    case 32: { constexpr int DT = 2; CALL; }     \
    case 48: { constexpr int DT = 3; CALL; }     \
    case 64: { constexpr int DT = 4; CALL; }     \
    case 96: { constexpr int DT = 6; CALL; }     \
    case 128: { constexpr int DT = 8; CALL; }    \
    case 256: { constexpr int DT = 16; CALL; }   \
    default: return ERR_UNSUPPORTED;             \
  }

}  // namespace

// 1 if the MFMA kernels take this geometry, else 0 (the caller uses the plain kernel).
extern "C" int dinfer_attn_mfma_supports(int head_dim, int page_size, int heads, int kv_heads) {
  switch (head_dim) {
    case 32: case 48: case 64: case 96: case 128: case 256: break;
    default: return 0;
  }
  if (!(page_size > 0 && page_size % 8 == 0 && kv_heads > 0 && heads % kv_heads == 0)) return 0;
  // the kernels keep the elements of one page (all kv heads) in 32-bit arithmetic
  return (int64_t)kv_heads * page_size * head_dim < (int64_t)1 << 30 ? 1 : 0;
}

// skip_single: requests with one row are left to the split-K kernel.
extern "C" int dinfer_attn_flash(const void* q, int64_t ld_q, void* out, int64_t ld_out, const void* k_cache,
                                 const void* v_cache, const int32_t* block_table, int64_t max_blocks,
                                 const int32_t* cu_seqlens, const int32_t* seq_lens, int num_reqs, int max_q_len,
                                 float scale, int window, int heads, int kv_heads, int head_dim, int page_size,
                                 int skip_single, hipStream_t stream) {
  if (num_reqs <= 0 || max_q_len <= 0) return OK;
  if (!dinfer_attn_mfma_supports(head_dim, page_size, heads, kv_heads)) return ERR_UNSUPPORTED;
  if (window < 0 || max_blocks <= 0 || ld_q % 8 || ld_out % 4 || !aligned16(q) || !aligned16(k_cache) ||
      !aligned16(v_cache) || ((uintptr_t)out % 8))
    return ERR_BAD_SHAPE;
  DINFER_DISPATCH_HEAD_DIM(head_dim, return launch_flash<DT>(
      (const bf16*)q, ld_q, (bf16*)out, ld_out, (const bf16*)k_cache, (const bf16*)v_cache, block_table, max_blocks,
      cu_seqlens, seq_lens, num_reqs, max_q_len, scale, window, heads, kv_heads, page_size, skip_single, stream));
}

// Single-row requests only. cu_seqlens null: every request brings exactly one row (row b belongs to
// request b). cu_seqlens given: requests with one row are served, the others are left alone.
// Each request's visible keys are cut into `splits` (1..256) equal parts, one wave each.
// part: float workspace of num_reqs * heads * splits * (head_dim + 4) elements.
extern "C" int dinfer_attn_decode(const void* q, int64_t ld_q, void* out, int64_t ld_out, float* part,
                                  int64_t part_elems, const void* k_cache, const void* v_cache,
                                  const int32_t* block_table, int64_t max_blocks, const int32_t* cu_seqlens,
                                  const int32_t* seq_lens, int num_reqs, int splits, float scale, int window,
                                  int heads, int kv_heads, int head_dim, int page_size, hipStream_t stream) {
  if (num_reqs <= 0) return OK;
  if (!dinfer_attn_mfma_supports(head_dim, page_size, heads, kv_heads)) return ERR_UNSUPPORTED;
  if (heads / kv_heads > 16) return ERR_UNSUPPORTED;
  if (window < 0 || max_blocks <= 0 || splits <= 0 || splits > MAX_SPLITS || ld_q % 8 || !aligned16(q) ||
      !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(part) || num_reqs > 65535 || kv_heads > 65535)
    return ERR_BAD_SHAPE;
  if ((int64_t)num_reqs * heads * splits * (head_dim + 4) > part_elems) return 5;
  DINFER_DISPATCH_HEAD_DIM(head_dim, return (launch_decode<DT, false>(
      (const bf16*)q, ld_q, (bf16*)out, ld_out, part, (const bf16*)k_cache, (const bf16*)v_cache, block_table,
      max_blocks, cu_seqlens, seq_lens, num_reqs, splits, scale, window, heads, kv_heads, page_size, DecodePost{},
      stream)));
}

// 1 if dinfer_attn_decode_post takes this head size (both elements of a rotated pair must lie in one lane).
extern "C" int dinfer_attn_decode_post_supports(int head_dim) { return head_dim == 64 || head_dim == 128 || head_dim == 256; }

// dinfer_attn_decode for a step in which every request brings exactly one row, with what otherwise runs as a kernel of
// its own before it: q [rows, ld_q], k_new and v_new (rows of the same stride) come as the q|k|v product left them.
// q and k get their per-head RMSNorm (gains q_gain and k_gain of head_dim bf16 elements; null: none) and are
// rotated by the angles of positions[row] (cos_sin [positions, head_dim] float: cos of the head_dim / 2 angles, then
// sin; pairs (i, i + head_dim / 2); null: no rotation); the new key and value go to slot_mapping[row] of the pages
// (null or negative: nowhere; then the pages must already hold them). q, k_new and v_new are left as they were.
extern "C" int dinfer_attn_decode_post(const void* q, const void* k_new, const void* v_new, int64_t ld_q, void* out,
                                       int64_t ld_out, float* part, int64_t part_elems, void* k_cache, void* v_cache,
                                       const int32_t* block_table, int64_t max_blocks, const int32_t* seq_lens,
                                       int num_reqs, int splits, float scale, int window, int heads, int kv_heads,
                                       int head_dim, int page_size, const void* q_gain, const void* k_gain,
                                       float eps, float gain_offset, const int32_t* positions,
                                       const float* cos_sin, const int64_t* slot_mapping, hipStream_t stream) {
  if (num_reqs <= 0) return OK;
  if (!dinfer_attn_mfma_supports(head_dim, page_size, heads, kv_heads) || !dinfer_attn_decode_post_supports(head_dim))
    return ERR_UNSUPPORTED;
  if (heads / kv_heads > 16) return ERR_UNSUPPORTED;
  if (window < 0 || max_blocks <= 0 || splits <= 0 || splits > MAX_SPLITS || ld_q % 8 || !aligned16(q) ||
      !aligned16(k_new) || !aligned16(v_new) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(part) ||
      !aligned16(q_gain) || !aligned16(k_gain) || !aligned16(cos_sin) || num_reqs > 65535 || kv_heads > 65535 ||
      (cos_sin && !positions) || (!q_gain != !k_gain))
    return ERR_BAD_SHAPE;
  if ((int64_t)num_reqs * heads * splits * (head_dim + 4) > part_elems) return 5;
  DecodePost post{(const bf16*)q_gain, (const bf16*)k_gain, eps, gain_offset, positions, cos_sin, slot_mapping,
                  (const bf16*)k_new, (const bf16*)v_new, (bf16*)k_cache, (bf16*)v_cache};
  switch (head_dim) {
    case 64: return launch_decode<4, true>((const bf16*)q, ld_q, (bf16*)out, ld_out, part, (const bf16*)k_cache,
                                           (const bf16*)v_cache, block_table, max_blocks, nullptr, seq_lens, num_reqs,
                                           splits, scale, window, heads, kv_heads, page_size, post, stream);
    case 128: return launch_decode<8, true>((const bf16*)q, ld_q, (bf16*)out, ld_out, part, (const bf16*)k_cache,
                                            (const bf16*)v_cache, block_table, max_blocks, nullptr, seq_lens, num_reqs,
                                            splits, scale, window, heads, kv_heads, page_size, post, stream);
    default: return launch_decode<16, true>((const bf16*)q, ld_q, (bf16*)out, ld_out, part, (const bf16*)k_cache,
                                            (const bf16*)v_cache, block_table, max_blocks, nullptr, seq_lens, num_reqs,
                                            splits, scale, window, heads, kv_heads, page_size, post, stream);
  }
}
