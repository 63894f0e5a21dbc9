// C[M,N] = A[M,K] . W[N,K]^T for few rows (M <= 64), bf16 operands, float
// accumulation, bf16 or float output: the matrix product of decode steps and of
// the LM head, where time is the time to stream W from HBM once.
//
// v_mfma_f32_16x16x32_bf16 with the weight as the A operand: a tile is 16 weight
// rows (n) x 16 tokens (m), contracted over k in steps of 64.
//
// Loads are shaped for the memory path, not for the MFMA: lane l reads the
// 16-byte piece l % 8 of row l / 8, so that eight lanes read one whole 128-byte
// line and an instruction touches 8 lines (with the MFMA's own lane order, one
// row per lane, it touches 64 line-quads and the load-return path of the CU was
// busy 75% of the time, measured). Each wave turns a tile into MFMA order through
// a 2.3 KB strip of LDS of its own (rows padded to 144 bytes: both the writes and
// the reads are free of bank conflicts); a wave's LDS operations complete in
// order, so the strip needs no barrier. Activations go the same way.
//
// The waves of a workgroup take consecutive runs of k of the same rows (split-K
// inside the workgroup). Partial sums meet in LDS and are added in wave order,
// then stored once. No atomics: the result of a given launch shape is reproducible.
//
//   MT = ceil(M / 16) token tiles share every weight fragment (registers),
//   RT weight-row tiles share every activation fragment.
//
// K must be a multiple of 8 (16-byte loads); any M <= 64, any N.
//
// Two more forms take the norm kernels out of a decode layer (a kernel costs 3 to 5 us however small):
//   SINK    the product is added to the residual stream in place (one rounding), and what the next RMSNorm
//           needs leaves with it: the new stream times that norm's gain (XG), and per token and 16 columns (8 in
//           the form whose workgroups take 24 rows) the sum of squares of the new stream (rounded as stored), in float;
//   SCALED  the consumer of those: A is XG, and every token's result is multiplied by
//           rsqrt(sum of its partial sums of squares / width + eps) before it is stored (or gated).
// Together: y = (x g) W^T / rms(x) instead of ((x / rms(x)) g) W^T, the same value rounded at other places.
//
// Reference behaviour: crates/kernels/cuda/gemm_small_m.cu:42-114,148-285
// (weight read once, split-K, M <= 32).
#include <type_traits>

#include "common.cuh"

using namespace dinfer;

namespace {

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
  return z;
}

// Orders a wave's LDS writes before its reads of what other lanes wrote (and the reverse): the hardware
// runs a wave's LDS operations in order, this keeps the compiler from moving them across.
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// 16 bytes of the weight; STREAM: read past the caches (a large weight is read once per launch, and
// whole lines at a time: measured 10% faster from about 40 MB on, slightly slower below)
template <bool STREAM>
__device__ __forceinline__ bf16x8 ld_weight(const bf16* p) {
  if constexpr (STREAM)
    return __builtin_nontemporal_load((const bf16x8*)p);
  else
    return *(const bf16x8*)p;
}

template <class O>
__device__ __forceinline__ void store4(O* p, f32x4 v);
template <>
__device__ __forceinline__ void store4<float>(float* p, f32x4 v) {
  p[0] = v[0]; p[1] = v[1]; p[2] = v[2]; p[3] = v[3];
}
template <>
__device__ __forceinline__ void store4<bf16>(bf16* p, f32x4 v) {
  p[0] = (bf16)v[0]; p[1] = (bf16)v[1]; p[2] = (bf16)v[2]; p[3] = (bf16)v[3];
}


enum : int { PLAIN = 0, SCALED = 1, SINK = 2 };

// LDS of a workgroup: a strip per wave while streaming, then the partial sums of every wave
__host__ __device__ inline size_t lds_core_bytes(int waves, int rt, int mt) {
  const size_t strips = (size_t)waves * 16 * 144, sums = (size_t)waves * rt * mt * 64 * sizeof(f32x4);
  return strips > sums ? strips : sums;
}

// What the SCALED and SINK forms need beside the product's own operands.
struct NormLink {
  const float* stats;  // SCALED: [M][ld_stats] partial sums of squares, `cols` of them a token
  float* stats_out;    // SINK: where this product's partial sums go, one a token and 16 columns (CUT: 8)
  int64_t ld_stats;
  int cols;
  float eps, inv_width;
  bf16* xg;            // SINK: the new stream times the next norm's gain
  int64_t ld_xg;
  const void* gain;    // SINK: that gain, bf16 or float (gain_f32), plus gain_offset
  int gain_f32;
  float gain_offset;
};

// GATED (RT == 2): W is [2N, K], rows [0, N) the gate and [N, 2N) the up projection; the workgroup's
// two row tiles are gate rows n0.. and up rows N + n0.., and the epilogue stores
// silu(gate) * up into C [M, N]: the activation costs no pass of its own.
// CUT (not GATED): the last 8 rows of the workgroup's last tile are left out, so a workgroup takes
// 16 RT - 8 weight rows: with two tiles 24 rows, which makes 256 workgroups of N = 6,144 where 32 rows make 192.
// The waves a SIMD that a form is to keep room for (its registers are held to that): the form of one token tile and
// two row tiles that is no producer of a carried norm (the gate/up pair, q/k/v, the LM head) runs with workgroups of
// 4 or 8 waves, six workgroups of 4 on a CU, and loses a tenth of its rate at five (measured when two more registers
// cost it the sixth). The other forms take what they need.
constexpr int waves_a_simd(int mt, int rt, int mode, bool cut) { return mt == 1 && rt == 2 && mode != SINK && !cut ? 6 : 1; }

template <int MT, int RT, class O, bool GATED, bool STREAM, int MODE = PLAIN, bool CUT = false>
__global__ void __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(waves_a_simd(MT, RT, MODE, CUT), 8))) gemm_small_m_kernel(const bf16* __restrict__ A, int64_t lda,
                                                            const bf16* __restrict__ W, int64_t ldw,
                                                            O* __restrict__ C, int64_t ldc, int M, int N, int K,
                                                            NormLink link = NormLink{}) {
  static_assert(!GATED || RT == 2, "the gated form pairs one gate tile with one up tile");
  static_assert(!CUT || !GATED, "the gated form pairs whole tiles");
  constexpr int ROWS = 16 * RT - (CUT ? 8 : 0);  // weight rows of a workgroup (not GATED)
  // 64-wide k steps in flight per wave: as many as the register file takes at 16 waves a workgroup
  constexpr int UNROLL = RT == 3 ? (MT == 1 ? 2 : 1) : MT <= 2 ? (4 / RT > 0 ? 4 / RT : 1) : (2 / RT > 0 ? 2 / RT : 1);
  constexpr int ROW_BYTES = 144;              // 64 k of a row and 16 bytes of padding
  constexpr int STRIP_BYTES = 16 * ROW_BYTES;  // one tile of 16 rows
  extern __shared__ __attribute__((aligned(16))) char smem[];  // a strip per wave; afterwards [waves][RT * MT][64 lanes][4] sums
  float* red = (float*)smem;
  const int nw = blockDim.x >> 6;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, i16 = lane & 15, g4 = lane >> 4;
  const int lrow = lane >> 3, lpiece = lane & 7;  // what this lane loads: piece lpiece of rows lrow and lrow + 8
  const int n0 = GATED ? blockIdx.x * 16 : blockIdx.x * ROWS;
  const int n_end = GATED ? N : (n0 + ROWS < N ? n0 + ROWS : N);  // rows from here on are not this workgroup's
  char* strip = smem + wave * STRIP_BYTES;
  char* put = strip + lrow * ROW_BYTES + lpiece * 16;  // where this lane's loads go (rows lrow, + 8)
  const char* get = strip + i16 * ROW_BYTES + g4 * 16;  // its MFMA operands: row i16, pieces g4 and 4 + g4

  const bf16* wp[RT][2];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      int n = (GATED ? n0 : n0 + r * 16) + lrow + 8 * h;
      if (n >= N) n = N - 1;  // rows past the end are computed and dropped
      if (GATED && r == 1) n += N;
      wp[r][h] = W + (int64_t)n * ldw + 8 * lpiece;
    }
  const bf16* ap[MT][2];
  bool arow[MT][2];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int m = t * 16 + lrow + 8 * h;
      arow[t][h] = m < M;
      ap[t][h] = A + (int64_t)(arow[t][h] ? m : 0) * lda + 8 * lpiece;
    }
  f32x4 acc[RT][MT];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // SINK: what the epilogue adds to and multiplies by is fetched now, where the latency hides behind the first
  // weights (for the first slot a thread sums; a workgroup with fewer threads than slots fetches the rest when it
  // gets there)
  float res0[4] = {0.f, 0.f, 0.f, 0.f}, gain0[4] = {0.f, 0.f, 0.f, 0.f};
  if constexpr (MODE == SINK) {
    const int x = threadIdx.x;
    if (x < RT * MT * 64) {
      const int tile = x >> 6, ln = x & 63;
      const int m = (tile % MT) * 16 + (ln & 15), n = n0 + (tile / MT) * 16 + 4 * (ln >> 4);
      if (m < M) {
        const bf16* hp = (const bf16*)C + (int64_t)m * ldc + n;
        for (int e = 0; e < 4 && n + e < n_end; ++e) {
          res0[e] = (float)hp[e];
          gain0[e] = (link.gain_f32 ? ((const float*)link.gain)[n + e] : (float)((const bf16*)link.gain)[n + e]) +
                     link.gain_offset;
        }
      }
    }
  }

  // k steps of 64; wave w takes a contiguous run of them, so its loads walk each row in long pieces
  const int steps = (K + 63) / 64;
  const int per_wave = (steps + nw - 1) / nw;
  const int s_begin = wave * per_wave;
  const int s_end = s_begin + per_wave < steps ? s_begin + per_wave : steps;
  // One round: the loads of UNROLL steps, then their MFMAs. `masked` is a type: the rounds that lie wholly inside the
  // wave's run and inside k load without a condition, so that the compiler issues them in one go and lets the first
  // MFMAs start when the first loads are back (under a condition every load is a branch of its own, and the first use
  // of any waits for all of them: measured 0.3 to 1.3 us a product at the 8B sizes); the last round of a run that
  // does not divide evenly asks. (Rows of A past M are then copies of row 0, computed and dropped like weight rows
  // past N.)
  auto round = [&](int s0, auto masked) {
    constexpr bool MASKED = decltype(masked)::value;
    bf16x8 wraw[UNROLL][RT][2], araw[UNROLL][MT][2];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int kk = (s0 + u) * 64;
      const bool ok = !MASKED || (kk + 8 * lpiece < K && (s0 + u) < s_end);
#pragma unroll
      for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          if (CUT && r == RT - 1 && h == 1)
            wraw[u][r][h] = zero8();
          else if constexpr (MASKED)
            wraw[u][r][h] = ok ? ld_weight<STREAM>(wp[r][h] + kk) : zero8();
          else
            wraw[u][r][h] = ld_weight<STREAM>(wp[r][h] + kk);
        }
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          if constexpr (MASKED)
            araw[u][t][h] = (ok && arow[t][h]) ? *(const bf16x8*)(ap[t][h] + kk) : zero8();
          else
            araw[u][t][h] = *(const bf16x8*)(ap[t][h] + kk);
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      // through the strip, tile by tile: what every lane loaded goes in by rows, the MFMA operands come out
      bf16x8 af[MT][2];
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        *(bf16x8*)put = araw[u][t][0];
        *(bf16x8*)(put + 8 * ROW_BYTES) = araw[u][t][1];
        wave_sync();
        af[t][0] = *(const bf16x8*)get;
        af[t][1] = *(const bf16x8*)(get + 64);
        wave_sync();
      }
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        *(bf16x8*)put = wraw[u][r][0];
        *(bf16x8*)(put + 8 * ROW_BYTES) = wraw[u][r][1];
        wave_sync();
        const bf16x8 wf0 = *(const bf16x8*)get, wf1 = *(const bf16x8*)(get + 64);
        wave_sync();
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf0, af[t][0], acc[r][t], 0, 0, 0);
          acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf1, af[t][1], acc[r][t], 0, 0, 0);
        }
      }
    }
  };
  // whole steps of k end at K / 64; the rounds before `plain_end` touch nothing else
  const int whole = K / 64 < s_end ? K / 64 : s_end;
  const int plain_end = whole > s_begin ? s_begin + (whole - s_begin) / UNROLL * UNROLL : s_begin;
  int s0 = s_begin;
  for (; s0 < plain_end; s0 += UNROLL) round(s0, std::false_type{});
  for (; s0 < s_end; s0 += UNROLL) round(s0, std::true_type{});
  // SCALED: every token's 1 / rms from the producer's partial sums, added in a fixed order; kept behind the
  // strips and the sums (the launch sizes LDS for it)
  float* rs = (float*)(smem + lds_core_bytes(nw, RT, MT));
  if constexpr (MODE == SCALED) {
    for (int m = wave; m < M; m += nw) {
      float a = 0.f;
      for (int j = lane; j < link.cols; j += 64) a += link.stats[(int64_t)m * link.ld_stats + j];
      a = wave_sum(a);
      if (lane == 0) rs[m] = rsqrtf(a * link.inv_width + link.eps);
    }
  }
  __syncthreads();  // the strips are done with: the same memory now takes the sums

  // partial sums of the waves meet in LDS
  f32x4* slot = (f32x4*)red + ((int64_t)wave * RT * MT) * 64 + lane;
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int t = 0; t < MT; ++t) slot[(r * MT + t) * 64] = acc[r][t];
  __syncthreads();
  // thread x sums slot x of every wave, in wave order; slot = (tile, lane): 4 consecutive n of one token
  for (int x = threadIdx.x; x < (GATED ? 1 : RT) * MT * 64; x += blockDim.x) {
    f32x4 s = ((const f32x4*)red)[x];
    for (int w = 1; w < nw; ++w) {
      const f32x4 v = ((const f32x4*)red)[(int64_t)w * RT * MT * 64 + x];
      s[0] += v[0]; s[1] += v[1]; s[2] += v[2]; s[3] += v[3];
    }
    const int tile = x >> 6, ln = x & 63;
    const int r = tile / MT, t = tile % MT;
    const int m = t * 16 + (ln & 15);
    const int n = n0 + r * 16 + 4 * (ln >> 4);
    float scale = 1.f;
    if constexpr (MODE == SCALED) scale = m < M ? rs[m] : 0.f;
    if (GATED) {  // slot x of the up tile lies MT * 64 slots further on
      f32x4 u = ((const f32x4*)red)[MT * 64 + x];
      for (int w = 1; w < nw; ++w) {
        const f32x4 v = ((const f32x4*)red)[(int64_t)w * RT * MT * 64 + MT * 64 + x];
        u[0] += v[0]; u[1] += v[1]; u[2] += v[2]; u[3] += v[3];
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float g = s[e] * scale;
        s[e] = (g / (1.f + expf(-g))) * (u[e] * scale);
      }
    } else if constexpr (MODE == SCALED) {
#pragma unroll
      for (int e = 0; e < 4; ++e) s[e] *= scale;
    }
    if constexpr (MODE == SINK) {
      // C is the residual stream: read, added to, rounded once, written back; the same lanes feed the next norm
      float ss = 0.f;
      if (m < M) {
        bf16* hp = (bf16*)C + (int64_t)m * ldc + n;
        bf16* xp = link.xg + (int64_t)m * link.ld_xg + n;
        const bool first = x == (int)threadIdx.x;
        bf16x4 hv, xv;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float res = res0[e], g = gain0[e];
          if (!first && n + e < n_end) {
            res = (float)hp[e];
            g = (link.gain_f32 ? ((const float*)link.gain)[n + e] : (float)((const bf16*)link.gain)[n + e]) + link.gain_offset;
          }
          const bf16 h = (bf16)(res + s[e]);
          const float hf = n + e < n_end ? (float)h : 0.f;
          hv[e] = h;
          ss += hf * hf;
          xv[e] = (bf16)(hf * g);
        }
        if (n + 3 < n_end && ((ldc | link.ld_xg) & 3) == 0 && (((uintptr_t)C | (uintptr_t)link.xg) & 7) == 0) {
          *(bf16x4*)hp = hv;  // four columns as one 8-byte store
          *(bf16x4*)xp = xv;
        } else {
          for (int e = 0; e < 4 && n + e < n_end; ++e) hp[e] = hv[e], xp[e] = xv[e];
        }
      }
      if constexpr (CUT) {
        // 8 columns of a token lie in the two lanes ln and ln + 16 (n0 is a multiple of 8, so they share n / 8)
        ss += __shfl_xor(ss, 16, 64);
        if (((ln >> 4) & 1) == 0 && m < M && n < n_end) link.stats_out[(int64_t)m * link.ld_stats + (n >> 3)] = ss;
      } else {
        // the tile's 16 columns of a token lie in the four lanes ln, ln + 16, + 32, + 48
        ss += __shfl_xor(ss, 16, 64);
        ss += __shfl_xor(ss, 32, 64);
        if ((ln >> 4) == 0 && m < M && n0 + r * 16 < N) link.stats_out[(int64_t)m * link.ld_stats + (n0 >> 4) + r] = ss;
      }
    } else if (m < M) {
      O* cp = C + (int64_t)m * ldc + n;
      if (n + 3 < n_end) {
        store4<O>(cp, s);
      } else {
        for (int e = 0; e < 4 && n + e < n_end; ++e) cp[e] = from_f32<O>(s[e]);
      }
    }
  }
}

inline bool streams_weight(int64_t rows, int64_t K) { return rows * K * (int64_t)sizeof(bf16) >= (int64_t)40 << 20; }

inline size_t lds_bytes(int waves, int rt, int mt) { return lds_core_bytes(waves, rt, mt); }
constexpr size_t RS_BYTES = 64 * sizeof(float);  // SCALED: a token's 1 / rms, behind the rest

// Two row tiles a workgroup leave CUs without work (fewer than 256 workgroups) where 24 rows a workgroup would not
// (measured on weights taken in turn, K = 4,096: N = 6,144 in 256 workgroups 12.4 us at 8 tokens, N = 6,176 in 193
// workgroups of 32 rows 13.2; 11.5 against 12.2 at one token, 13.7 against 15.0 at 16).
inline bool cut_pays(int N) { return N / 32 < 256 && (N + 23) / 24 <= 256; }
// Likewise 40 rows a workgroup (three tiles, the last 8 rows left out; 8 waves with two k steps of loads in flight
// each) where 32 rows give 257 to 511 workgroups, some CUs two and most one, and 40 give 256 or fewer: N = 10,240,
// K = 5,120 at 8 tokens 26.6 -> 21.2 us (with one k step in flight and 4 waves: 31.1).
inline bool wide_cut_pays(int N) { return (N + 31) / 32 > 256 && (N + 39) / 40 <= 256; }

// And 8 rows a workgroup (one tile less 8 rows) for a weight of so few rows that 16 a workgroup leave half the CUs
// and more without work (1,024 rows: 64 workgroups).
inline bool narrow_cut_pays(int N) { return (N + 15) / 16 <= 128; }

// One launch of the kernel in the form <MT, RT, O, GATED, ., MODE, CUT>, reading the weight past the caches where
// it is large.
template <int MT, int RT, class O, bool GATED, int MODE, bool CUT>
int go(unsigned blocks, int waves, size_t lds, hipStream_t stream, const bf16* A, int64_t lda, const bf16* W, int64_t ldw,
       O* C, int64_t ldc, int M, int N, int K, const NormLink& link = NormLink{}) {
  if (streams_weight(GATED ? 2 * (int64_t)N : N, K))
    gemm_small_m_kernel<MT, RT, O, GATED, true, MODE, CUT><<<blocks, waves * 64, lds, stream>>>(A, lda, W, ldw, C, ldc, M, N, K, link);
  else
    gemm_small_m_kernel<MT, RT, O, GATED, false, MODE, CUT><<<blocks, waves * 64, lds, stream>>>(A, lda, W, ldw, C, ldc, M, N, K, link);
  return launch_status();
}

template <int MT, int RT, class O>
int launch(const bf16* A, int64_t lda, const bf16* W, int64_t ldw, O* C, int64_t ldc, int M, int N, int K, int waves,
           hipStream_t stream) {
  const size_t lds = lds_bytes(waves, RT, MT);
  if constexpr (RT == 1 && MT <= 2 && sizeof(O) == sizeof(bf16)) {
    if (narrow_cut_pays(N))
      return go<MT, RT, O, false, PLAIN, true>((unsigned)((N + 7) / 8), waves, lds, stream, A, lda, W, ldw, C, ldc, M, N, K);
  }
  if constexpr (RT == 2 && MT <= 2 && sizeof(O) == sizeof(bf16)) {
    if (cut_pays(N))
      return go<MT, RT, O, false, PLAIN, true>((unsigned)((N + 23) / 24), waves, lds, stream, A, lda, W, ldw, C, ldc, M, N, K);
  }
  return go<MT, RT, O, false, PLAIN, false>((unsigned)((N + 16 * RT - 1) / (16 * RT)), waves, lds, stream, A, lda, W, ldw, C,
                                            ldc, M, N, K);
}

template <int MT>
int launch_gated(const bf16* A, int64_t lda, const bf16* W, int64_t ldw, bf16* C, int64_t ldc, int M, int N, int K,
                 int waves, hipStream_t stream) {
  return go<MT, 2, bf16, true, PLAIN, false>((unsigned)((N + 15) / 16), waves, lds_bytes(waves, 2, MT), stream, A, lda, W, ldw,
                                             C, ldc, M, N, K);
}

template <class O>
int dispatch(const bf16* A, int64_t lda, const bf16* W, int64_t ldw, O* C, int64_t ldc, int M, int N, int K, int rt,
             int waves, hipStream_t stream) {
  const int mt = (M + 15) / 16;
#define GO(MT_, RT_) return launch<MT_, RT_, O>(A, lda, W, ldw, C, ldc, M, N, K, waves, stream)
  if (mt == 1) { if (rt == 1) GO(1, 1); if (rt == 2) GO(1, 2); if (rt == 4) GO(1, 4); }
  if (mt == 2) { if (rt == 1) GO(2, 1); if (rt == 2) GO(2, 2); if (rt == 4) GO(2, 4); }
  if (mt == 3) { if (rt == 1) GO(3, 1); if (rt == 2) GO(3, 2); }
  if (mt == 4) { if (rt == 1) GO(4, 1); if (rt == 2) GO(4, 2); }
#undef GO
  return ERR_UNSUPPORTED;
}

// The SCALED and SINK forms: up to 32 rows, bf16 out, one or two row tiles.
template <int MT, int RT, int MODE>
int launch_linked(const bf16* A, int64_t lda, const bf16* W, int64_t ldw, bf16* C, int64_t ldc, int M, int N, int K,
                  int waves, const NormLink& link, hipStream_t stream) {
  const size_t lds = lds_bytes(waves, RT, MT) + RS_BYTES;
  if constexpr (RT == 2 && MT == 1 && MODE == SCALED) {
    if (wide_cut_pays(N))  // three tiles less 8 rows, 8 waves
      return go<MT, 3, bf16, false, MODE, true>((unsigned)((N + 39) / 40), 8, lds_bytes(8, 3, MT) + RS_BYTES, stream, A, lda, W,
                                                ldw, C, ldc, M, N, K, link);
  }
  if constexpr (RT == 1 && MT == 1) {
    if (narrow_cut_pays(N))
      return go<MT, RT, bf16, false, MODE, true>((unsigned)((N + 7) / 8), waves, lds, stream, A, lda, W, ldw, C, ldc, M, N, K, link);
  }
  if constexpr (RT == 2 && MT == 1) {
    if (cut_pays(N))
      return go<MT, RT, bf16, false, MODE, true>((unsigned)((N + 23) / 24), waves, lds, stream, A, lda, W, ldw, C, ldc, M, N, K, link);
  }
  return go<MT, RT, bf16, false, MODE, false>((unsigned)((N + 16 * RT - 1) / (16 * RT)), waves, lds, stream, A, lda, W, ldw, C,
                                              ldc, M, N, K, link);
}

template <int MODE>
int dispatch_linked(const bf16* A, int64_t lda, const bf16* W, int64_t ldw, bf16* C, int64_t ldc, int M, int N, int K,
                    int rt, int waves, const NormLink& link, hipStream_t stream) {
  const int mt = (M + 15) / 16;
#define GO(MT_, RT_) return launch_linked<MT_, RT_, MODE>(A, lda, W, ldw, C, ldc, M, N, K, waves, link, stream)
  if (mt == 1) { if (rt == 1) GO(1, 1); if (rt == 2) GO(1, 2); }
  if (mt == 2) { if (rt == 1) GO(2, 1); if (rt == 2) GO(2, 2); }
#undef GO
  return ERR_UNSUPPORTED;
}

template <int MT>
int launch_gated_scaled(const bf16* A, int64_t lda, const bf16* W, int64_t ldw, bf16* C, int64_t ldc, int M, int N, int K,
                        int waves, const NormLink& link, hipStream_t stream) {
  return go<MT, 2, bf16, true, SCALED, false>((unsigned)((N + 15) / 16), waves, lds_bytes(waves, 2, MT) + RS_BYTES, stream, A,
                                              lda, W, ldw, C, ldc, M, N, K, link);
}

// Row tiles a workgroup (16 weight rows each) for up to 16 tokens. Measured inside whole decode steps on MI355X (256
// CUs): with one row tile there is one workgroup per 16 columns, and from 257 to 511 of them the CUs are loaded
// unevenly (320 workgroups: a quarter of the CUs get two); half as many workgroups of twice the work finish no later
// and each wave keeps more loads in flight. N = 5,120: 14B-sized steps 6.93 -> 6.60 ms at 8 tokens, 6.35 -> 5.91 at one;
// N = 6,144 (K = 4,096): 3.93 -> 3.88 ms. At N = 4,096 (256 workgroups, one a CU) two row tiles lose (4.00 ms). From
// N = 8,192 on, two row tiles when there are more than a few tokens (measured on the kernel alone).
inline int few_rows_row_tiles(int64_t M, int64_t N) {
  if (N > 4096 && N < 8192) return 2;
  return N >= 8192 && M > 4 ? 2 : 1;
}

// Waves of a workgroup (they share K): 8, or 4 with two row tiles of a wide weight; 16 for a small square weight with
// one workgroup a CU, where 8 waves a CU keep too few loads in flight (N = K = 4,096: 3.93 -> 3.90 ms a step; with
// K = 12,288 or N = 5,120 sixteen lose). Every wave gets at least four k steps (K = 1,024: 4 waves, measured).
inline int few_rows_waves(int mt, int rt, int64_t N, int64_t K) {
  int nw = (rt == 1 || N < 8192) ? 8 : 4;
  if (mt == 1 && rt == 1 && N <= 4096 && K <= 4096) nw = 16;
  const int64_t steps = (K + 63) / 64;
  while (nw > 1 && steps < 4 * nw) nw /= 2;
  return nw;
}

// Row tiles and waves of a launch, as dinfer_gemm_small_m chooses them (at most two row tiles here).
// scaled: the launch is the consumer of a carried norm, which has a form of 40 rows a workgroup (launched from the
// two-tile case).
inline void shape_for(int64_t M, int64_t N, int64_t K, int* rt_out, int* nw_out, bool scaled = false) {
  const int mt = (int)(M + 15) / 16;
  int rt = mt >= 2 ? ((N >= 6144 || streams_weight(N, K)) ? 2 : 1) : few_rows_row_tiles(M, N);
  if (scaled && mt == 1 && wide_cut_pays((int)N)) rt = 2;
  int nw = few_rows_waves(mt, rt, N, K);
  while (nw > 1 && lds_bytes(nw, rt, mt) + RS_BYTES > 64 * 1024) nw /= 2;
  *rt_out = rt, *nw_out = nw;
}

inline bool linked_operands_ok(const void* A, int64_t lda, const void* W, int64_t ldw, int64_t ldc, int64_t M, int64_t N,
                               int64_t K) {
  return M > 0 && M <= 32 && N > 0 && K > 0 && K % 8 == 0 && lda >= K && ldw >= K && ldc >= N && lda % 8 == 0 &&
         ldw % 8 == 0 && N <= 0x3fffffff && K <= 0x7fffffff && !((uintptr_t)A % 16) && !((uintptr_t)W % 16);
}

}  // namespace

// row_tiles_per_block (1, 2 or 4; at most 2 for M > 32) and waves (1..16) shape the launch;
// 0 lets the library choose from the sizes.
extern "C" int dinfer_gemm_small_m(int out_f32, const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                                   int64_t ldc, int64_t M, int64_t N, int64_t K, int row_tiles_per_block, int waves,
                                   hipStream_t stream) {
  if (M <= 0 || N <= 0) return OK;
  if (M > 64) return ERR_UNSUPPORTED;
  if (K <= 0 || K % 8 || lda < K || ldw < K || ldc < N || lda % 8 || ldw % 8 || N > 0x7fffffff || K > 0x7fffffff ||
      ((uintptr_t)A % 16) || ((uintptr_t)W % 16))
    return ERR_BAD_SHAPE;
  const int mt = (int)(M + 15) / 16;
  int rt = row_tiles_per_block, nw = waves;
  // measured on MI355X (K = 4096 and 12288, N from 4096 to 151936): one row tile and 8 waves a workgroup,
  // two row tiles and 4 waves from N = 8192 on when there are more than a few tokens; with two token tiles
  // and more, two row tiles from N = 6144 on and for every weight large enough to be read past the caches
  // (32 tokens: N = K = 4096 9.1 us with one row tile, 11.2 with two; N = K = 5120 24.0 with one, 18.3 with
  // two); four row tiles for a vocabulary-sized N at 17 to 32 tokens
  if (rt == 0)
    rt = mt >= 2 ? ((mt == 2 && N >= 65536) ? 4 : ((N >= 6144 || streams_weight(N, K)) ? 2 : 1)) : few_rows_row_tiles(M, N);
  if (nw == 0) nw = few_rows_waves(mt, rt, N, K);
  while (nw > 1 && lds_bytes(nw, rt, mt) > 64 * 1024) nw /= 2;
  if (nw < 1 || nw > 16) return ERR_BAD_SHAPE;
  if (lds_bytes(nw, rt, mt) > 64 * 1024) return ERR_UNSUPPORTED;
  if (out_f32)
    return dispatch<float>((const bf16*)A, lda, (const bf16*)W, ldw, (float*)C, ldc, (int)M, (int)N, (int)K, rt, nw,
                           stream);
  return dispatch<bf16>((const bf16*)A, lda, (const bf16*)W, ldw, (bf16*)C, ldc, (int)M, (int)N, (int)K, rt, nw,
                        stream);
}


// out[:M] = silu(A . Wg^T) * (A . Wu^T) with W = [Wg; Wu] stacked [2N, K], M <= 32, bf16 in and out:
// the two projections of a gated feed-forward and its activation in one weight-streaming kernel.
extern "C" int dinfer_gemm_small_m_gated(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc,
                                         int64_t M, int64_t N, int64_t K, int waves, hipStream_t stream) {
  if (M <= 0 || N <= 0) return OK;
  if (M > 32) return ERR_UNSUPPORTED;
  if (K <= 0 || K % 8 || lda < K || ldw < K || ldc < N || lda % 8 || ldw % 8 || N > 0x3fffffff || K > 0x7fffffff ||
      ((uintptr_t)A % 16) || ((uintptr_t)W % 16))
    return ERR_BAD_SHAPE;
  const int mt = (int)(M + 15) / 16;
  int nw = waves;
  if (nw == 0) {
    const int64_t tiles = (N + 15) / 16;
    nw = 4;
    while (nw < 16 && tiles * nw < 768) nw *= 2;
    const int64_t steps = (K + 63) / 64;
    while (nw > 1 && steps < 2 * nw) nw /= 2;
  }
  if (nw < 1 || nw > 16 || lds_bytes(nw, 2, mt) > 64 * 1024) return ERR_BAD_SHAPE;
  if (mt == 1)
    return launch_gated<1>((const bf16*)A, lda, (const bf16*)W, ldw, (bf16*)C, ldc, (int)M, (int)N, (int)K, nw, stream);
  return launch_gated<2>((const bf16*)A, lda, (const bf16*)W, ldw, (bf16*)C, ldc, (int)M, (int)N, (int)K, nw, stream);
}


// C[:M] = (A . W^T) scaled per row by rsqrt(sum(stats[m][0..cols)) / width + eps): A is the residual stream times the
// gain of an RMSNorm (dinfer_gemm_small_m_sink wrote both it and stats), so C is W applied to the normed stream.
// gated: W = [gate; up] stacked [2N, K] and C[M,N] = silu(scaled gate) * scaled up. M <= 32, bf16 in and out.
extern "C" int dinfer_gemm_small_m_scaled(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc,
                                          int64_t M, int64_t N, int64_t K, int gated, const float* stats, int64_t ld_stats,
                                          int64_t cols, float eps, int64_t width, hipStream_t stream) {
  if (M <= 0 || N <= 0) return OK;
  if (M > 32) return ERR_UNSUPPORTED;
  if (!linked_operands_ok(A, lda, W, ldw, ldc, M, N, K) || !stats || cols <= 0 || cols > ld_stats || width <= 0 ||
      cols > 0x7fffffff)
    return ERR_BAD_SHAPE;
  NormLink link{};
  link.stats = stats, link.ld_stats = ld_stats, link.cols = (int)cols, link.eps = eps, link.inv_width = 1.f / (float)width;
  const int mt = (int)(M + 15) / 16;
  if (gated) {
    const int64_t tiles = (N + 15) / 16;
    // up to 16 tokens: 8 waves, measured inside whole decode steps (8B sizes 3.86 -> 3.83 ms a step of 8 tokens, 14B 6.60
    // -> 6.52, 32B 13.82 -> 13.63; 2 or 16 waves lose 0.1 to 0.4 ms)
    int nw = mt == 1 ? 8 : 4;
    while (nw < 16 && tiles * nw < 768) nw *= 2;
    const int64_t steps = (K + 63) / 64;
    while (nw > 1 && steps < 2 * nw) nw /= 2;
    while (nw > 1 && lds_bytes(nw, 2, mt) + RS_BYTES > 64 * 1024) nw /= 2;
    if (mt == 1)
      return launch_gated_scaled<1>((const bf16*)A, lda, (const bf16*)W, ldw, (bf16*)C, ldc, (int)M, (int)N, (int)K, nw, link, stream);
    return launch_gated_scaled<2>((const bf16*)A, lda, (const bf16*)W, ldw, (bf16*)C, ldc, (int)M, (int)N, (int)K, nw, link, stream);
  }
  int rt, nw;
  shape_for(M, N, K, &rt, &nw, true);
  return dispatch_linked<SCALED>((const bf16*)A, lda, (const bf16*)W, ldw, (bf16*)C, ldc, (int)M, (int)N, (int)K, rt, nw, link,
                                 stream);
}

// H[:M] += A . W^T in place (H bf16, the residual stream; summed in float, rounded once), and for the RMSNorm that
// reads H next: XG[:M] = H * (gain + gain_offset), and stats[m][j] = sum of squares of H[m] over columns g j .. g j + g - 1
// with g = 16, or 8 for the sizes dinfer_gemm_small_m_sink_stats_columns says so; ceil(N / g) of them a token. M <= 32.
extern "C" int dinfer_gemm_small_m_sink_stats_columns(int64_t M, int64_t N, int64_t K) {
  int rt, nw;
  shape_for(M, N, K, &rt, &nw);
  return M <= 16 && ((rt == 2 && cut_pays((int)N)) || (rt == 1 && narrow_cut_pays((int)N))) ? 8 : 16;
}

extern "C" int dinfer_gemm_small_m_sink(const void* A, int64_t lda, const void* W, int64_t ldw, void* H, int64_t ldh, void* XG,
                                        int64_t ld_xg, const void* gain, int gain_f32, float gain_offset, float* stats,
                                        int64_t ld_stats, int64_t M, int64_t N, int64_t K, hipStream_t stream) {
  if (M <= 0 || N <= 0) return OK;
  if (M > 32) return ERR_UNSUPPORTED;
  if (!linked_operands_ok(A, lda, W, ldw, ldh, M, N, K) || !H || !XG || !gain || !stats || ld_xg < N)
    return ERR_BAD_SHAPE;
  const int64_t g = dinfer_gemm_small_m_sink_stats_columns(M, N, K);
  if (ld_stats < (N + g - 1) / g) return ERR_BAD_SHAPE;
  NormLink link{};
  link.stats_out = stats, link.ld_stats = ld_stats, link.xg = (bf16*)XG, link.ld_xg = ld_xg, link.gain = gain;
  link.gain_f32 = gain_f32, link.gain_offset = gain_offset;
  int rt, nw;
  shape_for(M, N, K, &rt, &nw);
  return dispatch_linked<SINK>((const bf16*)A, lda, (const bf16*)W, ldw, (bf16*)H, ldh, (int)M, (int)N, (int)K, rt, nw, link,
                               stream);
}
