// C[M,N] = A[M,K] . W[N,K]^T for few rows (M <= 64), bf16 operands, float
// accumulation, bf16 or float output: the matrix product of decode steps and of
// the LM head, where time is the time to stream W from HBM once.
//
// v_mfma_f32_16x16x32_bf16 with the weight as the A operand: a tile is 16 weight
// rows (n) x 16 tokens (m), contracted over k. Lane l = (i = l % 16, g = l / 16)
// loads 32 contiguous bytes W[n0 + i][kk + 16 g .. + 16] and feeds them to two
// MFMAs; the activations are loaded with the same k mapping, so a wave reads
// 128 contiguous bytes of each of its 16 rows per step, and the waves of a
// workgroup take consecutive runs of k of the same rows (split-K inside the
// workgroup). Partial sums meet in LDS and are added in wave order, then stored
// once. No atomics: the result of a given launch shape is reproducible.
//
//   MT = ceil(M / 16) token tiles share every weight fragment (registers),
//   RT weight-row tiles share every activation fragment.
//
// K must be a multiple of 8 (16-byte loads); any M <= 64, any N.
//
// Reference behaviour: crates/kernels/cuda/gemm_small_m.cu:42-114,148-285
// (weight read once, split-K, M <= 32).
#include "common.cuh"

using namespace dinfer;

namespace {

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
  return z;
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


// GATED (RT == 2): W is [2N, K], rows [0, N) the gate and [N, 2N) the up projection; the workgroup's
// two row tiles are gate rows n0.. and up rows N + n0.., and the epilogue stores
// silu(gate) * up into C [M, N]: the activation costs no pass of its own.
template <int MT, int RT, class O, bool GATED = false>
__global__ void __launch_bounds__(1024) gemm_small_m_kernel(const bf16* __restrict__ A, int64_t lda,
                                                            const bf16* __restrict__ W, int64_t ldw,
                                                            O* __restrict__ C, int64_t ldc, int M, int N, int K) {
  static_assert(!GATED || RT == 2, "the gated form pairs one gate tile with one up tile");
  // 64-wide k steps in flight per wave: as many as the register file takes at 16 waves a workgroup
  constexpr int UNROLL = MT <= 2 ? (4 / RT > 0 ? 4 / RT : 1) : (2 / RT > 0 ? 2 / RT : 1);
  extern __shared__ float red[];  // [waves][RT * MT][64 lanes][4]
  const int nw = blockDim.x >> 6;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, i16 = lane & 15, g4 = lane >> 4;
  const int n0 = GATED ? blockIdx.x * 16 : blockIdx.x * 16 * RT;

  const bf16* wp[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    int n = GATED ? n0 + i16 : n0 + r * 16 + i16;
    if (n >= N) n = N - 1;  // rows past the end are computed and dropped
    if (GATED && r == 1) n += N;
    wp[r] = W + (int64_t)n * ldw + 16 * g4;
  }
  const bf16* ap[MT];
  bool arow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + i16;
    arow[t] = m < M;
    ap[t] = A + (int64_t)(arow[t] ? m : 0) * lda + 16 * g4;
  }
  f32x4 acc[RT][MT];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // k steps of 64; wave w takes a contiguous run of them, so its loads walk each row in long pieces
  const int steps = (K + 63) / 64;
  const int per_wave = (steps + nw - 1) / nw;
  const int s_begin = wave * per_wave;
  const int s_end = s_begin + per_wave < steps ? s_begin + per_wave : steps;
  for (int s0 = s_begin; s0 < s_end; s0 += UNROLL) {
    bf16x8 wf[UNROLL][RT][2], af[UNROLL][MT][2];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int kk = (s0 + u) * 64;
      const int k = kk + 16 * g4;
      const bool ok0 = k < K && (s0 + u) < s_end, ok1 = k + 8 < K && (s0 + u) < s_end;
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        wf[u][r][0] = ok0 ? *(const bf16x8*)(wp[r] + kk) : zero8();
        wf[u][r][1] = ok1 ? *(const bf16x8*)(wp[r] + kk + 8) : zero8();
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        af[u][t][0] = (ok0 && arow[t]) ? *(const bf16x8*)(ap[t] + kk) : zero8();
        af[u][t][1] = (ok1 && arow[t]) ? *(const bf16x8*)(ap[t] + kk + 8) : zero8();
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][r][0], af[u][t][0], acc[r][t], 0, 0, 0);
          acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][r][1], af[u][t][1], acc[r][t], 0, 0, 0);
        }
  }

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
    if (GATED) {  // slot x of the up tile lies MT * 64 slots further on
      f32x4 u = ((const f32x4*)red)[MT * 64 + x];
      for (int w = 1; w < nw; ++w) {
        const f32x4 v = ((const f32x4*)red)[(int64_t)w * RT * MT * 64 + MT * 64 + x];
        u[0] += v[0]; u[1] += v[1]; u[2] += v[2]; u[3] += v[3];
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) s[e] = (s[e] / (1.f + expf(-s[e]))) * u[e];
    }
    const int tile = x >> 6, ln = x & 63;
    const int r = tile / MT, t = tile % MT;
    const int m = t * 16 + (ln & 15);
    const int n = n0 + r * 16 + 4 * (ln >> 4);
    if (m < M) {
      O* cp = C + (int64_t)m * ldc + n;
      if (n + 3 < N) {
        store4<O>(cp, s);
      } else {
        for (int e = 0; e < 4 && n + e < N; ++e) cp[e] = from_f32<O>(s[e]);
      }
    }
  }
}

template <int MT, int RT, class O>
int launch(const bf16* A, int64_t lda, const bf16* W, int64_t ldw, O* C, int64_t ldc, int M, int N, int K, int waves,
           hipStream_t stream) {
  const int row_tiles = (N + 16 * RT - 1) / (16 * RT);
  const size_t lds = (size_t)waves * RT * MT * 64 * sizeof(f32x4);
  gemm_small_m_kernel<MT, RT, O><<<(unsigned)row_tiles, waves * 64, lds, stream>>>(A, lda, W, ldw, C, ldc, M, N, K);
  return launch_status();
}

template <int MT>
int launch_gated(const bf16* A, int64_t lda, const bf16* W, int64_t ldw, bf16* C, int64_t ldc, int M, int N, int K,
                 int waves, hipStream_t stream) {
  const int col_tiles = (N + 15) / 16;
  const size_t lds = (size_t)waves * 2 * MT * 64 * sizeof(f32x4);
  gemm_small_m_kernel<MT, 2, bf16, true><<<(unsigned)col_tiles, waves * 64, lds, stream>>>(A, lda, W, ldw, C, ldc, M, N, K);
  return launch_status();
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
  if (rt == 0) rt = mt >= 2 ? 2 : ((N >= 6144 && M > 4) ? 2 : 1);  // measured on MI355X
  if (nw == 0) {
    // about 2048 waves in flight, each with at least two k steps
    const int64_t tiles = (N + 16 * rt - 1) / (16 * rt);
    nw = 4;
    while (nw < 16 && tiles * nw < (rt == 1 ? 2048 : 768)) nw *= 2;
    const int64_t steps = (K + 63) / 64;
    while (nw > 1 && steps < 2 * nw) nw /= 2;
  }
  while (nw > 1 && (size_t)nw * rt * mt * 64 * sizeof(f32x4) > 64 * 1024) nw /= 2;
  if (nw < 1 || nw > 16) return ERR_BAD_SHAPE;
  if ((size_t)nw * rt * mt * 64 * sizeof(f32x4) > 64 * 1024) return ERR_UNSUPPORTED;
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
  if (nw < 1 || nw > 16 || (size_t)nw * 2 * mt * 64 * sizeof(f32x4) > 64 * 1024) return ERR_BAD_SHAPE;
  if (mt == 1)
    return launch_gated<1>((const bf16*)A, lda, (const bf16*)W, ldw, (bf16*)C, ldc, (int)M, (int)N, (int)K, nw, stream);
  return launch_gated<2>((const bf16*)A, lda, (const bf16*)W, ldw, (bf16*)C, ldc, (int)M, (int)N, (int)K, nw, stream);
}
