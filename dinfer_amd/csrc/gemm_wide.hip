// C[M,N] = A[M,K] . W[N,K]^T for 17 to 64 rows and a weight of many rows (the gate and up projections of a
// feed-forward, the LM head), bf16 operands, float accumulation: the products of a decode step of 17 to 64
// requests whose weight is so tall that 96 of its rows a workgroup still make a workgroup for every CU.
//
// At these row counts a weight-streaming kernel's trouble is the activations: every workgroup needs all of A
// (64 rows x K: 512 KB at K = 4,096), and what it loads of A crosses the same path into the CU as the weight it
// streams. Here A costs that path no registers and no waiting: a workgroup is 8 waves, wave w owns the 64-wide
// k steps w, w + 8, w + 16, ... and fetches the fragments of A it will need itself, one step ahead, straight into
// LDS (a buffer load that writes LDS: 16 bytes a lane, laid down in lane order, which is the order of the MFMA's
// B operand when lane l asks for A[16 t + l % 16][k + 8 (l / 16) ..]). Nobody else reads them, so the waves never
// meet while they stream: each is a chain of [fragments of the next step on their way into LDS | 12 weight loads of
// the next step in flight (6 tiles of 16 rows x 64 k, line-shaped: lane l reads piece l % 8 of row l / 8) | this
// step's 48 MFMAs]. The wait for the fragments is written out (see fetch_a), the compiler counts the weight loads
// itself. A's fragments are read from LDS once per step and serve all six
// weight tiles, so LDS carries a sixth of what a wave-per-tile layout would ask of it.
//
// At the end the eight waves' partial sums meet in LDS, two tiles at a time, and are added in wave order (no
// atomics). GATED: W is [2N, K] = [gate; up]; a workgroup takes gate rows n0 .. n0 + 48 and the up rows of the
// same columns, and stores silu(gate) * up. SCALED: every token's result is multiplied by
// rsqrt(sum of its partial sums of squares / width + eps) first (the consumer of a norm carried by the product
// before it, as in gemm.hip).
//
// v_mfma_f32_16x16x32_bf16, weight as the A operand. K a multiple of 512, N of 16, M <= 64.
//
// Reference behaviour: crates/kernels/src/gemm.rs:605-647 (the product; the reference hands these row counts to its
// vendor library), crates/kernels/cuda/activation.cu:8-16 (the gated activation).
#include <type_traits>

#include "common.cuh"

using namespace dinfer;

namespace {

constexpr int WAVES = 8;
constexpr int RT = 6;              // weight tiles of 16 rows a workgroup
constexpr int CHUNK = WAVES * 64;  // k between two steps of one wave
constexpr int ROW_BYTES = 144;     // strip: 64 k of a row and 16 bytes of padding
constexpr int STRIP_BYTES = 16 * ROW_BYTES;

// Orders a wave's LDS writes before its reads of what other lanes wrote (and the reverse): the hardware
// runs a wave's LDS operations in order, this keeps the compiler from moving them across.
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// Waits until at most N of the wave's vector memory loads are in flight (s_waitcnt with the other counters left
// open: vmcnt is bits 3:0 and 15:14 of the operand, expcnt 6:4, lgkmcnt 11:8); nothing is scheduled across it.
template <int N>
__device__ __forceinline__ void wait_for_loads() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
  __builtin_amdgcn_sched_barrier(0);
}

// What the SCALED form needs beside the product's own operands.
struct Scale {
  const float* stats;  // [M][ld_stats] partial sums of squares, `cols` of them a token
  int64_t ld_stats;
  int cols;
  float eps, inv_width;
};

template <int MT, bool GATED, class O, bool SCALED>
__global__ void __launch_bounds__(WAVES * 64) gemm_wide_kernel(const bf16* __restrict__ A, int64_t lda,
                                                              const bf16* __restrict__ W, int64_t ldw,
                                                              O* __restrict__ C, int64_t ldc, int M, int N, int K,
                                                              Scale link) {
  // a wave's fragments of A for one step: [wave][half of the step][token tile][lane], two buffers in turn; afterwards
  // the waves' partial sums
  __shared__ __attribute__((aligned(16))) bf16x8 stage0[WAVES * 2 * 4][64];
  __shared__ __attribute__((aligned(16))) bf16x8 stage1[WAVES * 2 * 4][64];
  __shared__ __attribute__((aligned(16))) char strips[WAVES * STRIP_BYTES];
  __shared__ float rs[64];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63, i16 = lane & 15, g4 = lane >> 4;
  const int lrow = lane >> 3, lpiece = lane & 7;
  char* const strip = strips + wave * STRIP_BYTES;
  char* const put = strip + lrow * ROW_BYTES + lpiece * 16;
  const char* const get = strip + i16 * ROW_BYTES + g4 * 16;

  // the workgroup's six tiles: GATED three of the gate and the same three of the up projection, else six in a row.
  // A tile past the weight's end is replaced by the last one (computed, never stored).
  const int tiles = N >> 4;  // N % 16 == 0
  const int tile0 = blockIdx.x * (GATED ? 3 : RT);
  auto tile_row = [&](int r) {
    int j = tile0 + (GATED ? r % 3 : r);
    j = j < tiles ? j : tiles - 1;
    return (GATED && r >= 3 ? N : 0) + j * 16;
  };
  // Addresses are a scalar base (what the wave and the tile decide) plus one 32-bit offset in bytes a lane, to which
  // the step's k is added inside the loop: so the compiler sees the widening of that sum where the load is and picks
  // the form of load that takes its base from scalar registers (no lane holds a 64-bit address; hoisted out of the
  // loop, the widened offsets took a register pair each and the 64-row form spilled inside its loop).
  const char* const Wb = (const char*)W;
  const uint32_t w_lane = (uint32_t)(lrow * (int)ldw + 8 * lpiece) * 2u;  // inside a tile: row l / 8, piece l % 8
  const uint32_t w_half = (uint32_t)(16 * ldw);                            // eight rows further on
  auto tile_base = [&](int r) { return Wb + ((int64_t)tile_row(r) * ldw + wave * 64) * 2; };
  uint32_t a_lane[MT];  // inside A: row 16 t + l % 16 (past the end: a copy of the last row, dropped), piece l / 16
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + i16;
    a_lane[t] = (uint32_t)((m < M ? m : M - 1) * (int)lda + 8 * g4) * 2u;
  }
  // This wave's fragments of A for the step at k0, on their way into `stage`. The loads are buffer loads (a
  // descriptor of A, an offset a lane), not global ones: after a global load into LDS the compiler waits for every
  // load in flight at the next thing that depends on any of them, which was once a step and drained the wave's queue
  // of weights each time. A buffer load into LDS it counts among the loads in flight like any other, but it does not
  // reliably order a later read of that LDS behind it (it looks at the first such load into an object only), so the
  // wait before the fragments are read is written out in `compute`, and nothing may move across the end of this.
  const __amdgpu_buffer_rsrc_t a_desc =
      __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, (int)(((int64_t)(M - 1) * lda + K) * 2), 0x00020000);
  auto fetch_a = [&](bf16x8 (&stage)[WAVES * 2 * 4][64], int k0) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int t = 0; t < MT; ++t)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(a_desc,
                                                 (__attribute__((address_space(3))) void*)&stage[(wave * 2 + h) * 4 + t][0],
                                                 16, (int)a_lane[t], (k0 + wave * 64 + 32 * h) * 2, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // the 16 rows x 64 k of tile r at k0, in the line-shaped order
  auto fetch_w = [&](bf16x8 (&dst)[2], int r, int k0) {
    const char* p = tile_base(r);
    const uint32_t o = w_lane + (uint32_t)(k0 * 2);
    dst[0] = __builtin_nontemporal_load((const bf16x8*)(p + o));
    dst[1] = __builtin_nontemporal_load((const bf16x8*)(p + (o + w_half)));
  };

  f32x4 acc[RT][MT];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // One step: A's fragments out of LDS, then tile by tile: the weights that arrived go through the strip into MFMA
  // order, the same registers take the loads of the next step's tile at once (k_next < 0: there is none), 8 MFMAs.
  // (`more` is a type, so that the last step is code of its own: a branch around a load would make the compiler wait
  // for every load in flight wherever it needs one of them)
  bf16x8 w[RT][2];
  auto compute = [&](const bf16x8 (&stage)[WAVES * 2 * 4][64], auto more, int k_next) {
    // Loads return in the order they were issued. Behind this step's fragments came the 12 weight loads of this step
    // and, unless this is the last step, the 2 MT fragment loads of the next: when no more than those are in flight,
    // the fragments are in LDS.
    wait_for_loads<12 + (decltype(more)::value ? 2 * MT : 0)>();
    bf16x8 af[MT][2];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      af[t][0] = stage[(wave * 2 + 0) * 4 + t][lane];
      af[t][1] = stage[(wave * 2 + 1) * 4 + t][lane];
    }
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      *(bf16x8*)put = w[r][0];
      *(bf16x8*)(put + 8 * ROW_BYTES) = w[r][1];
      if constexpr (decltype(more)::value) {
        fetch_w(w[r], r, k_next);
      }
      wave_sync();
      const bf16x8 wf0 = *(const bf16x8*)get, wf1 = *(const bf16x8*)(get + 64);
      wave_sync();
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf0, af[t][0], acc[r][t], 0, 0, 0);
        acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf1, af[t][1], acc[r][t], 0, 0, 0);
      }
    }
  };

  // K % CHUNK == 0. Workgroup b starts its walk at step b % steps and wraps round: workgroups that all stood at the
  // same k would ask the same few memory channels at any moment when a row is a power of two long (measured on
  // reads alone, 8 KB rows: 5.7 TB/s in step, 6.5 staggered).
  const int steps = K / CHUNK;
  const int first = blockIdx.x % steps;
  auto k_of = [&](int it) {
    const int s = it + first;
    return (s < steps ? s : s - steps) * CHUNK;
  };
  fetch_a(stage0, k_of(0));
#pragma unroll
  for (int r = 0; r < RT; ++r) fetch_w(w[r], r, k_of(0));
  // even steps stage in stage0, odd ones in stage1
  constexpr std::true_type MORE{};
  constexpr std::false_type LAST{};
  int it = 0;
  for (; it + 2 < steps; it += 2) {
    fetch_a(stage1, k_of(it + 1));
    compute(stage0, MORE, k_of(it + 1));
    fetch_a(stage0, k_of(it + 2));
    compute(stage1, MORE, k_of(it + 2));
  }
  if (it + 1 < steps) {
    fetch_a(stage1, k_of(it + 1));
    compute(stage0, MORE, k_of(it + 1));
    compute(stage1, LAST, 0);
  } else {
    compute(stage0, LAST, 0);
  }

  if constexpr (SCALED) {
    for (int m = wave; m < M; m += WAVES) {
      float a = 0.f;
      for (int j = lane; j < link.cols; j += 64) a += link.stats[(int64_t)m * link.ld_stats + j];
      a = wave_sum(a);
      if (lane == 0) rs[m] = rsqrtf(a * link.inv_width + link.eps);
    }
  }
  // The partial sums meet, two tiles a round (GATED: a gate tile and its up tile): [wave][2][MT][lane] of f32x4,
  // 64 KB at MT = 4, in the staging buffers in turn; thread x adds slot x of every wave, in wave order.
  const int n_first = blockIdx.x * (GATED ? 48 : 96);
#pragma unroll
  for (int round = 0; round < 3; ++round) {
    f32x4* const red = (f32x4*)(round == 1 ? &stage1[0][0] : &stage0[0][0]);
    const int ra = GATED ? round : 2 * round, rb = GATED ? round + 3 : 2 * round + 1;
    __syncthreads();  // every wave is done with what this buffer held
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      red[((wave * 2 + 0) * MT + t) * 64 + lane] = acc[ra][t];
      red[((wave * 2 + 1) * MT + t) * 64 + lane] = acc[rb][t];
    }
    __syncthreads();
    for (int x = threadIdx.x; x < (GATED ? 1 : 2) * MT * 64; x += WAVES * 64) {
      f32x4 s = red[x];
      for (int w = 1; w < WAVES; ++w) {
        const f32x4 v = red[w * 2 * MT * 64 + x];
        s[0] += v[0]; s[1] += v[1]; s[2] += v[2]; s[3] += v[3];
      }
      const int which = x / (MT * 64), t = (x >> 6) % MT, ln = x & 63;
      const int m = t * 16 + (ln & 15);
      const int n = n_first + (GATED ? round : 2 * round + which) * 16 + 4 * (ln >> 4);
      float scale = 1.f;
      if constexpr (SCALED) scale = m < M ? rs[m] : 0.f;
      if constexpr (GATED) {
        f32x4 u = red[MT * 64 + x];
        for (int w = 1; w < WAVES; ++w) {
          const f32x4 v = red[w * 2 * MT * 64 + MT * 64 + x];
          u[0] += v[0]; u[1] += v[1]; u[2] += v[2]; u[3] += v[3];
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float g = s[e] * scale;
          s[e] = (g / (1.f + expf(-g))) * (u[e] * scale);
        }
      } else if constexpr (SCALED) {
#pragma unroll
        for (int e = 0; e < 4; ++e) s[e] *= scale;
      }
      if (m < M && n < N) {  // N % 16 == 0: all four columns or none
        O* cp = C + (int64_t)m * ldc + n;
#pragma unroll
        for (int e = 0; e < 4; ++e) cp[e] = from_f32<O>(s[e]);
      }
    }
  }
}

template <int MT, bool GATED, class O>
int launch(const bf16* A, int64_t lda, const bf16* W, int64_t ldw, O* C, int64_t ldc, int M, int N, int K,
           const Scale* link, hipStream_t stream) {
  const unsigned blocks = (unsigned)((N + (GATED ? 47 : 95)) / (GATED ? 48 : 96));
  if (link)
    gemm_wide_kernel<MT, GATED, O, true><<<blocks, WAVES * 64, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K, *link);
  else
    gemm_wide_kernel<MT, GATED, O, false><<<blocks, WAVES * 64, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K, Scale{});
  return launch_status();
}

}  // namespace

// 1 if dinfer_gemm_wide takes these sizes (the caller uses another product otherwise).
extern "C" int dinfer_gemm_wide_supports(int64_t M, int64_t N, int64_t K) {
  return M > 0 && M <= 64 && N > 0 && N % 16 == 0 && K > 0 && K % CHUNK == 0 && N <= 0x7fffffff - 96 && K <= 1 << 24;
}

// C[M,N] = A . W^T for up to 64 rows. gated: W is [2N, K] = [gate; up] and C[M,N] = silu(A . gate^T) * (A . up^T).
// out_f32: C is float (not gated). stats non-null: every row m of the result is multiplied by
// rsqrt(sum(stats[m, :cols]) / width + eps) first (before the activation, when gated).
extern "C" int dinfer_gemm_wide(int out_f32, const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc,
                                int64_t M, int64_t N, int64_t K, int gated, const float* stats, int64_t ld_stats,
                                int cols, float eps, int64_t width, hipStream_t stream) {
  if (M <= 0 || N <= 0) return OK;
  if (!dinfer_gemm_wide_supports(M, N, K)) return ERR_UNSUPPORTED;
  if (lda < K || ldw < K || ldc < N || lda > 1 << 23 || ldw > 1 << 24 || lda % 8 || ldw % 8 || ((uintptr_t)A % 16) || ((uintptr_t)W % 16) ||
      (gated && out_f32) || (stats && (cols <= 0 || width <= 0 || ld_stats < cols)))
    return ERR_BAD_SHAPE;
  Scale link{stats, ld_stats, cols, eps, width > 0 ? 1.f / (float)width : 0.f};
  const Scale* lp = stats ? &link : nullptr;
  const int mt = (int)(M + 15) / 16;
#define GO(MT_)                                                                                                          \
  if (gated) return launch<MT_, true, bf16>((const bf16*)A, lda, (const bf16*)W, ldw, (bf16*)C, ldc, (int)M, (int)N, (int)K, lp, stream); \
  if (out_f32) return launch<MT_, false, float>((const bf16*)A, lda, (const bf16*)W, ldw, (float*)C, ldc, (int)M, (int)N, (int)K, lp, stream); \
  return launch<MT_, false, bf16>((const bf16*)A, lda, (const bf16*)W, ldw, (bf16*)C, ldc, (int)M, (int)N, (int)K, lp, stream);
  if (mt == 1) { GO(1) }
  if (mt == 2) { GO(2) }
  if (mt == 3) { GO(3) }
  GO(4)
#undef GO
}
