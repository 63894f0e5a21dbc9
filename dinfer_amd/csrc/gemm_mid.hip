// C[M,N] = A[M,K] . W[N,K]^T for 17 to 64 rows (any M <= 64 works), bf16 operands, float
// accumulation: the matrix products of a decode step at batch sizes where the weight-streaming
// kernel for few rows spends most of its loads on the activations (every workgroup of 16 or 32
// weight rows reads all of A again: four token tiles cost four times the loads of the weight).
// On this chip the vector-memory path of a CU holds a bounded number of bytes in flight, so a byte
// of A from L2 costs that path almost what a byte of W from HBM costs: A must be loaded few times.
//
// Here a workgroup of 8 waves owns a run of k (a "slice") and keeps that slice of A, all M rows of
// it, in LDS for its whole life: up to 129 KB of the 160 KB a CU has (a slice of 1,024 at 64 rows,
// of 2,048 at 32), laid out as the MFMA's B operand reads it (rows padded by 16 bytes, no bank
// conflicts). After this one fill and one barrier the waves never meet again. A workgroup walks
// several groups of 8 x RT x 16 weight rows, one workgroup a CU; each wave streams its RT tiles
// of 16 rows with the line-shaped loads of the few-row kernel (lane l reads piece l % 8 of row
// l / 8; a strip of LDS of its own turns a tile into MFMA order), two rounds of loads in flight
// across the groups' ends, and reads the activations' fragments from LDS: no load of A in the loop.
// Every load is unconditional (addresses past the end are pulled back inside): a branch around a
// load makes the compiler wait for everything in flight wherever it needs one of them.
//
// Slices of k are different workgroups (blockIdx.y); each writes float partial sums
// P[slice][MT * 16][N] (a token's row is contiguous, so that the pass over them can take a token a workgroup), and
// gemm_mid_reduce_kernel adds them in slice order (no atomics: a launch shape gives the same bits every time), applies
// silu(gate) * up for the gated form, and rounds once. gemm_mid_reduce_norm_kernel is that pass for a product that
// completes the residual stream before an RMSNorm: it adds into the stream and writes the norm's output as well.
//
// v_mfma_f32_16x16x32_bf16, weight as the A operand: a tile is 16 weight rows x 16 tokens.
// K must be a multiple of 8 (16-byte loads), N of 4.
//
// Reference behaviour: crates/kernels/src/gemm.rs:605-647 (the product itself; the reference hands
// these row counts to its vendor library).
#include "common.cuh"
#include "gemm_mid.h"

#include <mutex>

using namespace dinfer;

namespace {

constexpr int WAVES = 8;
constexpr int ROW_BYTES = 144;     // strip: 64 k of a row and 16 bytes of padding
constexpr int STRIP_BYTES = 16 * ROW_BYTES;
constexpr int MAX_LDS = 160 * 1024;

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

template <bool STREAM>
__device__ __forceinline__ bf16x8 ld_weight(const bf16* p) {
  if constexpr (STREAM)
    return __builtin_nontemporal_load((const bf16x8*)p);
  else
    return *(const bf16x8*)p;
}

template <int MT, int RT, bool STREAM>
__global__ void __launch_bounds__(WAVES * 64) gemm_mid_m_kernel(const bf16* __restrict__ A, int64_t lda,
                                                                const bf16* __restrict__ W, int64_t ldw,
                                                                float* __restrict__ P, int M, int N, int K, int ks, int groups) {
  // 64-wide k steps per round of loads; two rounds (16 loads of 16 bytes a lane) are in flight
  constexpr int UN = RT >= 4 ? 1 : 4 / RT;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int a_stride = ks * 2 + 16;  // bytes of a row of the slice in LDS; ks % 64 == 0, so 16 mod 128: no bank conflicts
  char* const strips = smem + MT * 16 * a_stride;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, i16 = lane & 15, g4 = lane >> 4;
  const int lrow = lane >> 3, lpiece = lane & 7;
  const int k_begin = blockIdx.y * ks;
  const int k_end = k_begin + ks < K ? k_begin + ks : K;
  const int units = (k_end - k_begin + 63) / 64;
  // this workgroup's groups of WAVES * RT * 16 weight rows: blockIdx.x, blockIdx.x + gridDim.x, ...
  const int chunks = gridDim.x;
  const int iters = (groups - (int)blockIdx.x + chunks - 1) / chunks;
  const int rps = (units + UN - 1) / UN;  // rounds per group of rows
  const int total = iters * rps;
  auto first_row = [&](int it) { return (((int)blockIdx.x + it * chunks) * WAVES + wave) * (RT * 16); };

  // Every load below is unconditional (addresses past the slice are pulled back inside it): a branch around
  // a load would make the compiler wait for all loads in flight wherever it needs one of them. What a lane
  // reads in place of k past the slice's end meets zeros of A in LDS.
  const int k_last = k_end - k_begin - 8;  // offset of the slice's last 16-byte piece
  const bf16* wp[RT][2];
  auto set_rows = [&](int it) {
    const int n0 = first_row(it);
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        int n = n0 + r * 16 + lrow + 8 * h;
        if (n >= N) n = N - 1;  // rows past the end are computed and dropped
        wp[r][h] = W + (int64_t)n * ldw + k_begin + 8 * lpiece;
      }
  };
  set_rows(0);
  bf16x8 buf[2][UN][RT][2];
  int l_it = 0, l_r = 0;  // the round the next load_round fetches: rounds are fetched in the order they are computed
  auto load_round = [&](int b) {
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      int kk = (l_r * UN + u) * 64 + 8 * lpiece;
      kk = (kk < k_last ? kk : k_last) - 8 * lpiece;
#pragma unroll
      for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int h = 0; h < 2; ++h) buf[b][u][r][h] = ld_weight<STREAM>(wp[r][h] + kk);
    }
    if (l_r + 1 < rps) {
      ++l_r;
    } else if (l_it + 1 < iters) {
      l_r = 0;
      set_rows(++l_it);
    }  // past the last round: the same round again (an odd number of rounds fetches one too many)
  };
  load_round(0);  // the first weights are on their way while the slice of A is fetched
  load_round(1);
  {
    // all of the slice at once: up to 16 loads of 16 bytes a thread in flight, then into LDS
    const int pieces = ks >> 3;  // 16-byte pieces of a row of the slice
    const int total_pieces = MT * 16 * pieces;
    constexpr int BATCH = 16;
    for (int c0 = threadIdx.x; c0 < total_pieces; c0 += BATCH * WAVES * 64) {
      bf16x8 v[BATCH];
      int where[BATCH];
#pragma unroll
      for (int i = 0; i < BATCH; ++i) {
        const int c = c0 + i * WAVES * 64;
        const int row = c / pieces, piece = c - row * pieces;
        const int k = 8 * piece;
        const bool real = row < M && k <= k_last;
        v[i] = *(const bf16x8*)(A + (int64_t)(row < M ? row : M - 1) * lda + k_begin + (k <= k_last ? k : k_last));
        if (!real) v[i] = zero8();
        where[i] = c < total_pieces ? row * a_stride + piece * 16 : -1;
      }
#pragma unroll
      for (int i = 0; i < BATCH; ++i)
        if (where[i] >= 0) *(bf16x8*)(smem + where[i]) = v[i];
    }
  }
  __syncthreads();

  char* const strip = strips + wave * STRIP_BYTES;
  char* const put = strip + lrow * ROW_BYTES + lpiece * 16;
  const char* const get = strip + i16 * ROW_BYTES + g4 * 16;
  const char* const a_get = smem + i16 * a_stride + g4 * 16;
  // partial sums of this slice: [MT * 16][N]
  f32x4* const out = (f32x4*)P + (int64_t)blockIdx.y * (N >> 2) * (MT * 16);

  f32x4 acc[RT][MT];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  int c_it = 0, c_r = 0;  // the round the next compute_round works on
  auto compute_round = [&](int b) {
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      if (c_r * UN + u >= units) break;  // uniform
      bf16x8 af[MT][2];
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const char* ag = a_get + t * 16 * a_stride + (c_r * UN + u) * 128;
        af[t][0] = *(const bf16x8*)ag;
        af[t][1] = *(const bf16x8*)(ag + 64);
      }
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        *(bf16x8*)put = buf[b][u][r][0];
        *(bf16x8*)(put + 8 * ROW_BYTES) = buf[b][u][r][1];
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
    if (c_r + 1 < rps) {
      ++c_r;
      return;
    }
    // the group's rows are complete for this slice. lane: token t * 16 + i16, weight rows n0 + r * 16 + 4 g4 + {0..3}
    const int n0 = first_row(c_it);
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      const int n = n0 + r * 16 + 4 * g4;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        if (n < N) out[(int64_t)(t * 16 + i16) * (N >> 2) + (n >> 2)] = acc[r][t];  // N % 4 == 0: all four or none
        acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
    }
    c_r = 0;
    ++c_it;
  };

  // two rounds are in flight while a round is computed; the last pair has nothing left to fetch
  int q = 0;
  for (; q + 2 < total; q += 2) {
    compute_round(0);
    load_round(0);
    compute_round(1);
    load_round(1);
  }
  compute_round(0);
  if (q + 1 < total) compute_round(1);
}

// C[m][n] = sum over slices of P[s][m][n] in slice order; GATED: a row of P is the gate's N columns and then the up
// projection's, and C[m][n] = silu(sum gate) * sum up. One thread per token and four columns.
template <class O, bool GATED>
__global__ void __launch_bounds__(256) gemm_mid_reduce_kernel(const float* __restrict__ P, int mp, int slices,
                                                              O* __restrict__ C, int64_t ldc, int M, int N) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int quads = N >> 2;
  if (i >= (int64_t)quads * M) return;
  const int m = (int)(i / quads), q = (int)(i % quads);
  const int row_quads = GATED ? 2 * quads : quads;
  const int64_t slice_stride = (int64_t)row_quads * mp;
  const f32x4* p = (const f32x4*)P + (int64_t)m * row_quads + q;
  f32x4 g = *p, u;
  if (GATED) u = p[quads];
  for (int s = 1; s < slices; ++s) {
    const f32x4 v = p[s * slice_stride];
    g[0] += v[0]; g[1] += v[1]; g[2] += v[2]; g[3] += v[3];
    if (GATED) {
      const f32x4 w = p[s * slice_stride + quads];
      u[0] += w[0]; u[1] += w[1]; u[2] += w[2]; u[3] += w[3];
    }
  }
  O* c = C + (int64_t)m * ldc + 4 * q;
#pragma unroll
  for (int e = 0; e < 4; ++e) c[e] = from_f32<O>(GATED ? (g[e] / (1.f + expf(-g[e]))) * u[e] : g[e]);
}

// The pass over the partial sums for a product that completes the residual stream before an RMSNorm, a token a
// workgroup: H[m][n] += sum over slices of P[s][m][n] (the float sum of the slices in their order and the stream,
// rounded once), and OUT[m][n] = H[m][n] / sqrt(mean(H[m]^2) + eps) * (gain[n] + gain_offset), from the rounded H as
// the norm's own kernel reads it. Stands for this file's pass, the add and the norm: two kernels of about 5 us fewer a
// layer. A thread keeps its columns (four at a time, up to QMAX times) between the sum and the division.
constexpr int SINK_THREADS = 1024, SINK_QMAX = 2;
__global__ void __launch_bounds__(SINK_THREADS) gemm_mid_reduce_norm_kernel(
    const float* __restrict__ P, int mp, int slices, bf16* __restrict__ H, int64_t ldh, bf16* __restrict__ OUT,
    int64_t ld_out, const void* __restrict__ gain, int gain_f32, float gain_offset, float eps, int N) {
  __shared__ float red[16];
  const int m = blockIdx.x, quads = N >> 2;
  const int64_t slice_stride = (int64_t)quads * mp;
  const f32x4* p = (const f32x4*)P + (int64_t)m * quads;
  bf16* h = H + (int64_t)m * ldh;
  float v[SINK_QMAX][4], g[SINK_QMAX][4];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < SINK_QMAX; ++j) {
    const int q = threadIdx.x + j * SINK_THREADS;
    if (q < quads) {
      f32x4 a = p[q];
      const bf16x4 old = *(const bf16x4*)(h + 4 * q);
      if (gain_f32) {
        const f32x4 gv = *(const f32x4*)((const float*)gain + 4 * q);
#pragma unroll
        for (int e = 0; e < 4; ++e) g[j][e] = gv[e] + gain_offset;
      } else {
        const bf16x4 gv = *(const bf16x4*)((const bf16*)gain + 4 * q);
#pragma unroll
        for (int e = 0; e < 4; ++e) g[j][e] = (float)gv[e] + gain_offset;
      }
      // (eight slices' loads at a time: the pass is a chain of trips to L2 otherwise; added in slice order)
      int s = 1;
      for (; s + 8 <= slices; s += 8) {
        f32x4 b[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) b[i] = p[(s + i) * slice_stride + q];
#pragma unroll
        for (int i = 0; i < 8; ++i) { a[0] += b[i][0]; a[1] += b[i][1]; a[2] += b[i][2]; a[3] += b[i][3]; }
      }
      for (; s + 2 <= slices; s += 2) {
        const f32x4 b0 = p[s * slice_stride + q], b1 = p[(s + 1) * slice_stride + q];
        a[0] += b0[0]; a[1] += b0[1]; a[2] += b0[2]; a[3] += b0[3];
        a[0] += b1[0]; a[1] += b1[1]; a[2] += b1[2]; a[3] += b1[3];
      }
      for (; s < slices; ++s) {
        const f32x4 b = p[s * slice_stride + q];
        a[0] += b[0]; a[1] += b[1]; a[2] += b[2]; a[3] += b[3];
      }
      bf16x4 r;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        r[e] = (bf16)(a[e] + (float)old[e]);
        v[j][e] = (float)r[e];
        ss += v[j][e] * v[j][e];
      }
      *(bf16x4*)(h + 4 * q) = r;
    }
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)N + eps);
  bf16* o = OUT + (int64_t)m * ld_out;
#pragma unroll
  for (int j = 0; j < SINK_QMAX; ++j) {
    const int q = threadIdx.x + j * SINK_THREADS;
    if (q < quads) {
      bf16x4 y;
#pragma unroll
      for (int e = 0; e < 4; ++e) y[e] = (bf16)(v[j][e] * inv * g[j][e]);
      *(bf16x4*)(o + 4 * q) = y;
    }
  }
}

inline bool streams_weight(int64_t rows, int64_t K) { return rows * K * (int64_t)sizeof(bf16) >= (int64_t)40 << 20; }

inline int64_t lds_bytes(int mt, int ks) { return (int64_t)mt * 16 * (ks * 2 + 16) + WAVES * STRIP_BYTES; }

struct Shape {
  int ks, rt, slices, chunks;
  int64_t groups;
};

constexpr int CUS = 256;

// Workgroups for a slice length and row tiles per wave: one per CU if the sizes allow, each with as many
// groups of rows as the others. Returns the bytes on the critical path of the busiest CU (weights streamed,
// the fill, its share of the partial sums written and read again), the figure candidates are compared by.
inline double layout(int64_t M, int64_t rows, int64_t K, int ks, int rt, Shape* s) {
  const int64_t slices = (K + ks - 1) / ks;
  const int64_t groups = (rows + WAVES * 16 * rt - 1) / (WAVES * 16 * rt);
  int64_t per = (groups * slices + CUS - 1) / CUS;  // groups of rows a workgroup walks
  if (per < 1) per = 1;
  const int64_t chunks = (groups + per - 1) / per;
  per = (groups + chunks - 1) / chunks;
  s->ks = ks, s->rt = rt, s->slices = (int)slices, s->chunks = (int)chunks, s->groups = groups;
  const int64_t k_eff = K < ks ? K : ks;
  const double turns = (double)((chunks * slices + CUS - 1) / CUS);
  return turns * (double)(per * WAVES * 16 * rt * k_eff * 2 + M * k_eff * 2) + (double)(slices * M * rows * 8) / CUS;
}

inline bool choose(int64_t M, int64_t rows, int64_t K, int ks, int rt, Shape* s) {
  const int mt = (int)(M + 15) / 16;
  if (ks > 0 && (ks % 64 || lds_bytes(mt, ks) > MAX_LDS)) return false;
  if (rt != 0 && rt != 1 && rt != 2 && rt != 4) return false;
  double best = -1.;
  for (int k = 4096; k >= 256; k -= 128) {  // longest first: of equal costs the one with the fewest slices stays
    if (ks > 0 && k != 4096) break;
    const int len = ks > 0 ? ks : k;
    if (lds_bytes(mt, len) > MAX_LDS) continue;
    for (int r = 1; r <= 2; r *= 2) {
      if (rt > 0 && r != 1) break;
      Shape c;
      const double cost = layout(M, rows, K, len, rt > 0 ? rt : r, &c);
      if (best < 0. || cost < best) best = cost, *s = c;
    }
  }
  return best >= 0. && s->slices <= 65535;
}

template <int MT, int RT, bool STREAM>
int launch(const bf16* A, int64_t lda, const bf16* W, int64_t ldw, float* P, int M, int N, int K, const Shape& s,
           hipStream_t stream) {
  const size_t lds = (size_t)lds_bytes(MT, s.ks);
  if (hipFuncSetAttribute((const void*)gemm_mid_m_kernel<MT, RT, STREAM>, hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)lds) != hipSuccess)
    return ERR_LAUNCH;
  gemm_mid_m_kernel<MT, RT, STREAM><<<dim3((unsigned)s.chunks, (unsigned)s.slices), WAVES * 64, lds, stream>>>(
      A, lda, W, ldw, P, M, N, K, s.ks, (int)s.groups);
  return launch_status();
}

template <int MT>
int launch_rt(const bf16* A, int64_t lda, const bf16* W, int64_t ldw, float* P, int M, int N, int K, const Shape& s,
              hipStream_t stream) {
  const bool st = streams_weight(N, K);
#define GO(RT_) \
  return st ? launch<MT, RT_, true>(A, lda, W, ldw, P, M, N, K, s, stream) \
            : launch<MT, RT_, false>(A, lda, W, ldw, P, M, N, K, s, stream)
  if (s.rt == 1) GO(1);
  if (s.rt == 2) GO(2);
  GO(4);
#undef GO
}

}  // namespace

// Bytes of workspace that dinfer_gemm_mid_m needs for these sizes (ks, rt: as passed there).
extern "C" int dinfer_gemm_mid_m_workspace(int64_t M, int64_t N, int64_t K, int gated, int ks, int rt, int64_t* bytes) {
  if (M <= 0 || M > 64 || N <= 0 || K <= 0 || !bytes) return ERR_BAD_SHAPE;
  Shape s;
  const int64_t rows = gated ? 2 * N : N;
  if (!choose(M, rows, K, ks, rt, &s)) return ERR_UNSUPPORTED;
  *bytes = (int64_t)s.slices * rows * (((M + 15) / 16) * 16) * (int64_t)sizeof(float);
  return OK;
}

namespace {

// The slices' partial sums of A . W^T (W of `rows` rows) into `P` (at least `capacity` bytes); *slices: how many.
int partial_sums(const void* A, int64_t lda, const void* W, int64_t ldw, int64_t M, int64_t rows, int64_t K, int ks, int rt,
                 void* P_, int64_t capacity, int too_small, int* slices, hipStream_t stream) {
  if (M > 64) return ERR_UNSUPPORTED;
  if (K <= 0 || K % 8 || rows % 4 || lda < K || ldw < K || lda % 8 || ldw % 8 || rows > 0x7fffffff || K > 0x7fffffff ||
      ((uintptr_t)A % 16) || ((uintptr_t)W % 16))
    return ERR_BAD_SHAPE;
  Shape s;
  if (!choose(M, rows, K, ks, rt, &s)) return ERR_UNSUPPORTED;
  const int mt = (int)(M + 15) / 16;
  const int64_t need = (int64_t)s.slices * rows * (mt * 16) * (int64_t)sizeof(float);
  if (!P_ || capacity < need || ((uintptr_t)P_ % 16)) return too_small;
  float* P = (float*)P_;
  int st;
#define GO(MT_) st = launch_rt<MT_>((const bf16*)A, lda, (const bf16*)W, ldw, P, (int)M, (int)rows, (int)K, s, stream)
  if (mt == 1) GO(1);
  else if (mt == 2) GO(2);
  else if (mt == 3) GO(3);
  else GO(4);
#undef GO
  *slices = s.slices;
  return st;
}

// The product and the pass that adds up its slices, with the partial sums in `P` (at least `capacity` bytes).
int run_mid_m(int out_f32, const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, int64_t M, int64_t N,
              int64_t K, int gated, int ks, int rt, void* P_, int64_t capacity, int too_small, hipStream_t stream) {
  if (M <= 0 || N <= 0) return OK;
  if (N % 4 || ldc < N || (gated && out_f32)) return M > 64 ? ERR_UNSUPPORTED : ERR_BAD_SHAPE;
  struct { int slices; } s{0};
  const int mt = (int)(M + 15) / 16;
  const float* P = (const float*)P_;
  const int st = partial_sums(A, lda, W, ldw, M, gated ? 2 * N : N, K, ks, rt, P_, capacity, too_small, &s.slices, stream);
  if (st != OK) return st;
  const unsigned blocks = (unsigned)(((int64_t)(mt * 16) * (N / 4) + 255) / 256);
  if (gated)
    gemm_mid_reduce_kernel<bf16, true><<<blocks, 256, 0, stream>>>(P, mt * 16, s.slices, (bf16*)C, ldc, (int)M, (int)N);
  else if (out_f32)
    gemm_mid_reduce_kernel<float, false><<<blocks, 256, 0, stream>>>(P, mt * 16, s.slices, (float*)C, ldc, (int)M, (int)N);
  else
    gemm_mid_reduce_kernel<bf16, false><<<blocks, 256, 0, stream>>>(P, mt * 16, s.slices, (bf16*)C, ldc, (int)M, (int)N);
  return launch_status();
}

}  // namespace

// C[M,N] = A . W^T for up to 64 rows. gated: W is [2N, K] = [gate; up] and C[M,N] = silu(A . gate^T) * (A . up^T).
// ks: k per slice (a multiple of 64; 0: as long as LDS holds), rt: tiles of 16 weight rows per wave (1, 2, 4; 0:
// chosen from the sizes). Partial sums go through `workspace` (dinfer_gemm_mid_m_workspace bytes, 16-byte aligned).
extern "C" int dinfer_gemm_mid_m(int out_f32, const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc,
                                 int64_t M, int64_t N, int64_t K, int gated, int ks, int rt, void* workspace,
                                 int64_t workspace_bytes, hipStream_t stream) {
  return run_mid_m(out_f32, A, lda, W, ldw, C, ldc, M, N, K, gated, ks, rt, workspace, workspace_bytes, ERR_WORKSPACE, stream);
}

// H[:M] += A . W^T in place (H bf16, the residual stream) and OUT[:M] = the RMSNorm of the new H (gain [N] bf16 or
// float, each plus gain_offset; eps): the product, the add and the norm that reads the stream next, in two kernels.
// N % 4 == 0 and N <= 8,192; ks, rt, workspace as for dinfer_gemm_mid_m (not gated).
extern "C" int dinfer_gemm_mid_m_sink(const void* A, int64_t lda, const void* W, int64_t ldw, void* H, int64_t ldh, void* OUT,
                                      int64_t ld_out, const void* gain, int gain_f32, float gain_offset, float eps,
                                      int64_t M, int64_t N, int64_t K, int ks, int rt, void* workspace,
                                      int64_t workspace_bytes, hipStream_t stream) {
  if (M <= 0 || N <= 0) return OK;
  if (N > 4 * SINK_THREADS * SINK_QMAX) return ERR_UNSUPPORTED;
  if (N % 4 || ldh < N || ld_out < N || ldh % 4 || ld_out % 4 || !gain || ((uintptr_t)H % 8) || ((uintptr_t)OUT % 8) ||
      ((uintptr_t)gain % (gain_f32 ? 16 : 8)))
    return ERR_BAD_SHAPE;
  int slices = 0;
  const int st = partial_sums(A, lda, W, ldw, M, N, K, ks, rt, workspace, workspace_bytes, ERR_WORKSPACE, &slices, stream);
  if (st != OK) return st;
  const int mt = (int)(M + 15) / 16;
  gemm_mid_reduce_norm_kernel<<<(unsigned)M, SINK_THREADS, 0, stream>>>((const float*)workspace, mt * 16, slices, (bf16*)H, ldh,
                                                                       (bf16*)OUT, ld_out, gain, gain_f32, gain_offset, eps,
                                                                       (int)N);
  return launch_status();
}

// ---- the same product for callers that cannot allocate ---------------------------------------------------------
// The partial sums go through a device array that is part of this library's code object: every GPU the library
// runs on holds its own copy, at its own address, from the moment the code object is loaded there until the
// process ends. In host code the array's name stands for that symbol, it is no device address: the address on
// the current device comes from hipGetSymbolAddress, once per device, and only that pointer is ever handed to
// a kernel.
static __device__ __align__(256) unsigned char scratch[DINFER_GEMM_MID_STATIC_BYTES];

namespace {

constexpr int MAX_DEVICES = 64;
void* scratch_ptr[MAX_DEVICES];   // by device ordinal; nullptr until that device has been set up
std::mutex scratch_mutex;

// The address of `scratch` on the current device (asked for once per device and kept).
int scratch_on_current_device(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return ERR_LAUNCH;
  std::lock_guard<std::mutex> guard(scratch_mutex);
  if (!scratch_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
      (void)hipGetLastError();
      return ERR_LAUNCH;
    }
    scratch_ptr[dev] = p;
  }
  *out = scratch_ptr[dev];
  return OK;
}

}  // namespace

extern "C" int dinfer_gemm_mid_m_static_init(void) {
  void* p;
  return scratch_on_current_device(&p);
}

extern "C" int64_t dinfer_gemm_mid_m_static_capacity(void) { return DINFER_GEMM_MID_STATIC_BYTES; }

extern "C" int dinfer_gemm_mid_m_static(int out_f32, const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                                        int64_t ldc, int64_t M, int64_t N, int64_t K, int gated, int ks, int rt,
                                        hipStream_t stream) {
  if (M <= 0 || N <= 0) return OK;
  void* p = nullptr;
  const int st = scratch_on_current_device(&p);
  if (st != OK) return st;
  // Nothing of the array has to start at zero: every slice writes all of its partial sums (all rows of every
  // token tile, all columns) before the second kernel, later on the same stream, reads them.
  return run_mid_m(out_f32, A, lda, W, ldw, C, ldc, M, N, K, gated, ks, rt, p, DINFER_GEMM_MID_STATIC_BYTES,
                   ERR_SCRATCH_LIMIT, stream);
}
