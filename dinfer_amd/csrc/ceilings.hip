// What this chip delivers to a kernel that does nothing else: the two ceilings a measurement is priced against
// beside the vendor's figures.
//
//   stream_read   every workgroup reads its share of a buffer with 16-byte loads, several in flight a lane, and
//                 keeps a sum so that the loads cannot be dropped: bytes / time is the HBM read rate a streaming
//                 kernel can reach (the buffer is far larger than the caches).
//   mfma_loop     every wave runs chains of independent v_mfma_f32_32x32x16_bf16 on registers, no memory at all:
//                 flops / time is the dense bf16 matrix rate the matrix pipes sustain at the clock they hold.
//                 (Measured on MI355X: 2.1 PFLOP/s with this instruction, 1.3 to 1.4 with v_mfma_f32_16x16x32_bf16,
//                 whatever the number of chains and waves: the smaller tile does not reach the larger one's rate.)
//
// Reference behaviour: the reference prices its kernels against measured copy and matrix rates in its micro-benches
// (crates/kernels/benches, cold_shape); these two kernels are the same two measurements for gfx950.
#include "common.cuh"

using namespace dinfer;

namespace {

constexpr int READ_THREADS = 512;
constexpr int READ_AHEAD = 4;   // 16-byte loads in flight a lane

// A workgroup reads 32 KB in one piece (four loads a lane, 8 KB apart), then the piece a whole grid further on.
// (Eight loads a lane, each a grid apart, with workgroups of 256 reach 6.2 TB/s where this form reaches 7.0.)
__global__ void __launch_bounds__(READ_THREADS) stream_read_kernel(const f32x4* __restrict__ p, int64_t n16,
                                                                   float* __restrict__ out) {
  constexpr int64_t PIECE = (int64_t)READ_THREADS * READ_AHEAD;
  const int64_t stride = (int64_t)gridDim.x * PIECE;
  int64_t i = (int64_t)blockIdx.x * PIECE + threadIdx.x;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (; i + (READ_AHEAD - 1) * READ_THREADS < n16; i += stride) {
    f32x4 v[READ_AHEAD];
#pragma unroll
    for (int j = 0; j < READ_AHEAD; ++j) v[j] = __builtin_nontemporal_load(p + i + j * READ_THREADS);
#pragma unroll
    for (int j = 0; j < READ_AHEAD; ++j) acc += v[j];
  }
  // the last, incomplete piece
  for (int j = 0; j < READ_AHEAD; ++j)
    if (i + j * READ_THREADS < n16) acc += __builtin_nontemporal_load(p + i + j * READ_THREADS);
  const float s = wave_sum(acc[0] + acc[1] + acc[2] + acc[3]);
  if ((threadIdx.x & 63) == 0) out[blockIdx.x * (READ_THREADS / 64) + (threadIdx.x >> 6)] = s;
}

constexpr int CHAINS = 4;   // independent accumulators a wave: enough to hide the latency of one MFMA

__global__ void __launch_bounds__(256) mfma_loop_kernel(int iters, float* __restrict__ out) {
  bf16x8 a, b;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    a[e] = (bf16)(0.37f * (float)((threadIdx.x * 7 + e * 13) % 31 - 15));
    b[e] = (bf16)(0.11f * (float)((threadIdx.x * 5 + e * 3) % 29 - 14));
  }
  f32x16 acc[CHAINS];
#pragma unroll
  for (int c = 0; c < CHAINS; ++c)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[c][e] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int c = 0; c < CHAINS; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < CHAINS; ++c)
#pragma unroll
    for (int e = 0; e < 16; ++e) s += acc[c][e];
  out[(int64_t)blockIdx.x * 256 + threadIdx.x] = s;   // keeps the chains alive
}

}  // namespace

// Reads `bytes` (a multiple of 16, 16-byte aligned) once with `blocks` workgroups; out: blocks * 8 floats.
extern "C" int dinfer_stream_read(const void* p, int64_t bytes, int blocks, float* out, hipStream_t stream) {
  if (!p || !out || bytes <= 0 || bytes % 16 || ((uintptr_t)p % 16) || blocks <= 0 || blocks > 1 << 20) return ERR_BAD_SHAPE;
  stream_read_kernel<<<(unsigned)blocks, READ_THREADS, 0, stream>>>((const f32x4*)p, bytes / 16, out);
  return launch_status();
}

// `blocks` workgroups of 4 waves each run iters * 4 MFMAs of 32 x 32 x 16 a wave: 2 * 32 * 32 * 16 flops each.
// out: blocks * 256 floats. *flops: what the launch computes.
extern "C" int dinfer_mfma_loop(int iters, int blocks, float* out, int64_t* flops, hipStream_t stream) {
  if (iters <= 0 || blocks <= 0 || blocks > 1 << 20 || !out) return ERR_BAD_SHAPE;
  if (flops) *flops = (int64_t)blocks * 4 * iters * CHAINS * 2 * 32 * 32 * 16;
  mfma_loop_kernel<<<(unsigned)blocks, 256, 0, stream>>>(iters, out);
  return launch_status();
}
