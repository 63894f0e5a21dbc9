// Shared device helpers for the gfx950 kernels: storage types, 64-wide wave
// reductions, workgroup reductions through LDS, and host-side argument checks.
//
// Every kernel is templated on the storage type S (float or bf16); arithmetic
// is always done in float. A value is rounded to S exactly once, on store.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dinfer {

using bf16 = __bf16;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int WAVE = 64;

// dtype codes of the C ABI
enum : int { DT_F32 = 0, DT_BF16 = 1 };

// Error codes of the C ABI. 0 is success; the Python side turns the others
// into exceptions with the text of dinfer_error_string().
enum : int {
  OK = 0,
  ERR_BAD_DTYPE = 1,
  ERR_BAD_SHAPE = 2,
  ERR_UNSUPPORTED = 3,
  ERR_LAUNCH = 4,
  ERR_WORKSPACE = 5,
  ERR_SCRATCH_LIMIT = 6,
};

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return (float)v; }

template <class S>
__device__ __forceinline__ S from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16 from_f32<bf16>(float v) { return (bf16)v; }

// A norm gain or similar small parameter vector may be stored in 32-bit even
// when activations are bf16; `wf32` selects the element type at run time.
template <class S>
__device__ __forceinline__ float ld_param(const void* p, int64_t i, bool wf32) {
  return wf32 ? ((const float*)p)[i] : to_f32(((const S*)p)[i]);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}

// Workgroup-wide sum; every thread gets the result. `red` has >= 16 floats.
// blockDim.x must be a multiple of 64 and at most 1024.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) red[w] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += red[i];  // fixed order: same result in every thread
  return t;
}
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) red[w] = v;
  __syncthreads();
  float t = -INFINITY;
  for (int i = 0; i < nw; ++i) t = fmaxf(t, red[i]);
  return t;
}

static inline int launch_status() { return hipGetLastError() == hipSuccess ? OK : ERR_LAUNCH; }

// One rotated pair (a, b) -> (a cos - b sin, b cos + a sin) and one step of a sum of squares, with their roundings
// spelled out: the kernels that norm and rotate a head (alone, or on the way into an attention kernel) must leave the
// same bits, whatever the compiler would fuse in each of them.
__device__ __forceinline__ float rotated_first(float a, float b, float c, float s) {
#pragma clang fp contract(off)
  const float t = b * s;
  return __builtin_fmaf(a, c, -t);
}
__device__ __forceinline__ float rotated_second(float a, float b, float c, float s) {
#pragma clang fp contract(off)
  const float t = a * s;
  return __builtin_fmaf(b, c, t);
}
__device__ __forceinline__ float add_square(float sum, float x) { return __builtin_fmaf(x, x, sum); }

// K pages. One kv head of one page is [D / 8][page][8]: the 8-element pieces of consecutive keys lie
// next to each other, so lanes that read the same piece of consecutive keys (the rows of an MFMA
// operand) read contiguous memory. Needs D % 8 == 0. Offset of element d of the key at `off`:
__host__ __device__ __forceinline__ int64_t k_page_offset(int off, int d, int page) {
  return ((int64_t)(d >> 3) * page + off) * 8 + (d & 7);
}

}  // namespace dinfer

#define DINFER_DISPATCH_DTYPE(dtype, ...)         \
  do {                                            \
    if ((dtype) == dinfer::DT_F32) {              \
      using S = float;                            \
      __VA_ARGS__;                                \
    } else if ((dtype) == dinfer::DT_BF16) {      \
      using S = dinfer::bf16;                     \
      __VA_ARGS__;                                \
    } else {                                      \
      return dinfer::ERR_BAD_DTYPE;               \
    }                                             \
  } while (0)
