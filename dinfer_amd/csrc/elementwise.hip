// Embedding row gather, gated activation (SwiGLU), residual add and dtype
// widening. All of them are memory-bound; rows are moved in 16-byte pieces
// when sizes and pointers allow it.
//
// Reference behaviour: crates/kernels/cuda/activation.cu:8-16,80-99,121-129
// (silu(x) = x / (1 + exp(-x)), an id outside [0, vocab) reads row 0) and
// crates/kernels/cuda/elementwise.cu:42-46 (add in float, one rounding).
#include "common.cuh"

using namespace dinfer;

namespace {

template <class S>
__global__ void __launch_bounds__(256) embedding_kernel(const int32_t* __restrict__ ids, const S* __restrict__ table,
                                                        S* __restrict__ out, int64_t vocab, int64_t width, int vec_ok,
                                                        const int32_t* __restrict__ from,
                                                        const int32_t* __restrict__ last) {
  const int64_t t = blockIdx.x;
  // from[t] >= 0: the token is not known to the host yet, it is that one of the tokens the step before sampled
  int64_t id = ids[t];
  if (from) {
    const int32_t at = from[t];
    if (at >= 0) id = last[at];
  }
  if (id < 0 || id >= vocab) id = 0;
  const S* src = table + id * width;
  S* dst = out + t * width;
  if (vec_ok) {
    const int64_t n16 = width * (int64_t)sizeof(S) / 16;
    const uint4* s4 = (const uint4*)src;
    uint4* d4 = (uint4*)dst;
    for (int64_t i = threadIdx.x; i < n16; i += blockDim.x) d4[i] = s4[i];
  } else {
    for (int64_t i = threadIdx.x; i < width; i += blockDim.x) dst[i] = src[i];
  }
}

__device__ __forceinline__ float silu(float x) { return x / (1.f + expf(-x)); }

// in [T, 2*inter] with row stride ld_in: gate = cols [0, inter), up = cols [inter, 2*inter).
template <class S>
__global__ void __launch_bounds__(256) swiglu_kernel(const S* __restrict__ in, S* __restrict__ out, int64_t inter,
                                                     int64_t ld_in) {
  const int64_t t = blockIdx.y;
  const S* g = in + t * ld_in;
  const S* u = g + inter;
  S* o = out + t * inter;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < inter; i += (int64_t)gridDim.x * blockDim.x)
    o[i] = from_f32<S>(silu(to_f32(g[i])) * to_f32(u[i]));
}

// 8 bf16 per thread and iteration; needs inter % 8 == 0 and 16-byte aligned rows.
__global__ void __launch_bounds__(256) swiglu_bf16x8_kernel(const bf16* __restrict__ in, bf16* __restrict__ out,
                                                            int64_t inter, int64_t ld_in) {
  const int64_t t = blockIdx.y;
  const bf16x8* g = (const bf16x8*)(in + t * ld_in);
  const bf16x8* u = (const bf16x8*)(in + t * ld_in + inter);
  bf16x8* o = (bf16x8*)(out + t * inter);
  const int64_t n8 = inter / 8;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += (int64_t)gridDim.x * blockDim.x) {
    const bf16x8 gv = g[i], uv = u[i];
    bf16x8 r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = (bf16)(silu((float)gv[j]) * (float)uv[j]);
    o[i] = r;
  }
}

// dst[i] = round(float(dst[i]) + float(src[i]))
template <class S>
__global__ void __launch_bounds__(256) add_inplace_kernel(S* __restrict__ dst, const S* __restrict__ src, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = from_f32<S>(to_f32(dst[i]) + to_f32(src[i]));
}

template <class S>
__global__ void __launch_bounds__(256) widen_kernel(const S* __restrict__ src, float* __restrict__ dst, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = to_f32(src[i]);
}

// x[r][c] = cap * tanh(x[r][c] * scale / cap) (cap <= 0: x * scale), in place, rows of `width` at stride ld
template <class S>
__global__ void __launch_bounds__(256) scale_softcap_kernel(S* __restrict__ x, int64_t ld, int64_t width, float scale,
                                                            float cap) {
  S* row = x + (int64_t)blockIdx.y * ld;
  const float inv = cap > 0.f ? 1.f / cap : 0.f;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < width; i += (int64_t)gridDim.x * blockDim.x) {
    float v = to_f32(row[i]) * scale;
    if (cap > 0.f) v = cap * tanhf(v * inv);
    row[i] = from_f32<S>(v);
  }
}

// Fills n 32-bit words; used where a captured graph must not hold a memset node.
__global__ void __launch_bounds__(256) fill_u32_kernel(uint32_t* __restrict__ dst, uint32_t v, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    dst[i] = v;
}

inline unsigned blocks_for(int64_t n, int per_block, unsigned cap) {
  int64_t b = (n + per_block - 1) / per_block;
  if (b < 1) b = 1;
  return (unsigned)(b > cap ? cap : b);
}

}  // namespace

// src, last (both or neither): where src[t] >= 0, token t's id is last[src[t]] instead of ids[t].
extern "C" int dinfer_embedding(int dtype, const int32_t* ids, const void* table, void* out, int64_t tokens,
                                int64_t vocab, int64_t width, const int32_t* src, const int32_t* last,
                                hipStream_t stream) {
  if (tokens <= 0) return OK;
  if (vocab <= 0 || width <= 0 || tokens > 0x7fffffff || (!src != !last)) return ERR_BAD_SHAPE;
  DINFER_DISPATCH_DTYPE(dtype, {
    const bool vec = (width * sizeof(S)) % 16 == 0 && ((uintptr_t)table % 16 == 0) && ((uintptr_t)out % 16 == 0);
    embedding_kernel<S><<<(unsigned)tokens, 256, 0, stream>>>(ids, (const S*)table, (S*)out, vocab, width, vec ? 1 : 0,
                                                              src, last);
  });
  return launch_status();
}

// act: 0 = silu. Anything else is refused.
extern "C" int dinfer_gated_act(int dtype, int act, const void* in, void* out, int64_t tokens, int64_t inter,
                                int64_t ld_in, hipStream_t stream) {
  if (tokens <= 0) return OK;
  if (act != 0) return ERR_UNSUPPORTED;
  if (inter <= 0 || ld_in < 2 * inter || tokens > 65535 * 1024LL) return ERR_BAD_SHAPE;
  // grid.y is limited to 65535 rows; larger batches are cut into slabs
  for (int64_t t0 = 0; t0 < tokens; t0 += 65535) {
    const int64_t nt = tokens - t0 < 65535 ? tokens - t0 : 65535;
    if (dtype == DT_BF16) {
      const bf16* ip = (const bf16*)in + t0 * ld_in;
      bf16* op = (bf16*)out + t0 * inter;
      const bool vec = inter % 8 == 0 && ld_in % 8 == 0 && ((uintptr_t)ip % 16 == 0) && ((uintptr_t)op % 16 == 0);
      if (vec)
        swiglu_bf16x8_kernel<<<dim3(blocks_for(inter / 8, 256, 64), (unsigned)nt), 256, 0, stream>>>(ip, op, inter, ld_in);
      else
        swiglu_kernel<bf16><<<dim3(blocks_for(inter, 256, 64), (unsigned)nt), 256, 0, stream>>>(ip, op, inter, ld_in);
    } else if (dtype == DT_F32) {
      swiglu_kernel<float><<<dim3(blocks_for(inter, 256, 64), (unsigned)nt), 256, 0, stream>>>(
          (const float*)in + t0 * ld_in, (float*)out + t0 * inter, inter, ld_in);
    } else {
      return ERR_BAD_DTYPE;
    }
  }
  return launch_status();
}

// x[:rows, :width] (row stride ld) *= scale, then softly capped at +-cap (cap * tanh(x / cap); cap <= 0: no cap).
extern "C" int dinfer_scale_softcap(int dtype, void* x, int64_t ld, int64_t rows, int64_t width, float scale, float cap,
                                    hipStream_t stream) {
  if (rows <= 0 || width <= 0) return OK;
  if (ld < width || rows > 65535) return ERR_BAD_SHAPE;
  DINFER_DISPATCH_DTYPE(dtype, {
    scale_softcap_kernel<S><<<dim3(blocks_for(width, 256, 256), (unsigned)rows), 256, 0, stream>>>((S*)x, ld, width, scale, cap);
  });
  return launch_status();
}

extern "C" int dinfer_add_inplace(int dtype, void* dst, const void* src, int64_t n, hipStream_t stream) {
  if (n <= 0) return OK;
  DINFER_DISPATCH_DTYPE(dtype, {
    add_inplace_kernel<S><<<blocks_for(n, 256, 4096), 256, 0, stream>>>((S*)dst, (const S*)src, n);
  });
  return launch_status();
}

extern "C" int dinfer_widen(int dtype, const void* src, float* dst, int64_t n, hipStream_t stream) {
  if (n <= 0) return OK;
  DINFER_DISPATCH_DTYPE(dtype, {
    widen_kernel<S><<<blocks_for(n, 256, 4096), 256, 0, stream>>>((const S*)src, dst, n);
  });
  return launch_status();
}

extern "C" int dinfer_fill_u32(void* dst, uint32_t value, int64_t n_words, hipStream_t stream) {
  if (n_words <= 0) return OK;
  fill_u32_kernel<<<blocks_for(n_words, 256, 4096), 256, 0, stream>>>((uint32_t*)dst, value, n_words);
  return launch_status();
}
