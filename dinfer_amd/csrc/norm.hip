// RMSNorm over the last dimension, one workgroup per row, with three optional
// fusions that each save one pass over the activations:
//   * residual add:  r = round(x + r) is written back, then the norm is taken
//     of the rounded r (the value the next layer will also read);
//   * row gather:    only the listed rows of x are normed (final norm before
//     the LM head);
//   * weight offset: y = x * inv * (w + offset), offset 0 for plain gains and
//     1 for gains stored around zero.
// ss, inv and all products are float; one rounding on store.
//
// Reference behaviour: crates/kernels/cuda/norm.cu:41-116,192-221 and
// rmsnorm_core.cuh:63-81 (inv = 1/sqrt(ss/n + eps), weight multiplies
// directly), norm.cu:69-85 (the add is rounded before it is normed).
#include "common.cuh"

using namespace dinfer;

namespace {

template <class S>
__global__ void __launch_bounds__(256) rmsnorm_kernel(const S* __restrict__ x, S* __restrict__ residual,
                                                      const int32_t* __restrict__ rows, const void* __restrict__ w,
                                                      int wf32, S* __restrict__ out, int64_t width, int64_t ld_x,
                                                      int64_t ld_res, float eps, float w_offset) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const int64_t src = rows ? (int64_t)rows[r] : r;
  const S* xr = x + src * ld_x;
  S* rr = residual ? residual + src * ld_res : nullptr;
  S* o = out + r * width;
  float ss = 0.f;
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x) {
    float v = to_f32(xr[i]);
    if (rr) {
      const S s = from_f32<S>(v + to_f32(rr[i]));
      rr[i] = s;
      v = to_f32(s);
    }
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
  const S* src2 = rr ? rr : xr;  // each thread re-reads only what it wrote itself
  for (int64_t i = threadIdx.x; i < width; i += blockDim.x)
    o[i] = from_f32<S>(to_f32(src2[i]) * inv * (ld_param<S>(w, i, wf32) + w_offset));
}

// bf16 rows whose width is a multiple of 8 and at most 256*8*ITERS: each
// thread keeps its 8-element pieces in registers between the two phases.
template <int ITERS>
__global__ void __launch_bounds__(256) rmsnorm_bf16x8_kernel(const bf16* __restrict__ x, bf16* __restrict__ residual,
                                                             const int32_t* __restrict__ rows,
                                                             const void* __restrict__ w, int wf32,
                                                             bf16* __restrict__ out, int64_t width, int64_t ld_x,
                                                             int64_t ld_res, float eps, float w_offset) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const int64_t src = rows ? (int64_t)rows[r] : r;
  const bf16x8* xr = (const bf16x8*)(x + src * ld_x);
  bf16x8* rr = residual ? (bf16x8*)(residual + src * ld_res) : nullptr;
  bf16x8* o = (bf16x8*)(out + r * width);
  const int n8 = (int)(width / 8);
  float v[ITERS][8];
  float g[ITERS][8];  // the gains: loaded with the row, not after the sum (one memory round trip less)
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = it * 256 + threadIdx.x;
    if (i < n8) {
      const bf16x8 xv = xr[i];
      if (wf32) {
        const float* wp = (const float*)w + (int64_t)i * 8;
#pragma unroll
        for (int j = 0; j < 8; ++j) g[it][j] = wp[j] + w_offset;
      } else {
        const bf16x8 wv = ((const bf16x8*)w)[i];
#pragma unroll
        for (int j = 0; j < 8; ++j) g[it][j] = (float)wv[j] + w_offset;
      }
      if (rr) {
        const bf16x8 rv = rr[i];
        bf16x8 s;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          s[j] = (bf16)((float)xv[j] + (float)rv[j]);
          v[it][j] = (float)s[j];
        }
        rr[i] = s;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[it][j] = (float)xv[j];
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += v[it][j] * v[it][j];
    }
  }
  ss = block_sum(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = it * 256 + threadIdx.x;
    if (i < n8) {
      bf16x8 y;
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = (bf16)(v[it][j] * inv * g[it][j]);
      o[i] = y;
    }
  }
}

inline bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }

}  // namespace

// x [*, width] with row stride ld_x; residual (may be null) has row stride
// ld_res and is updated in place; rows (may be null) lists the n_rows source
// rows; out is dense [n_rows, width]. w has `width` elements, float if w_f32.
extern "C" int dinfer_rmsnorm(int dtype, const void* x, void* residual, const int32_t* rows, const void* w, int w_f32,
                              void* out, int64_t n_rows, int64_t width, int64_t ld_x, int64_t ld_res, float eps,
                              float w_offset, hipStream_t stream) {
  if (n_rows <= 0) return OK;
  if (width <= 0 || ld_x < width || (residual && ld_res < width) || n_rows > 0x7fffffff) return ERR_BAD_SHAPE;
  if (dtype == DT_BF16) {
    const bool vec = width % 8 == 0 && ld_x % 8 == 0 && (!residual || ld_res % 8 == 0) && aligned16(x) &&
                     aligned16(out) && aligned16(w) && (!residual || aligned16(residual)) && width <= 256 * 8 * 4;
    const bf16* xp = (const bf16*)x;
    bf16* rp = (bf16*)residual;
    bf16* op = (bf16*)out;
    if (vec && width <= 256 * 8) {
      rmsnorm_bf16x8_kernel<1><<<(unsigned)n_rows, 256, 0, stream>>>(xp, rp, rows, w, w_f32, op, width, ld_x, ld_res,
                                                                     eps, w_offset);
    } else if (vec && width <= 256 * 8 * 2) {
      rmsnorm_bf16x8_kernel<2><<<(unsigned)n_rows, 256, 0, stream>>>(xp, rp, rows, w, w_f32, op, width, ld_x, ld_res,
                                                                     eps, w_offset);
    } else if (vec) {
      rmsnorm_bf16x8_kernel<4><<<(unsigned)n_rows, 256, 0, stream>>>(xp, rp, rows, w, w_f32, op, width, ld_x, ld_res,
                                                                     eps, w_offset);
    } else {
      rmsnorm_kernel<bf16><<<(unsigned)n_rows, 256, 0, stream>>>(xp, rp, rows, w, w_f32, op, width, ld_x, ld_res, eps,
                                                                 w_offset);
    }
  } else if (dtype == DT_F32) {
    rmsnorm_kernel<float><<<(unsigned)n_rows, 256, 0, stream>>>((const float*)x, (float*)residual, rows, w, 1,
                                                                (float*)out, width, ld_x, ld_res, eps, w_offset);
  } else {
    return ERR_BAD_DTYPE;
  }
  return launch_status();
}
