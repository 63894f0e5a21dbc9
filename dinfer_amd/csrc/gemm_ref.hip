// C[M,N] = A[M,K] . W[N,K]^T with float accumulation on the vector ALUs: the
// matrix product of the 32-bit path (no matrix-core instruction, no reduced
// precision mode) and the reference beside the MFMA kernels. Any M, N, K.
//
// Every output element is summed over k = 0..K-1 in ascending order by one
// thread, so a row's result does not depend on M, on the other rows of the
// batch or on where its tile lies.
//
// Reference behaviour: crates/layers/src/nn.rs:16-76 (y = x . W^T, W stored
// [out, in] row-major, float accumulation, one rounding on store).
#include "common.cuh"

using namespace dinfer;

namespace {

constexpr int BM = 64, BN = 64, BK = 16;

template <class S, class O>
__global__ void __launch_bounds__(256) gemm_ref_kernel(const S* __restrict__ A, int64_t lda, const S* __restrict__ W,
                                                       int64_t ldw, O* __restrict__ C, int64_t ldc, int M, int N,
                                                       int K) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += BK) {
    // 64 rows x 16 k per operand = 1024 elements, 4 per thread
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int idx = e * 256 + threadIdx.x;
      const int r = idx >> 4, kk = idx & 15;
      const int gk = k0 + kk;
      const int gm = m0 + r, gn = n0 + r;
      As[kk][r] = (gm < M && gk < K) ? to_f32(A[(int64_t)gm * lda + gk]) : 0.f;
      Ws[kk][r] = (gn < N && gk < K) ? to_f32(W[(int64_t)gn * ldw + gk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + ty * 4 + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn < N) C[(int64_t)gm * ldc + gn] = from_f32<O>(acc[i][j]);
    }
  }
}

}  // namespace

// out_f32 != 0: C is float whatever the input type (LM head logits).
extern "C" int dinfer_gemm_ref(int dtype, int out_f32, const void* A, int64_t lda, const void* W, int64_t ldw,
                               void* C, int64_t ldc, int64_t M, int64_t N, int64_t K, hipStream_t stream) {
  if (M <= 0 || N <= 0) return OK;
  if (K <= 0 || lda < K || ldw < K || ldc < N || M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff)
    return ERR_BAD_SHAPE;
  const int64_t gy = (M + BM - 1) / BM;
  if (gy > 65535) return ERR_UNSUPPORTED;
  const dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)gy);
  if (dtype == DT_F32) {
    gemm_ref_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)A, lda, (const float*)W, ldw, (float*)C,
                                                            ldc, (int)M, (int)N, (int)K);
  } else if (dtype == DT_BF16) {
    if (out_f32)
      gemm_ref_kernel<bf16, float><<<grid, 256, 0, stream>>>((const bf16*)A, lda, (const bf16*)W, ldw, (float*)C, ldc,
                                                             (int)M, (int)N, (int)K);
    else
      gemm_ref_kernel<bf16, bf16><<<grid, 256, 0, stream>>>((const bf16*)A, lda, (const bf16*)W, ldw, (bf16*)C, ldc,
                                                            (int)M, (int)N, (int)K);
  } else {
    return ERR_BAD_DTYPE;
  }
  return launch_status();
}
