// C interface of libdinfer_gemm_mid: matrix products C[M,N] = A[M,K] . W[N,K]^T of 17 to 64 rows (any M <= 64),
// bf16 operands, float accumulation, the slice of A resident in LDS (gemm_mid.hip). Every function returns 0 or
// one of the error codes of common.cuh; kernels are launched on `stream` of the current device.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// Bytes of workspace dinfer_gemm_mid_m needs for these sizes (ks, rt as passed there).
int dinfer_gemm_mid_m_workspace(int64_t M, int64_t N, int64_t K, int gated, int ks, int rt, int64_t* bytes);

// The product; partial sums of the k slices go through `workspace`, which the caller owns.
int dinfer_gemm_mid_m(int out_f32, const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, int64_t M,
                      int64_t N, int64_t K, int gated, int ks, int rt, void* workspace, int64_t workspace_bytes,
                      hipStream_t stream);

// ---- For callers that cannot allocate -----------------------------------------------------------------------------
// No counterpart in the reference (rayze-ai/dinfer hands these row counts to its vendor library, which takes a
// workspace from the caller). These are for callers that may not call hipMalloc or anything that does: code under HIP
// graph capture, tight serving loops, harnesses that forbid allocation.
//
// dinfer_gemm_mid_m_static is dinfer_gemm_mid_m with the same kernels and the same result bit for bit, its partial
// sums in a device array that is part of the library (DINFER_GEMM_MID_STATIC_BYTES on every GPU the library is
// loaded on, held until the process ends) instead of a workspace argument. It allocates and frees nothing, in
// device or pinned memory. Sizes whose partial sums (slices x 16-row-padded M x N floats, N doubled when gated:
// what dinfer_gemm_mid_m_workspace reports) exceed the array are refused with ERR_SCRATCH_LIMIT (6) and nothing
// is launched. The limit holds the down projections of 8B, 14B and 32B sized models at 64 rows.
//
// All calls on one GPU share that GPU's array, and a call leaves its partial sums behind: two calls whose kernels
// may overlap on one GPU (different streams, or graphs replayed side by side) race; calls on one stream are
// ordered and safe. Nothing in the array has to start at zero, so nothing is cleared.
//
// dinfer_gemm_mid_m_static_init looks the array's address up for the current device; call it once per device at
// set-up. The product's first call on a device does the same if it was not called, which a caller under graph
// capture should not rely on.
#define DINFER_GEMM_MID_STATIC_BYTES (32 << 20)
int dinfer_gemm_mid_m_static_init(void);
int64_t dinfer_gemm_mid_m_static_capacity(void);
int dinfer_gemm_mid_m_static(int out_f32, const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc,
                             int64_t M, int64_t N, int64_t K, int gated, int ks, int rt, hipStream_t stream);

#ifdef __cplusplus
}
#endif
