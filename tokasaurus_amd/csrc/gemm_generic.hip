// C[M,N] = A[M,K] * W[N,K]^T (+ residual[M,N]) with plain 32-bit multiply-adds:
// the matrix product of the true 32-bit path, and the fallback of the bfloat16
// path for shapes the MFMA kernels refuse.  Operands are row-major with K
// contiguous; any M, N, K.  Each output element sums its K products in
// ascending k, whatever M is, so a row's result does not depend on the batch.
#include "common.h"

#define GT_BM 64
#define GT_BN 64
#define GT_BK 16

template <typename T, typename TO>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const T* __restrict__ A, int lda,
                                                           const T* __restrict__ W,
                                                           TO* __restrict__ C, int ldc,
                                                           const T* __restrict__ residual,
                                                           int ldr, int M, int N, int K) {
  __shared__ float As[GT_BK][GT_BM + 1];
  __shared__ float Ws[GT_BK][GT_BN + 1];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * GT_BM, n0 = blockIdx.x * GT_BN;
  const int ty = tid / 16, tx = tid % 16;
  const int lr = tid / 4, lk = (tid % 4) * 4;  // loader: row within tile, first k
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += GT_BK) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int k = k0 + lk + q;
      const int am = m0 + lr, wn = n0 + lr;
      As[lk + q][lr] = (am < M && k < K) ? to_f32<T>(A[(size_t)am * lda + k]) : 0.f;
      Ws[lk + q][lr] = (wn < N && k < K) ? to_f32<T>(W[(size_t)wn * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GT_BK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (residual) {
        // the product is materialised in the storage type, then added (x + proj)
        v = round_to<T>(v) + to_f32<T>(residual[(size_t)m * ldr + n]);
      }
      C[(size_t)m * ldc + n] = from_f32<TO>(v);
    }
  }
}

// out_f32: write C as 32-bit floats whatever the storage type (the logits).
TK_API int tk_gemm_generic(int dt, const void* A, int lda, const void* W, void* C, int ldc,
                               const void* residual, int ldr, int M, int N, int K, int out_f32,
                               hipStream_t stream) {
  TK_REQUIRE(M >= 0 && N > 0 && K > 0 && lda >= K && ldc >= N, "gemm_generic: bad sizes M=%d N=%d K=%d lda=%d ldc=%d",
             M, N, K, lda, ldc);
  TK_REQUIRE(!residual || ldr >= N, "gemm_generic: residual stride %d < N %d", ldr, N);
  if (M == 0) return 0;
  dim3 grid((N + GT_BN - 1) / GT_BN, (M + GT_BM - 1) / GT_BM);
  TK_REQUIRE(grid.y < 65536, "gemm_generic: M=%d needs too many row tiles", M);
  if (dt == TK_F32) {
    hipLaunchKernelGGL((gemm_generic_kernel<float, float>), grid, dim3(256), 0, stream,
                       (const float*)A, lda, (const float*)W, (float*)C, ldc,
                       (const float*)residual, ldr, M, N, K);
  } else if (out_f32) {
    hipLaunchKernelGGL((gemm_generic_kernel<bf16_t, float>), grid, dim3(256), 0, stream,
                       (const bf16_t*)A, lda, (const bf16_t*)W, (float*)C, ldc,
                       (const bf16_t*)residual, ldr, M, N, K);
  } else {
    hipLaunchKernelGGL((gemm_generic_kernel<bf16_t, bf16_t>), grid, dim3(256), 0, stream,
                       (const bf16_t*)A, lda, (const bf16_t*)W, (bf16_t*)C, ldc,
                       (const bf16_t*)residual, ldr, M, N, K);
  }
  TK_CHECK_LAUNCH("gemm_generic");
  return 0;
}
