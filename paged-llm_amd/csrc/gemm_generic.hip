// C[M, N] = A[M, K] * W[N, K]^T with float accumulation, for any M, N, K and either element
// type.  This is the plain matrix product of the true 32-bit path (operands stay float: no
// reduced-precision matrix mode) and the fallback for shapes the MFMA kernels refuse.
//
// 64 x 64 output tile per workgroup of 256 threads, 4 x 4 outputs per thread, K walked in
// slabs of 16 through LDS.  Every output element is summed over k in ascending order by one
// thread, so its value does not depend on M or on the tile it falls in: the same row gives
// the same bits in any batch.
#include "common.h"

using namespace pllm;

constexpr int BM = 64, BN = 64, BK = 16;

template <typename TA, typename TC>
__global__ __launch_bounds__(256) void gemm_nt_kernel(const TA* __restrict__ A, int lda, const TA* __restrict__ W, int ldw,
                                                      TC* __restrict__ C, int ldc, int M, int N, int K) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += BK) {
    // 64 rows x 16 k per operand: 1024 elements, 4 per thread; consecutive threads walk k first.
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int idx = tid + e * 256;
      const int r = idx / BK, kk = idx % BK;
      const int k = k0 + kk;
      const int am = m0 + r, wn = n0 + r;
      As[kk][r] = (am < M && k < K) ? to_f32(A[(size_t)am * lda + k]) : 0.f;
      Ws[kk][r] = (wn < N && k < K) ? to_f32(W[(size_t)wn * ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][tm + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tn + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + tm + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tn + j;
      if (n < N) C[(size_t)m * ldc + n] = from_f32<TC>(acc[i][j]);
    }
  }
}

// out_dtype may be PLLM_F32 with bf16 operands (logits).
PLLM_API int pllm_gemm_nt(int dtype, int out_dtype, const void* A, int lda, const void* W, int ldw, void* C, int ldc,
                          int M, int N, int K, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0) return -2;
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM), block(256);
  if (dtype == PLLM_F32 && out_dtype == PLLM_F32)
    hipLaunchKernelGGL((gemm_nt_kernel<float, float>), grid, block, 0, stream, (const float*)A, lda, (const float*)W, ldw,
                       (float*)C, ldc, M, N, K);
  else if (dtype == PLLM_BF16 && out_dtype == PLLM_BF16)
    hipLaunchKernelGGL((gemm_nt_kernel<bf16, bf16>), grid, block, 0, stream, (const bf16*)A, lda, (const bf16*)W, ldw,
                       (bf16*)C, ldc, M, N, K);
  else if (dtype == PLLM_BF16 && out_dtype == PLLM_F32)
    hipLaunchKernelGGL((gemm_nt_kernel<bf16, float>), grid, block, 0, stream, (const bf16*)A, lda, (const bf16*)W, ldw,
                       (float*)C, ldc, M, N, K);
  else
    return -3;
  PLLM_RETURN_LAST_ERROR();
}
