// C[M, N] = X[M, K] * W[N, K]^T in bfloat16 with float accumulation for up to 64 rows, float or
// bfloat16 out.  The engine uses it where it wants float results for more rows than the fused
// decode kernel takes (logits of many rows); it streams the weights once.
//
// One workgroup of 4 wavefronts owns NT tiles of 16 weight rows.  The wavefronts split K between
// them in interleaved slabs of 128 and each multiplies its slab with v_mfma_f32_16x16x32_bf16: the
// weight tile is the A operand (16 rows x 32 k), the rows of X are the B operand (32 k x 16 rows),
// both fetched from global memory with 16-byte loads laid out so that the four lanes that share a
// row read 64 contiguous bytes per instruction.  The four partial sums are added through LDS in
// wave order and written once: every output is summed in one fixed order.
#include "common.h"

using namespace pllm;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

constexpr int kWaves = 4;
constexpr int kSlab = 128;  // k elements one wavefront consumes per step

__device__ __forceinline__ bf16x8 load8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

template <int MT, int NT>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const bf16* __restrict__ X, int ldx, const bf16* __restrict__ W, int ldw,
                                                          void* __restrict__ C, int ldc, int M, int N, int K, int out_f32) {
  __shared__ float part[kWaves][NT * MT * 256];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int n_base = blockIdx.x * NT * 16;

  const bf16* wrow[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) wrow[t] = W + (size_t)min(n_base + t * 16 + r, N - 1) * ldw;   // clamped; masked at the store

  floatx4 acc[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[t][m] = floatx4{0.f, 0.f, 0.f, 0.f};

  for (int ks = wave * kSlab; ks < K; ks += kWaves * kSlab) {
    bf16x8 wreg[NT][4], xreg[MT][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int kk = ks + j * 32 + g * 8;
      const bool in_k = kk < K;                               // K is a multiple of 8: whole pieces only
#pragma unroll
      for (int t = 0; t < NT; ++t) wreg[t][j] = in_k ? load8(wrow[t] + kk) : zero8();
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const int row = m * 16 + r;
        xreg[m][j] = (in_k && row < M) ? load8(X + (size_t)row * ldx + kk) : zero8();
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m)
          acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wreg[t][j], xreg[m][j], acc[t][m], 0, 0, 0);
  }

  // acc[t][m][i] is the element (weight row g*4 + i of tile t, X row m*16 + r).
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int i = 0; i < 4; ++i) part[wave][((t * MT + m) * 4 + i) * 64 + lane] = acc[t][m][i];
  __syncthreads();

  constexpr int kEntries = NT * MT * 4;
  for (int e = wave; e < kEntries; e += kWaves) {
    const int i = e & 3, m = (e >> 2) % MT, t = (e >> 2) / MT;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) v += part[w][e * 64 + lane];
    const int row = m * 16 + r;
    const int n = n_base + t * 16 + g * 4 + i;
    if (row < M && n < N) {
      if (out_f32) ((float*)C)[(size_t)row * ldc + n] = v;
      else ((bf16*)C)[(size_t)row * ldc + n] = __float2bfloat16(v);
    }
  }
}

template <int MT, int NT>
static int launch(const bf16* X, int ldx, const bf16* W, int ldw, void* C, int ldc, int M, int N, int K, int out_f32,
                  hipStream_t stream) {
  dim3 grid((N + NT * 16 - 1) / (NT * 16)), block(256);
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, NT>), grid, block, 0, stream, X, ldx, W, ldw, C, ldc, M, N, K, out_f32);
  return (int)hipGetLastError();
}

PLLM_API int pllm_gemm_skinny(const void* X, int ldx, const void* W, int ldw, void* C, int ldc, int M, int N, int K,
                              int out_f32, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || (K & 7) || (ldx & 7) || (ldw & 7)) return -2;
  const bf16* x = (const bf16*)X;
  const bf16* w = (const bf16*)W;
  switch ((M + 15) / 16) {
    case 1: return launch<1, 1>(x, ldx, w, ldw, C, ldc, M, N, K, out_f32, stream);
    case 2: return launch<2, 1>(x, ldx, w, ldw, C, ldc, M, N, K, out_f32, stream);
    case 3: return launch<3, 2>(x, ldx, w, ldw, C, ldc, M, N, K, out_f32, stream);
    default: return launch<4, 2>(x, ldx, w, ldw, C, ldc, M, N, K, out_f32, stream);
  }
}
