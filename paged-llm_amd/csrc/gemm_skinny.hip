// C[M, N] = X[M, K] * W[N, K]^T in bfloat16 with float accumulation for few rows (M <= 64):
// the decode-time products, which only stream the weights once from HBM.
//
// One workgroup of 4 wavefronts owns NT tiles of 16 weight rows.  The wavefronts split K between
// them in interleaved slabs of 128 (so that at any moment they read neighbouring 256-byte pieces
// of the same rows) and each multiplies its slab with v_mfma_f32_16x16x32_bf16: the weight tile is
// the A operand (16 rows x 32 k), the activations are the B operand (32 k x 16 rows of X).  Each
// lane fetches 64 contiguous bytes of one weight row per slab with four 16-byte loads; the same k
// assignment is used for X, so the order of k inside an instruction does not matter.  The four
// partial sums are added through LDS in wave order and written once.
//
// When N is small the grid is also split over K (grid.y): every workgroup writes its partial tile
// to a workspace, and the last one to arrive for a tile (an atomic counter that it resets) adds
// the partials in split order, so the result does not depend on which one was last.
//
// GATED mode: W is [gate rows; up rows] (2*I rows); a workgroup pairs tile t of the gate rows
// with tile t of the up rows and writes silu(gate) * up, [M, I].
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

template <int MT, int NT, bool GATED>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const bf16* __restrict__ X, int ldx, const bf16* __restrict__ W, int ldw,
                                                          void* __restrict__ C, int ldc, int M, int N, int K, int out_f32,
                                                          float* __restrict__ workspace, int* __restrict__ counters) {
  __shared__ float part[kWaves][NT * MT * 256];
  __shared__ int is_last;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int ksplit = gridDim.y, kpart = blockIdx.y;
  // Rows of the tiles of this workgroup.  GATED: N is the number of gate rows (= up rows).
  constexpr int kTilesOut = GATED ? NT / 2 : NT;
  const int n_base = blockIdx.x * kTilesOut * 16;

  const bf16* wrow[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    int n = n_base + (GATED ? (t % kTilesOut) : t) * 16 + r;
    if (n >= N) n = N - 1;                                    // stay inside the matrix; masked at the store
    if (GATED && t >= kTilesOut) n += N;                      // the up rows follow the gate rows
    wrow[t] = W + (size_t)n * ldw;
  }

  floatx4 acc[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[t][m] = floatx4{0.f, 0.f, 0.f, 0.f};

  // k slabs are dealt round-robin over all wavefronts of all splits of this tile.
  const int stride = ksplit * kWaves * kSlab;
  for (int ks = (kpart * kWaves + wave) * kSlab; ks < K; ks += stride) {
    bf16x8 wreg[NT][4], xreg[MT][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int kk = ks + j * 32 + g * 8;
      const bool in_k = kk < K;                               // K is a multiple of 8: whole chunks only
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

  // Thread `tid` now owns, for every (t, m, i), the lane slot tid & 63 of entry e = tid >> 6 + 4 * j.
  constexpr int kEntries = NT * MT * 4;                        // float4-slots per lane
  float* ws = workspace;
  if (ksplit > 1) {
    // Partial tile of this split: [block][split][entry][lane]
    float* mine = ws + ((size_t)blockIdx.x * ksplit + kpart) * kEntries * 64;
    for (int e = wave; e < kEntries; e += kWaves) {
      float s = 0.f;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) s += part[w][e * 64 + lane];
      mine[e * 64 + lane] = s;
    }
    __threadfence();
    __syncthreads();
    if (tid == 0) {
      const int seen = atomicAdd(&counters[blockIdx.x], 1);
      is_last = (seen == ksplit - 1);
      if (is_last) counters[blockIdx.x] = 0;                  // ready for the next launch
    }
    __syncthreads();
    if (!is_last) return;
    __threadfence();
  }

  for (int e = wave; e < kEntries; e += kWaves) {
    // entry e = ((t * MT + m) * 4 + i)
    const int i = e & 3, m = (e >> 2) % MT, t = (e >> 2) / MT;
    if (GATED && t >= kTilesOut) continue;
    auto total = [&](int entry) {
      float s = 0.f;
      if (ksplit > 1) {
        const float* base = ws + (size_t)blockIdx.x * ksplit * kEntries * 64 + entry * 64 + lane;
        for (int p = 0; p < ksplit; ++p) s += base[(size_t)p * kEntries * 64];
      } else {
#pragma unroll
        for (int w = 0; w < kWaves; ++w) s += part[w][entry * 64 + lane];
      }
      return s;
    };
    float v = total(e);
    if (GATED) {
      const float u = total(((t + kTilesOut) * MT + m) * 4 + i);
      v = (v / (1.f + expf(-v))) * u;
    }
    const int row = m * 16 + r;
    const int n = n_base + t * 16 + g * 4 + i;
    if (row < M && n < N) {
      if (out_f32) ((float*)C)[(size_t)row * ldc + n] = v;
      else ((bf16*)C)[(size_t)row * ldc + n] = __float2bfloat16(v);
    }
  }
}

template <int MT, int NT, bool GATED>
static int launch(const bf16* X, int ldx, const bf16* W, int ldw, void* C, int ldc, int M, int N, int K, int out_f32,
                  int ksplit, float* workspace, int* counters, hipStream_t stream) {
  constexpr int tiles_out = GATED ? NT / 2 : NT;
  dim3 grid((N + tiles_out * 16 - 1) / (tiles_out * 16), ksplit), block(256);
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, NT, GATED>), grid, block, 0, stream, X, ldx, W, ldw, C, ldc, M, N, K, out_f32,
                     workspace, counters);
  return (int)hipGetLastError();
}

// Bytes of workspace and number of counters a call with these sizes needs (ksplit > 1 only).
PLLM_API long pllm_gemm_skinny_workspace_floats(int M, int N, int ksplit) {
  const long mt = (M + 15) / 16;
  const long blocks = (N + 15) / 16;
  return blocks * ksplit * (2 * mt * 4) * 64 * 2;              // upper bound over the tile choices below
}

// gated != 0: W has 2*N rows ([gate; up]) and C is [M, N] = silu(X Wg^T) * (X Wu^T).
PLLM_API int pllm_gemm_skinny(const void* X, int ldx, const void* W, int ldw, void* C, int ldc, int M, int N, int K,
                              int out_f32, int gated, int ksplit, float* workspace, int* counters, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || (K & 7) || (ldx & 7) || (ldw & 7) || ksplit < 1) return -2;
  if (ksplit > 1 && (!workspace || !counters)) return -2;
  const bf16* x = (const bf16*)X;
  const bf16* w = (const bf16*)W;
  const int mt = (M + 15) / 16;
#define PLLM_GO(MT_, NT_, G_) return launch<MT_, NT_, G_>(x, ldx, w, ldw, C, ldc, M, N, K, out_f32, ksplit, workspace, counters, stream)
  if (gated) {
    switch (mt) { case 1: PLLM_GO(1, 2, true); case 2: PLLM_GO(2, 2, true); case 3: PLLM_GO(3, 2, true); default: PLLM_GO(4, 2, true); }
  }
  switch (mt) { case 1: PLLM_GO(1, 1, false); case 2: PLLM_GO(2, 1, false); case 3: PLLM_GO(3, 2, false); default: PLLM_GO(4, 2, false); }
#undef PLLM_GO
  return -3;
}
