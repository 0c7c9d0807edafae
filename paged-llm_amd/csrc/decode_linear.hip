// Linear layers of a decode step (at most 16 rows) in bfloat16, each fused with what surrounds it,
// because at these sizes a kernel launch costs as much as the weights take to stream:
//
//   prologue (optional)   rows = x (+ delta), the residual sum in float rounded once; the new
//                         residual is written out by workgroup 0; RMS norm of the rows in float
//   product               rows[M, K] * W[N, K]^T on the matrix cores, float accumulation
//   epilogue              plain (bfloat16 or float out) | silu(gate) * up | rotary encoding of q and
//                         k and the write of k, v into their cache pages
//
// One workgroup owns NT tiles of 16 weight rows and all of K.  Its wavefronts deal the K slabs of
// 128 round-robin; each lane fetches 64 contiguous bytes of a weight row per slab (four 16-byte
// loads) as the A operand of v_mfma_f32_16x16x32_bf16.  The first slab's weights are requested
// before the prologue runs, so the prologue hides behind HBM latency.  The rows (after the norm)
// sit in LDS and are the B operand of every wavefront.  Partial sums of the wavefronts are added
// through LDS in wave order: every output is summed in one fixed order.
#include "common.h"

using namespace pllm;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

constexpr int kSlab = 128;
constexpr int kPad = 8;            // bf16 elements of padding per LDS row (spreads rows over banks)

enum { EPI_BF16 = 0, EPI_F32 = 1, EPI_GATED = 2, EPI_ROPE_KV = 3 };

struct DecodeLinearParams {
  const bf16* x; int ldx;
  const bf16* delta; int ldd;
  const float* norm_w; float eps;
  bf16* x_out; int ldxo;
  const int* row_index;
  const bf16* W; int ldw;
  void* out; int ldo;
  int M, N, K;
  // EPI_ROPE_KV
  const int* positions; const float* cos_t; const float* sin_t; const int* slots;
  bf16* k_pages; bf16* v_pages;
  int num_heads, num_kv_heads, head_dim, block_size;
};

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

template <int NT, int EPI, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void decode_linear_kernel(const DecodeLinearParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  bf16* xs = reinterpret_cast<bf16*>(lds_raw);                 // [M][K + kPad]
  float* part = reinterpret_cast<float*>(lds_raw);             // [WAVES][NT * 256], reuses the space after the product
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int M = p.M, N = p.N, K = p.K;
  const int row_len = K + kPad;

  // ---- rows of W for this workgroup's tiles
  const bf16* wrow[NT];
  int tile_col[NT];                                            // first output column of each tile
  if (EPI == EPI_GATED) {
    const int n = min(blockIdx.x * 16 + r, N - 1);
    wrow[0] = p.W + (size_t)n * p.ldw;
    wrow[NT - 1] = p.W + (size_t)(n + N) * p.ldw;              // up rows follow the gate rows
    tile_col[0] = tile_col[NT - 1] = blockIdx.x * 16;
  } else if (EPI == EPI_ROPE_KV) {
    const int half = p.head_dim >> 1, per_head = half >> 4;
    const int head = blockIdx.x / per_head, j = blockIdx.x - head * per_head;
    tile_col[0] = head * p.head_dim + j * 16;
    tile_col[NT - 1] = tile_col[0] + half;
    wrow[0] = p.W + (size_t)(tile_col[0] + r) * p.ldw;
    wrow[NT - 1] = p.W + (size_t)(tile_col[NT - 1] + r) * p.ldw;
  } else {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      tile_col[t] = (blockIdx.x * NT + t) * 16;
      wrow[t] = p.W + (size_t)min(tile_col[t] + r, N - 1) * p.ldw;
    }
  }

  // ---- request the first slab of weights, then build the rows in LDS while it travels
  const int num_slabs = (K + kSlab - 1) / kSlab;
  bf16x8 wreg[NT][4];
  auto load_w = [&](int slab, bf16x8 (&dst)[NT][4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int kk = slab * kSlab + g * 32 + j * 8;
#pragma unroll
      for (int t = 0; t < NT; ++t) dst[t][j] = (kk < K) ? *reinterpret_cast<const bf16x8*>(wrow[t] + kk) : zero8();
    }
  };
  if (wave < num_slabs) load_w(wave, wreg);

  for (int m = wave; m < M; m += WAVES) {
    const size_t src = p.row_index ? (size_t)p.row_index[m] : (size_t)m;
    const bf16* xr = p.x + src * p.ldx;
    bf16* dst = xs + (size_t)m * row_len;
    float ss = 0.f;
    // pass 1: the (summed) row goes to LDS exactly as it is stored in bfloat16
    for (int k0 = lane * 8; k0 < K; k0 += 512) {
      bf16x8 v = *reinterpret_cast<const bf16x8*>(xr + k0);
      if (p.delta) {
        const bf16x8 d = *reinterpret_cast<const bf16x8*>(p.delta + src * p.ldd + k0);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (__bf16)((float)v[i] + (float)d[i]);       // float sum, rounded once
        if (p.x_out && blockIdx.x == 0) *reinterpret_cast<bf16x8*>(p.x_out + src * p.ldxo + k0) = v;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += (float)v[i] * (float)v[i];
      *reinterpret_cast<bf16x8*>(dst + k0) = v;
    }
    if (p.norm_w) {
      // pass 2: scale in place (each lane rereads only what it wrote)
      const float inv = rsqrtf(wave_sum(ss) / (float)K + p.eps);
      for (int k0 = lane * 8; k0 < K; k0 += 512) {
        bf16x8 v = *reinterpret_cast<const bf16x8*>(dst + k0);
        const float4 w0 = *reinterpret_cast<const float4*>(p.norm_w + k0), w1 = *reinterpret_cast<const float4*>(p.norm_w + k0 + 4);
        const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (__bf16)(((float)v[i] * inv) * w[i]);
        *reinterpret_cast<bf16x8*>(dst + k0) = v;
      }
    }
  }
  __syncthreads();

  // ---- product: this wavefront's slabs
  floatx4 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
  for (int slab = wave; slab < num_slabs; slab += WAVES) {
    bf16x8 wnext[NT][4];
    const bool more = slab + WAVES < num_slabs;
    if (more) load_w(slab + WAVES, wnext);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int kk = slab * kSlab + g * 32 + j * 8;
      const bf16x8 xb = (r < M && kk < K) ? *reinterpret_cast<const bf16x8*>(xs + (size_t)r * row_len + kk) : zero8();
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wreg[t][j], xb, acc[t], 0, 0, 0);
    }
    if (more) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j) wreg[t][j] = wnext[t][j];
    }
  }
  __syncthreads();                                              // everyone is done with the rows: reuse LDS
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) part[(size_t)wave * (NT * 256) + (t * 4 + i) * 64 + lane] = acc[t][i];
  __syncthreads();

  // ---- epilogue: work item (i, lane) holds output row m = r and tile column g * 4 + i
  if (tid >= 256) return;
  const int i = tid >> 6;                                       // lane is tid & 63 again
  auto total = [&](int t) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) s += part[(size_t)w * (NT * 256) + (t * 4 + i) * 64 + lane];
    return s;
  };
  const int m = r, c = g * 4 + i;
  if (m >= M) return;
  if (EPI == EPI_BF16 || EPI == EPI_F32) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int n = tile_col[t] + c;
      if (n < N) {
        const float v = total(t);
        if (EPI == EPI_F32) ((float*)p.out)[(size_t)m * p.ldo + n] = v;
        else ((bf16*)p.out)[(size_t)m * p.ldo + n] = __float2bfloat16(v);
      }
    }
  } else if (EPI == EPI_GATED) {
    const int n = tile_col[0] + c;
    if (n < N) {
      const float gate = total(0), up = total(NT - 1);
      ((bf16*)p.out)[(size_t)m * p.ldo + n] = __float2bfloat16((gate / (1.f + expf(-gate))) * up);
    }
  } else {  // EPI_ROPE_KV
    const int d = p.head_dim, half = d >> 1;
    const int head = tile_col[0] / d, ri = tile_col[0] - head * d + c;          // rotation index in [0, half)
    float lo = total(0), hi = total(NT - 1);
    const int nh = p.num_heads, nkv = p.num_kv_heads;
    if (head < nh + nkv) {
      // q and k are rounded to bfloat16 by the projection before they are rotated
      lo = __bfloat162float(__float2bfloat16(lo));
      hi = __bfloat162float(__float2bfloat16(hi));
      float cs = 1.f, sn = 0.f;
      if (p.cos_t) {
        const int pos = p.positions[m];
        cs = p.cos_t[(size_t)pos * half + ri];
        sn = p.sin_t[(size_t)pos * half + ri];
      }
      const bf16 out_lo = __float2bfloat16(lo * cs - hi * sn), out_hi = __float2bfloat16(hi * cs + lo * sn);
      if (head < nh) {
        bf16* q = (bf16*)p.out + (size_t)m * p.ldo + (size_t)head * d;
        q[ri] = out_lo;
        q[ri + half] = out_hi;
      } else {
        const int slot = p.slots[m];
        if (slot >= 0) {
          const int page = slot / p.block_size, off = slot - page * p.block_size;
          bf16* k = p.k_pages + (((size_t)page * nkv + (head - nh)) * p.block_size + off) * d;
          k[ri] = out_lo;
          k[ri + half] = out_hi;
        }
      }
    } else {
      const int slot = p.slots[m];
      if (slot >= 0) {
        const int page = slot / p.block_size, off = slot - page * p.block_size;
        bf16* v = p.v_pages + ((size_t)page * nkv + (head - nh - nkv)) * d * p.block_size + off;
        v[(size_t)ri * p.block_size] = __float2bfloat16(lo);
        v[(size_t)(ri + half) * p.block_size] = __float2bfloat16(hi);
      }
    }
  }
}

template <int NT, int EPI, int WAVES>
static int launch(const DecodeLinearParams& p, int blocks, size_t lds, hipStream_t stream) {
  auto kernel = decode_linear_kernel<NT, EPI, WAVES>;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(WAVES * 64), lds, stream, p);
  return (int)hipGetLastError();
}

// Largest LDS allocation of one workgroup on the current device.
PLLM_API long pllm_max_lds_bytes() {
  int dev = 0, v = 0;
  if (hipGetDevice(&dev) != hipSuccess) return -1;
  if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) return -1;
  return v;
}

// Bytes of LDS a call needs; the caller checks them against the device's limit.
PLLM_API long pllm_decode_linear_lds_bytes(int M, int K, int waves) {
  const long rows = (long)M * (K + kPad) * 2;
  const long reduce = (long)waves * 2 * 256 * 4;
  return rows > reduce ? rows : reduce;
}

PLLM_API int pllm_decode_linear(int epi, const void* x, int ldx, const void* delta, int ldd, const float* norm_w, float eps,
                                void* x_out, int ldxo, const int* row_index, const void* W, int ldw, void* out, int ldo, int M,
                                int N, int K, const int* positions, const float* cos_t, const float* sin_t, const int* slots,
                                void* k_pages, void* v_pages, int num_heads, int num_kv_heads, int head_dim, int block_size,
                                hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 16 || K <= 0 || (K & 7) || (ldx & 7) || (ldw & 7) || (delta && (ldd & 7)) || (x_out && (ldxo & 7))) return -2;
  DecodeLinearParams p;
  p.x = (const bf16*)x; p.ldx = ldx; p.delta = (const bf16*)delta; p.ldd = ldd; p.norm_w = norm_w; p.eps = eps;
  p.x_out = (bf16*)x_out; p.ldxo = ldxo; p.row_index = row_index; p.W = (const bf16*)W; p.ldw = ldw; p.out = out; p.ldo = ldo;
  p.M = M; p.N = N; p.K = K; p.positions = positions; p.cos_t = cos_t; p.sin_t = sin_t; p.slots = slots;
  p.k_pages = (bf16*)k_pages; p.v_pages = (bf16*)v_pages; p.num_heads = num_heads; p.num_kv_heads = num_kv_heads;
  p.head_dim = head_dim; p.block_size = block_size;
  const int waves = (K >= 4096) ? 16 : 8;
  const size_t lds = (size_t)pllm_decode_linear_lds_bytes(M, K, waves);
  const int tiles = (N + 15) / 16;
#define GO(NT_, EPI_, BLOCKS_)                                                        \
  return waves == 16 ? launch<NT_, EPI_, 16>(p, BLOCKS_, lds, stream) : launch<NT_, EPI_, 8>(p, BLOCKS_, lds, stream)
  switch (epi) {
    case EPI_BF16: GO(1, EPI_BF16, tiles);
    case EPI_F32: GO(1, EPI_F32, tiles);
    case EPI_GATED: GO(2, EPI_GATED, tiles);
    case EPI_ROPE_KV: {
      if (head_dim % 32 || (!slots) || !k_pages || !v_pages || N != (num_heads + 2 * num_kv_heads) * head_dim) return -2;
      GO(2, EPI_ROPE_KV, (num_heads + 2 * num_kv_heads) * (head_dim / 32));
    }
  }
#undef GO
  return -3;
}
