// Shared device helpers for the gfx950 kernels: element types, 32-bit conversions,
// wavefront (64 lanes) and workgroup reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#define PLLM_API extern "C" __attribute__((visibility("default")))

// Element type codes shared with the Python side.
enum { PLLM_F32 = 0, PLLM_BF16 = 1 };

typedef __hip_bfloat16 bf16;

namespace pllm {

constexpr int kWave = 64;

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16 x) { return __bfloat162float(x); }

template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float x) { return __float2bfloat16(x); }  // round to nearest even

// The gate's activation in a gated product, out = act(gate) * up, chosen by the feed-forward's configuration:
// SiLU, z / (1 + exp(-z)), or GELU in its tanh form, 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))).
enum { PLLM_ACT_SILU = 0, PLLM_ACT_GELU_TANH = 1, PLLM_ACT_COUNT = 2 };

__device__ __forceinline__ float gate_activation(float z, int act) {
  if (act == PLLM_ACT_GELU_TANH) return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  return z / (1.f + expf(-z));
}

// Terms of an attention score beside the scaled dot product x = scale * q.k, for mixers that have them:
//   score(query position i, key position n, head h) = cap(x) + slopes[h] * (n - i),   cap(x) = c tanh(x / c) for c > 0,
// and a logit sinks[h] that takes part in the softmax's sum and in nothing else (a key with no value).
struct ScoreTerms {
  float cap;            // 0: the product as it is
  const float* slopes;  // [heads] floats or null
  const float* sinks;   // [heads] floats or null
  __host__ __device__ bool any() const { return cap > 0.f || slopes || sinks; }
};
__device__ __forceinline__ float capped_score(float x, float cap) { return cap > 0.f ? cap * tanhf(x / cap) : x; }

// One rotary pair turned by the angle whose cosine and sine are c and s.  Products and sums are rounded one by one (no
// fused multiply-add), in every kernel that rotates: what one kernel writes into the cache and what another computes
// for the same position are then the same bits, and equal to what plain float arithmetic gives.
__device__ __forceinline__ void rotate_pair(float lo, float hi, float c, float s, float& out_lo, float& out_hi) {
#pragma clang fp contract(off)
  out_lo = lo * c - hi * s;
  out_hi = hi * c + lo * s;
}

// Raw 16-bit pattern <-> float, for vector loads of bf16 data.
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // NaN stays NaN
  u += 0x7fffu + ((u >> 16) & 1u);                                           // round to nearest even
  return (uint16_t)(u >> 16);
}

// Reductions over a wavefront without LDS traffic or lane-index arithmetic: two swaps inside groups of
// four lanes, a mirror inside groups of 8 and of 16 (data-parallel-primitive moves; after each step all
// lanes of the group hold the group's result), then the four rows of 16 are read out and combined in row
// order.  Every lane gets the result; the order of operations is fixed.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
constexpr int kDppSwap1 = 0xB1;        // quad_perm [1, 0, 3, 2]
constexpr int kDppSwap2 = 0x4E;        // quad_perm [2, 3, 0, 1]
constexpr int kDppHalfMirror = 0x141;  // lane i <- lane 7 - i of its group of 8
constexpr int kDppMirror = 0x140;      // lane i <- lane 15 - i of its row of 16
__device__ __forceinline__ float row_lane(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<kDppSwap1>(v);
  v += dpp_move<kDppSwap2>(v);
  v += dpp_move<kDppHalfMirror>(v);
  v += dpp_move<kDppMirror>(v);
  return ((row_lane(v, 0) + row_lane(v, 16)) + row_lane(v, 32)) + row_lane(v, 48);
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<kDppSwap1>(v));
  v = fmaxf(v, dpp_move<kDppSwap2>(v));
  v = fmaxf(v, dpp_move<kDppHalfMirror>(v));
  v = fmaxf(v, dpp_move<kDppMirror>(v));
  return fmaxf(fmaxf(row_lane(v, 0), row_lane(v, 16)), fmaxf(row_lane(v, 32), row_lane(v, 48)));
}

// Sum over a workgroup whose size is a multiple of 64 (at most 1024). `scratch` holds 16 floats
// of LDS.  Every thread gets the total; the order of additions depends only on the block size.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nwaves; ++i) t += scratch[i];
  return t;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = scratch[0];
  for (int i = 1; i < nwaves; ++i) t = fmaxf(t, scratch[i]);
  return t;
}

}  // namespace pllm

// Every entry point returns the hipError_t of its launches as an int (0 = success).
#define PLLM_RETURN_LAST_ERROR() return (int)hipGetLastError()
