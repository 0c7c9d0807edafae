// Next-token choice from float logits [rows, vocab], one workgroup of 1024 threads per row.
//
// Greedy rows (temperature < 1e-5) take the first index of the maximum.  Other rows draw from
//   softmax(logits / max(T, 1e-5)) restricted by top-k and top-p,
// where, as in pagedllm/sampler.py:21-35, a token stays if fewer than top_k tokens have a larger
// logit and the probability mass of the tokens with a larger logit is at most top_p.  Both tests
// depend only on the token's own logit, so the kept set is {logit >= threshold}; the threshold is
// found by bisection over the ordered bit patterns of float (32 passes over the row, which stays
// in cache), not by a sort.  Tokens with equal logits are kept or dropped together.
//
// The draw is the inverse CDF in index order with one uniform number per row from Philox4x32-10
// keyed by (seed, request key, step), so a request's tokens do not depend on its neighbours.
#include "common.h"

using namespace pllm;

constexpr int kThreads = 1024;

__device__ __forceinline__ uint32_t mulhi32(uint32_t a, uint32_t b) { return __umulhi(a, b); }

// Philox4x32 with 10 rounds (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3").
__device__ __forceinline__ uint32_t philox_first_word(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = mulhi32(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = mulhi32(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n1 = lo1, n2 = hi0 ^ c3 ^ k1, n3 = lo0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  return c0;
}

// Order-preserving map float -> uint32 (larger float, larger key).
__device__ __forceinline__ uint32_t float_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct ArgMax { float v; int i; };
__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {
  return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

__device__ ArgMax block_argmax(ArgMax a, ArgMax* scratch) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    ArgMax b; b.v = __shfl_xor(a.v, o, 64); b.i = __shfl_xor(a.i, o, 64);
    a = better(a, b);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = a;
  __syncthreads();
  ArgMax t = scratch[0];
  for (int w = 1; w < nwaves; ++w) t = better(t, scratch[w]);
  if (t.i == 0x7fffffff) t.i = 0;  // a row of NaN: still a valid token id
  return t;
}

__global__ __launch_bounds__(kThreads) void sample_kernel(const float* __restrict__ logits, int vocab, const float* __restrict__ temperature,
                                                          const int* __restrict__ top_k, const float* __restrict__ top_p,
                                                          const long long* __restrict__ request_key, const int* __restrict__ step,
                                                          unsigned long long seed, int* __restrict__ out) {
  __shared__ float fscratch[16];
  __shared__ ArgMax ascratch[16];
  __shared__ float chunk_sum[kThreads];
  __shared__ int chosen;
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* z = logits + (size_t)row * vocab;

  ArgMax best; best.v = -INFINITY; best.i = 0x7fffffff;
  for (int i = tid; i < vocab; i += kThreads) { ArgMax c; c.v = z[i]; c.i = i; best = better(best, c); }
  best = block_argmax(best, ascratch);
  const float temp = temperature[row];
  if (temp < 1e-5f) {
    if (tid == 0) out[row] = best.i;
    return;
  }
  const float inv_t = 1.f / fmaxf(temp, 1e-5f);
  const float zmax = best.v;
  // weight of token i (unnormalised probability)
  auto weight = [&](float v) { return expf((v - zmax) * inv_t); };

  float part = 0.f;
  for (int i = tid; i < vocab; i += kThreads) part += weight(z[i]);
  const float total = block_sum(part, fscratch);

  int k = top_k[row];
  if (k <= 0 || k > vocab) k = vocab;
  const float p = top_p[row];
  uint32_t threshold = 0;  // keep tokens whose key >= threshold; 0 keeps all
  if (k < vocab || p < 1.f) {
    // Largest key value `c` whose tokens fail neither test is monotone: find the smallest kept key.
    // kept(v)  <=>  count(key > v) < k  and  mass(key > v) <= p * total.   Bisection on v.
    uint32_t lo_key = 0, hi_key = float_key(zmax);  // hi_key is always kept (nothing is larger)
    while (lo_key < hi_key) {
      const uint32_t mid = lo_key + ((hi_key - lo_key) >> 1);
      float cnt = 0.f, mass = 0.f;
      for (int i = tid; i < vocab; i += kThreads) {
        const float v = z[i];
        if (float_key(v) > mid) { cnt += 1.f; mass += weight(v); }
      }
      cnt = block_sum(cnt, fscratch);
      mass = block_sum(mass, fscratch);
      const bool kept = cnt < (float)k && mass <= p * total;
      if (kept) hi_key = mid; else lo_key = mid + 1;
    }
    threshold = hi_key;
  }

  // Inverse CDF in index order over contiguous chunks, one chunk per thread.
  const int chunk = (vocab + kThreads - 1) / kThreads;
  const int begin = tid * chunk, end = min(begin + chunk, vocab);
  float mine = 0.f;
  for (int i = begin; i < end; ++i) { const float v = z[i]; if (float_key(v) >= threshold) mine += weight(v); }
  chunk_sum[tid] = mine;
  if (tid == 0) chosen = -1;
  __syncthreads();
  if (tid == 0) {
    const long long key = request_key[row];
    const uint32_t bits = philox_first_word((uint32_t)step[row], 0u, (uint32_t)key, (uint32_t)(key >> 32),
                                            (uint32_t)seed, (uint32_t)(seed >> 32));
    const float u = (float)(bits >> 8) * (1.0f / 16777216.0f);  // [0, 1)
    float kept_total = 0.f;
    for (int t = 0; t < kThreads; ++t) kept_total += chunk_sum[t];
    const float target = u * kept_total;
    // Find the chunk, then the token inside it.
    float run = 0.f;
    int t = 0;
    for (; t < kThreads - 1; ++t) {
      if (run + chunk_sum[t] > target) break;
      run += chunk_sum[t];
    }
    int pick = -1, last_kept = -1;
    const int b = t * chunk, e = min(b + chunk, vocab);
    for (int i = b; i < e; ++i) {
      const float v = z[i];
      if (float_key(v) < threshold) continue;
      last_kept = i;
      run += weight(v);
      if (run > target) { pick = i; break; }
    }
    if (pick < 0) pick = last_kept >= 0 ? last_kept : best.i;  // rounding at the very end of the range
    chosen = pick;
  }
  __syncthreads();
  if (tid == 0) out[row] = chosen;
}

PLLM_API int pllm_sample(const float* logits, int rows, int vocab, const float* temperature, const int* top_k,
                         const float* top_p, const long long* request_key, const int* step, unsigned long long seed,
                         int* out, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0) return -2;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(kThreads), 0, stream, logits, vocab, temperature, top_k, top_p,
                     request_key, step, seed, out);
  PLLM_RETURN_LAST_ERROR();
}

// Greedy only: first index of the maximum of each row.
__global__ __launch_bounds__(kThreads) void argmax_kernel(const float* __restrict__ logits, int vocab, int* __restrict__ out) {
  __shared__ ArgMax ascratch[16];
  const float* z = logits + (size_t)blockIdx.x * vocab;
  ArgMax best; best.v = -INFINITY; best.i = 0x7fffffff;
  if ((vocab & 3) == 0 && (reinterpret_cast<uintptr_t>(z) & 15) == 0) {
    // pieces of four, four pieces requested before the first is looked at: the row is read by one compute
    // unit, so what counts is how many loads are under way
    const float4* z4 = reinterpret_cast<const float4*>(z);
    const int pieces = vocab >> 2;
    for (int i = threadIdx.x; i < pieces; i += 4 * kThreads) {
      float4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = i + u * kThreads;
        v[u] = j < pieces ? z4[j] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = i + u * kThreads;
        if (j >= pieces) continue;
        const float e[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
        for (int k = 0; k < 4; ++k) { ArgMax c; c.v = e[k]; c.i = 4 * j + k; best = better(best, c); }
      }
    }
  } else {
    for (int i = threadIdx.x; i < vocab; i += kThreads) { ArgMax c; c.v = z[i]; c.i = i; best = better(best, c); }
  }
  best = block_argmax(best, ascratch);
  if (threadIdx.x == 0) out[blockIdx.x] = best.i;
}

PLLM_API int pllm_argmax(const float* logits, int rows, int vocab, int* out, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0) return -2;
  hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(kThreads), 0, stream, logits, vocab, out);
  PLLM_RETURN_LAST_ERROR();
}
