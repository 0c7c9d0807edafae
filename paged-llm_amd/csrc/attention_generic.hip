// Paged causal attention, plain version: one wavefront per (query token, query head), any head
// size up to 256, any page size, either element type, everything in float.  It serves the true
// 32-bit path and every shape the MFMA kernel refuses.
//
//   q            [total_q, num_heads, d] with row stride q_stride (elements)
//   k_pages      [pages, kv_heads, block_size, d]
//   v_pages      [pages, kv_heads, d, block_size]      (transposed inside a page)
//   block_tables [num_seqs, bt_stride] int32; entry i holds positions i*block_size .. +block_size-1
//   cu_seqlens_q [num_seqs+1], seq_lens_k [num_seqs] (context length including the new tokens)
// Query i of a sequence sits at position seq_len_k - num_q + i and sees keys n <= that position
// (and n > position - window when window > 0).  Query head j reads kv head j / (heads / kv_heads).
// A score may carry further terms (a cap, a slope times the distance, a sink per head: ScoreTerms).
//
// Keys are walked in tiles of 64 aligned to absolute positions 0, 64, 128, ..., so the order of
// every sum for one (token, head) is the same however the tokens were cut into steps or batched.
// Table entries past the context, and slots past it inside the last page, are never read.
#include "common.h"

using namespace pllm;

constexpr int kMaxHeadDim = 256;

template <typename T>
__global__ __launch_bounds__(64) void paged_attention_generic_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    T* __restrict__ out, int out_stride, const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ cu_seqlens_q, const int* __restrict__ seq_lens_k, int num_seqs, int num_heads,
    int num_kv_heads, int head_dim, int block_size, float scale, int window, ScoreTerms terms) {
  __shared__ float q_s[kMaxHeadDim];
  __shared__ float p_s[64];
  __shared__ int page_s[64];
  const int lane = threadIdx.x;
  const int tok = blockIdx.x, head = blockIdx.y;

  // Sequence of this token: last s with cu[s] <= tok.
  int lo = 0, hi = num_seqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu_seqlens_q[mid] <= tok) lo = mid; else hi = mid - 1;
  }
  const int seq = lo;
  const int q_begin = cu_seqlens_q[seq], num_q = cu_seqlens_q[seq + 1] - q_begin;
  const int len_k = seq_lens_k[seq];
  const int q_pos = len_k - num_q + (tok - q_begin);
  const int kvh = head / (num_heads / num_kv_heads);
  const int* bt = block_tables + (size_t)seq * bt_stride;

  for (int i = lane; i < head_dim; i += 64) q_s[i] = to_f32(q[(size_t)tok * q_stride + (size_t)head * head_dim + i]);
  __syncthreads();

  const int first_key = (window > 0 && q_pos - window + 1 > 0) ? q_pos - window + 1 : 0;
  const int dims_per_lane = (head_dim + 63) / 64;  // <= 4
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  if (terms.sinks) { m = terms.sinks[head]; l = 1.f; }          // as if one key with this score and no value had been seen
  const float slope = terms.slopes ? terms.slopes[head] : 0.f;

  for (int n0 = (first_key / 64) * 64; n0 <= q_pos; n0 += 64) {
    const int n = n0 + lane;
    const bool visible = n >= first_key && n <= q_pos;
    float s = -INFINITY;
    int page = 0;
    if (visible) {
      page = bt[n / block_size];
      const T* kr = k_pages + (((size_t)page * num_kv_heads + kvh) * block_size + (n % block_size)) * head_dim;
      float dot = 0.f;
      for (int i = 0; i < head_dim; ++i) dot = fmaf(q_s[i], to_f32(kr[i]), dot);
      s = capped_score(dot * scale, terms.cap);
      if (terms.slopes) s += slope * (float)(n - q_pos);
    }
    const float m_new = fmaxf(m, wave_max(s));   // finite: the tile holds at least one visible key
    const float alpha = expf(m - m_new);          // 0 on the first tile (without a sink)
    const float p = visible ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
    __syncthreads();
    p_s[lane] = p;
    page_s[lane] = page;
    __syncthreads();
    const int count = (q_pos - n0 + 1 < 64) ? q_pos - n0 + 1 : 64;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (r >= dims_per_lane) break;
      const int i = lane + r * 64;
      if (i >= head_dim) break;
      float a = acc[r] * alpha;
      for (int j = 0; j < count; ++j) {
        const float pj = p_s[j];
        if (pj != 0.f) {
          const int nj = n0 + j;
          a = fmaf(pj, to_f32(v_pages[(((size_t)page_s[j] * num_kv_heads + kvh) * head_dim + i) * block_size + (nj % block_size)]), a);
        }
      }
      acc[r] = a;
    }
  }
  const float inv_l = 1.f / l;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int i = lane + r * 64;
    if (r < dims_per_lane && i < head_dim)
      out[(size_t)tok * out_stride + (size_t)head * head_dim + i] = from_f32<T>(acc[r] * inv_l);
  }
}

PLLM_API int pllm_paged_attention_generic(int dtype, const void* q, int q_stride, const void* k_pages, const void* v_pages,
                                          void* out, int out_stride, const int* block_tables, int bt_stride,
                                          const int* cu_seqlens_q, const int* seq_lens_k, int num_seqs, int total_q,
                                          int num_heads, int num_kv_heads, int head_dim, int block_size, float scale,
                                          int window, float score_cap, const float* slopes, const float* sinks,
                                          hipStream_t stream) {
  if (total_q <= 0 || num_seqs <= 0) return 0;
  if (head_dim > kMaxHeadDim || head_dim <= 0 || num_kv_heads <= 0 || num_heads % num_kv_heads) return -2;
  if (!(score_cap >= 0.f)) return -2;
  const ScoreTerms terms{score_cap, slopes, sinks};
  dim3 grid(total_q, num_heads), block(64);
  if (dtype == PLLM_F32)
    hipLaunchKernelGGL(paged_attention_generic_kernel<float>, grid, block, 0, stream, (const float*)q, q_stride,
                       (const float*)k_pages, (const float*)v_pages, (float*)out, out_stride, block_tables, bt_stride,
                       cu_seqlens_q, seq_lens_k, num_seqs, num_heads, num_kv_heads, head_dim, block_size, scale, window, terms);
  else
    hipLaunchKernelGGL(paged_attention_generic_kernel<bf16>, grid, block, 0, stream, (const bf16*)q, q_stride,
                       (const bf16*)k_pages, (const bf16*)v_pages, (bf16*)out, out_stride, block_tables, bt_stride,
                       cu_seqlens_q, seq_lens_k, num_seqs, num_heads, num_kv_heads, head_dim, block_size, scale, window, terms);
  PLLM_RETURN_LAST_ERROR();
}
