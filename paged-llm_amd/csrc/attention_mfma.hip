// Paged causal attention in bfloat16 on the matrix cores, for prompt portions and for decoding.
// Compiled once per head size (-DHEAD_DIM=16..256 in steps of 16).
//
// Work item = (sequence, kv head, tile of columns, partition of keys), one wavefront each.
// A *column* is a (query token, query head of the kv head's group) pair, numbered
// c = token * G + head_in_group, so the G heads that share a kv head sit side by side and every
// loaded key/value tile serves all of them: a decode step has G columns, a prompt portion
// num_q * G.  A wavefront owns 16 * NCB columns.
//
// Scores are computed transposed, S^T = K Q^T, with v_mfma_f32_16x16x32_bf16: the A operand is a
// tile of 16 keys (each lane loads 16 contiguous bytes of one key row straight from the page),
// the B operand is Q^T, held in registers for the whole kernel.  The result leaves every lane
// with 4 keys of ONE column, so the softmax statistics of a column live in one lane (and its
// three mirror lanes), and the probabilities are already in B-operand layout for O^T = V^T P^T.
// V pages are stored transposed ([d, block_size]), so the A operand of that product (16 channels
// x 32 keys) is two 8-byte loads per lane.  Nothing goes through LDS.
//
// Keys are walked in blocks of 64 aligned to absolute positions; partitions (split-K for
// decoding) are aligned multiples of 64 as well, and are merged by a second kernel.  Softmax
// statistics, the running output and the merge are float; probabilities are rounded to bfloat16
// for the second product, as the reference's kernel does (pagedllm/attention/triton_kernel.py:88).
// Page-table entries past the context are never read; values of keys that no column of the tile
// may see are zeroed, so stale or non-finite data in reused pages cannot leak (0 * NaN).
#include "common.h"

using namespace pllm;

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<16..256, multiple of 16>"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "head size must be 16..256 in steps of 16");

// -DSCORE_TERMS=1 compiles the kernels with the further terms of a score (a cap, a slope times the distance, a sink
// per head: ScoreTerms in common.h) as one more argument.  Without it there is no such argument: `terms` then names a
// constant that says "none", and everything that reads it is compiled out.
#ifndef SCORE_TERMS
#define SCORE_TERMS 0
#endif
constexpr bool kTerms = SCORE_TERMS != 0;
#if SCORE_TERMS
#define PLLM_TERMS_PARAM , ScoreTerms terms
#define PLLM_TERMS_ARG , terms
#else
#define PLLM_TERMS_PARAM
#define PLLM_TERMS_ARG
static constexpr ScoreTerms terms{0.f, nullptr, nullptr};
#endif

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float floatx4;

// Lengths and page tables are read through the constant address space: what a launch is given there does not change
// while it runs, and a load from that address space at an address that is the same in all lanes is a scalar load
// whatever else the kernel does (the compiler otherwise makes vector loads of them as soon as anything it cannot see
// through stands in front, and a vector load's result arrives only behind every vector load requested before it).
typedef const int __attribute__((address_space(4))) * ConstantInts;
__device__ __forceinline__ ConstantInts as_constant(const int* p) { return (ConstantInts)p; }

constexpr int D = HEAD_DIM;
constexpr int KSTEPS = (D + 31) / 32;   // MFMA steps over the head dimension for Q K^T
constexpr int DBLOCKS = D / 16;          // 16-channel blocks of the output
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

// v_exp_f32: 2^x, with 2^-inf = 0 and tiny results flushed to zero (harmless in a softmax).
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Further terms of the scores (kernels compiled with them): the 16 raw products of one column in a block of 64 keys
// (s[kt][i] belongs to key n0 + kt * 16 + g * 4 + i) are brought to their final form in log2 units,
//   log2(e) * (cap(scale * s) + slope * (n - query position)),
// with c tanh(x / c) = c (1 - 2 / (2^(2 log2(e) x / c) + 1)): right at both ends (2^inf = inf gives c, 2^-inf = 0
// gives -c) and within c * 2^-23 everywhere, far below what rounding the probabilities to bfloat16 leaves.  Which
// terms there are is the same for the whole launch, so each is a branch around sixteen scores, not inside them.
struct ScoreForm {
  float sl2;        // log2(e) * scale
  float cap_l2;     // log2(e) * cap                  (cap > 0)
  float cap_in;     // 2 log2(e) * scale / cap: what the raw product is multiplied by inside the power of two
  bool capped, sloped;
  __device__ __forceinline__ bool any() const { return capped || sloped; }
};
__device__ __forceinline__ ScoreForm score_form(const ScoreTerms& t, float scale) {
  constexpr float l2e = 1.4426950408889634f;
  ScoreForm f;
  f.sl2 = scale * l2e;
  f.capped = t.cap > 0.f;
  f.sloped = t.slopes != nullptr;
  f.cap_l2 = f.capped ? t.cap * l2e : 0.f;
  f.cap_in = f.capped ? 2.f * l2e * scale / t.cap : 0.f;
  return f;
}
__device__ __forceinline__ void final_scores(const ScoreForm& f, float slope_l2, float distance0, float (&s)[4][4]) {
  if (f.capped) {
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        s[kt][i] = fmaf(-2.f * f.cap_l2, __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(s[kt][i] * f.cap_in) + 1.f), f.cap_l2);
  } else {
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) s[kt][i] *= f.sl2;
  }
  if (f.sloped) {                                               // slope_l2 = log2(e) * slope; distance0 = n0 + g * 4 - query position
    const float base = slope_l2 * distance0;
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
      for (int i = 0; i < 4; ++i) s[kt][i] += fmaf(slope_l2, (float)(kt * 16 + i), base);
  }
}

// The four lanes that mirror a column are 16 lanes apart.  v_permlane16_swap exchanges the odd rows (of 16 lanes)
// of one register with the even rows of another, v_permlane32_swap the upper half of one with the lower half of
// the other; applied to two copies of a value they leave every lane with its own row's (half's) value in one
// register and the neighbour row's (half's) in the other, without a trip through the LDS crossbar.
__device__ __forceinline__ void rows_swapped(float v, float& mine_or_left, float& right_or_mine) {
  const auto t = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  mine_or_left = __uint_as_float(t[0]);
  right_or_mine = __uint_as_float(t[1]);
}
__device__ __forceinline__ void halves_swapped(float v, float& lower, float& upper) {
  const auto t = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  lower = __uint_as_float(t[0]);
  upper = __uint_as_float(t[1]);
}
__device__ __forceinline__ float group_max(float v) {      // over the 4 lanes that mirror a column
  float a, b;
  rows_swapped(v, a, b);
  v = fmaxf(a, b);
  halves_swapped(v, a, b);
  return fmaxf(a, b);
}
__device__ __forceinline__ float group_sum(float v) {      // the same four terms in the same order in every lane
  float a, b;
  rows_swapped(v, a, b);
  v = a + b;
  halves_swapped(v, a, b);
  return a + b;
}

// Partials of one (token, head, partition): [m (log2 units), l, acc[D]].
constexpr int kPartialFloats = D + 2;

template <int NCB, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void paged_attention_mfma_kernel(
    const bf16* __restrict__ q, int q_stride, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
    bf16* __restrict__ out, int out_stride, const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ cu_seqlens_q, const int* __restrict__ seq_lens_k, int num_heads, int num_kv_heads,
    int block_size, float scale, int window, int partition_size, int num_partitions, float* __restrict__ partials PLLM_TERMS_PARAM) {
  // Fetch all arguments in one go (left alone, the compiler fetches each where it is first used, and every fetch is
  // a wait of its own in the chain lengths -> page table -> keys).
  constexpr bool kLookupsTogether = D <= 64;
  if constexpr (kLookupsTogether)
    asm volatile("" ::"s"(q), "s"(q_stride), "s"(k_pages), "s"(v_pages), "s"(out), "s"(out_stride), "s"(block_tables), "s"(bt_stride),
                 "s"(cu_seqlens_q), "s"(seq_lens_k), "s"(num_heads), "s"(num_kv_heads), "s"(block_size), "s"(scale), "s"(window),
                 "s"(partition_size), "s"(num_partitions), "s"(partials));
  // The wavefront's index is the same in all its lanes; saying so keeps everything derived from it (key ranges,
  // page-table entries, page addresses) in scalar registers.
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), r = lane & 15, g = lane >> 4;
  const int bs_shift = __builtin_ctz(block_size);              // pages hold a power of two of positions
  const int seq = blockIdx.z;
  const int kvh = blockIdx.y / num_partitions, part = blockIdx.y - kvh * num_partitions;
  const int G = num_heads / num_kv_heads;
  const int q_begin = as_constant(cu_seqlens_q)[seq], num_q = as_constant(cu_seqlens_q)[seq + 1] - q_begin;
  const int len_k = as_constant(seq_lens_k)[seq];
  if constexpr (kLookupsTogether) asm volatile("" ::"s"(q_begin), "s"(num_q), "s"(len_k));       // (all three requested here, with one wait)
  const int num_cols = num_q * G;
  const int col0 = blockIdx.x * 16 * NCB;
  if (col0 >= num_cols) return;
  const int last_col = min(col0 + 16 * NCB, num_cols) - 1;
  const int pos0 = len_k - num_q;                               // position of the sequence's first query
  const int qpos_min = pos0 + col0 / G, qpos_max = pos0 + last_col / G;
  // Keys any column of this tile may see: [vis_lo, vis_hi)
  const int vis_hi = qpos_max + 1;
  const int vis_lo = (window > 0 && qpos_min - window + 1 > 0) ? qpos_min - window + 1 : 0;
  int k_lo = vis_lo & ~63, k_hi = vis_hi;
  if (partition_size > 0) {
    k_lo = max(k_lo, part * partition_size);
    k_hi = min(k_hi, (part + 1) * partition_size);
  }
  if (k_lo >= k_hi) return;                                     // nothing of this partition is visible

  // ---- this lane's column in each column block, and Q^T in B-operand layout
  int my_qpos[NCB], my_first[NCB];
  bool my_valid[NCB];
  size_t my_out[NCB];
  bf16x8 qreg[NCB][KSTEPS];
  float my_slope[NCB], my_sink[NCB];                            // (with further score terms only; both in log2 units)
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    const int c = col0 + cb * 16 + r;
    my_valid[cb] = c < num_cols;
    const int tok = my_valid[cb] ? c / G : 0, hg = my_valid[cb] ? c - tok * G : 0;
    my_qpos[cb] = my_valid[cb] ? pos0 + tok : -1;               // -1: sees nothing
    my_first[cb] = (window > 0 && my_qpos[cb] - window + 1 > 0) ? my_qpos[cb] - window + 1 : 0;
    const size_t row = (size_t)(q_begin + tok) * q_stride + (size_t)(kvh * G + hg) * D;
    my_out[cb] = (size_t)(q_begin + tok) * out_stride + (size_t)(kvh * G + hg) * D;
    if constexpr (kTerms) {
      my_slope[cb] = (terms.slopes && my_valid[cb]) ? terms.slopes[kvh * G + hg] * kLog2e : 0.f;
      my_sink[cb] = (terms.sinks && my_valid[cb]) ? terms.sinks[kvh * G + hg] * kLog2e : -INFINITY;
    }
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int dd = s * 32 + g * 8;
      qreg[cb][s] = (my_valid[cb] && dd < D) ? *reinterpret_cast<const bf16x8*>(q + row + dd) : zero8();
    }
  }

  floatx4 acc[NCB][DBLOCKS];
  float m_run[NCB], l_run[NCB];
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    m_run[cb] = -INFINITY;
    l_run[cb] = 0.f;
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) acc[cb][db] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  const float sl2 = scale * kLog2e;
  [[maybe_unused]] const ScoreForm form = score_form(terms, scale);
  if constexpr (kTerms) {
    // A head's sink enters as the state of a softmax that has seen one key with that score and no value.  Of the
    // wavefronts that share a column, the first one of the partition that holds the column's first visible key
    // has it (that partition has work for this column, and the merge counts it).
    if (terms.sinks) {
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) {
        const bool here = my_valid[cb] && wave == 0 && (partition_size == 0 || part == my_first[cb] / partition_size);
        if (here) {
          m_run[cb] = my_sink[cb];
          l_run[cb] = g == 0 ? 1.f : 0.f;                         // (the four lanes of a column are added at the end)
        }
      }
    }
  }
  ConstantInts bt = as_constant(block_tables) + (size_t)seq * bt_stride;
  const size_t page_elems = (size_t)block_size * D;             // one kv head's part of a page
  const size_t page_stride = page_elems * num_kv_heads;

  // One block = 64 keys = four tiles of 16.  All of a block's keys and values are requested
  // together, and (when the wavefronts of a workgroup share the keys) the next block is
  // requested before the current one is used, so that a wavefront waits for memory once, not once
  // per dependent step.
  struct KVBlock {
    bf16x8 k[4][KSTEPS];
    bf16x4 v[4][DBLOCKS];
    bool on[4];
  };
  const int last_tile = (k_hi - 1) & ~15;
  auto load_block = [&](KVBlock& blk, int n0) {
    // The four tiles' page-table entries first, together (a tile past the range looks the range's last tile up
    // again, so no entry past the context is read): one wait, not one per tile.
    int pages[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) pages[kt] = bt[min(n0 + kt * 16, last_tile) >> bs_shift];
    // (here, not each where its tile begins.  Only for the head sizes whose kernels have registers to spare: at 128 the
    //  form with eight wavefronts takes all 256, and holding it to this order made it spill, 112 -> 125 us for 64 sequences
    //  of 2048 keys.)
    if constexpr (kLookupsTogether) asm volatile("" ::"s"(pages[0]), "s"(pages[1]), "s"(pages[2]), "s"(pages[3]));
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      const int nk = n0 + kt * 16;
      blk.on[kt] = nk < k_hi;                                   // uniform
      if (!blk.on[kt]) continue;
      const int page = pages[kt];
      const int off = nk & (block_size - 1);
      const size_t base = (size_t)page * page_stride + (size_t)kvh * page_elems;
      const bf16* krow = k_pages + base + (size_t)(off + r) * D;
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        const int dd = s * 32 + g * 8;
        blk.k[kt][s] = (dd < D) ? *reinterpret_cast<const bf16x8*>(krow + dd) : zero8();
      }
      const bf16* vrow = v_pages + base + off + g * 4;          // + channel * block_size
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db) blk.v[kt][db] = *reinterpret_cast<const bf16x4*>(vrow + (size_t)(db * 16 + r) * block_size);
    }
  };
  auto compute_block = [&](KVBlock& blk, int n0) {
    // Every key of the block visible to every column?  Then no masking is needed.
    const bool interior = (n0 + 63 <= qpos_min) && (n0 >= (window > 0 ? max(qpos_max - window + 1, 0) : 0)) && (n0 + 64 <= k_hi) &&
                          (col0 + 16 * NCB <= num_cols);
    // ---- S^T = K Q^T for four tiles of 16 keys
    floatx4 s_t[4][NCB];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) s_t[kt][cb] = floatx4{0.f, 0.f, 0.f, 0.f};
      if (!blk.on[kt]) continue;
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
          s_t[kt][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.k[kt][s], qreg[cb][s], s_t[kt][cb], 0, 0, 0);
    }

    // ---- online softmax per column; lane holds keys n0 + kt*16 + g*4 + i of its column
    bf16x8 p_op[2][NCB];                                        // B operands of the second product
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
      float sc[4][4];
      float mx = -INFINITY;
      float mul = sl2;
      if constexpr (kTerms) {
        if (form.any()) {
          float s[4][4];
#pragma unroll
          for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) s[kt][i] = s_t[kt][cb][i];
          final_scores(form, my_slope[cb], (float)(n0 + g * 4 - my_qpos[cb]), s);
#pragma unroll
          for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) s_t[kt][cb][i] = s[kt][i];
          mul = 1.f;
        }
      }
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v = s_t[kt][cb][i] * mul;
          if (!interior) {
            const int n = n0 + kt * 16 + g * 4 + i;
            const bool vis = blk.on[kt] && n <= my_qpos[cb] && n >= my_first[cb];
            v = vis ? v : -INFINITY;
          }
          sc[kt][i] = v;
          mx = fmaxf(mx, v);
        }
      mx = group_max(mx);
      const float m_new = fmaxf(m_run[cb], mx);
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;  // a column that has seen nothing yet
      const float alpha = fast_exp2(m_run[cb] - m_safe);
      m_run[cb] = m_new;
      float psum = 0.f;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = fast_exp2(sc[kt][i] - m_safe);
          psum += p;
          p_op[kt >> 1][cb][(kt & 1) * 4 + i] = (__bf16)p;
        }
      l_run[cb] = l_run[cb] * alpha + psum;                     // per lane; mirrored lanes are added at the end
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db) acc[cb][db] *= alpha;
    }

    // ---- O^T += V^T P^T : A operand = 16 channels x 32 keys (k slots 0-3: tile 2a, 4-7: tile 2a+1)
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      if (!blk.on[2 * a]) continue;
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db) {
        bf16x8 vreg;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int kt = 2 * a + h;
          bf16x4 v4;
          if (blk.on[kt]) {
            v4 = blk.v[kt][db];
            if (!interior) {
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                const int n = n0 + kt * 16 + g * 4 + i;
                if (n >= vis_hi || n < vis_lo) v4[i] = (__bf16)0.0f;
              }
            }
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) v4[i] = (__bf16)0.0f;
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) vreg[h * 4 + i] = v4[i];
        }
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
          acc[cb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vreg, p_op[a][cb], acc[cb][db], 0, 0, 0);
      }
    }
  };

  // With several wavefronts per work item the blocks are dealt round-robin; their partial
  // results are merged through LDS below.
  constexpr int kStride = WAVES * 64;
  // Registers of one block: with small heads two blocks fit and the next one travels while the current
  // one is used; with large heads one block is all there is room for (the caller then sizes partitions
  // so that a wavefront has a single block).
  constexpr bool kTwoBlocks = 4 * KSTEPS * 4 + 4 * DBLOCKS * 2 <= 64;
  if constexpr (WAVES > 1 && kTwoBlocks) {
    KVBlock blk_a, blk_b;
    int n0 = k_lo + wave * 64;
    if (n0 < k_hi) {
      load_block(blk_a, n0);
      while (true) {
        const int n1 = n0 + kStride;
        const bool has1 = n1 < k_hi;
        if (has1) load_block(blk_b, n1);
        compute_block(blk_a, n0);
        if (!has1) break;
        const int n2 = n1 + kStride;
        const bool has2 = n2 < k_hi;
        if (has2) load_block(blk_a, n2);
        compute_block(blk_b, n1);
        if (!has2) break;
        n0 = n2;
      }
    }
  } else {
    KVBlock blk;
    for (int n0 = k_lo + (WAVES > 1 ? wave * 64 : 0); n0 < k_hi; n0 += kStride) {
      load_block(blk, n0);
      compute_block(blk, n0);
    }
  }

  if (WAVES > 1) {
    // ---- merge the wavefronts: common maximum per column, rescale, add in wave order
    extern __shared__ float lds[];
    float* m_s = lds;                                            // [WAVES][NCB * 16]
    float* l_s = lds + WAVES * NCB * 16;                         // [WAVES][NCB * 16]
    float* acc_s = lds + 2 * WAVES * NCB * 16;                   // [WAVES][NCB * DBLOCKS * 4][64]
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
      if (g == 0) m_s[(wave * NCB + cb) * 16 + r] = m_run[cb];
    __syncthreads();
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
      float mx = -INFINITY;
      for (int w = 0; w < WAVES; ++w) mx = fmaxf(mx, m_s[(w * NCB + cb) * 16 + r]);
      const float f = (m_run[cb] == -INFINITY) ? 0.f : fast_exp2(m_run[cb] - mx);
      const float l_tot = group_sum(l_run[cb]) * f;
      if (g == 0) l_s[(wave * NCB + cb) * 16 + r] = l_tot;
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc_s[((size_t)(wave * NCB + cb) * DBLOCKS * 4 + db * 4 + i) * 64 + lane] = acc[cb][db][i] * f;
    }
    __syncthreads();
    // entry e = (cb, db, i); thread (e, lane) owns column cb*16 + r, channel db*16 + g*4 + i
    for (int e = wave; e < NCB * DBLOCKS * 4; e += WAVES) {
      const int cb = e / (DBLOCKS * 4), rest = e - cb * DBLOCKS * 4, db = rest >> 2, i = rest & 3;
      const int c = col0 + cb * 16 + r;
      if (c >= num_cols) continue;
      float o = 0.f, l_tot = 0.f;
      for (int w = 0; w < WAVES; ++w) {
        o += acc_s[((size_t)(w * NCB + cb) * DBLOCKS * 4 + rest) * 64 + lane];
        l_tot += l_s[(w * NCB + cb) * 16 + r];
      }
      const int tok = c / G, hg = c - tok * G;
      if (partition_size > 0) {
        // this workgroup's partition: unnormalised sum, its maximum and its weight, for the merge kernel
        float* dst = partials + (((size_t)(q_begin + tok) * num_heads + (kvh * G + hg)) * num_partitions + part) * kPartialFloats;
        if (rest == 0 && g == 0) {
          float mx = -INFINITY;
          for (int w = 0; w < WAVES; ++w) mx = fmaxf(mx, m_s[(w * NCB + cb) * 16 + r]);
          dst[0] = mx;
          dst[1] = l_tot;
        }
        dst[2 + db * 16 + g * 4 + i] = o;
      } else {
        // (times the reciprocal, as the one-wavefront form below and the merge kernel have it: with all keys in one
        //  wavefront's block the three give the same bits)
        out[(size_t)(q_begin + tok) * out_stride + (size_t)(kvh * G + hg) * D + db * 16 + g * 4 + i] = __float2bfloat16(o * (1.f / l_tot));
      }
    }
    return;
  }

  // ---- write: lane holds channels db*16 + g*4 + i of its column
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    if (!my_valid[cb]) continue;
    const float l_tot = group_sum(l_run[cb]);
    if (partition_size > 0) {
      const int c = col0 + cb * 16 + r;
      const int tok = c / G, hg = c - tok * G;
      float* dst = partials + (((size_t)(q_begin + tok) * num_heads + (kvh * G + hg)) * num_partitions + part) * kPartialFloats;
      if (g == 0) { dst[0] = m_run[cb]; dst[1] = l_tot; }
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[2 + db * 16 + g * 4 + i] = acc[cb][db][i];
    } else {
      const float inv = 1.f / l_tot;
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db) {
        bf16x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = (__bf16)(acc[cb][db][i] * inv);
        *reinterpret_cast<bf16x4*>(out + my_out[cb] + db * 16 + g * 4) = o;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Prompt portions: one workgroup per (sequence, kv head, 128 columns), of KG groups of four wavefronts.
// A step covers 64 * KG keys: the four wavefronts of group kg work on keys kg * 64 .. kg * 64 + 63 of the
// step, each for its own 32 columns, so a step is fetched once into LDS (each wavefront fetches the 16
// keys and values of one tile: one page lookup, uniform in the wavefront) and the next step travels while
// the current one is used: global -> registers while computing, registers -> the other LDS buffer, one
// barrier per step.  With KG = 2 the two groups hold two halves of every column's softmax, merged through
// LDS at the end (group 0 first): a compute unit then holds two wavefronts per SIMD with equal work, which
// overlap each other's matrix, vector and LDS phases (one wavefront alone leaves the SIMD idle for
// most of its chain of dependent steps).
//
// LDS layouts: keys [64 rows][D + 8] (row = key), values [D rows][64 + 8] (row = channel) with the
// keys of each half of 32 stored in operand order (lane group g, tile h, key i -> g*8 + h*4 + i), so
// that both A operands are single 16-byte reads and rows that differ by one land 36 banks apart.
constexpr int kKRow = D + 8;                 // elements per key row in LDS
constexpr int kVRow = 64 + 8;                // elements per channel row in LDS
constexpr int kKChunks = 16 * D / 8;         // 16-byte pieces of one tile of keys (16 rows of D)
constexpr int kVChunks = 2 * D;              // 16-byte pieces of one tile of values (D channels x 2 halves of 8 keys)
constexpr int kKPerLane = (kKChunks + 63) / 64;
constexpr int kVPerLane = (kVChunks + 63) / 64;

struct MaskedTag { static constexpr bool value = true; };
struct PlainTag { static constexpr bool value = false; };

template <int NCB, int KG>
__global__ __launch_bounds__(256 * KG, (D <= 96 || KG == 2) ? 2 : 1) void paged_attention_prefill_kernel(
    const bf16* __restrict__ q, int q_stride, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
    bf16* __restrict__ out, int out_stride, const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ cu_seqlens_q, const int* __restrict__ seq_lens_k, int num_heads, int num_kv_heads,
    int block_size, float scale, int window, const int* __restrict__ work, int partition_size, int num_partitions,
    float* __restrict__ partials PLLM_TERMS_PARAM) {
  extern __shared__ __attribute__((aligned(16))) unsigned char prefill_lds[];
  constexpr int kKTile = 64 * kKRow, kVTile = D * kVRow;         // elements of one group's keys / values of a step
  // keys [2 buffers][KG][64 rows][kKRow], then values [2 buffers][KG][D rows][kVRow].  Addresses are formed
  // from the LDS symbol where they are used: a pointer kept in a register may be spilled, and comes back as
  // a generic pointer whose accesses are no longer LDS instructions.
#define PLLM_K_TILE(buf, group) (reinterpret_cast<bf16*>(prefill_lds) + ((buf) * KG + (group)) * kKTile)
#define PLLM_V_TILE(buf, group) (reinterpret_cast<bf16*>(prefill_lds) + 2 * KG * kKTile + ((buf) * KG + (group)) * kVTile)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, g = lane >> 4;
  const int cw = wave & 3, kg = wave >> 2;                      // column share and key group of this wavefront
  // The wavefront's index is the same in all its lanes; saying so keeps what the fetches derive from it (the tile's
  // page-table entry and page address) in scalar registers.  (Used for the fetches only: with the column share
  // and key group declared uniform as well the compiler needs more vector registers than large heads leave.)
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int bs_shift = __builtin_ctz(block_size);
  // Workgroups are handed out x first.  With a work list (pairs of sequence and tile, those with the most keys
  // first): blockIdx.x = kv head, blockIdx.y = entry of the list, so the longest pieces of work of all sequences
  // start first and no workgroup is launched for nothing.  Without one: blockIdx.x = (sequence, kv head),
  // blockIdx.y = tile slot counted from every sequence's last tile; sequences with fewer tiles than the
  // longest leave their other slots empty.
  int seq, kvh, listed_tile = -1;
  if (work) {
    kvh = blockIdx.x;
    seq = work[2 * blockIdx.y];
    listed_tile = work[2 * blockIdx.y + 1];
    if (seq < 0) return;                                          // an unused entry of a list of fixed length
  } else {
    seq = blockIdx.x / num_kv_heads;
    kvh = blockIdx.x - seq * num_kv_heads;
  }
  const int G = num_heads / num_kv_heads;
  const int q_begin = cu_seqlens_q[seq], num_q = cu_seqlens_q[seq + 1] - q_begin;
  const int len_k = seq_lens_k[seq];
  const int num_cols = num_q * G;
  constexpr int kWgCols = 4 * 16 * NCB;
  const int my_tiles = (num_cols + kWgCols - 1) / kWgCols;
  const int tile = work ? listed_tile : my_tiles - 1 - (int)blockIdx.y;
  if (tile < 0 || tile >= my_tiles) return;                     // no such tile in this sequence
  const int wg_col0 = tile * kWgCols;
  const int pos0 = len_k - num_q;
  // key range of the whole workgroup
  const int wg_last = min(wg_col0 + kWgCols, num_cols) - 1;
  const int wg_qmin = pos0 + wg_col0 / G, wg_qmax = pos0 + wg_last / G;
  int k_hi = wg_qmax + 1;
  int k_lo = ((window > 0 && wg_qmin - window + 1 > 0) ? wg_qmin - window + 1 : 0) & ~63;
  // With partitions (few tiles, long contexts: too few workgroups to fill the GPU otherwise) blockIdx.z takes one
  // aligned partition of the keys and leaves a partial result for the merge kernel.
  const int part = blockIdx.z;
  if (partition_size > 0) {
    k_lo = max(k_lo, part * partition_size);
    k_hi = min(k_hi, (part + 1) * partition_size);
    if (k_lo >= k_hi) return;                                   // nothing of this partition is visible to the tile
  }
  // this wavefront's columns
  const int col0 = wg_col0 + cw * 16 * NCB;
  const bool wave_on = col0 < num_cols;
  const int last_col = min(col0 + 16 * NCB, num_cols) - 1;
  const int qpos_min = pos0 + col0 / G, qpos_max = wave_on ? pos0 + last_col / G : -1;
  const int vis_hi = qpos_max + 1;
  const int vis_lo = (window > 0 && qpos_min - window + 1 > 0) ? qpos_min - window + 1 : 0;

  int my_qpos[NCB], my_first[NCB];
  bool my_valid[NCB];
  size_t my_out[NCB];
  bf16x8 qreg[NCB][KSTEPS];
  float my_slope[NCB], my_sink[NCB];                            // (with further score terms only; both in log2 units)
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    const int c = col0 + cb * 16 + r;
    my_valid[cb] = c < num_cols;
    const int tok = my_valid[cb] ? c / G : 0, hg = my_valid[cb] ? c - tok * G : 0;
    my_qpos[cb] = my_valid[cb] ? pos0 + tok : -1;
    my_first[cb] = (window > 0 && my_qpos[cb] - window + 1 > 0) ? my_qpos[cb] - window + 1 : 0;
    const size_t row = (size_t)(q_begin + tok) * q_stride + (size_t)(kvh * G + hg) * D;
    my_out[cb] = (size_t)(q_begin + tok) * out_stride + (size_t)(kvh * G + hg) * D;
    if constexpr (kTerms) {
      my_slope[cb] = (terms.slopes && my_valid[cb]) ? terms.slopes[kvh * G + hg] * kLog2e : 0.f;
      my_sink[cb] = (terms.sinks && my_valid[cb]) ? terms.sinks[kvh * G + hg] * kLog2e : -INFINITY;
    }
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) {
      const int dd = s * 32 + g * 8;
      qreg[cb][s] = (my_valid[cb] && dd < D) ? *reinterpret_cast<const bf16x8*>(q + row + dd) : zero8();
    }
  }
  floatx4 acc[NCB][DBLOCKS];
  float m_run[NCB], l_run[NCB];
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    m_run[cb] = -INFINITY;
    l_run[cb] = 0.f;
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) acc[cb][db] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  const float sl2 = scale * kLog2e;
  [[maybe_unused]] const ScoreForm form = score_form(terms, scale);
  if constexpr (kTerms) {
    // A head's sink enters as the state of a softmax that has seen one key with that score and no value.  Of the
    // key groups that share a column, the first one of the partition that holds the column's first visible key
    // has it (that partition has work for this column, and the merge counts it).
    if (terms.sinks) {
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) {
        const bool here = my_valid[cb] && kg == 0 && (partition_size == 0 || part == my_first[cb] / partition_size);
        if (here) {
          m_run[cb] = my_sink[cb];
          l_run[cb] = g == 0 ? 1.f : 0.f;                         // (the four lanes of a column are added at the end)
        }
      }
    }
  }
  const int* bt = block_tables + (size_t)seq * bt_stride;
  const size_t page_elems = (size_t)block_size * D;
  const size_t page_stride = page_elems * num_kv_heads;

  // ---- fetch of one tile (16 keys) per wavefront: wavefront w fetches tile w of the step.  Everything but the
  //      lane's own offset is uniform (page-table entry, page address), so it stays in scalar registers.  A tile
  //      past the range is fetched as the range's last tile again: the loads are unconditional (the count of loads
  //      in flight is then known at every wait), no table entry past the context is read, and what lands in LDS
  //      for keys past the range is never used (the masked version drops scores and values by position).
  struct Fetched {
    bf16x8 k[kKPerLane], v[kVPerLane];
  };
  const int last_tile = (k_hi - 1) & ~15;
  auto page_of = [&](int n0) -> int { return bt[min(n0 + wave_u * 16, last_tile) >> bs_shift]; };
  auto fetch = [&](Fetched& f, int n0, int page) {
    const int nk = min(n0 + wave_u * 16, last_tile);
    const int off = nk & (block_size - 1);
    const size_t base = (size_t)page * page_stride + (size_t)kvh * page_elems;
    const bf16* kbase = k_pages + base + (size_t)off * D;        // 16 rows of D, contiguous
    const bf16* vbase = v_pages + base + off;                    // + channel * block_size + key
#pragma unroll
    for (int i = 0; i < kKPerLane; ++i) {
      const int c = lane + i * 64;
      f.k[i] = (c < kKChunks) ? *reinterpret_cast<const bf16x8*>(kbase + c * 8) : zero8();
    }
#pragma unroll
    for (int i = 0; i < kVPerLane; ++i) {
      const int c = lane + i * 64;                                // c = channel * 2 + half
      f.v[i] = (c < kVChunks) ? *reinterpret_cast<const bf16x8*>(vbase + (c >> 1) * block_size + (c & 1) * 8) : zero8();
    }
  };
  auto stash = [&](const Fetched& f, int buf) {
#pragma unroll
    for (int i = 0; i < kKPerLane; ++i) {
      const int c = lane + i * 64;
      if (c < kKChunks) {
        const int row = c / (D / 8), part = c - row * (D / 8);
        *reinterpret_cast<bf16x8*>(PLLM_K_TILE(buf, kg) + (cw * 16 + row) * kKRow + part * 8) = f.k[i];
      }
    }
    const int a = cw >> 1, h = cw & 1;                            // tile `cw` of the group is half h of its 32 keys a
#pragma unroll
    for (int i = 0; i < kVPerLane; ++i) {
      const int c = lane + i * 64;
      if (c < kVChunks) {
        const int ch = c >> 1, half = c & 1;
        bf16* dst = PLLM_V_TILE(buf, kg) + ch * kVRow + a * 32 + h * 4;
        // keys half*8 .. half*8+7 of the tile: lane groups g = half*2 and half*2 + 1, four keys each
        bf16x4 lo4, hi4;
#pragma unroll
        for (int j = 0; j < 4; ++j) { lo4[j] = f.v[i][j]; hi4[j] = f.v[i][4 + j]; }
        *reinterpret_cast<bf16x4*>(dst + (half * 2) * 8) = lo4;
        *reinterpret_cast<bf16x4*>(dst + (half * 2 + 1) * 8) = hi4;
      }
    }
  };

  // `masked` is a compile-time flag: blocks whose 64 keys every valid column of the wavefront may see take
  // the version without any comparison.  Columns past the end of the sequence (the last tile's surplus)
  // carry zero queries and are never stored; they go along with either version.
  // (inlined at both of its places in every build: left to itself the compiler makes a call of the larger forms, with
  //  the captured state passed through memory)
  auto compute = [&](int buf, int n0, auto masked_tag) __attribute__((always_inline)) {
    constexpr bool kMasked = decltype(masked_tag)::value;
    const bf16* kb = PLLM_K_TILE(buf, kg);
    const bf16* vb = PLLM_V_TILE(buf, kg);
    floatx4 s_t[4][NCB];
    if constexpr (!kMasked && KSTEPS <= 2) {
      // All key operands of the block are requested from LDS before the first product: the reads then wait
      // for each other's latency once, not one after the other between the matrix instructions.
      bf16x8 kop[4][KSTEPS];
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          const int dd = s * 32 + g * 8;
          kop[kt][s] = (dd < D) ? *reinterpret_cast<const bf16x8*>(kb + (kt * 16 + r) * kKRow + dd) : zero8();
        }
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) s_t[kt][cb] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
          for (int cb = 0; cb < NCB; ++cb) s_t[kt][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop[kt][s], qreg[cb][s], s_t[kt][cb], 0, 0, 0);
      }
    } else {
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) s_t[kt][cb] = floatx4{0.f, 0.f, 0.f, 0.f};
      if (kMasked && n0 + kt * 16 >= vis_hi) continue;            // uniform in the wavefront: nothing of this tile is visible
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        const int dd = s * 32 + g * 8;
        const bf16x8 kop = (dd < D) ? *reinterpret_cast<const bf16x8*>(kb + (kt * 16 + r) * kKRow + dd) : zero8();
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) s_t[kt][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop, qreg[cb][s], s_t[kt][cb], 0, 0, 0);
      }
    }
    }
    // Unmasked blocks: the value operands are requested from LDS here, so that they arrive during the softmax.
    constexpr bool kEarlyValues = !kMasked && DBLOCKS <= 4;
    bf16x8 v_early[kEarlyValues ? 2 : 1][kEarlyValues ? DBLOCKS : 1];
    if constexpr (kEarlyValues) {
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db) v_early[a][db] = *reinterpret_cast<const bf16x8*>(vb + (db * 16 + r) * kVRow + a * 32 + g * 8);
    }
    bf16x8 p_op[2][NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
      // The maximum is taken over the raw dot products (the scale is positive); the running
      // maximum m_run is kept in scaled log2 units.  (With further terms the scores are brought to their final
      // form in log2 units first, and the factor below is one.)
      float mul = sl2;
      if constexpr (kTerms) {
        if (form.any()) {
          float s[4][4];
#pragma unroll
          for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) s[kt][i] = s_t[kt][cb][i];
          final_scores(form, my_slope[cb], (float)(n0 + g * 4 - my_qpos[cb]), s);
#pragma unroll
          for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) s_t[kt][cb][i] = s[kt][i];
          mul = 1.f;
        }
      }
      float mx = -INFINITY;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (kMasked) {
            const int n = n0 + kt * 16 + g * 4 + i;
            if (!(n <= my_qpos[cb] && n >= my_first[cb])) s_t[kt][cb][i] = -INFINITY;
          }
          mx = fmaxf(mx, s_t[kt][cb][i]);
        }
      mx = group_max(mx) * mul;
      const float m_new = fmaxf(m_run[cb], mx);
      const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = fast_exp2(m_run[cb] - m_safe);
      m_run[cb] = m_new;
      float psum = 0.f;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = fast_exp2(fmaf(s_t[kt][cb][i], mul, -m_safe));
          psum += p;
          p_op[kt >> 1][cb][(kt & 1) * 4 + i] = (__bf16)p;
        }
      l_run[cb] = l_run[cb] * alpha + psum;
      if (!__all(alpha == 1.f)) {                                 // the maximum seldom moves after the first blocks
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db) acc[cb][db] *= alpha;
      }
    }
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      if (kMasked && n0 + a * 32 >= vis_hi) continue;
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db) {
        bf16x8 vreg;
        if constexpr (kEarlyValues) vreg = v_early[a][db];
        else vreg = *reinterpret_cast<const bf16x8*>(vb + (db * 16 + r) * kVRow + a * 32 + g * 8);
        if (kMasked) {
          // values of keys that no column of this wavefront may see are zeroed (stale data, 0 * NaN)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int n = n0 + (2 * a + (j >> 2)) * 16 + g * 4 + (j & 3);
            if (n >= vis_hi || n < vis_lo) vreg[j] = (__bf16)0.0f;
          }
        }
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) acc[cb][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vreg, p_op[a][cb], acc[cb][db], 0, 0, 0);
      }
    }
  };
  const int full_from = window > 0 ? max(qpos_max - window + 1, 0) : 0;   // blocks from here on are inside every column's window

  // ---- the steps.  Step i is computed from LDS while the next steps are on their way in registers: two sets
  //      of them (steps i + 1 and i + 2) for head sizes up to 64, one set (step i + 1) where a second would not
  //      fit.  After the computation step i + 1 is written to the other LDS buffer and the registers it leaves take
  //      the request for the step after those in flight, with the page-table entry that was looked up a step
  //      earlier: with two sets a fetch has two steps to arrive, and it never waits for its table entry.  Fetches
  //      and stashes past the last step repeat the last tile into a buffer nobody reads.
  constexpr int kStepKeys = 64 * KG;
  constexpr bool kTwoSets = D <= 64;
  constexpr int kAhead = kTwoSets ? 3 : 2;                        // the fetch issued in step i is for step i + kAhead
  Fetched set_a, set_b;
  int page_next;
  auto step = [&](int n0, int buf, Fetched& next) {               // `next` holds step n0 + kStepKeys
    const int mine = n0 + kg * 64;                                // this group's 64 keys of the step
    if (wave_on && mine < vis_hi && mine < k_hi && mine + 64 > vis_lo) {   // (k_hi: a partition's end, a multiple of 64)
      if (mine + 63 <= qpos_min && mine >= full_from) compute(buf, mine, PlainTag{});
      else compute(buf, mine, MaskedTag{});
    }
    // (the compiler may not move the requests up into the computation: their registers are free only here)
    __builtin_amdgcn_sched_barrier(0);
    stash(next, buf ^ 1);
    fetch(next, n0 + kAhead * kStepKeys, page_next);
    page_next = page_of(n0 + (kAhead + 1) * kStepKeys);
    __syncthreads();
  };
  fetch(set_a, k_lo, page_of(k_lo));
  if constexpr (kTwoSets) fetch(set_b, k_lo + kStepKeys, page_of(k_lo + kStepKeys));
  page_next = page_of(k_lo + (kAhead - 1) * kStepKeys);
  stash(set_a, 0);
  fetch(set_a, k_lo + (kAhead - 1) * kStepKeys, page_next);
  page_next = page_of(k_lo + kAhead * kStepKeys);
  __syncthreads();
  // (the loop is left from between the two steps, not around the second one: on every way back to its head the
  //  set that was requested first is the one that is stashed next, so the wait before a stash can leave the
  //  younger set's loads in flight)
  for (int n0 = k_lo;;) {
    if constexpr (kTwoSets) step(n0, 0, set_b); else step(n0, 0, set_a);
    n0 += kStepKeys;
    if (n0 >= k_hi) break;
    step(n0, 1, set_a);
    n0 += kStepKeys;
    if (n0 >= k_hi) break;
  }

  if (KG == 2) {
    // Group 1 hands its half of every column to group 0 through LDS (the last step ended with a barrier,
    // so the key and value buffers are free): per wavefront [NCB][DBLOCKS * 4 + 2][64 lanes] floats.
    float* hand = reinterpret_cast<float*>(prefill_lds) + (size_t)cw * NCB * (DBLOCKS * 4 + 2) * 64;
    if (kg == 1) {
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) {
        float* h = hand + cb * (DBLOCKS * 4 + 2) * 64 + lane;
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) h[(db * 4 + i) * 64] = acc[cb][db][i];
        h[DBLOCKS * 4 * 64] = m_run[cb];
        h[(DBLOCKS * 4 + 1) * 64] = l_run[cb];
      }
    }
    __syncthreads();
    if (kg == 0) {
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) {
        const float* h = hand + cb * (DBLOCKS * 4 + 2) * 64 + lane;
        const float m_other = h[DBLOCKS * 4 * 64], l_other = h[(DBLOCKS * 4 + 1) * 64];
        const float m_new = fmaxf(m_run[cb], m_other);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float a_mine = fast_exp2(m_run[cb] - m_safe), a_other = fast_exp2(m_other - m_safe);   // 2^-inf = 0: an empty half adds nothing
        l_run[cb] = l_run[cb] * a_mine + l_other * a_other;
        m_run[cb] = m_new;
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[cb][db][i] = acc[cb][db][i] * a_mine + h[(db * 4 + i) * 64] * a_other;
      }
    }
  }

#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    const float l_tot = group_sum(l_run[cb]);                     // every lane takes part in the exchange
    const float inv = 1.f / l_tot;
    if (!my_valid[cb] || kg != 0) continue;
    if (partition_size > 0) {                                     // unnormalised sum, maximum and weight of this partition
      const int c = col0 + cb * 16 + r;
      const int tok = c / G, hg = c - tok * G;
      float* dst = partials + (((size_t)(q_begin + tok) * num_heads + (kvh * G + hg)) * num_partitions + part) * kPartialFloats;
      if (g == 0) { dst[0] = m_run[cb]; dst[1] = l_tot; }
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[2 + db * 16 + g * 4 + i] = acc[cb][db][i];
      continue;
    }
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) {
      bf16x4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (__bf16)(acc[cb][db][i] * inv);
      *reinterpret_cast<bf16x4*>(out + my_out[cb] + db * 16 + g * 4) = o;
    }
  }
#undef PLLM_K_TILE
#undef PLLM_V_TILE
}

// Merge of the partitions of one (token, head), one wavefront each:
//   out = sum_p 2^(m_p - M) acc_p / sum_p 2^(m_p - M) l_p   over the partitions that hold a visible key,
// added in partition order.  The kernel is a chain of waits for memory, so the chain is kept short: with
// one query per sequence (decoding) the token is the sequence, and the partials of every partition are
// requested before the lengths that say which of them count have arrived (what does not count is dropped
// by a select, never multiplied: it may be anything).
template <bool ONE_QUERY>
__global__ __launch_bounds__(256) void attention_merge_kernel(const float* __restrict__ partials, bf16* __restrict__ out, int out_stride,
                                                             const int* __restrict__ cu_seqlens_q, const int* __restrict__ seq_lens_k,
                                                             int num_seqs, int total_q, int num_heads, int window, int partition_size,
                                                             int num_partitions) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= total_q * num_heads) return;
  const int tok = item / num_heads, head = item - tok * num_heads;
  const float* base = partials + (size_t)item * num_partitions * kPartialFloats;
  // maxima of up to 64 partitions at a time, one per lane, requested at once
  float m_mine = -INFINITY;
  if (lane < num_partitions) m_mine = base[(size_t)lane * kPartialFloats];
  // ... and behind them, before anything is waited for, the partial results of the first kEarly partitions (all there
  // are, for most contexts): a loop over a number of partitions that is known only at run time would request
  // them after the maxima and the lengths have arrived, four at a time, each time with a wait of its own.
  constexpr int kEarly = 8, kPerLane = (D + 63) / 64;
  float early_m[kEarly], early_l[kEarly], early_a[kEarly][kPerLane];
#pragma unroll
  for (int p = 0; p < kEarly; ++p) {
    const float* pp = base + (size_t)min(p, num_partitions - 1) * kPartialFloats;
    early_m[p] = pp[0];
    early_l[p] = pp[1];
#pragma unroll
    for (int j = 0; j < kPerLane; ++j) early_a[p][j] = pp[2 + min(lane + j * 64, D - 1)];
  }
  int seq = tok, q_begin = tok, num_q = 1;
  if (!ONE_QUERY) {
    int lo = 0, hi = num_seqs - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cu_seqlens_q[mid] <= tok) lo = mid; else hi = mid - 1;
    }
    seq = lo;
    q_begin = cu_seqlens_q[lo];
    num_q = cu_seqlens_q[lo + 1] - q_begin;
    if (tok < q_begin || tok >= q_begin + num_q) return;           // a row of none of this launch's sequences
  }
  const int qpos = seq_lens_k[seq] - num_q + (tok - q_begin);
  const int first_key = (window > 0 && qpos - window + 1 > 0) ? qpos - window + 1 : 0;
  const int p_lo = first_key / partition_size, p_hi = min(qpos / partition_size, num_partitions - 1);
  float M = (lane >= p_lo && lane <= p_hi) ? m_mine : -INFINITY;
  for (int p = 64 + lane; p <= p_hi; p += 64)
    if (p >= p_lo) M = fmaxf(M, base[(size_t)p * kPartialFloats]);
  M = wave_max(M);
  float l = 0.f;
  float o[(D + 63) / 64];
#pragma unroll
  for (int j = 0; j < (D + 63) / 64; ++j) o[j] = 0.f;
#pragma unroll
  for (int p = 0; p < kEarly; ++p) {                             // (in partition order, as below)
    const bool counts = p < num_partitions && p >= p_lo && p <= p_hi;
    const float w = counts ? fast_exp2(early_m[p] - M) : 0.f;
    l += counts ? w * early_l[p] : 0.f;
#pragma unroll
    for (int j = 0; j < kPerLane; ++j) o[j] += counts ? w * early_a[p][j] : 0.f;
  }
#pragma unroll 4
  for (int p = kEarly; p < num_partitions; ++p) {                // all of them: the loads wait for nothing
    const float* pp = base + (size_t)p * kPartialFloats;
    const bool counts = p >= p_lo && p <= p_hi;
    const float m_p = pp[0], l_p = pp[1];
    float a[(D + 63) / 64];
#pragma unroll
    for (int j = 0; j < (D + 63) / 64; ++j) a[j] = pp[2 + min(lane + j * 64, D - 1)];
    const float w = counts ? fast_exp2(m_p - M) : 0.f;
    l += counts ? w * l_p : 0.f;
#pragma unroll
    for (int j = 0; j < (D + 63) / 64; ++j) o[j] += counts ? w * a[j] : 0.f;
  }
  const float inv = 1.f / l;
#pragma unroll
  for (int j = 0; j < (D + 63) / 64; ++j) {
    const int i = lane + j * 64;
    if (i < D) out[(size_t)tok * out_stride + (size_t)head * D + i] = __float2bfloat16(o[j] * inv);
  }
}

PLLM_API int pllm_attention_mfma_head_dim() { return D; }

// Registers per lane (vector and accumulation registers together) of the decode kernel's form with `waves`
// wavefronts and one block of 16 columns, as the runtime reports them for the compiled kernel; -1 for another form.
// Two workgroups of four wavefronts share a compute unit only up to 256: a test holds the kernel to that, since a
// few registers more halve its throughput for large batches.
PLLM_API int pllm_attention_decode_registers(int waves) {
  hipFuncAttributes attr;
  const void* fn = waves == 4 ? reinterpret_cast<const void*>(paged_attention_mfma_kernel<1, 4>)
                 : waves == 8 ? reinterpret_cast<const void*>(paged_attention_mfma_kernel<1, 8>) : nullptr;
  if (!fn || hipFuncGetAttributes(&attr, fn) != hipSuccess) return -1;
  return attr.numRegs;
}

// Bytes per lane that the same two forms keep outside registers (spilled registers): 0 as long as they fit.
PLLM_API int pllm_attention_decode_spill_bytes(int waves) {
  hipFuncAttributes attr;
  const void* fn = waves == 4 ? reinterpret_cast<const void*>(paged_attention_mfma_kernel<1, 4>)
                 : waves == 8 ? reinterpret_cast<const void*>(paged_attention_mfma_kernel<1, 8>) : nullptr;
  if (!fn || hipFuncGetAttributes(&attr, fn) != hipSuccess) return -1;
  return (int)attr.localSizeBytes;
}

static int num_compute_units() {
  static int cus = 0;
  if (!cus) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) cus = prop.multiProcessorCount;
    if (cus <= 0) cus = 256;
  }
  return cus;
}

static long pllm_max_lds() {
  static long cached = 0;
  if (!cached) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) == hipSuccess) cached = v;
    if (cached <= 0) cached = 64 * 1024;
  }
  return cached;
}

// LDS floats of the several-wavefront variant.
// LDS of the prompt kernel with kg key groups: two buffers of keys and values per group, reused at the
// end for the hand-over of group 1's halves (four wavefronts x 2 column blocks).
constexpr size_t prefill_lds_bytes(int kg) {
  const size_t buffers = (size_t)2 * kg * (64 * kKRow + D * kVRow) * sizeof(bf16);
  const size_t hand = (size_t)4 * 2 * (DBLOCKS * 4 + 2) * 64 * sizeof(float);
  return buffers > hand ? buffers : hand;
}
static size_t merge_lds_bytes(int ncb, int waves) { return (size_t)(2 * waves * ncb * 16 + waves * ncb * DBLOCKS * 4 * 64) * sizeof(float); }

// waves == 1: every work item is one wavefront that walks its key range.
// waves in {4, 8}: the wavefronts of a workgroup share the key range of one work item (they take
//   its blocks of 64 keys in turn, with the next block already requested) and merge through LDS.
// partition_size == 0: a work item's key range is everything its queries may see; it writes the result.
// partition_size > 0 (a multiple of 64): num_partitions work items per tile each take one aligned
//   partition of the keys and write partials into `partials` (total_q * heads * num_partitions *
//   (D + 2) floats); a second kernel merges them.
static int launch_attention(const void* q, int q_stride, const void* k_pages, const void* v_pages, void* out,
                            int out_stride, const int* block_tables, int bt_stride, const int* cu_seqlens_q,
                            const int* seq_lens_k, int num_seqs, int total_q, int max_q_len, int num_heads,
                            int num_kv_heads, int block_size, float scale, int window, int partition_size,
                            int num_partitions, float* partials, int waves, int column_blocks, const int* work_list, int num_work,
                            int single_prompt, [[maybe_unused]] ScoreTerms terms, hipStream_t stream) {
  if (total_q <= 0 || num_seqs <= 0) return 0;
  if (num_kv_heads <= 0 || num_heads % num_kv_heads) return -2;
  const int G = num_heads / num_kv_heads;
  if (G > 64 || block_size < 16 || (block_size & (block_size - 1))) return -2;
  if (partition_size < 0 || (partition_size & 63) || (partition_size > 0 && (!partials || num_partitions < 1))) return -2;
  if (partition_size == 0) num_partitions = 1;
  const int max_cols = max_q_len * G;
  // column_blocks (1, 2 or 4 blocks of 16 columns per work item; 0 = as many as the columns need, up to 4)
  int ncb = max_cols <= 16 ? 1 : (max_cols <= 32 ? 2 : 4);
  if (column_blocks == 1 || column_blocks == 2 || column_blocks == 4) ncb = column_blocks < ncb ? column_blocks : ncb;
  else if (column_blocks != 0) return -2;
  const int tiles = (max_cols + 16 * ncb - 1) / (16 * ncb);
  if (num_kv_heads * num_partitions > 65535 || num_seqs > 65535) return -2;
  if (waves != 1 && waves != 4 && waves != 8) return -2;
  if (waves > 1 && (long)merge_lds_bytes(ncb, waves) > pllm_max_lds()) return -2;
  if (waves == 1 && max_cols > 64 && column_blocks != 1 && column_blocks != 4) {
    // prompt portions: workgroups of four wavefronts that share every block of keys through LDS
    constexpr int kCols = 4 * 16 * 2;
    const int ptiles = (max_cols + kCols - 1) / kCols;
    // The grid is (sequence x kv head, tile slot): workgroups are handed out in that order, so the last
    // tiles of all sequences (most keys) start first and the early tiles fill the tail; that keeps the compute
    // units evenly loaded for any number and length of prompts (pairing far and near tiles in one workgroup
    // was 5 % faster when the pairs filled the compute units exactly and up to 40 % slower just past that).
    if (ptiles > 65535 || num_work > 65535 || (work_list && num_work <= 0)) return -2;
    if (num_partitions > 65535) return -2;
    dim3 pgrid(num_kv_heads * num_seqs, ptiles, num_partitions);
    if (work_list) pgrid = dim3(num_kv_heads, num_work, num_partitions);
    // Two key groups (eight wavefronts, one workgroup per compute unit) for the head sizes that then still fit
    // into registers and LDS (up to 128): always where a wavefront of the four-wavefront kind needs more than half
    // of a SIMD's registers (head sizes above 96: two groups are then the only way to two wavefronts per SIMD,
    // measured 1.4 times faster at 128), else while the workgroups fit the compute units in one round, and for a
    // single sequence in two (its tiles, handed out longest first, pair up a long one and a short one per compute
    // unit: 2048 tokens 39.9 against 42.7 us; but two prompts of 1024 tokens 26.1 against 23.9 us, four of 512 19.4
    // against 16.0, sixteen of 256 31.5 against 19.7, and one of 2560 62.0 against 52.4: there two workgroups of the
    // four-wavefront kind per compute unit, each hiding the other's start and end, are faster).  `single_prompt`: the
    // caller says that all queries but a few are one sequence's (a step replayed from a graph holds a padding sequence
    // beside its portion, and its list of tiles has spare entries).
    constexpr bool two_fits = D <= 128 && prefill_lds_bytes(2) <= 160 * 1024;
    // (workgroups that find work: with a list exactly its entries; else a sequence has as many tiles as its own queries
    // need, one more than its share at most)
    const bool solo = num_seqs == 1 || single_prompt;
    const long tiles_of_queries = ((long)total_q * G + kCols - 1) / kCols;
    const long busy = (single_prompt ? tiles_of_queries : work_list ? (long)num_work : tiles_of_queries + (num_seqs - 1)) * num_kv_heads * num_partitions;
    const long cus = num_compute_units();
    const bool two = two_fits && (D > 96 || busy <= cus || (solo && busy <= 2 * cus));
    const size_t lds = prefill_lds_bytes(two ? 2 : 1);
    if ((long)lds > pllm_max_lds()) return -2;
    auto kern = paged_attention_prefill_kernel<2, 1>;
    if constexpr (two_fits) {
      if (two) kern = paged_attention_prefill_kernel<2, 2>;
    }
    if (lds > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL(kern, pgrid, dim3(two ? 512 : 256), lds, stream, (const bf16*)q, q_stride,
                       (const bf16*)k_pages, (const bf16*)v_pages, (bf16*)out, out_stride, block_tables, bt_stride, cu_seqlens_q,
                       seq_lens_k, num_heads, num_kv_heads, block_size, scale, window, work_list, partition_size, num_partitions, partials PLLM_TERMS_ARG);
    int perr = (int)hipGetLastError();
    if (perr || partition_size == 0) return perr;
    hipLaunchKernelGGL(attention_merge_kernel<false>, dim3((total_q * num_heads + 3) / 4), dim3(256), 0, stream, partials, (bf16*)out,
                       out_stride, cu_seqlens_q, seq_lens_k, num_seqs, total_q, num_heads, window, partition_size, num_partitions);
    return (int)hipGetLastError();
  }
  dim3 grid(tiles, num_kv_heads * num_partitions, num_seqs), block(64 * waves);
  const size_t lds = waves > 1 ? merge_lds_bytes(ncb, waves) : 0;
#define PLLM_LAUNCH(NCB_, WAVES_)                                                                                                    \
  do {                                                                                                                               \
    auto kern = paged_attention_mfma_kernel<NCB_, WAVES_>;                                                                           \
    if (lds > 48 * 1024) {                                                                                                           \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
      if (e != hipSuccess) return (int)e;                                                                                            \
    }                                                                                                                                \
    hipLaunchKernelGGL(kern, grid, block, lds, stream, (const bf16*)q, q_stride, (const bf16*)k_pages, (const bf16*)v_pages,         \
                       (bf16*)out, out_stride, block_tables, bt_stride, cu_seqlens_q, seq_lens_k, num_heads, num_kv_heads,           \
                       block_size, scale, window, partition_size, num_partitions, partials PLLM_TERMS_ARG);                          \
  } while (0)
#define PLLM_BY_WAVES(NCB_)                                                                          \
  do {                                                                                               \
    if (waves == 1) PLLM_LAUNCH(NCB_, 1); else if (waves == 4) PLLM_LAUNCH(NCB_, 4);                 \
    else PLLM_LAUNCH(NCB_, 8);                                                                       \
  } while (0)
  if (ncb == 1) PLLM_BY_WAVES(1); else if (ncb == 2) PLLM_BY_WAVES(2); else PLLM_BY_WAVES(4);
#undef PLLM_BY_WAVES
#undef PLLM_LAUNCH
  int err = (int)hipGetLastError();
  if (err) return err;
  if (partition_size > 0) {
    // one query per sequence: total_q == num_seqs and no sequence is empty (max_q_len bounds them all)
    if (max_q_len == 1 && total_q == num_seqs)
      hipLaunchKernelGGL(attention_merge_kernel<true>, dim3((total_q * num_heads + 3) / 4), dim3(256), 0, stream, partials, (bf16*)out,
                         out_stride, cu_seqlens_q, seq_lens_k, num_seqs, total_q, num_heads, window, partition_size, num_partitions);
    else
      hipLaunchKernelGGL(attention_merge_kernel<false>, dim3((total_q * num_heads + 3) / 4), dim3(256), 0, stream, partials, (bf16*)out,
                         out_stride, cu_seqlens_q, seq_lens_k, num_seqs, total_q, num_heads, window, partition_size, num_partitions);
    err = (int)hipGetLastError();
  }
  return err;
}

PLLM_API int pllm_paged_attention_mfma(const void* q, int q_stride, const void* k_pages, const void* v_pages, void* out,
                                       int out_stride, const int* block_tables, int bt_stride, const int* cu_seqlens_q,
                                       const int* seq_lens_k, int num_seqs, int total_q, int max_q_len, int num_heads,
                                       int num_kv_heads, int block_size, float scale, int window, int partition_size,
                                       int num_partitions, float* partials, int waves, int column_blocks, const int* work_list, int num_work,
                                       hipStream_t stream) {
  return launch_attention(q, q_stride, k_pages, v_pages, out, out_stride, block_tables, bt_stride, cu_seqlens_q, seq_lens_k, num_seqs,
                          total_q, max_q_len, num_heads, num_kv_heads, block_size, scale, window, partition_size, num_partitions,
                          partials, waves, column_blocks, work_list, num_work, 0, ScoreTerms{0.f, nullptr, nullptr}, stream);
}

// The same with a hint for the prompt kernel's form (single_prompt: all queries but a few belong to one sequence) and
// with further terms of the score: score_cap > 0 caps the scaled products (c tanh(x / c)), slopes [heads]
// adds slope * (key position - query position), sinks [heads] gives every head a logit that takes part in the
// softmax's sum only (null: none).  A library compiled without -DSCORE_TERMS=1 refuses any of them.
PLLM_API int pllm_attention_mfma_score_terms() { return kTerms ? 1 : 0; }

PLLM_API int pllm_paged_attention_mfma_terms(const void* q, int q_stride, const void* k_pages, const void* v_pages, void* out,
                                             int out_stride, const int* block_tables, int bt_stride, const int* cu_seqlens_q,
                                             const int* seq_lens_k, int num_seqs, int total_q, int max_q_len, int num_heads,
                                             int num_kv_heads, int block_size, float scale, int window, int partition_size,
                                             int num_partitions, float* partials, int waves, int column_blocks, const int* work_list,
                                             int num_work, int single_prompt, float score_cap, const float* slopes, const float* sinks,
                                             hipStream_t stream) {
  const ScoreTerms given{score_cap, slopes, sinks};
  if (!(score_cap >= 0.f) || (given.any() && !kTerms)) return -2;
  return launch_attention(q, q_stride, k_pages, v_pages, out, out_stride, block_tables, bt_stride, cu_seqlens_q, seq_lens_k, num_seqs,
                          total_q, max_q_len, num_heads, num_kv_heads, block_size, scale, window, partition_size, num_partitions,
                          partials, waves, column_blocks, work_list, num_work, single_prompt, given, stream);
}

// What the library that holds the no-allocation entry point needs from this one (see attention_noalloc.h): the head
// size it was compiled for, the entry point above, and a call that makes the device queries of the launch code now
// (they are made lazily otherwise, at the first launch, which may be inside a stream capture).
#include "attention_noalloc.h"

static int warm_up_device_queries() { return (num_compute_units() > 0 && pllm_max_lds() > 0) ? 0 : -1; }

PLLM_API const pllm_attention_api* pllm_attention_mfma_api() {
  static const pllm_attention_api api = {D, &pllm_paged_attention_mfma, &warm_up_device_queries};
  return &api;
}
