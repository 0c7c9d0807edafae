// Linear layers for 17 to a few hundred rows in bfloat16 (decode steps of many requests, short prompts, steps that
// hold prompt portions beside decoded tokens): out[M, N] = x[M, K] W[N, K]^T.  At these sizes the product is bound by
// streaming W from memory once; what has to be kept from spoiling that is the traffic of the rows, which every
// workgroup needs in full.
//
// Weights come in the tiled layout that `tile_weight` (ops.py) makes when a model is loaded: tiles of 16 weight rows x
// 32 columns of K, each 1 KB in the order of the matrix instruction's operand (lane g * 16 + r holds row r, columns
// 8 g .. 8 g + 7), the tiles of one block of 16 rows one after the other along K.  A wavefront's load of a tile is 1 KB
// of contiguous memory (measured: 5.2 TB/s for a matrix of 46 MB, against 4.3 TB/s when the same operand is gathered
// from 16 rows of a row-major matrix) and lands in the registers the matrix instruction reads.
//
// A workgroup owns NT blocks of 16 weight rows and MT tiles of 16 input rows (all rows of the step up to 128; more rows
// are further workgroups along y, which find the weights in the caches) over a range of K, in stages of 256 columns:
//
//   8 compute wavefronts   wavefront c takes columns 32 c .. 32 c + 31 of every stage: its NT weight tiles straight
//                          from memory, DW stages ahead in registers; the rows' operands from LDS; NT x MT matrix
//                          instructions (v_mfma_f32_16x16x32_bf16) per stage into its own accumulators
//   4 loader wavefronts    bring the rows of a stage (MT * 16 rows x 256 columns) from memory (cache hits) straight into
//                          LDS (global_load_lds, 16 bytes per lane, no registers in between), R stages deep.  They are
//                          wavefronts of their own because a wavefront's loads return in the order they were issued:
//                          rows asked for by a wavefront that also streams weights would wait behind the weights.
//                          A lane's 16 bytes are chosen so that four neighbouring lanes read 64 contiguous bytes of a row
//                          (measured twice as fast out of the caches as 16 lanes on 16 rows), and the piece is put where
//                          the compute wavefront's lane finds it without bank conflicts (pieces of a row XOR-ed with the
//                          row's quarter).
//
// One workgroup barrier per stage (an s_barrier alone: it does not wait for loads under way, so the weights keep
// streaming across it).  At the end the eight wavefronts' sums are added through LDS in wavefront order and the epilogue
// runs: bfloat16 or float out, act(gate) * up, the rotary encoding of q and k with the write of k and v into their cache
// pages, or float partial sums of a range of K ([splits, M, N]: matrices with few rows are cut along K so that every
// compute unit streams; whoever consumes them adds the ranges in order).
// Every output element is summed in one fixed order that does not depend on the number of rows.
#include "common.h"
#include <type_traits>

using namespace pllm;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

constexpr int kComputeWaves = 8, kLoaderWaves = 4, kStreamThreads = (kComputeWaves + kLoaderWaves) * 64;
constexpr int kChunkK = 32;                          // columns of one matrix instruction: a wavefront's share of a stage
constexpr int kStageK = kComputeWaves * kChunkK;     // 256
constexpr int kTileElems = 16 * kChunkK;             // 512 elements, 1 KB

enum { SL_BF16 = 0, SL_F32 = 1, SL_GATED = 2, SL_PARTIAL = 3, SL_ROPE_KV = 4 };

struct StreamLinearParams {
  const bf16* x; int ldx;
  int activation;             // SL_GATED: the gate's activation (PLLM_ACT_*); here it fills a gap, and the arguments keep their places
  const bf16* wt;             // tiled weights [blocks of 16 rows][K / 32][64 lanes][8]
  void* out; int ldo;         // SL_PARTIAL: float [splits][M][ldo]
  int M, N, K;                // N: outputs (gated: half the weight rows)
  int ksteps;                 // K / 32
  int num_stages;             // stages of 256 columns that K has
  int stages_per_split;
  // SL_ROPE_KV: W = [q; k; v] rows tiled in units of 8 lower-half elements of a head and their 8 partners
  const int* positions; const float* cos_t; const float* sin_t; const int* slots;
  bf16* k_pages; bf16* v_pages;
  int num_heads, num_kv_heads, head_dim, block_size;
};

template <int N_>
__device__ __forceinline__ void wait_loads_but() {   // until at most N_ of this wavefront's loads are still under way
  static_assert(N_ >= 0 && N_ < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt((N_ & 0xf) | ((N_ >> 4) << 14) | 0x0f70);
}

__device__ __forceinline__ void stage_barrier() { asm volatile("s_barrier" ::: "memory"); }

template <int EPI, int NT, int MT, int R, int DW>
__global__ __launch_bounds__(kStreamThreads) void stream_linear_kernel(const StreamLinearParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char sl_lds[];
  constexpr int kSlotBytes = kComputeWaves * MT * 1024;          // the rows of one stage
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nb = blockIdx.x, row0 = blockIdx.y * (MT * 16), split = blockIdx.z;
  const int first_stage = split * p.stages_per_split;
  const int nstages = min(p.stages_per_split, p.num_stages - first_stage);     // at least one (the host sees to it)
  // Workgroups walk their stages from different starting points (the order of an output's sums then depends on its
  // place in the matrix, not on the batch): all of them asking the caches for the same rows at the same moment was
  // measured at little more than half the rate.
  const int start = (int)((blockIdx.x * 5u) % (unsigned)nstages);
  auto stage_at = [&](int s) { const int t = s + start; return first_stage + (t >= nstages ? t - nstages : t); };
  floatx4 acc[NT][MT];

  if (wave >= kComputeWaves) {
    // ---- loaders: the rows of stage s into slot s % R, R - 1 stages ahead of the stage being computed
    const int l = wave - kComputeWaves;
    const int r = lane >> 2, g = (lane & 3) ^ (r >> 2);          // four lanes per row; the row's pieces in XOR-ed order
    constexpr int kPerStage = 2 * MT;                            // loads of one loader per stage (8 * MT blocks of 1 KB for four)
    auto issue = [&](int s) {
      const int k_stage = stage_at(s) * kStageK;
      unsigned char* slot = sl_lds + (s % R) * kSlotBytes;
#pragma unroll
      for (int i = 0; i < kPerStage; ++i) {
        const int b = l + i * kLoaderWaves, c = b / MT, t = b - c * MT;        // block b: the operands of compute wavefront c, tile t
        const int row = min(row0 + t * 16 + r, p.M - 1);                       // rows past M repeat the last one: never stored
        const int k = min(k_stage + c * kChunkK + g * 8, p.K - 8);             // (a chunk past K is not computed)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(p.x + (size_t)row * p.ldx + k),
                                         (__attribute__((address_space(3))) void*)(slot + b * 1024), 16, 0, 0);
      }
    };
#pragma unroll
    for (int s = 0; s < R - 1; ++s) {
      if (s < nstages) issue(s);
    }
    for (int s = 0; s < nstages; ++s) {
      // stage s has landed when at most the loads of the stages behind it are under way
      if (R >= 3 && s + 1 < nstages) wait_loads_but<(R >= 3 ? (R - 2) * kPerStage : 0)>(); else wait_loads_but<0>();
      stage_barrier();                                           // everybody is done with stage s - 1: its slot is free
      if (s + R - 1 < nstages) issue(s + R - 1);
    }
  } else {
    // ---- compute: this wavefront's 32 columns of every stage
#pragma unroll
    for (int u = 0; u < NT; ++u) {
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[u][t] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    const bf16* wbase = p.wt + (size_t)nb * NT * p.ksteps * kTileElems + lane * 8;
    bf16x8 wbuf[DW][NT];
    auto load_w = [&](int s, bf16x8 (&dst)[NT]) {                // unconditional: a stage past the range rereads the last one
      const int ks = min(stage_at(min(s, nstages - 1)) * kComputeWaves + wave, p.ksteps - 1);
#pragma unroll
      for (int u = 0; u < NT; ++u) dst[u] = *reinterpret_cast<const bf16x8*>(wbase + ((size_t)u * p.ksteps + ks) * kTileElems);
    };
#pragma unroll
    for (int d = 0; d < DW; ++d) load_w(d, wbuf[d]);
    const int r = lane & 15, g = lane >> 4;
    const unsigned char* mine = sl_lds + wave * MT * 1024 + (r * 4 + (g ^ (r >> 2))) * 16;      // where the loaders put this lane's operands
    int slot = 0;
    // One stage: wait for the rows, fetch this lane's operands (all requested before the first is used), multiply, and
    // refill the registers the weights came from with the stage DW further on.  LAST: the stages that the rounds below
    // leave over; they refill nothing.  (A K that is no multiple of 256 cuts one stage short: wavefronts without columns
    // in it skip the products.)
    auto stage = [&](int s, bf16x8 (&w)[NT], auto last) {
      constexpr bool LAST = decltype(last)::value;
      stage_barrier();
      bf16x8 xf[MT];
#pragma unroll
      for (int t = 0; t < MT; ++t) xf[t] = *reinterpret_cast<const bf16x8*>(mine + slot * kSlotBytes + t * 1024);
      asm volatile("" ::: "memory");                             // (the requests stay together in front of the products)
      if (stage_at(s) * kComputeWaves + wave < p.ksteps) {
#pragma unroll
        for (int t = 0; t < MT; ++t) {
#pragma unroll
          for (int u = 0; u < NT; ++u) acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u], xf[t], acc[u][t], 0, 0, 0);
        }
      }
      if (!LAST) load_w(s + DW, w);
      slot = slot + 1 == R ? 0 : slot + 1;
    };
    // Rounds of DW stages without a condition inside (the compiler then knows how many loads are under way at every
    // use and waits for the oldest only), as long as a whole round lies before the last stage.
    int s = 0;
    for (; s + DW < nstages; s += DW) {
#pragma unroll
      for (int d = 0; d < DW; ++d) stage(s + d, wbuf[d], std::false_type{});
    }
#pragma unroll
    for (int d = 0; d < DW; ++d) {
      if (s + d < nstages) stage(s + d, wbuf[d], std::true_type{});
    }
  }

  // ---- the eight wavefronts' sums through LDS, added in wavefront order; epilogue
  floatx4* part = reinterpret_cast<floatx4*>(sl_lds);            // [8][NT][MT][64 lanes]: a lane's four sums are four weight rows of one input row
  stage_barrier();                                               // the last stage's operands are read
  if (wave < kComputeWaves) {
#pragma unroll
    for (int u = 0; u < NT; ++u) {
#pragma unroll
      for (int t = 0; t < MT; ++t) part[((wave * NT + u) * MT + t) * 64 + lane] = acc[u][t];
    }
  }
  __syncthreads();
  constexpr bool kPaired = EPI == SL_GATED || EPI == SL_ROPE_KV;  // tile rows 8-15 are the partners of rows 0-7
  for (int v = tid; v < NT * MT * 64; v += kStreamThreads) {
    const int tile = v >> 6, ln = v & 63, u = tile / MT, t = tile - u * MT;
    const int r = ln & 15, g = ln >> 4;
    const int m = row0 + t * 16 + r;                             // input row; this lane's sums are tile rows 4 g .. 4 g + 3
    if (m >= p.M || (kPaired && g >= 2)) continue;
    auto total = [&](int l) {
      floatx4 s = part[(u * MT + t) * 64 + l];
#pragma unroll
      for (int w = 1; w < kComputeWaves; ++w) s += part[((w * NT + u) * MT + t) * 64 + l];
      return s;
    };
    const floatx4 a = total(ln);
    const int unit = nb * NT + u;
    if (EPI == SL_GATED) {
      // a tile holds 8 gate rows and, 8 tile rows further, the up rows of the same outputs
      const floatx4 up = total(ln + 32);
      const int n = unit * 8 + g * 4;
      bf16 o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = __float2bfloat16(gate_activation(a[i], p.activation) * up[i]);
      bf16* dst = (bf16*)p.out + (size_t)m * p.ldo + n;
      if (n + 3 < p.N && (p.ldo & 3) == 0) *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(o);
      else {
#pragma unroll
        for (int i = 0; i < 4; ++i) if (n + i < p.N) dst[i] = o[i];
      }
    } else if (EPI == SL_ROPE_KV) {
      // a tile holds 8 elements of the lower half of a head and their partners in the upper half (element i turns with i + d/2)
      const floatx4 hi = total(ln + 32);
      const int d = p.head_dim, half = d >> 1, per_head = half >> 3;
      const int head = unit / per_head, ri = (unit - head * per_head) * 8 + g * 4;
      const int nh = p.num_heads, nkv = p.num_kv_heads;
      if (head >= nh + 2 * nkv) continue;                        // (the zero rows that pad the tiled weights)
      if (head < nh + nkv) {
        floatx4 cs = {1.f, 1.f, 1.f, 1.f}, sn = {0.f, 0.f, 0.f, 0.f};
        if (p.cos_t) {
          const size_t at = (size_t)p.positions[m] * half + ri;
          cs = *reinterpret_cast<const floatx4*>(p.cos_t + at);
          sn = *reinterpret_cast<const floatx4*>(p.sin_t + at);
        }
        bf16 lo_out[4], hi_out[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // q and k are rounded to bfloat16 by the projection before they are rotated
          const float lo = __bfloat162float(__float2bfloat16(a[i])), up = __bfloat162float(__float2bfloat16(hi[i]));
          float rl, ru;
          rotate_pair(lo, up, cs[i], sn[i], rl, ru);
          lo_out[i] = __float2bfloat16(rl);
          hi_out[i] = __float2bfloat16(ru);
        }
        bf16* dst = nullptr;
        if (head < nh) dst = (bf16*)p.out + (size_t)m * p.ldo + (size_t)head * d + ri;
        else {
          const int slot = p.slots[m];
          if (slot >= 0) {
            const int page = slot / p.block_size, off = slot - page * p.block_size;
            dst = p.k_pages + (((size_t)page * nkv + (head - nh)) * p.block_size + off) * d + ri;
          }
        }
        if (dst) {                                               // (8-byte stores: ri and d / 2 are multiples of four)
          *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(lo_out);
          *reinterpret_cast<uint2*>(dst + half) = *reinterpret_cast<const uint2*>(hi_out);
        }
      } else {
        const int slot = p.slots[m];
        if (slot >= 0) {
          const int page = slot / p.block_size, off = slot - page * p.block_size;
          bf16* vdst = p.v_pages + ((size_t)page * nkv + (head - nh - nkv)) * d * p.block_size + off;     // values lie transposed in a page
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            vdst[(size_t)(ri + i) * p.block_size] = __float2bfloat16(a[i]);
            vdst[(size_t)(ri + half + i) * p.block_size] = __float2bfloat16(hi[i]);
          }
        }
      }
    } else {
      const int n = unit * 16 + g * 4;
      if (EPI == SL_BF16) {
        bf16 o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = __float2bfloat16(a[i]);
        bf16* dst = (bf16*)p.out + (size_t)m * p.ldo + n;
        if (n + 3 < p.N && (p.ldo & 3) == 0) *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(o);
        else {
#pragma unroll
          for (int i = 0; i < 4; ++i) if (n + i < p.N) dst[i] = o[i];
        }
      } else {
        float* dst = (float*)p.out + ((size_t)(EPI == SL_PARTIAL ? split : 0) * p.M + m) * p.ldo + n;
        if (n + 3 < p.N && (p.ldo & 3) == 0) *reinterpret_cast<floatx4*>(dst) = a;
        else {
#pragma unroll
          for (int i = 0; i < 4; ++i) if (n + i < p.N) dst[i] = a[i];
        }
      }
    }
  }
}

template <int EPI, int NT, int MT, int R, int DW>
static int launch_stream(const StreamLinearParams& p, dim3 grid, hipStream_t stream) {
  constexpr size_t slots = (size_t)R * kComputeWaves * MT * 1024, sums = (size_t)kComputeWaves * NT * MT * 1024;
  constexpr size_t lds = slots > sums ? slots : sums;
  static_assert(lds <= 160 * 1024, "LDS of one compute unit");
  auto kernel = stream_linear_kernel<EPI, NT, MT, R, DW>;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  hipLaunchKernelGGL(kernel, grid, dim3(kStreamThreads), lds, stream, p);
  return (int)hipGetLastError();
}

// Rows of a workgroup along y: as few blocks as 128 rows each allow, evenly filled, in tiles of 32 rows.
PLLM_API int pllm_stream_linear_row_blocks(int M) { return (M + 127) / 128; }

// nt: blocks of 16 weight rows per workgroup (1 to 4); the tiled weights hold a multiple of 24 blocks (zero rows at the end).
// splits > 1 with epi SL_PARTIAL only.
PLLM_API int pllm_stream_linear(int epi, const void* x, int ldx, const void* wt, void* out, int ldo, int M, int N, int K,
                                int weight_blocks, int nt, int splits, const int* positions, const float* cos_t, const float* sin_t,
                                const int* slots, void* k_pages, void* v_pages, int num_heads, int num_kv_heads, int head_dim,
                                int block_size, int activation, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K % kChunkK) || (ldx & 7) || nt < 1 || nt > 4 || weight_blocks <= 0 || (weight_blocks % 24) || splits < 1) return -2;
  if (splits > 1 && epi != SL_PARTIAL) return -2;
  if (epi == SL_ROPE_KV && (head_dim <= 0 || (head_dim % 16) || !slots || !k_pages || !v_pages || !positions ||
                            N != (num_heads + 2 * num_kv_heads) * head_dim || block_size <= 0 || (ldo & 3))) return -2;
  const int rows_of_w = epi == SL_GATED ? 2 * N : N;
  if ((long)weight_blocks * 16 < rows_of_w) return -2;
  StreamLinearParams p;
  p.x = (const bf16*)x; p.ldx = ldx; p.wt = (const bf16*)wt; p.out = out; p.ldo = ldo; p.M = M; p.N = N; p.K = K;
  p.positions = positions; p.cos_t = cos_t; p.sin_t = sin_t; p.slots = slots; p.k_pages = (bf16*)k_pages; p.v_pages = (bf16*)v_pages;
  p.num_heads = num_heads; p.num_kv_heads = num_kv_heads; p.head_dim = head_dim; p.block_size = block_size;
  if (activation < 0 || activation >= PLLM_ACT_COUNT) return -2;
  p.activation = activation;
  p.ksteps = K / kChunkK;
  p.num_stages = (K + kStageK - 1) / kStageK;
  p.stages_per_split = (p.num_stages + splits - 1) / splits;
  if ((long)p.stages_per_split * (splits - 1) >= p.num_stages) return -2;      // (every range of K has a stage)
  const int m_blocks = pllm_stream_linear_row_blocks(M);
  const int rows = (M + m_blocks - 1) / m_blocks, mt = (rows + 31) / 32 * 2;    // 2, 4, 6 or 8 tiles of 16 rows
  if (nt >= 3 && mt > 4) return -2;
  const int n_blocks = ((rows_of_w + 15) / 16 + nt - 1) / nt;
  if (n_blocks > 65535 * 16 || m_blocks > 65535 || splits > 65535) return -2;
  const dim3 grid(n_blocks, m_blocks, splits);
#define PLLM_SL(EPI_, NT_, MT_, R_, DW_) return launch_stream<EPI_, NT_, MT_, R_, DW_>(p, grid, stream)
#define PLLM_SL_SHAPES(EPI_)                                          \
  do {                                                                \
    if (nt == 1) {                                                    \
      switch (mt) {                                                   \
        case 2: PLLM_SL(EPI_, 1, 2, 3, 8);                            \
        case 4: PLLM_SL(EPI_, 1, 4, 3, 8);                            \
        case 6: PLLM_SL(EPI_, 1, 6, 2, 8);                            \
        case 8: PLLM_SL(EPI_, 1, 8, 2, 8);                            \
      }                                                               \
    } else if (nt == 2) {                                             \
      switch (mt) {                                                   \
        case 2: PLLM_SL(EPI_, 2, 2, 3, 6);                            \
        case 4: PLLM_SL(EPI_, 2, 4, 3, 6);                            \
        case 6: PLLM_SL(EPI_, 2, 6, 2, 6);                            \
        case 8: PLLM_SL(EPI_, 2, 8, 2, 6);                            \
      }                                                               \
    } else if (nt == 3) {                                             \
      switch (mt) {                                                   \
        case 2: PLLM_SL(EPI_, 3, 2, 3, 6);                            \
        case 4: PLLM_SL(EPI_, 3, 4, 3, 6);                            \
      }                                                               \
    } else {                                                          \
      switch (mt) {                                                   \
        case 2: PLLM_SL(EPI_, 4, 2, 3, 4);                            \
        case 4: PLLM_SL(EPI_, 4, 4, 3, 4);                            \
      }                                                               \
    }                                                                 \
  } while (0)
  switch (epi) {
    case SL_BF16: PLLM_SL_SHAPES(SL_BF16); break;
    case SL_F32: PLLM_SL_SHAPES(SL_F32); break;
    case SL_GATED: PLLM_SL_SHAPES(SL_GATED); break;
    case SL_PARTIAL: PLLM_SL_SHAPES(SL_PARTIAL); break;
    case SL_ROPE_KV: PLLM_SL_SHAPES(SL_ROPE_KV); break;
  }
#undef PLLM_SL_SHAPES
#undef PLLM_SL
  return -3;
}

// ---------------------------------------------------------------------------------------------
// The same products for a few hundred rows (steps that hold a prompt portion, short prompts): tiles of up to 128 input
// rows x 128 weight rows per workgroup, along x the blocks of weight rows, along y the blocks of input rows, along z
// ranges of K.  With this many rows every workgroup of the kernel above would read all of them for its 32 weight rows;
// here both operands of a stage (64 columns of K) come into LDS once per workgroup, brought by the four loader
// wavefronts (the weights' tiles are 1 KB of contiguous memory each and land in operand order; the rows as above), and
// the eight compute wavefronts, as 2 x 4 over the tile (MTW tiles of 16 input rows x 2 blocks of 16 weight rows each),
// only read LDS and multiply.  No sums across wavefronts: each owns its outputs.  Epilogues as above.
constexpr int kTileBlocksN = 8;                      // blocks of 16 weight rows per workgroup, at most (NB: 8 or 4)
constexpr int kTileStageSteps = 2;                   // steps of 32 columns per stage

// MT: tiles of 16 input rows per workgroup (the upper row of wavefronts takes the larger half).
// What bounds a workgroup is what its compute unit can draw from the L2 (about 28 bytes a cycle when all compute units
// draw: cycle stamps show the loaders' requests queueing, a stage of 34 KB taking 1,250 cycles, whatever the number of
// stages in flight, with or without the products; four compute wavefronts as 2 x 2 with a third less LDS traffic took the
// same time), so a tile is as large as registers and LDS allow, and matrices of many rows and few hundred input rows,
// whose tiles cannot be large in both directions, stay with the library, which meets the same bound.
template <int EPI, int MT, int R, int NB>
__global__ __launch_bounds__(kStreamThreads) void tile_linear_kernel(const StreamLinearParams p) {
  constexpr int CW = kComputeWaves;
  extern __shared__ __attribute__((aligned(16))) unsigned char sl_lds[];
  constexpr int MTW = (MT + 1) / 2;                              // tiles of 16 input rows per wavefront (at most)
  constexpr int WN = CW / 2, NTW = NB / WN;                      // wavefronts along the weight rows, blocks of 16 weight rows each
  constexpr int kWBlocks = NB * kTileStageSteps, kXBlocks = MT * kTileStageSteps;
  constexpr int kSlotBytes = (kWBlocks + kXBlocks) * 1024;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nb = blockIdx.x, row0 = blockIdx.y * (MT * 16), split = blockIdx.z;
  const int first_stage = split * p.stages_per_split;           // (stages of 64 columns here)
  const int nstages = min(p.stages_per_split, p.num_stages - first_stage);
  floatx4 acc[MTW][NTW];

  if (wave >= CW) {
    const int l = wave - CW;
    const int xr = lane >> 2, xg = (lane & 3) ^ (xr >> 2);
    constexpr int kBlocks = kWBlocks + kXBlocks, kPerLoader = (kBlocks + kLoaderWaves - 1) / kLoaderWaves;
    static_assert(kWBlocks % kLoaderWaves == 0, "a loader's i-th block is a weight tile for all loaders or for none");
    // A loader's i-th block of a stage is the same block in every stage, kAdvance further along K: the addresses of the
    // first stage are worked out once (a dozen vector instructions each, which issued before every load made the loaders
    // the slowest part of a stage), a stage adds its offset.
    const bf16* base[kPerLoader];
#pragma unroll
    for (int i = 0; i < kPerLoader; ++i) {
      const int bb = min(l + i * kLoaderWaves, kBlocks - 1);     // (every loader issues the same number of loads per stage: the waits
                                                                 //  below count them; a loader whose share is one short repeats its last block)
      if (bb < kWBlocks) {
        const int u = bb / kTileStageSteps, st = bb - u * kTileStageSteps;
        base[i] = p.wt + (((size_t)(nb * NB + u) * p.ksteps + first_stage * kTileStageSteps + st) * 64 + lane) * 8;
      } else {
        const int bx = bb - kWBlocks, t = bx / kTileStageSteps, st = bx - t * kTileStageSteps;
        const int row = min(row0 + t * 16 + xr, p.M - 1);        // rows past M repeat the last one: never stored
        base[i] = p.x + (size_t)row * p.ldx + (first_stage * kTileStageSteps + st) * kChunkK + xg * 8;
      }
    }
    const bool odd_steps = p.ksteps & 1;                         // K no multiple of 64: the last stage has one step only
    auto issue = [&](int s) {
      unsigned char* slot = sl_lds + (s % R) * kSlotBytes;
      if (odd_steps && first_stage + s == p.num_stages - 1) {
        // the stage that K cuts short: its second step repeats the first (and is not computed)
        const int ks0 = (first_stage + s) * kTileStageSteps;
#pragma unroll
        for (int i = 0; i < kPerLoader; ++i) {
          const int bb = min(l + i * kLoaderWaves, kBlocks - 1);
          const bf16* src;
          if (bb < kWBlocks) src = p.wt + (((size_t)(nb * NB + bb / kTileStageSteps) * p.ksteps + ks0) * 64 + lane) * 8;
          else src = p.x + (size_t)min(row0 + ((bb - kWBlocks) / kTileStageSteps) * 16 + xr, p.M - 1) * p.ldx + ks0 * kChunkK + xg * 8;
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                           (__attribute__((address_space(3))) void*)(slot + bb * 1024), 16, 0, 0);
        }
        return;
      }
#pragma unroll
      for (int i = 0; i < kPerLoader; ++i) {
        const int bb = min(l + i * kLoaderWaves, kBlocks - 1);
        constexpr int kTileAdvance = kTileStageSteps * kTileElems, kRowAdvance = kTileStageSteps * kChunkK;
        const bf16* src = base[i] + (size_t)s * (i * kLoaderWaves < kWBlocks ? kTileAdvance : kRowAdvance);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                         (__attribute__((address_space(3))) void*)(slot + bb * 1024), 16, 0, 0);
      }
    };
#pragma unroll
    for (int s = 0; s < R - 1; ++s) {
      if (s < nstages) issue(s);
    }
    for (int s = 0; s < nstages; ++s) {
      // stage s has landed when at most the loads of the R - 2 stages behind it are under way (fewer near the end)
      const int behind = min(R - 2, nstages - 1 - s);
      if (behind >= 2) wait_loads_but<2 * kPerLoader>();
      else if (behind == 1) wait_loads_but<kPerLoader>();
      else wait_loads_but<0>();
      stage_barrier();
      if (s + R - 1 < nstages) issue(s + R - 1);
    }
  } else {
#pragma unroll
    for (int t = 0; t < MTW; ++t) {
#pragma unroll
      for (int u = 0; u < NTW; ++u) acc[t][u] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    const int wm = wave / WN, wn = wave - wm * WN;
    const int my_tiles = wm == 0 ? MTW : MT - MTW;               // (the same for the whole wavefront)
    const int r = lane & 15, g = lane >> 4;
    const unsigned char* my_w = sl_lds + (wn * NTW * kTileStageSteps) * 1024 + lane * 16;
    const unsigned char* my_x = sl_lds + (kWBlocks + wm * MTW * kTileStageSteps) * 1024 + (r * 4 + (g ^ (r >> 2))) * 16;
    int slot = 0;
    for (int s = 0; s < nstages; ++s) {
      stage_barrier();
      const int steps = min(kTileStageSteps, p.ksteps - (first_stage + s) * kTileStageSteps);
      // All operands of the stage are requested before the first product: the requests of the second step travel while
      // the first step's products run (asked for step by step, a wavefront waited for LDS twice per stage, 200 cycles each,
      // with its SIMD's other wavefront in the same place at the same time).
      bf16x8 wf[kTileStageSteps][NTW], xf[kTileStageSteps][MTW];
#pragma unroll
      for (int st = 0; st < kTileStageSteps; ++st) {
#pragma unroll
        for (int u = 0; u < NTW; ++u) wf[st][u] = *reinterpret_cast<const bf16x8*>(my_w + slot * kSlotBytes + (u * kTileStageSteps + st) * 1024);
        // (the lower row of wavefronts may have a tile less: it reads its last tile again and leaves the product out)
#pragma unroll
        for (int t = 0; t < MTW; ++t) xf[st][t] = *reinterpret_cast<const bf16x8*>(my_x + slot * kSlotBytes + (min(t, my_tiles - 1) * kTileStageSteps + st) * 1024);
      }
      asm volatile("" ::: "memory");
#pragma unroll
      for (int st = 0; st < kTileStageSteps; ++st) {
        if (st < steps) {
#pragma unroll
          for (int t = 0; t < MTW; ++t) {
            if (t < my_tiles) {
#pragma unroll
              for (int u = 0; u < NTW; ++u) acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[st][u], xf[st][t], acc[t][u], 0, 0, 0);
            }
          }
        }
      }
      slot = slot + 1 == R ? 0 : slot + 1;
    }

    // ---- epilogue: a lane's four sums are four weight rows (4 g .. 4 g + 3 of the tile) of input row r
    constexpr bool kPaired = EPI == SL_GATED || EPI == SL_ROPE_KV;
#pragma unroll
    for (int t = 0; t < MTW; ++t) {
#pragma unroll
      for (int u = 0; u < NTW; ++u) {
        const int m = t < my_tiles ? row0 + (wm * MTW + t) * 16 + r : p.M;
        const int unit = nb * NB + wn * NTW + u;
        const floatx4 a = acc[t][u];
        floatx4 partner = a;
        if (kPaired) {                                           // tile rows 8-15 (the lanes 32 further on) hold the partners of rows 0-7
#pragma unroll
          for (int i = 0; i < 4; ++i) partner[i] = __shfl_down(a[i], 32, 64);
        }
        if (m >= p.M || (kPaired && g >= 2)) continue;
        if (EPI == SL_GATED) {
          const int n = unit * 8 + g * 4;
          bf16 o[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) o[i] = __float2bfloat16(gate_activation(a[i], p.activation) * partner[i]);
          bf16* dst = (bf16*)p.out + (size_t)m * p.ldo + n;
          if (n + 3 < p.N && (p.ldo & 3) == 0) *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(o);
          else {
#pragma unroll
            for (int i = 0; i < 4; ++i) if (n + i < p.N) dst[i] = o[i];
          }
        } else if (EPI == SL_ROPE_KV) {
          const int d = p.head_dim, half = d >> 1, per_head = half >> 3;
          const int head = unit / per_head, ri = (unit - head * per_head) * 8 + g * 4;
          const int nh = p.num_heads, nkv = p.num_kv_heads;
          if (head >= nh + 2 * nkv) continue;
          if (head < nh + nkv) {
            floatx4 cs = {1.f, 1.f, 1.f, 1.f}, sn = {0.f, 0.f, 0.f, 0.f};
            if (p.cos_t) {
              const size_t at = (size_t)p.positions[m] * half + ri;
              cs = *reinterpret_cast<const floatx4*>(p.cos_t + at);
              sn = *reinterpret_cast<const floatx4*>(p.sin_t + at);
            }
            bf16 lo_out[4], hi_out[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const float lo = __bfloat162float(__float2bfloat16(a[i])), up = __bfloat162float(__float2bfloat16(partner[i]));
              float rl, ru;
              rotate_pair(lo, up, cs[i], sn[i], rl, ru);
              lo_out[i] = __float2bfloat16(rl);
              hi_out[i] = __float2bfloat16(ru);
            }
            bf16* dst = nullptr;
            if (head < nh) dst = (bf16*)p.out + (size_t)m * p.ldo + (size_t)head * d + ri;
            else {
              const int slot_kv = p.slots[m];
              if (slot_kv >= 0) {
                const int page = slot_kv / p.block_size, off = slot_kv - page * p.block_size;
                dst = p.k_pages + (((size_t)page * nkv + (head - nh)) * p.block_size + off) * d + ri;
              }
            }
            if (dst) {
              *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(lo_out);
              *reinterpret_cast<uint2*>(dst + half) = *reinterpret_cast<const uint2*>(hi_out);
            }
          } else {
            const int slot_kv = p.slots[m];
            if (slot_kv >= 0) {
              const int page = slot_kv / p.block_size, off = slot_kv - page * p.block_size;
              bf16* vdst = p.v_pages + ((size_t)page * nkv + (head - nh - nkv)) * d * p.block_size + off;
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                vdst[(size_t)(ri + i) * p.block_size] = __float2bfloat16(a[i]);
                vdst[(size_t)(ri + half + i) * p.block_size] = __float2bfloat16(partner[i]);
              }
            }
          }
        } else {
          const int n = unit * 16 + g * 4;
          if (EPI == SL_BF16) {
            bf16 o[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) o[i] = __float2bfloat16(a[i]);
            bf16* dst = (bf16*)p.out + (size_t)m * p.ldo + n;
            if (n + 3 < p.N && (p.ldo & 3) == 0) *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(o);
            else {
#pragma unroll
              for (int i = 0; i < 4; ++i) if (n + i < p.N) dst[i] = o[i];
            }
          } else {
            float* dst = (float*)p.out + ((size_t)(EPI == SL_PARTIAL ? split : 0) * p.M + m) * p.ldo + n;
            if (n + 3 < p.N && (p.ldo & 3) == 0) *reinterpret_cast<floatx4*>(dst) = a;
            else {
#pragma unroll
              for (int i = 0; i < 4; ++i) if (n + i < p.N) dst[i] = a[i];
            }
          }
        }
      }
    }
  }
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

template <int EPI, int MT, int R, int NB>
static int launch_tile(const StreamLinearParams& p, dim3 grid, hipStream_t stream) {
  constexpr size_t lds = (size_t)R * (NB * kTileStageSteps + MT * kTileStageSteps) * 1024;
  static_assert(lds <= 160 * 1024, "LDS of one compute unit");
  auto kernel = tile_linear_kernel<EPI, MT, R, NB>;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  hipLaunchKernelGGL(kernel, grid, dim3(kStreamThreads), lds, stream, p);
  return (int)hipGetLastError();
}

// Blocks of input rows of the tiled kernel when the product is cut into ranges of K: of at most 160 rows (10 tiles of 16),
// evenly filled.
PLLM_API int pllm_tile_linear_row_blocks(int M) { return (M + 159) / 160; }

// Tiles of 16 input rows per workgroup that the kernel is compiled for, for a block of `rows` input rows.
static int tile_rows_compiled(int rows) {
  const int mt = (rows + 15) / 16;
  return mt <= 2 ? 2 : mt <= 4 ? 4 : mt <= 6 ? 6 : mt <= 8 ? 8 : mt;       // (9 and 10 as they are)
}

// Shape of the tiles of a product in one range of K: blocks of input rows (evenly filled, of 32 to 160 rows) x tiles of
// 128 or 64 weight rows.  A workgroup has about 100 KB under way whatever its tile, so what counts first is how many
// workgroups run at once: the shape with the most workgroups that still fit the compute units in one round (q/k/v of
// 2560 x 2048 at 264 rows: 5 x 40 tiles of 64 x 64, 11.8 us, against 14.7 us as 3 x 40 and 16.9 us in the library with the
// rotary kernel behind it; 11264 x 2048 with the gated epilogue at 128 rows: 176 tiles of 128 x 64, 19.0 us, against 25.7
// as 88 tiles of 128 x 128), among equals the one that draws the fewest bytes, then the one with the fewest blocks of
// rows; the largest tiles when even those need more than one round.
static void tile_shape(int M, int weight_blocks16, int cus, int* m_blocks_out, int* nb_out) {
  long best_wgs = -1, best_bytes = 0;
  *m_blocks_out = pllm_tile_linear_row_blocks(M);
  *nb_out = kTileBlocksN;
  const int compiled[] = {10, 9, 8, 6, 4, 2};                   // tiles of 16 rows per block, the largest first
  for (int mt : compiled) {
    const int mb = (M + mt * 16 - 1) / (mt * 16);
    if (tile_rows_compiled(((M + mb - 1) / mb)) != mt) continue;  // (the same blocks, evenly filled, fit a smaller shape)
    for (int nb = kTileBlocksN; nb >= kTileBlocksN / 2; nb /= 2) {
      // (blocks of 144 and 160 rows only with tiles of 128 weight rows: twice the blocks of half the rows x tiles of 128
      //  are as many workgroups and draw fewer bytes, so the other shape would never be chosen and is not compiled)
      if (nb != kTileBlocksN && mt > 8) continue;
      const long n_blocks = (weight_blocks16 + nb - 1) / nb, wgs = n_blocks * mb;
      if (wgs > cus) continue;
      const long bytes = n_blocks * M + (long)mb * weight_blocks16 * 16;        // rows drawn, of K values each
      if (wgs > best_wgs || (wgs == best_wgs && bytes < best_bytes)) {
        best_wgs = wgs; best_bytes = bytes; *m_blocks_out = mb; *nb_out = nb;
      }
    }
  }
}

// What `tile_shape` chooses for M input rows and a matrix of `weight_rows` rows on `compute_units` compute units: rows per
// block of input rows (a multiple of 16) and weight rows per tile (128 or 64); returns the number of workgroups.
PLLM_API int pllm_tile_linear_shape(int M, int weight_rows, int compute_units, int* block_rows, int* tile_weight_rows) {
  if (M <= 0 || weight_rows <= 0 || compute_units <= 0) return -2;
  int m_blocks, nb;
  tile_shape(M, (weight_rows + 15) / 16, compute_units, &m_blocks, &nb);
  const int mt = tile_rows_compiled((M + m_blocks - 1) / m_blocks);
  *block_rows = mt * 16;
  *tile_weight_rows = nb * 16;
  return ((M + mt * 16 - 1) / (mt * 16)) * (((weight_rows + 15) / 16 + nb - 1) / nb);
}

// The tiled weights hold a multiple of 8 blocks (of 24, in fact).  splits > 1 with epi SL_PARTIAL only.
PLLM_API int pllm_tile_linear(int epi, const void* x, int ldx, const void* wt, void* out, int ldo, int M, int N, int K,
                              int weight_blocks, int splits, const int* positions, const float* cos_t,
                              const float* sin_t, const int* slots, void* k_pages, void* v_pages, int num_heads, int num_kv_heads,
                              int head_dim, int block_size, int activation, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K % kChunkK) || (ldx & 7) || weight_blocks <= 0 || (weight_blocks % kTileBlocksN) || splits < 1) return -2;
  if (splits > 1 && epi != SL_PARTIAL) return -2;
  if (epi == SL_ROPE_KV && (head_dim <= 0 || (head_dim % 16) || !slots || !k_pages || !v_pages || !positions ||
                            N != (num_heads + 2 * num_kv_heads) * head_dim || block_size <= 0 || (ldo & 3))) return -2;
  const int rows_of_w = epi == SL_GATED ? 2 * N : N;
  if ((long)weight_blocks * 16 < rows_of_w) return -2;
  StreamLinearParams p;
  p.x = (const bf16*)x; p.ldx = ldx; p.wt = (const bf16*)wt; p.out = out; p.ldo = ldo; p.M = M; p.N = N; p.K = K;
  p.positions = positions; p.cos_t = cos_t; p.sin_t = sin_t; p.slots = slots; p.k_pages = (bf16*)k_pages; p.v_pages = (bf16*)v_pages;
  p.num_heads = num_heads; p.num_kv_heads = num_kv_heads; p.head_dim = head_dim; p.block_size = block_size;
  if (activation < 0 || activation >= PLLM_ACT_COUNT) return -2;
  p.activation = activation;
  p.ksteps = K / kChunkK;
  p.num_stages = (p.ksteps + kTileStageSteps - 1) / kTileStageSteps;
  p.stages_per_split = (p.num_stages + splits - 1) / splits;
  if ((long)p.stages_per_split * (splits - 1) >= p.num_stages) return -2;
  // Cut into ranges of K (the caller's plan, which fills the GPU with them): blocks of up to 160 rows x 128 weight rows.
  // In one range: the shape that gives the most workgroups in one round.
  int m_blocks = pllm_tile_linear_row_blocks(M), nb_per = kTileBlocksN;
  if (epi != SL_PARTIAL) tile_shape(M, (rows_of_w + 15) / 16, num_compute_units(), &m_blocks, &nb_per);
  const bool narrow = nb_per != kTileBlocksN;
  const int rows = (M + m_blocks - 1) / m_blocks, mt = tile_rows_compiled(rows);     // tiles of 16 rows per workgroup: 2 to 10
  m_blocks = (M + mt * 16 - 1) / (mt * 16);                                     // (blocks are filled to whole tiles, the last one may be short)
  const int n_blocks = ((rows_of_w + 15) / 16 + nb_per - 1) / nb_per;
  if (m_blocks > 65535 || splits > 65535) return -2;
  const dim3 grid(n_blocks, m_blocks, splits);
  // (the kernel's row offset of a block along y is MT * 16: blocks are filled to whole tiles, the last one may be short)
#define PLLM_TL(EPI_, MT_)                                                                       \
  do {                                                                                           \
    if constexpr ((MT_) <= 8) {                                                                  \
      if (narrow) return launch_tile<EPI_, MT_, 4, kTileBlocksN / 2>(p, grid, stream);           \
    }                                                                                            \
    if (narrow) return -3;                                                                       \
    return launch_tile<EPI_, MT_, (MT_ > 8 ? 3 : 4), kTileBlocksN>(p, grid, stream);             \
  } while (0)
#define PLLM_TL_SHAPES(EPI_)                                                  \
  do {                                                                        \
    switch (mt) {                                                             \
      case 1: case 2: PLLM_TL(EPI_, 2);                                       \
      case 3: case 4: PLLM_TL(EPI_, 4);                                       \
      case 5: case 6: PLLM_TL(EPI_, 6);                                       \
      case 7: case 8: PLLM_TL(EPI_, 8);                                       \
      case 9: PLLM_TL(EPI_, 9);                                               \
      case 10: PLLM_TL(EPI_, 10);                                             \
    }                                                                         \
  } while (0)
  switch (epi) {
    case SL_BF16: PLLM_TL_SHAPES(SL_BF16); break;
    case SL_F32: PLLM_TL_SHAPES(SL_F32); break;
    case SL_GATED: PLLM_TL_SHAPES(SL_GATED); break;
    case SL_PARTIAL: PLLM_TL_SHAPES(SL_PARTIAL); break;
    case SL_ROPE_KV: PLLM_TL_SHAPES(SL_ROPE_KV); break;
  }
#undef PLLM_TL_SHAPES
#undef PLLM_TL
  return -3;
}
