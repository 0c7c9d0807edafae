// Linear layers of a decode step (at most 16 rows; plain rows up to 64, see the second kernel) in bfloat16, each fused with what surrounds it,
// because at these sizes a kernel launch costs as much as the weights take to stream:
//
//   prologue (optional)   rows = x (+ delta), the residual sum in float rounded once; the new
//                         residual is written out by workgroup 0; RMS norm in float: the elements
//                         take the norm's weights here, the row's 1 / rms goes onto the finished sums
//   product               rows[M, K] * W[N, K]^T on the matrix cores, float accumulation
//   epilogue              plain (bfloat16 or float out) | act(gate) * up | rotary encoding of q and
//                         k and the write of k, v into their cache pages
//
// One workgroup of 8 wavefronts owns units of 16 weight rows over all of K.  Its wavefronts deal the K
// slabs of 128 round-robin; per slab a lane issues four 16-byte loads of one weight row, laid out so that
// the four lanes that share a row read 64 contiguous bytes in each load instruction; the loaded pieces are
// the A operands of v_mfma_f32_16x16x32_bf16 (the rows use the same k assignment).  A wavefront first
// requests its share of the input rows (cache hits), then the first slabs of weights (HBM), and works on
// the rows while the weights travel.  The rows (after the norm) sit in LDS and are the B operand of every
// wavefront.  Partial sums of the wavefronts are added through LDS in wave order: every output is summed
// in one fixed order.
#include "common.h"

using namespace pllm;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;

constexpr int kSlab = 128;
constexpr int kPad = 8;            // bf16 elements of padding per LDS row (spreads rows over banks)
constexpr int kSquares = 512;      // floats of LDS for the rows' sums of squares: 16 rows x up to 32 column groups of 512

enum { EPI_BF16 = 0, EPI_F32 = 1, EPI_GATED = 2, EPI_ROPE_KV = 3 };

struct DecodeLinearParams {
  const bf16* x; int ldx;
  int activation;              // EPI_GATED: the gate's activation (PLLM_ACT_*); here it fills a gap, and the arguments keep their places
  const bf16* delta; int ldd;
  const float* norm_w; float eps;
  bf16* x_out; int ldxo;
  const int* row_index;
  const bf16* W; int ldw;
  const bf16* Wt;              // the same matrix in tiles of 16 rows x 32 columns in the matrix instruction's operand order (or null)
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

// One unit of work = 16 weight rows (one MFMA tile) over all of K:
//   plain        rows 16u .. 16u+15
//   gated        rows 0-7: gate rows 8u .. 8u+7, rows 8-15: the up rows of the same outputs
//   rotary/cache rows 0-7: columns j*8 .. j*8+7 of the lower half of a head, rows 8-15: their partners
//                in the upper half (element i turns with element i + d/2)
// so that both members of a pair are in one tile and the epilogue finds them in LDS.
//
// HALF (at most 8 input rows): a unit is 8 weight rows.  Tile rows 0-7 hold them for the even slab of a
// pair of K slabs, tile rows 8-15 hold the same weight rows for the odd slab; the B operand carries
// the input rows for the even slab in columns 0-7 and for the odd slab in columns 8-15.  The two
// diagonal 8 x 8 blocks of the result are the two halves of the sum; the other two are ignored.
// Twice as many units of half the size: small matrices then put work on every compute unit.
template <int EPI, bool HALF>
__device__ __forceinline__ int unit_row(const DecodeLinearParams& p, int unit, int r) {
  if (HALF) {
    const int rr = r & 7;
    if (EPI == EPI_ROPE_KV) {
      const int half = p.head_dim >> 1, per_head = half >> 2;
      const int head = unit / per_head, j = unit - head * per_head;
      return head * p.head_dim + j * 4 + (rr & 3) + (rr < 4 ? 0 : half);
    }
    return min(unit * 8 + rr, p.N - 1);
  }
  if (EPI == EPI_GATED) {
    const int n = min(unit * 8 + (r & 7), p.N - 1);
    return r < 8 ? n : n + p.N;                                 // up rows follow the gate rows
  }
  if (EPI == EPI_ROPE_KV) {
    const int half = p.head_dim >> 1, per_head = half >> 3;
    const int head = unit / per_head, j = unit - head * per_head;
    return head * p.head_dim + j * 8 + (r & 7) + (r < 8 ? 0 : half);
  }
  return min(unit * 16 + r, p.N - 1);
}

// Rotary epilogue for one pair (element ri of the lower half, its partner in the upper half) of
// head `head` of input row m: q is rotated and written out, k is rotated and written to its page,
// v is written to its (transposed) page.
__device__ __forceinline__ void rope_store(const DecodeLinearParams& p, int m, int head, int ri, float lo, float hi, float cs,
                                           float sn, int slot) {
  const int d = p.head_dim, half = d >> 1;
  const int nh = p.num_heads, nkv = p.num_kv_heads;
  if (head < nh + nkv) {
    // q and k are rounded to bfloat16 by the projection before they are rotated
    lo = __bfloat162float(__float2bfloat16(lo));
    hi = __bfloat162float(__float2bfloat16(hi));
    float rl, rh;
    rotate_pair(lo, hi, cs, sn, rl, rh);
    const bf16 out_lo = __float2bfloat16(rl), out_hi = __float2bfloat16(rh);
    if (head < nh) {
      bf16* q = (bf16*)p.out + (size_t)m * p.ldo + (size_t)head * d;
      q[ri] = out_lo;
      q[ri + half] = out_hi;
    } else {
      if (slot >= 0) {
        const int page = slot / p.block_size, off = slot - page * p.block_size;
        bf16* k = p.k_pages + (((size_t)page * nkv + (head - nh)) * p.block_size + off) * d;
        k[ri] = out_lo;
        k[ri + half] = out_hi;
      }
    }
  } else {
    if (slot >= 0) {
      const int page = slot / p.block_size, off = slot - page * p.block_size;
      bf16* v = p.v_pages + ((size_t)page * nkv + (head - nh - nkv)) * d * p.block_size + off;
      v[(size_t)ri * p.block_size] = __float2bfloat16(lo);
      v[(size_t)(ri + half) * p.block_size] = __float2bfloat16(hi);
    }
  }
}

// The rows into LDS (kernels whose input needs a residual sum and / or a norm): rows = x[row_index] (+ delta),
// the sum in float rounded once and written out by workgroup 0, the elements multiplied by the norm's
// weights, and the rows' sums of squares into `sq` ([M][column groups]).  `after_first_requests` is called once
// the first loads of the rows are issued: the caller requests its first weights there.
template <int WAVES, class Early>
__device__ __forceinline__ void stage_rows(const DecodeLinearParams& p, bf16* xs, float* sq, int row_len, int wave, int lane,
                                           Early&& after_first_requests) {
  const int M = p.M, K = p.K;
  // ---- the rows into LDS.  A wavefront owns a group of 64 pieces of 8 columns and walks rows with it, up
  // to kBatch rows at a time.  It requests the pieces of its first batch, then its weights, and only then
  // touches the first piece: loads return in the order they were issued, so the rows (cache hits) must not
  // queue behind the weights (HBM), and the weight loads carry no condition, so that the compiler can
  // count exactly how many loads may still be under way when a piece is used.  Sums of squares: per lane
  // over its 8 elements, over the wavefront, then over the column groups of a row in ascending order: one
  // fixed order, whatever else is in the batch.
  constexpr int kBatch = 4;
  const int ipr = ((K >> 3) + 63) >> 6;                         // column groups per row
  const int cg = min(ipr, WAVES), rpp = WAVES / cg;             // groups and rows under way at a time
  const int wc = wave % cg, wr = wave / cg;                     // this wavefront's first group and row
  const bool active = wr < rpp;
  int src_lane = lane < M ? lane : 0;                           // lane m holds the source row of input row m
  if (p.row_index) src_lane = p.row_index[src_lane];
  const bool has_delta = p.delta != nullptr, has_norm = p.norm_w != nullptr;
  bf16x8 xv[kBatch], dv[kBatch];
  float4 nw0, nw1;
  auto column = [&](int c) { return min((c * 64 + lane) * 8, K - 8); };   // loads stay inside the row ...
  auto inside = [&](int c) { return (c * 64 + lane) * 8 < K; };           // ... and this says whether they count
  auto issue = [&](int c, int m0) {                             // rows m0, m0 + rpp, ... of column group c
    const int k0 = column(c);
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const size_t src = (size_t)__builtin_amdgcn_readlane(src_lane, min(m0 + u * rpp, M - 1));
      xv[u] = *reinterpret_cast<const bf16x8*>(p.x + src * p.ldx + k0);
    }
    if (has_delta) {
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const size_t src = (size_t)__builtin_amdgcn_readlane(src_lane, min(m0 + u * rpp, M - 1));
        dv[u] = *reinterpret_cast<const bf16x8*>(p.delta + src * p.ldd + k0);
      }
    }
  };
  auto issue_norm = [&](int c) {
    if (has_norm) {
      nw0 = *reinterpret_cast<const float4*>(p.norm_w + column(c));
      nw1 = *reinterpret_cast<const float4*>(p.norm_w + column(c) + 4);
    }
  };
  auto sum_rows = [&](int c, int m0) {                          // pass 1 on the issued batch
    const int k0 = column(c);
    const bool in = inside(c);
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int m = m0 + u * rpp;
      if (!active || m >= M) continue;                          // the same for the whole wavefront
      bf16x8 v = xv[u];
      if (has_delta) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (__bf16)((float)v[i] + (float)dv[u][i]);     // float sum, rounded once
        if (p.x_out && blockIdx.x == 0 && in) {
          const size_t src = (size_t)__builtin_amdgcn_readlane(src_lane, m);
          *reinterpret_cast<bf16x8*>(p.x_out + src * p.ldxo + k0) = v;
        }
      }
      if (has_norm) {
        // The row's scale 1 / rms is applied to the finished sums (it is the same for the whole row);
        // here the elements take the norm's weights, and their squares are summed.
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) ss += (float)v[i] * (float)v[i];
        const float w[8] = {nw0.x, nw0.y, nw0.z, nw0.w, nw1.x, nw1.y, nw1.z, nw1.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (__bf16)((float)v[i] * w[i]);
        ss = wave_sum(in ? ss : 0.f);
        if (lane == 0) sq[m * ipr + c] = ss;
      }
      if (in) *reinterpret_cast<bf16x8*>(xs + (size_t)m * row_len + k0) = v;
    }
  };
  issue(wc, wr);
  issue_norm(wc);
  after_first_requests();                                       // the first unit's weights: on their way during all that follows
  sum_rows(wc, wr);
  for (int c = wc; c < ipr; c += cg) {
    if (c != wc) issue_norm(c);
    for (int m0 = (c == wc) ? wr + kBatch * rpp : wr; m0 < M; m0 += kBatch * rpp) {
      issue(c, m0);
      sum_rows(c, m0);
    }
  }
  __syncthreads();
}

// TILED (units of 16 rows only): the weights come from their tiled copy, in which the 16 rows x 32 columns that one
// load instruction of a wavefront fetches are 1 KB of contiguous memory, and a unit's tiles follow each other along K
// (measured: a matrix of 46 MB streams in 8.8 us that way and in 10.8 us gathered from 16 rows of the row-major matrix).
// The tiled copy orders its rows as the units here do (plain, gate with up, lower with upper half of a head).
template <int EPI, int WAVES, bool HALF, bool DIRECT, int PRE, bool TILED>
__global__ __launch_bounds__(WAVES * 64) void decode_linear_kernel(const DecodeLinearParams p, int num_units) {
  static_assert(!(TILED && HALF), "the tiled copy holds units of 16 rows");
  // Fetch the arguments the first loads depend on in one go (left alone, the compiler fetches each where
  // it is first used, and every fetch is a wait of its own).
  asm volatile("" ::"s"(p.x), "s"(p.delta), "s"(p.norm_w), "s"(p.row_index), "s"(p.W), "s"(p.x_out), "s"(p.ldx), "s"(p.ldd),
               "s"(p.ldw), "s"(p.ldxo), "s"(p.M), "s"(p.K), "s"(p.N), "s"(num_units));
  if (EPI == EPI_ROPE_KV) asm volatile("" ::"s"(p.positions), "s"(p.slots), "s"(p.cos_t), "s"(p.head_dim), "s"(p.num_heads), "s"(p.num_kv_heads));
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int M = p.M, N = p.N, K = p.K;
  const int row_len = K + kPad;
  bf16* xs = reinterpret_cast<bf16*>(lds_raw);                                       // [M][K + kPad] (not DIRECT)
  float* part = reinterpret_cast<float*>(lds_raw + (DIRECT ? 0 : (((size_t)M * row_len * 2 + 15) & ~(size_t)15)));   // [WAVES][256]
  float* sq = part + WAVES * 256;                               // [M][column groups] sums of squares, kSquares floats
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;

  // ---- request this wavefront's slabs of the first unit, then build the rows in LDS while they travel
  constexpr int kStep = HALF ? 2 * kSlab : kSlab;               // k range one wavefront consumes per step
  const int khalf = HALF ? (r >> 3) * kSlab : 0;                // HALF: tile rows / columns 8-15 work on the odd slab
  const int xrow = HALF ? (r & 7) : r;                          // input row this lane's B operand column belongs to
  const int num_slabs = (K + kStep - 1) / kStep;
  const int my_slabs = wave < num_slabs ? (num_slabs - wave + WAVES - 1) / WAVES : 0;
  // PRE slabs are in flight per wavefront (registers).  A unit is walked in rounds of PRE slabs (the last
  // round of a unit may hold slabs the wavefront does not have: they cost one cached address), and a
  // slot that has been consumed is refilled at once with the slab PRE positions further on, which may
  // belong to the next unit: the weights stream without a gap at unit boundaries.
  const int padded_slabs = max(PRE, (my_slabs + PRE - 1) / PRE * PRE);
  bf16x8 wbuf[PRE][4];
  auto load_w = [&](const bf16* wrow, int nth, bf16x8 (&dst)[4]) {      // nth slab of this wavefront of a unit's rows
    const int slab = wave + nth * WAVES;
    // No condition on the loads (the compiler would turn one into a branch around them, and could then no
    // longer tell how many loads are under way).  Past the end of K a lane rereads the row's last piece,
    // which meets zeros in the rows' operand; a slab this wavefront does not have is one address for all lanes.
    const bool mine = nth < my_slabs;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (TILED) {
        // (wrow: this lane's 16 bytes in the unit's first tile; tiles of 512 elements follow along K; past K the last tile again)
        const int ks = min(slab * 4 + j, (K >> 5) - 1);
        dst[j] = *reinterpret_cast<const bf16x8*>(mine ? wrow + (size_t)ks * 512 : p.Wt);
      } else {
        const int kk = slab * kStep + khalf + j * 32 + g * 8;
        dst[j] = *reinterpret_cast<const bf16x8*>(mine ? wrow + min(kk, K - 8) : p.W);
      }
    }
  };
  // DIRECT (rows that need no sum and no norm): the rows' operand comes straight from memory with the
  // weights of the same slab and never passes through LDS.  Tile columns past M read row M - 1; what they
  // produce is never stored.
  bf16x8 xbuf[DIRECT ? PRE : 1][4];
  const bf16* xsrc = p.x;
  if (DIRECT) {
    const int row = min(xrow, M - 1);
    xsrc = p.x + (size_t)(p.row_index ? p.row_index[row] : row) * p.ldx;
  }
  auto load_x = [&](int nth, bf16x8 (&dst)[4]) {
    const int slab = wave + nth * WAVES;
    const bool mine = nth < my_slabs;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int kk = slab * kStep + khalf + j * 32 + g * 8;
      const bf16x8 v = *reinterpret_cast<const bf16x8*>(mine ? xsrc + min(kk, K - 8) : p.x);
      dst[j] = kk < K ? v : zero8();                            // zeros past the end of K (the weights reread their last piece there)
    }
  };
  auto rows_of_unit = [&](int unit) {
    if (TILED) return p.Wt + ((size_t)unit * (K >> 5) * 64 + lane) * 8;
    return p.W + (size_t)unit_row<EPI, HALF>(p, unit, r) * p.ldw;
  };
  int unit = blockIdx.x;                                        // below num_units: the grid has no more workgroups than units
  const bf16* wrow = rows_of_unit(unit);
  auto request_first = [&]() {                                  // the first PRE slabs of the first unit, needed or not
    if (DIRECT) {
#pragma unroll
      for (int s = 0; s < PRE; ++s) load_x(s, xbuf[s]);
    }
#pragma unroll
    for (int s = 0; s < PRE; ++s) load_w(wrow, s, wbuf[s]);
  };

  // Rotary epilogue: what depends only on the input row is fetched early, not after the product.
  int rope_pos = 0, rope_slot = -1;
  auto rope_inputs = [&]() {
    if (EPI == EPI_ROPE_KV && tid < 256 && (HALF ? (r & 7) : r) < M && (!HALF || r < 8)) {
      rope_pos = p.cos_t ? p.positions[r] : 0;
      rope_slot = p.slots[r];
    }
  };
  if constexpr (DIRECT) {
    rope_inputs();
    request_first();
  } else {
  stage_rows<WAVES>(p, xs, sq, row_len, wave, lane, [&]() {
    rope_inputs();
    request_first();
  });
  }
  // 1 / rms of the input row this thread's results belong to (tile column r), from the sums of squares
  float row_scale = 1.f;
  if (!DIRECT && p.norm_w && r < M) {
    float total = 0.f;
    for (int j = 0; j < ((K >> 3) + 63) >> 6; ++j) total += sq[r * (((K >> 3) + 63) >> 6) + j];
    row_scale = rsqrtf(total * (1.f / (float)K) + p.eps);
  }

  auto x_operand = [&](int nth, int j, int s) {
    if (DIRECT) return xbuf[s][j];
    const int kk = (wave + nth * WAVES) * kStep + khalf + j * 32 + g * 8;
    return (xrow < M && kk < K) ? *reinterpret_cast<const bf16x8*>(xs + (size_t)xrow * row_len + kk) : zero8();
  };

  // ---- units of this workgroup, one after the other
  for (; unit < num_units; unit += gridDim.x) {
    floatx4 acc = floatx4{0.f, 0.f, 0.f, 0.f};
    float rope_cs = 1.f, rope_sn = 0.f;
    if (EPI == EPI_ROPE_KV && tid < 256 && p.cos_t) {
      // thread (i = tid >> 6, lane) will finish tile row g * 4 + i of input row r: fetch its angle now
      const int half = p.head_dim >> 1, per_head = HALF ? (half >> 2) : (half >> 3), rows = HALF ? 4 : 8;
      const int row = g * 4 + (tid >> 6);
      if (row < rows && r < M && (!HALF || r < 8)) {
        const int head = unit / per_head, ri = (unit - head * per_head) * rows + row;
        if (head < p.num_heads + p.num_kv_heads) {
          rope_cs = p.cos_t[(size_t)rope_pos * half + ri];
          rope_sn = p.sin_t[(size_t)rope_pos * half + ri];
        }
      }
    }
    const int next = unit + gridDim.x;
    const bf16* wrow_next = next < num_units ? rows_of_unit(next) : (TILED ? p.Wt : p.W);
    for (int base = 0; base < padded_slabs; base += PRE) {
#pragma unroll
      for (int s = 0; s < PRE; ++s) {
        const int nth = base + s;
        if (nth < my_slabs) {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wbuf[s][j], x_operand(nth, j, s), acc, 0, 0, 0);
        }
        const int ahead = nth + PRE;                            // refill the slot: this unit's slab, or the next unit's
        if (ahead < padded_slabs) {
          if (DIRECT) load_x(ahead, xbuf[s]);
          load_w(wrow, ahead, wbuf[s]);
        } else if (next < num_units) {
          if (DIRECT) load_x(ahead - padded_slabs, xbuf[s]);
          load_w(wrow_next, ahead - padded_slabs, wbuf[s]);
        }
      }
    }
    wrow = wrow_next;

    // acc[i] = element (tile row g*4 + i, input row r); add the wavefronts in wave order
#pragma unroll
    for (int i = 0; i < 4; ++i) part[wave * 256 + i * 64 + lane] = acc[i];
    __syncthreads();
    if (tid < 256) {
      const int i = tid >> 6;                                   // lane is tid & 63 again
      auto total = [&](int ln) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) s += part[w * 256 + i * 64 + ln];
        return s;
      };
      const int m = r, row = g * 4 + i;                         // column (input row) and row of the tile
      if (HALF) {
        // useful blocks: (rows 0-7, columns 0-7) + (rows 8-15, columns 8-15), 40 lanes further
        if (m < M && m < 8 && row < 8) {
          if (EPI == EPI_BF16 || EPI == EPI_F32) {
            const int n = unit * 8 + row;
            if (n < N) {
              const float v = (total(lane) + total(lane + 40)) * row_scale;
              if (EPI == EPI_F32) ((float*)p.out)[(size_t)m * p.ldo + n] = v;
              else ((bf16*)p.out)[(size_t)m * p.ldo + n] = __float2bfloat16(v);
            }
          } else if (EPI == EPI_ROPE_KV && row < 4) {
            const int d = p.head_dim, half = d >> 1, per_head = half >> 2;
            const int head = unit / per_head, ri = (unit - head * per_head) * 4 + row;
            const float lo = (total(lane) + total(lane + 40)) * row_scale, hi = (total(lane + 16) + total(lane + 56)) * row_scale;   // tile rows row + 4
            rope_store(p, m, head, ri, lo, hi, rope_cs, rope_sn, rope_slot);
          }
        }
      } else if (m < M) {
        if (EPI == EPI_BF16 || EPI == EPI_F32) {
          const int n = unit * 16 + row;
          if (n < N) {
            const float v = total(lane) * row_scale;
            if (EPI == EPI_F32) ((float*)p.out)[(size_t)m * p.ldo + n] = v;
            else ((bf16*)p.out)[(size_t)m * p.ldo + n] = __float2bfloat16(v);
          }
        } else if (EPI == EPI_GATED) {
          const int n = unit * 8 + row;
          if (row < 8 && n < N) {
            const float gate = total(lane) * row_scale, up = total(lane + 32) * row_scale;    // same outputs, 8 tile rows further
            ((bf16*)p.out)[(size_t)m * p.ldo + n] = __float2bfloat16(gate_activation(gate, p.activation) * up);
          }
        } else if (row < 8) {  // EPI_ROPE_KV
          const int d = p.head_dim, half = d >> 1, per_head = half >> 3;
          const int head = unit / per_head, ri = (unit - head * per_head) * 8 + row;   // rotation index in [0, half)
          rope_store(p, m, head, ri, total(lane) * row_scale, total(lane + 32) * row_scale, rope_cs, rope_sn, rope_slot);
        }
      }
    }
    __syncthreads();                                            // the partial sums are read: the buffer may be reused
  }
}

// 17 to 64 input rows (decoding with many requests): the same units, slabs and fixed order of sums, with
// MT tiles of 16 input rows side by side.  A weight slab is loaded once per wavefront and multiplied with
// each tile's rows, which come straight from memory (cache hits) beside it; there is no sum or norm in
// front of this form (the caller runs the norm on its own) and no LDS for the rows.
// XFIXED (K of at most PRE slabs per wavefront, 2048): a wavefront's share of the rows is the same for every
// unit, so it is loaded once and stays in registers; a workgroup with several units (the gate/up product) then
// reads the rows once instead of once per unit, which otherwise is four times what it streams of weights.
template <int EPI, int MT, bool XFIXED>
__global__ __launch_bounds__(512) void decode_linear_wide_kernel(const DecodeLinearParams p, int num_units) {
  constexpr int WAVES = 8, PRE = 2;
  asm volatile("" ::"s"(p.x), "s"(p.row_index), "s"(p.W), "s"(p.ldx), "s"(p.ldw), "s"(p.M), "s"(p.K), "s"(p.N), "s"(num_units));
  if (EPI == EPI_ROPE_KV) asm volatile("" ::"s"(p.positions), "s"(p.slots), "s"(p.cos_t), "s"(p.head_dim), "s"(p.num_heads), "s"(p.num_kv_heads));
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  float* part = reinterpret_cast<float*>(lds_raw);              // [WAVES][MT][256]
  const int M = p.M, N = p.N, K = p.K;
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int r = lane & 15, g = lane >> 4;
  const int num_slabs = (K + kSlab - 1) / kSlab;
  const int my_slabs = wave < num_slabs ? (num_slabs - wave + WAVES - 1) / WAVES : 0;
  const int padded_slabs = max(PRE, (my_slabs + PRE - 1) / PRE * PRE);
  bf16x8 wbuf[PRE][4], xbuf[PRE][MT][4];
  const int row0 = blockIdx.y * (MT * 16);                      // (a second line of workgroups takes the rows after the first MT tiles)
  const bf16* xsrc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {                                // tile columns past M read row M - 1; never stored
    const int row = min(row0 + t * 16 + r, M - 1);
    xsrc[t] = p.x + (size_t)(p.row_index ? p.row_index[row] : row) * p.ldx;
  }
  auto load_w = [&](const bf16* wrow, int nth, bf16x8 (&dst)[4]) {      // unconditional, as in the kernel above
    const int slab = wave + nth * WAVES;
    const bool mine = nth < my_slabs;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int kk = slab * kSlab + j * 32 + g * 8;
      dst[j] = *reinterpret_cast<const bf16x8*>(mine ? wrow + min(kk, K - 8) : p.W);
    }
  };
  auto load_x = [&](int nth, bf16x8 (&dst)[MT][4]) {
    const int slab = wave + nth * WAVES;
    const bool mine = nth < my_slabs;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int kk = slab * kSlab + j * 32 + g * 8;
        const bf16x8 v = *reinterpret_cast<const bf16x8*>(mine ? xsrc[t] + min(kk, K - 8) : p.x);
        dst[t][j] = kk < K ? v : zero8();
      }
    }
  };
  auto rows_of_unit = [&](int unit) { return p.W + (size_t)unit_row<EPI, false>(p, unit, r) * p.ldw; };
  int unit = blockIdx.x;
  const bf16* wrow = rows_of_unit(unit);
  int rope_pos[MT], rope_slot[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    rope_pos[t] = 0;
    rope_slot[t] = -1;
    if (EPI == EPI_ROPE_KV && tid < 256 && row0 + t * 16 + r < M) {
      rope_pos[t] = p.cos_t ? p.positions[row0 + t * 16 + r] : 0;
      rope_slot[t] = p.slots[row0 + t * 16 + r];
    }
  }
#pragma unroll
  for (int s = 0; s < PRE; ++s) {
    load_x(s, xbuf[s]);
    load_w(wrow, s, wbuf[s]);
  }

  for (; unit < num_units; unit += gridDim.x) {
    floatx4 acc[MT];
    float rope_cs[MT], rope_sn[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
      rope_cs[t] = 1.f;
      rope_sn[t] = 0.f;
    }
    if (EPI == EPI_ROPE_KV && tid < 256 && p.cos_t) {
      const int half = p.head_dim >> 1, per_head = half >> 3;
      const int row = g * 4 + (tid >> 6);
      const int head = unit / per_head, ri = (unit - head * per_head) * 8 + row;
      if (row < 8 && head < p.num_heads + p.num_kv_heads) {
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          if (row0 + t * 16 + r < M) {
            rope_cs[t] = p.cos_t[(size_t)rope_pos[t] * half + ri];
            rope_sn[t] = p.sin_t[(size_t)rope_pos[t] * half + ri];
          }
        }
      }
    }
    const int next = unit + gridDim.x;
    const bf16* wrow_next = next < num_units ? rows_of_unit(next) : p.W;
    for (int base = 0; base < padded_slabs; base += PRE) {
#pragma unroll
      for (int s = 0; s < PRE; ++s) {
        const int nth = base + s;
        if (nth < my_slabs) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wbuf[s][j], xbuf[s][t][j], acc[t], 0, 0, 0);
          }
        }
        const int ahead = nth + PRE;
        if (ahead < padded_slabs) {
          if (!XFIXED) load_x(ahead, xbuf[s]);
          load_w(wrow, ahead, wbuf[s]);
        } else if (next < num_units) {
          if (!XFIXED) load_x(ahead - padded_slabs, xbuf[s]);
          load_w(wrow_next, ahead - padded_slabs, wbuf[s]);
        }
      }
    }
    wrow = wrow_next;

#pragma unroll
    for (int t = 0; t < MT; ++t) {
#pragma unroll
      for (int i = 0; i < 4; ++i) part[(wave * MT + t) * 256 + i * 64 + lane] = acc[t][i];
    }
    __syncthreads();
    if (tid < 256) {
      const int i = tid >> 6, row = g * 4 + i;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        auto total = [&](int ln) {
          float s = 0.f;
#pragma unroll
          for (int w = 0; w < WAVES; ++w) s += part[(w * MT + t) * 256 + i * 64 + ln];
          return s;
        };
        const int m = row0 + t * 16 + r;
        if (m >= M) continue;
        if (EPI == EPI_BF16 || EPI == EPI_F32) {
          const int n = unit * 16 + row;
          if (n < N) {
            const float v = total(lane);
            if (EPI == EPI_F32) ((float*)p.out)[(size_t)m * p.ldo + n] = v;
            else ((bf16*)p.out)[(size_t)m * p.ldo + n] = __float2bfloat16(v);
          }
        } else if (EPI == EPI_GATED) {
          const int n = unit * 8 + row;
          if (row < 8 && n < N) {
            const float gate = total(lane), up = total(lane + 32);
            ((bf16*)p.out)[(size_t)m * p.ldo + n] = __float2bfloat16(gate_activation(gate, p.activation) * up);
          }
        } else if (row < 8) {  // EPI_ROPE_KV
          const int half = p.head_dim >> 1, per_head = half >> 3;
          const int head = unit / per_head, ri = (unit - head * per_head) * 8 + row;
          rope_store(p, m, head, ri, total(lane), total(lane + 32), rope_cs[t], rope_sn[t], rope_slot[t]);
        }
      }
    }
    __syncthreads();
  }
}

template <int EPI>
static int launch_wide(const DecodeLinearParams& p, int units, int blocks, int cus, hipStream_t stream) {
  int tiles = (p.M + 15) / 16, lines = 1;
  // A matrix with so few units that one workgroup each leaves compute units idle (the output and q/k/v products of a
  // 2048-wide model): two lines of workgroups, each with half of the row tiles, all resident at once (half of the compute
  // units per line).  Every unit's weights are then read by two workgroups (with a number of workgroups per line that
  // is a multiple of the L2s' number both sit behind the same L2, and the second read is a hit), each of which fetches
  // half the rows and finishes half the sums.  2048 x 2048: 11.5 -> 7.9 us at 64 rows, 7.8 -> 6.1 us at 32 rows;
  // 2560 x 2048 (160 units, so some workgroups take two): 11.7 -> 10.2 us at 64 rows.  More workgroups than compute
  // units lose: four lines of one tile at 64 rows 9.6 us, 160 units in two full lines 13.0 us.
  if (tiles >= 3 && units <= cus) {
    tiles = 2;
    lines = 2;
    blocks = min(blocks, cus / 2);
  } else if (tiles == 2 && 2 * units <= cus) {
    tiles = 1;
    lines = 2;
  }
  const size_t lds = (size_t)8 * tiles * 256 * sizeof(float);
  const bool fixed = (p.K + kSlab - 1) / kSlab <= 2 * 8;      // at most PRE slabs for each of the 8 wavefronts
#define PLLM_WIDE(MT_)                                                                                                                     \
  do {                                                                                                                                     \
    if (fixed) hipLaunchKernelGGL((decode_linear_wide_kernel<EPI, MT_, true>), dim3(blocks, lines), dim3(512), lds, stream, p, units);     \
    else hipLaunchKernelGGL((decode_linear_wide_kernel<EPI, MT_, false>), dim3(blocks, lines), dim3(512), lds, stream, p, units);          \
  } while (0)
  switch (tiles) {
    case 1: PLLM_WIDE(1); break;
    case 2: PLLM_WIDE(2); break;
    case 3: PLLM_WIDE(3); break;
    case 4: PLLM_WIDE(4); break;
    default: return -2;
  }
#undef PLLM_WIDE
  return (int)hipGetLastError();
}

template <int EPI, int WAVES, bool HALF, bool DIRECT, int PRE, bool TILED = false>
static int launch(const DecodeLinearParams& p, int units, int blocks, size_t lds, hipStream_t stream) {
  auto kernel = decode_linear_kernel<EPI, WAVES, HALF, DIRECT, PRE, TILED>;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(WAVES * 64), lds, stream, p, units);
  return (int)hipGetLastError();
}

// Largest LDS allocation of one workgroup on the current device.
PLLM_API long pllm_max_lds_bytes() {
  int dev = 0, v = 0;
  if (hipGetDevice(&dev) != hipSuccess) return -1;
  if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) return -1;
  return v;
}

// LDS of one compute unit (what resident workgroups share); on this GPU the same as one workgroup's limit.
static long pllm_lds_bytes_per_cu() {
  static long bytes = 0;
  if (!bytes) {
    const long v = pllm_max_lds_bytes();
    bytes = v > 0 ? v : 64 * 1024;
  }
  return bytes;
}

// Bytes of LDS a call needs; the caller checks them against the device's limit.
PLLM_API long pllm_decode_linear_lds_bytes(int M, int K, int waves) {
  const long rows = (((long)M * (K + kPad) * 2) + 15) & ~15L;
  return rows + (long)waves * 256 * 4 + kSquares * 4;
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

// W: the row-major matrix; Wt (optional, K a multiple of 32, at most 16 rows): its tiled copy, taken whenever the units
// are of 16 rows (W may then be null).
PLLM_API int pllm_decode_linear(int epi, const void* x, int ldx, const void* delta, int ldd, const float* norm_w, float eps,
                                void* x_out, int ldxo, const int* row_index, const void* W, int ldw, const void* Wt, void* out, int ldo, int M,
                                int N, int K, const int* positions, const float* cos_t, const float* sin_t, const int* slots,
                                void* k_pages, void* v_pages, int num_heads, int num_kv_heads, int head_dim, int block_size,
                                int activation, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (activation < 0 || activation >= PLLM_ACT_COUNT) return -2;
  if (M > 64 || (M > 16 && (delta || norm_w)) || K <= 0 || (K & 7) || (ldx & 7) || (W && (ldw & 7)) || (delta && (ldd & 7)) || (x_out && (ldxo & 7))) return -2;
  if ((!W && !Wt) || (Wt && (K & 31)) || (!W && M > 16)) return -2;
  DecodeLinearParams p;
  p.x = (const bf16*)x; p.ldx = ldx; p.delta = (const bf16*)delta; p.ldd = ldd; p.norm_w = norm_w; p.eps = eps;
  p.x_out = (bf16*)x_out; p.ldxo = ldxo; p.row_index = row_index; p.W = (const bf16*)W; p.ldw = ldw; p.Wt = (const bf16*)Wt; p.out = out; p.ldo = ldo;
  p.M = M; p.N = N; p.K = K; p.positions = positions; p.cos_t = cos_t; p.sin_t = sin_t; p.slots = slots;
  p.k_pages = (bf16*)k_pages; p.v_pages = (bf16*)v_pages; p.num_heads = num_heads; p.num_kv_heads = num_kv_heads;
  p.head_dim = head_dim; p.block_size = block_size; p.activation = activation;
  int units;
  switch (epi) {
    case EPI_BF16: case EPI_F32: units = (N + 15) / 16; break;
    case EPI_GATED: units = (N + 7) / 8; break;
    case EPI_ROPE_KV:
      if (head_dim % 16 || !slots || !k_pages || !v_pages || N != (num_heads + 2 * num_kv_heads) * head_dim) return -2;
      units = (num_heads + 2 * num_kv_heads) * (head_dim / 16);
      break;
    default: return -3;
  }
  // Shape of the work.  A unit of 8 weight rows (at most 8 input rows, not the gated product) when that
  // leaves the busiest compute unit with at most 3/4 of what units of 16 would give it to stream.  One or two workgroups per
  // compute unit: two overlap one's prologue and reduction with the other's streaming, and are taken when
  // their rows fit into LDS side by side and the busiest compute unit gets no more units that way; more
  // units than workgroups are dealt evenly, and a workgroup walks its units with the next one's weights
  // already on their way.
  const int cus = num_compute_units();
  constexpr int waves = 8;
  if (M > 16) {                                                 // tiles of 16 rows side by side, one workgroup per compute unit
    const int per_block = (units + cus - 1) / cus, blocks = (units + per_block - 1) / per_block;
    switch (epi) {
      case EPI_BF16: return launch_wide<EPI_BF16>(p, units, blocks, cus, stream);
      case EPI_F32: return launch_wide<EPI_F32>(p, units, blocks, cus, stream);
      case EPI_GATED: return launch_wide<EPI_GATED>(p, units, blocks, cus, stream);
      case EPI_ROPE_KV: return launch_wide<EPI_ROPE_KV>(p, units, blocks, cus, stream);
    }
    return -3;
  }
  // Rows that need no sum and no norm are read straight from memory (no LDS for them, any K).
  const bool direct = !delta && !norm_w;
  if (!direct && (long)M * (((K >> 3) + 63) >> 6) > kSquares) return -2;
  const size_t lds = direct ? (size_t)waves * 256 * sizeof(float) : (size_t)pllm_decode_linear_lds_bytes(M, K, waves);
  auto ceil_div = [](int a, int b) { return (a + b - 1) / b; };
  // (units of 8 rows read the row-major matrix; with only the tiled copy at hand the units stay at 16)
  const bool half = W && M <= 8 && epi != EPI_GATED && K >= 512 && 2 * ceil_div(2 * units, cus) <= 3 * ceil_div(units, cus);   // at most 3/4
  const bool tiled = Wt && !half;
  if (half) units *= 2;
  const int per_block2 = ceil_div(units, 2 * cus), blocks2 = ceil_div(units, per_block2);
  const int busiest2 = per_block2 * (blocks2 > cus ? 2 : 1), busiest1 = ceil_div(units, cus);
  const bool two = 2 * lds <= (size_t)pllm_lds_bytes_per_cu() && busiest2 <= busiest1;
  const int per_block = two ? per_block2 : busiest1;
  const int blocks = ceil_div(units, per_block);
  // Slabs in flight per wavefront: two, or three when a wavefront of a workgroup with plain rows has three slabs of a
  // unit (the down projection: K = 5632 is 22 slabs of 256 for 8 wavefronts), so that all of them travel at once.
#define GO(EPI_, HALF_)                                                                                                   \
  do {                                                                                                                    \
    const int step = (HALF_) ? 2 * kSlab : kSlab, most = ((K + step - 1) / step + waves - 1) / waves;                     \
    if (!(HALF_) && tiled) {                                                                                              \
      if (direct && most == 3) return launch<EPI_, waves, false, true, 3, true>(p, units, blocks, lds, stream);           \
      if (direct) return launch<EPI_, waves, false, true, 2, true>(p, units, blocks, lds, stream);                        \
      return launch<EPI_, waves, false, false, 2, true>(p, units, blocks, lds, stream);                                   \
    }                                                                                                                     \
    if (direct && most == 3) return launch<EPI_, waves, HALF_, true, 3>(p, units, blocks, lds, stream);                   \
    if (direct) return launch<EPI_, waves, HALF_, true, 2>(p, units, blocks, lds, stream);                                \
    return launch<EPI_, waves, HALF_, false, 2>(p, units, blocks, lds, stream);                                           \
  } while (0)
  if (half) {
    switch (epi) {
      case EPI_BF16: GO(EPI_BF16, true);
      case EPI_F32: GO(EPI_F32, true);
      case EPI_ROPE_KV: GO(EPI_ROPE_KV, true);
    }
  }
  switch (epi) {
    case EPI_BF16: GO(EPI_BF16, false);
    case EPI_F32: GO(EPI_F32, false);
    case EPI_GATED: GO(EPI_GATED, false);
    case EPI_ROPE_KV: GO(EPI_ROPE_KV, false);
  }
#undef GO
  return -3;
}
