// Row-wise and element-wise kernels of the decoder: embedding gather, RMS norm (with the
// residual sum fused in), SiLU-gated product, rotary position encoding fused with the write of
// K and V into their pages, page copies.  All arithmetic is done in float; the element type T
// (float or bfloat16) is only the storage type.
#include "common.h"

using namespace pllm;

// ---------------------------------------------------------------------------------------------
// Embedding: out[t, :] = table[ids[t], :]
template <typename T>
__global__ void embed_gather_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                    T* __restrict__ out, int hidden, int vocab) {
  const int t = blockIdx.x;
  int id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // the host has checked the range; never fault
  const T* src = table + (size_t)id * hidden;
  T* dst = out + (size_t)t * hidden;
  constexpr int V = 16 / sizeof(T);                              // elements per 16-byte piece
  if (hidden % V == 0 && ((uintptr_t)table % 16) == 0 && ((uintptr_t)out % 16) == 0) {
    const uint4* s4 = reinterpret_cast<const uint4*>(src);
    uint4* d4 = reinterpret_cast<uint4*>(dst);
    for (int i = threadIdx.x; i < hidden / V; i += blockDim.x) d4[i] = s4[i];
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = src[i];
  }
}

PLLM_API int pllm_embed_gather(int dtype, const int* ids, const void* table, void* out, int num_tokens,
                               int hidden, int vocab, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  dim3 grid(num_tokens), block(256);
  if (dtype == PLLM_F32)
    hipLaunchKernelGGL(embed_gather_kernel<float>, grid, block, 0, stream, ids, (const float*)table, (float*)out, hidden, vocab);
  else
    hipLaunchKernelGGL(embed_gather_kernel<bf16>, grid, block, 0, stream, ids, (const bf16*)table, (bf16*)out, hidden, vocab);
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// RMS norm of one row per workgroup, optionally after adding `delta` to the residual stream:
//   s = x[src] + delta[src]   (sum in float, rounded to T: that rounded value is the new residual)
//   out[r] = T( (s * rsqrt(mean(s^2) + eps)) * w )
// `row_index` (optional) picks the source rows, so the last norm runs only on rows whose logits
// are wanted.  `x_out` (optional) receives the new residual rows (may alias x).
// The sum may also come as float partial sums of `splits` ranges of a product's inner dimension (`parts`:
// [splits][rows of x][hidden], `part_stride` floats from one range to the next): they are added in order, in float,
// and take delta's place.
template <typename T>
__global__ void rmsnorm_kernel(const T* x, const T* __restrict__ delta, const int* __restrict__ row_index,
                               const float* __restrict__ w, float eps, T* __restrict__ out, T* x_out, int hidden,
                               const float* __restrict__ parts, int splits, size_t part_stride) {
  extern __shared__ float lds[];
  float* row = lds;             // [hidden]
  float* scratch = lds + hidden;  // [16]
  const int r = blockIdx.x;
  const size_t src = row_index ? (size_t)row_index[r] : (size_t)r;
  const T* xr = x + src * hidden;
  T* o = out + (size_t)r * hidden;
  constexpr int V = 16 / sizeof(T);                              // elements per 16-byte piece
  struct alignas(16) Piece { T v[V]; };
  const bool wide = hidden % V == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
                    (!delta || ((uintptr_t)delta % 16) == 0) && (!x_out || ((uintptr_t)x_out % 16) == 0);
  float acc = 0.f;
  if (wide) {
    for (int c = threadIdx.x; c < hidden / V; c += blockDim.x) {
      Piece px = reinterpret_cast<const Piece*>(xr)[c];
      if (delta) {
        const Piece pd = reinterpret_cast<const Piece*>(delta + src * hidden)[c];
#pragma unroll
        for (int j = 0; j < V; ++j) px.v[j] = from_f32<T>(to_f32(px.v[j]) + to_f32(pd.v[j]));
        if (x_out) reinterpret_cast<Piece*>(x_out + src * hidden)[c] = px;
      } else if (parts) {
        float d[V];
#pragma unroll
        for (int j = 0; j < V; ++j) d[j] = 0.f;
        for (int sp = 0; sp < splits; ++sp) {
#pragma unroll
          for (int j = 0; j < V; ++j) d[j] += parts[sp * part_stride + src * hidden + (size_t)c * V + j];
        }
#pragma unroll
        for (int j = 0; j < V; ++j) px.v[j] = from_f32<T>(to_f32(px.v[j]) + d[j]);
        if (x_out) reinterpret_cast<Piece*>(x_out + src * hidden)[c] = px;
      }
#pragma unroll
      for (int j = 0; j < V; ++j) {
        const float v = to_f32(px.v[j]);
        row[c * V + j] = v;
        acc += v * v;
      }
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
      float v = to_f32(xr[i]);
      if (delta || parts) {
        float d = 0.f;
        if (delta) d = to_f32(delta[src * hidden + i]);
        else for (int sp = 0; sp < splits; ++sp) d += parts[sp * part_stride + src * hidden + i];
        v = to_f32(from_f32<T>(v + d));
        if (x_out) x_out[src * hidden + i] = from_f32<T>(v);
      }
      row[i] = v;
      acc += v * v;
    }
  }
  const float total = block_sum(acc, scratch);
  const float inv = rsqrtf(total / (float)hidden + eps);
  if (wide) {
    for (int c = threadIdx.x; c < hidden / V; c += blockDim.x) {
      Piece po;
#pragma unroll
      for (int j = 0; j < V; ++j) po.v[j] = from_f32<T>((row[c * V + j] * inv) * w[c * V + j]);
      reinterpret_cast<Piece*>(o)[c] = po;
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = from_f32<T>((row[i] * inv) * w[i]);
  }
}

// The same for rows of at most 64 * WPR * P pieces of 16 bytes: WPR wavefronts per row keep the row in registers
// (P pieces per lane).  WPR = 1: no LDS and no barrier, a workgroup of four wavefronts does four rows (many rows:
// prompts).  WPR = 4: a workgroup per row, the wavefronts' sums of squares added through LDS in wavefront order (a
// few dozen to a few hundred rows: with one wavefront per row such a step would keep a handful of compute units busy,
// each walking a whole row and its addends: 4.9 us for 64 rows of 2048, 8.5 us for 128 rows with four ranges of
// partial sums).  The sum of squares is taken per lane over its pieces in order, then over the wavefront.
template <typename T, int P, int WPR>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const T* x, const T* __restrict__ delta, const int* __restrict__ row_index,
                                                           const float* __restrict__ w, float eps, T* __restrict__ out, T* x_out,
                                                           int hidden, int rows, const float* __restrict__ parts, int splits,
                                                           size_t part_stride) {
  constexpr int V = 16 / sizeof(T);
  struct alignas(16) Piece { T v[V]; };
  constexpr int kStride = 64 * WPR;                              // lanes that share a row
  const int lane = WPR == 1 ? (threadIdx.x & 63) : threadIdx.x;
  const int r = WPR == 1 ? blockIdx.x * 4 + (threadIdx.x >> 6) : blockIdx.x;
  if (r >= rows) return;
  const size_t src = row_index ? (size_t)row_index[r] : (size_t)r;
  const int pieces = hidden / V;
  const Piece* xr = reinterpret_cast<const Piece*>(x + src * hidden);
  Piece px[P], pd[P];
  // The norm's weights are requested with the row (for rows of up to 8 pieces per lane, which leaves registers for
  // them): asked for where they are used, behind the sum, they would cost a second wait for memory.
  constexpr bool kWeightsEarly = P <= 8;
  struct alignas(16) Weights { float v[V]; };
  Weights pw[kWeightsEarly ? P : 1];
#pragma unroll
  for (int i = 0; i < P; ++i) {
    const int c = min(lane + i * kStride, pieces - 1);                // inside the row; what lies past it is not used
    px[i] = xr[c];
    if (delta) pd[i] = reinterpret_cast<const Piece*>(delta + src * hidden)[c];
  }
  if constexpr (kWeightsEarly) {
#pragma unroll
    for (int i = 0; i < P; ++i) pw[i] = reinterpret_cast<const Weights*>(w)[min(lane + i * kStride, pieces - 1)];
  }
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < P; ++i) {
    const int c = lane + i * kStride;
    if (c >= pieces) continue;
    if (delta) {
#pragma unroll
      for (int j = 0; j < V; ++j) px[i].v[j] = from_f32<T>(to_f32(px[i].v[j]) + to_f32(pd[i].v[j]));
      if (x_out) reinterpret_cast<Piece*>(x_out + src * hidden)[c] = px[i];
    } else if (parts) {
      // The ranges' float sums of this piece, added in order (16-byte loads: hidden is a multiple of V, the buffer
      // aligned).  The first kEarly ranges (all there are, for most launches) are requested together before any is
      // added: a loop over a number of ranges known only at run time asks for one, waits, adds, and asks for the
      // next, a round trip to memory each.  A range past the last repeats it and is dropped by a select.
      struct alignas(16) Four { float v[4]; };
      constexpr int kEarly = P == 1 ? 8 : (P == 2 ? 4 : 2);
      Four early[kEarly][V / 4];
#pragma unroll
      for (int sp = 0; sp < kEarly; ++sp) {
        const Four* pp = reinterpret_cast<const Four*>(parts + min(sp, splits - 1) * part_stride + src * hidden + (size_t)c * V);
#pragma unroll
        for (int q = 0; q < V / 4; ++q) early[sp][q] = pp[q];
      }
      float d[V];
#pragma unroll
      for (int j = 0; j < V; ++j) d[j] = 0.f;
#pragma unroll
      for (int sp = 0; sp < kEarly; ++sp)
#pragma unroll
        for (int j = 0; j < V; ++j) d[j] += sp < splits ? early[sp][j / 4].v[j % 4] : 0.f;
      for (int sp = kEarly; sp < splits; ++sp) {
        const Four* pp = reinterpret_cast<const Four*>(parts + sp * part_stride + src * hidden + (size_t)c * V);
#pragma unroll
        for (int q = 0; q < V / 4; ++q) {
          const Four f = pp[q];
#pragma unroll
          for (int j = 0; j < 4; ++j) d[q * 4 + j] += f.v[j];
        }
      }
#pragma unroll
      for (int j = 0; j < V; ++j) px[i].v[j] = from_f32<T>(to_f32(px[i].v[j]) + d[j]);
      if (x_out) reinterpret_cast<Piece*>(x_out + src * hidden)[c] = px[i];
    }
#pragma unroll
    for (int j = 0; j < V; ++j) acc += to_f32(px[i].v[j]) * to_f32(px[i].v[j]);
  }
  float total = wave_sum(acc);
  if constexpr (WPR > 1) {
    __shared__ float wave_totals[WPR];
    if ((threadIdx.x & 63) == 0) wave_totals[threadIdx.x >> 6] = total;
    __syncthreads();
    total = wave_totals[0];
#pragma unroll
    for (int wv = 1; wv < WPR; ++wv) total += wave_totals[wv];
  }
  const float inv = rsqrtf(total / (float)hidden + eps);
  Piece* o = reinterpret_cast<Piece*>(out + (size_t)r * hidden);
#pragma unroll
  for (int i = 0; i < P; ++i) {
    const int c = lane + i * kStride;
    if (c >= pieces) continue;
    Piece po;
#pragma unroll
    for (int j = 0; j < V; ++j) po.v[j] = from_f32<T>((to_f32(px[i].v[j]) * inv) * (kWeightsEarly ? pw[i].v[j] : w[c * V + j]));
    o[c] = po;
  }
}

template <typename T>
static int launch_rmsnorm(const T* x, const T* delta, const int* row_index, const float* w, float eps, T* out, T* x_out, int rows,
                           int hidden, const float* parts, int splits, size_t part_stride, hipStream_t stream) {
  constexpr int V = 16 / sizeof(T);
  const bool wide = hidden % V == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)w % 16) == 0 &&
                    (!delta || ((uintptr_t)delta % 16) == 0) && (!x_out || ((uintptr_t)x_out % 16) == 0) &&
                    (!parts || (((uintptr_t)parts % 16) == 0 && part_stride % 4 == 0));
  const int per_lane = wide ? (hidden / V + 63) / 64 : 0;
  dim3 grid4((rows + 3) / 4), block(256);
  // few rows (decode steps of many requests, short prompt portions): a workgroup per row
  if (wide && rows <= 1024 && per_lane >= 2 && per_lane <= 16) {
    const int per_thread = (hidden / V + 255) / 256;
#define PLLM_ROW_WG(P_) hipLaunchKernelGGL((rmsnorm_rows_kernel<T, P_, 4>), dim3(rows), block, 0, stream, x, delta, row_index, w, eps, out, x_out, hidden, rows, parts, splits, part_stride)
    if (per_thread <= 1) PLLM_ROW_WG(1); else if (per_thread <= 2) PLLM_ROW_WG(2); else PLLM_ROW_WG(4);
#undef PLLM_ROW_WG
    return (int)hipGetLastError();
  }
#define PLLM_ROWS(P_) hipLaunchKernelGGL((rmsnorm_rows_kernel<T, P_, 1>), grid4, block, 0, stream, x, delta, row_index, w, eps, out, x_out, hidden, rows, parts, splits, part_stride)
  if (wide && per_lane <= 2) PLLM_ROWS(2);
  else if (wide && per_lane <= 4) PLLM_ROWS(4);
  else if (wide && per_lane <= 8) PLLM_ROWS(8);
  else if (wide && per_lane <= 16) PLLM_ROWS(16);
  else {
    const size_t lds = ((size_t)hidden + 16) * sizeof(float);   // the row as floats, and the reduction's scratch
    if (lds > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(rmsnorm_kernel<T>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return (int)e;
    }
    hipLaunchKernelGGL(rmsnorm_kernel<T>, dim3(rows), block, lds, stream, x, delta, row_index, w, eps, out, x_out, hidden, parts, splits, part_stride);
  }
#undef PLLM_ROWS
  return (int)hipGetLastError();
}

PLLM_API int pllm_rmsnorm(int dtype, const void* x, const void* delta, const int* row_index, const float* w, float eps,
                          void* out, void* x_out, int rows, int hidden, const float* parts, int splits, long part_stride,
                          hipStream_t stream) {
  if (rows <= 0) return 0;
  if (parts && (delta || splits < 1 || part_stride < 0)) return -2;
  if (((size_t)hidden + 16) * sizeof(float) > 160 * 1024) return -2;  // a row must fit the LDS of the one-row-per-workgroup kernel
  if (dtype == PLLM_F32)
    return launch_rmsnorm<float>((const float*)x, (const float*)delta, row_index, w, eps, (float*)out, (float*)x_out, rows, hidden, parts, splits,
                                (size_t)part_stride, stream);
  return launch_rmsnorm<bf16>((const bf16*)x, (const bf16*)delta, row_index, w, eps, (bf16*)out, (bf16*)x_out, rows, hidden, parts, splits,
                              (size_t)part_stride, stream);
}

// ---------------------------------------------------------------------------------------------
// A projection's bias: out[t, i] = in[t, i] + bias[i], the sums of the product and the bias both float, rounded once
// to the output's type (projections with a bias take their product as float sums and come through here).
template <typename T>
__global__ void add_bias_kernel(const float* __restrict__ in, int ld_in, const float* __restrict__ bias, T* __restrict__ out, int ld_out,
                                int cols, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t t = idx / cols;
  const int i = (int)(idx - t * cols);
  out[t * ld_out + i] = from_f32<T>(in[t * ld_in + i] + bias[i]);
}

PLLM_API int pllm_add_bias(int dtype, const float* in, int ld_in, const float* bias, void* out, int ld_out, int rows, int cols,
                           hipStream_t stream) {
  const size_t total = (size_t)rows * cols;
  if (total == 0) return 0;
  if (cols > ld_in || cols > ld_out) return -2;
  dim3 block(256), grid((unsigned)((total + 255) / 256));
  if (dtype == PLLM_F32) hipLaunchKernelGGL(add_bias_kernel<float>, grid, block, 0, stream, in, ld_in, bias, (float*)out, ld_out, cols, total);
  else hipLaunchKernelGGL(add_bias_kernel<bf16>, grid, block, 0, stream, in, ld_in, bias, (bf16*)out, ld_out, cols, total);
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// Gated activation: out[t, i] = act(gu[t, i]) * gu[t, inter + i] (gate_activation in common.h).
template <typename T, int V>
__global__ void gate_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, size_t total, int act) {
  // Each thread handles V consecutive outputs of one row (V = 1, or a 16-byte piece).
  struct alignas(sizeof(T) * V) Piece { T v[V]; };
  const size_t idx = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * V;
  if (idx >= total) return;
  const size_t t = idx / inter;
  const int i = (int)(idx - t * inter);
  const Piece pg = *reinterpret_cast<const Piece*>(gu + t * 2 * inter + i);
  const Piece pu = *reinterpret_cast<const Piece*>(gu + t * 2 * inter + inter + i);
  Piece po;
#pragma unroll
  for (int j = 0; j < V; ++j) {
    const float g = to_f32(pg.v[j]), u = to_f32(pu.v[j]);
    po.v[j] = from_f32<T>(gate_activation(g, act) * u);
  }
  *reinterpret_cast<Piece*>(out + idx) = po;
}

PLLM_API int pllm_gate_mul(int dtype, int activation, const void* gate_up, void* out, int num_tokens, int inter, hipStream_t stream) {
  const size_t total = (size_t)num_tokens * inter;
  if (total == 0) return 0;
  if (activation < 0 || activation >= PLLM_ACT_COUNT) return -2;
  const int elem = dtype == PLLM_F32 ? 4 : 2, wide = 16 / elem;
  const bool vec = inter % wide == 0 && ((uintptr_t)gate_up % 16) == 0 && ((uintptr_t)out % 16) == 0;
  const size_t items = vec ? total / wide : total;
  dim3 block(256), grid((unsigned)((items + 255) / 256));
  if (dtype == PLLM_F32) {
    if (vec) hipLaunchKernelGGL((gate_mul_kernel<float, 4>), grid, block, 0, stream, (const float*)gate_up, (float*)out, inter, total, activation);
    else hipLaunchKernelGGL((gate_mul_kernel<float, 1>), grid, block, 0, stream, (const float*)gate_up, (float*)out, inter, total, activation);
  } else {
    if (vec) hipLaunchKernelGGL((gate_mul_kernel<bf16, 8>), grid, block, 0, stream, (const bf16*)gate_up, (bf16*)out, inter, total, activation);
    else hipLaunchKernelGGL((gate_mul_kernel<bf16, 1>), grid, block, 0, stream, (const bf16*)gate_up, (bf16*)out, inter, total, activation);
  }
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// Rotary encoding of q and k fused with the cache write.  The first rotary_dim elements of a head are
// rotated: pair i is (i, i + rotary_dim/2) (half-split) or (2i, 2i + 1) (interleaved) and turns by the
// angle whose cos/sin stand in column i of the float tables [positions, rotary_dim/2].  q is rotated in place inside the fused projection buffer
//   qkv[t] = [ q heads | k heads | v heads ],  row stride `row_stride` elements.
// Rotated k goes to k_pages [page, kv_head, offset, d]; v goes, transposed, to
// v_pages [page, kv_head, d, offset].  slot = page * block_size + offset; slot < 0 skips the write.
// With write_kv == 0 only q is rotated (a layer that reads another layer's cache).
template <typename T>
__global__ void rope_scatter_kernel(T* __restrict__ qkv, int row_stride, const int* __restrict__ positions,
                                    const float* __restrict__ cos_table, const float* __restrict__ sin_table,
                                    const int* __restrict__ slot_mapping, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                    int num_heads, int num_kv_heads, int head_dim, int block_size, int write_kv,
                                    int rotary_dim, int interleaved, int num_tokens, int value_groups) {
  // With value_groups > 0 the workgroups past the first num_tokens write the values: one for 16 tokens in a row.
  // Values sit transposed in a page ([channel][position]), so a token alone writes single elements a page's
  // width apart; 16 tokens whose slots follow each other inside one page (a prompt portion) fill whole rows of
  // 16 positions, written in 16-byte pieces.
  if (value_groups > 0 && (int)blockIdx.x >= num_tokens) {
    const int t0 = ((int)blockIdx.x - num_tokens) * 16, n = min(16, num_tokens - t0);
    // The 16 slots with one load (lane j of every wavefront holds token j's), not one after the other.
    const int lane = threadIdx.x & 63;
    const int my_slot = lane < n ? slot_mapping[t0 + lane] : -1;
    const int s0 = __builtin_amdgcn_readlane(my_slot, 0);
    const bool in_a_row = __all(lane >= 16 || my_slot == s0 + lane) && n == 16 && s0 >= 0 &&      // (uniform in the workgroup)
                          (s0 & (block_size - 1)) + 16 <= block_size && ((s0 * sizeof(T)) & 15) == 0 &&
                          ((uintptr_t)v_pages & 15) == 0 && ((block_size * sizeof(T)) & 15) == 0;
    const size_t v_at = (size_t)(num_heads + num_kv_heads) * head_dim;
    for (int w = threadIdx.x; w < num_kv_heads * head_dim; w += blockDim.x) {
      const int kvh = w / head_dim, i = w - kvh * head_dim;
      if (in_a_row) {
        const int page = s0 / block_size, off = s0 - page * block_size;
        struct alignas(16) Row { T v[16]; } out;
#pragma unroll
        for (int j = 0; j < 16; ++j) out.v[j] = qkv[(size_t)(t0 + j) * row_stride + v_at + w];
        *reinterpret_cast<Row*>(v_pages + (((size_t)page * num_kv_heads + kvh) * head_dim + i) * block_size + off) = out;
      } else {
#pragma unroll
        for (int j = 0; j < 16; ++j) {                           // (tokens past the last one hold -1)
          const int slot = __builtin_amdgcn_readlane(my_slot, j);
          if (slot < 0) continue;
          const int page = slot / block_size, off = slot - page * block_size;
          v_pages[(((size_t)page * num_kv_heads + kvh) * head_dim + i) * block_size + off] = qkv[(size_t)(t0 + j) * row_stride + v_at + w];
        }
      }
    }
    return;
  }
  const int t = blockIdx.x;
  const int half = rotary_dim >> 1;                      // pairs per head, and the tables' row length
  const int pos = positions[t];
  const float* cs = cos_table ? cos_table + (size_t)pos * half : nullptr;  // no tables: no rotation
  const float* sn = sin_table ? sin_table + (size_t)pos * half : nullptr;
  T* row = qkv + (size_t)t * row_stride;
  const int slot = write_kv ? slot_mapping[t] : -1;
  const int page = slot >= 0 ? slot / block_size : 0;
  const int off = slot >= 0 ? slot - page * block_size : 0;

  const int rot_heads = write_kv ? num_heads + num_kv_heads : num_heads;
  struct alignas(16) Piece { T v[8]; };
  const bool wide = rotary_dim == head_dim && !interleaved && (half % 8 == 0) && ((uintptr_t)qkv % 16) == 0 &&
                    (row_stride % 8 == 0) && ((uintptr_t)k_pages % 16) == 0;
  if (wide) {
    // 8 pairs per work item: 16-byte pieces of the lower and the upper half of a head
    const int per_head = half / 8;
    for (int w = threadIdx.x; w < rot_heads * per_head; w += blockDim.x) {
      const int head = w / per_head, i = (w - head * per_head) * 8;
      T* h = row + (size_t)head * head_dim;
      const Piece lo = *reinterpret_cast<const Piece*>(h + i), hi = *reinterpret_cast<const Piece*>(h + i + half);
      Piece out_lo, out_hi;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float c = cs ? cs[i + j] : 1.f, s = sn ? sn[i + j] : 0.f;
        const float l = to_f32(lo.v[j]), u = to_f32(hi.v[j]);
        float rl, ru;
        rotate_pair(l, u, c, s, rl, ru);
        out_lo.v[j] = from_f32<T>(rl);
        out_hi.v[j] = from_f32<T>(ru);
      }
      T* dst = nullptr;
      if (head < num_heads) dst = h;
      else if (slot >= 0) dst = k_pages + (((size_t)page * num_kv_heads + (head - num_heads)) * block_size + off) * head_dim;
      if (dst) {
        *reinterpret_cast<Piece*>(dst + i) = out_lo;
        *reinterpret_cast<Piece*>(dst + i + half) = out_hi;
      }
    }
  } else {
    // Any rotary width and either pairing: pair i of a head is (i, i + half) or, interleaved, (2i, 2i + 1);
    // elements from rotary_dim on are not rotated (of k they are copied to the page as they are).
    for (int w = threadIdx.x; w < rot_heads * half; w += blockDim.x) {
      const int head = w / half, i = w - head * half;
      const int a = interleaved ? 2 * i : i, b = interleaved ? 2 * i + 1 : i + half;
      T* h = row + (size_t)head * head_dim;
      const float lo = to_f32(h[a]), hi = to_f32(h[b]);
      const float c = cs ? cs[i] : 1.f, s = sn ? sn[i] : 0.f;
      float rl, ru;
      rotate_pair(lo, hi, c, s, rl, ru);
      const T out_lo = from_f32<T>(rl), out_hi = from_f32<T>(ru);
      if (head < num_heads) {
        h[a] = out_lo;
        h[b] = out_hi;
      } else if (slot >= 0) {
        const int kvh = head - num_heads;
        T* dst = k_pages + (((size_t)page * num_kv_heads + kvh) * block_size + off) * head_dim;
        dst[a] = out_lo;
        dst[b] = out_hi;
      }
    }
    const int tail = head_dim - rotary_dim;
    if (tail > 0 && slot >= 0) {
      for (int w = threadIdx.x; w < num_kv_heads * tail; w += blockDim.x) {
        const int kvh = w / tail, i = rotary_dim + (w - kvh * tail);
        k_pages[(((size_t)page * num_kv_heads + kvh) * block_size + off) * head_dim + i] = row[(size_t)(num_heads + kvh) * head_dim + i];
      }
    }
  }
  if (slot >= 0 && value_groups == 0) {
    const T* v = row + (size_t)(num_heads + num_kv_heads) * head_dim;
    for (int w = threadIdx.x; w < num_kv_heads * head_dim; w += blockDim.x) {
      const int kvh = w / head_dim, i = w - kvh * head_dim;
      v_pages[(((size_t)page * num_kv_heads + kvh) * head_dim + i) * block_size + off] = v[w];
    }
  }
}

// rotary_dim: how many leading elements of a head are rotated (even, at most head_dim; the tables hold
// rotary_dim / 2 columns); interleaved: pairs are (2i, 2i + 1) instead of (i, i + rotary_dim / 2).
PLLM_API int pllm_rope_scatter(int dtype, void* qkv, int row_stride, const int* positions, const float* cos_table,
                               const float* sin_table, const int* slot_mapping, void* k_pages, void* v_pages,
                               int num_tokens, int num_heads, int num_kv_heads, int head_dim, int block_size,
                               int write_kv, int rotary_dim, int interleaved, hipStream_t stream) {
  if (num_tokens <= 0) return 0;
  if (rotary_dim < 0 || rotary_dim > head_dim || (rotary_dim & 1)) return -2;
  // Many tokens (prompt portions) and pages that hold 16 positions of a row: the values are written by workgroups of
  // their own, 16 tokens each.  (A few hundred tokens are done sooner without: the kernel then ends with its longest
  // workgroup, and one that gathers 16 tokens is longer than one that scatters a single token.)
  const int value_groups = (write_kv && num_tokens >= 512 && block_size >= 16) ? (num_tokens + 15) / 16 : 0;
  dim3 grid(num_tokens + value_groups), block(256);
  if (dtype == PLLM_F32)
    hipLaunchKernelGGL(rope_scatter_kernel<float>, grid, block, 0, stream, (float*)qkv, row_stride, positions, cos_table,
                       sin_table, slot_mapping, (float*)k_pages, (float*)v_pages, num_heads, num_kv_heads, head_dim,
                       block_size, write_kv, rotary_dim, interleaved, num_tokens, value_groups);
  else
    hipLaunchKernelGGL(rope_scatter_kernel<bf16>, grid, block, 0, stream, (bf16*)qkv, row_stride, positions, cos_table,
                       sin_table, slot_mapping, (bf16*)k_pages, (bf16*)v_pages, num_heads, num_kv_heads, head_dim,
                       block_size, write_kv, rotary_dim, interleaved, num_tokens, value_groups);
  PLLM_RETURN_LAST_ERROR();
}

// ---------------------------------------------------------------------------------------------
// Page copies (copy-on-write): pages[dst[i]] = pages[src[i]], `page_elems` elements each.
template <typename T>
__global__ void copy_pages_kernel(T* __restrict__ pages, const int* __restrict__ src, const int* __restrict__ dst,
                                  size_t page_elems) {
  const T* s = pages + (size_t)src[blockIdx.x] * page_elems;
  T* d = pages + (size_t)dst[blockIdx.x] * page_elems;
  for (size_t i = (size_t)blockIdx.y * blockDim.x + threadIdx.x; i < page_elems; i += (size_t)gridDim.y * blockDim.x) d[i] = s[i];
}

PLLM_API int pllm_copy_pages(int dtype, void* pages, const int* src, const int* dst, int num_copies, long page_elems,
                             hipStream_t stream) {
  if (num_copies <= 0 || page_elems <= 0) return 0;
  unsigned gy = (unsigned)((page_elems + 255) / 256);
  if (gy > 64) gy = 64;
  dim3 grid(num_copies, gy), block(256);
  if (dtype == PLLM_F32)
    hipLaunchKernelGGL(copy_pages_kernel<float>, grid, block, 0, stream, (float*)pages, src, dst, (size_t)page_elems);
  else
    hipLaunchKernelGGL(copy_pages_kernel<bf16>, grid, block, 0, stream, (bf16*)pages, src, dst, (size_t)page_elems);
  PLLM_RETURN_LAST_ERROR();
}
