// Next-token choice from float logits [rows, vocab], one workgroup of 1024 threads per row.
//
// Greedy rows (temperature < 1e-5) take the first index of the maximum.  Other rows draw from
//   softmax(logits / max(T, 1e-5)) restricted by top-k and top-p,
// where, as in pagedllm/sampler.py:21-35, a token stays if fewer than top_k tokens have a larger
// logit and the probability mass of the tokens with a larger logit is at most top_p.  Both tests
// depend only on the token's own logit, so the kept set is {logit >= threshold}; the threshold is
// found by a search over the ordered bit patterns of float that moves from token to token (a few
// passes over the row, which stays in registers or in cache), not by a sort.  Tokens with equal
// logits are kept or dropped together.
//
// The draw is the inverse CDF over the kept tokens in a fixed order (thread by thread) with one uniform
// number per row from Philox4x32-10 keyed by (seed, request key, step), so a request's tokens do not
// depend on its neighbours; every sum is taken in an order that depends on the row's length only.
//
// Few rows of a long vocabulary with a small top_k (the usual settings of a decode step) would leave the GPU to as
// many workgroups as there are rows, each walking its whole row a dozen times.  For them the row is first cut into
// chunks, one workgroup each (sample_candidates_kernel): a chunk hands on every logit that may be among the row's
// top_k largest, a few more than top_k of its own, and its share of the sum of weights; the search and the draw then
// run over those few hundred candidates (the same kernel, on the candidates instead of the row).  A row whose chunks
// have too many candidates (many equal logits) goes the long way.
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

// Largest / smallest of one unsigned value per thread over the workgroup (scratch: 16 words of LDS).
__device__ __forceinline__ uint32_t float_as_uint_max(uint32_t v, float* scratch) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = max(v, (uint32_t)__shfl_xor((int)v, o, 64));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) reinterpret_cast<uint32_t*>(scratch)[wave] = v;
  __syncthreads();
  uint32_t t = reinterpret_cast<uint32_t*>(scratch)[0];
  for (int w = 1; w < nwaves; ++w) t = max(t, reinterpret_cast<uint32_t*>(scratch)[w]);
  return t;
}
__device__ __forceinline__ uint32_t float_as_uint_min(uint32_t v, float* scratch) { return ~float_as_uint_max(~v, scratch); }

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

// ---------------------------------------------------------------------------------------------
// The row is walked in passes.  A thread's elements are the same in every pass and come in the same order:
// with rows of whole 16-byte pieces, piece c * 512 + tid for c = 0, 1, ...; else element c * 512 + tid.
// The sampling kernel's workgroup has 512 threads (eight wavefronts, so that a thread may hold up to 256 registers): rows of
// up to 64 elements per thread (32768 logits) are read once and stay in registers; longer rows are read again in each
// pass (cache hits), eight requests under way at a time.
constexpr int kSampleThreads = 512;
constexpr int kSlots = 64;                   // elements per thread that registers hold
// elements per thread that the end of the search keeps in registers: 16 for a row that is read from memory (each pass
// before that is long), 8 for a row in registers (which leave no room for more)
template <bool IN_REGS> constexpr int kWindowSlots = IN_REGS ? 8 : 16;

__device__ __forceinline__ float key_value(uint32_t k) {       // inverse of float_key
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

struct Four { float a, b, c, d; };          // sums / extremes of one pass, reduced over the workgroup together
__device__ __forceinline__ void block_reduce_pass(float& mass, int& cnt, uint32_t& below, uint32_t& above, int& low_most, int& high_most,
                                                  float* fs, int* is) {
  // mass, cnt: sums; below: maximum; above: minimum; low_most / high_most: maxima.  Fixed order: wavefront, then wavefronts.
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    mass += __shfl_xor(mass, o, 64);
    cnt += __shfl_xor(cnt, o, 64);
    below = max(below, (uint32_t)__shfl_xor((int)below, o, 64));
    above = min(above, (uint32_t)__shfl_xor((int)above, o, 64));
    low_most = max(low_most, __shfl_xor(low_most, o, 64));
    high_most = max(high_most, __shfl_xor(high_most, o, 64));
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) {
    fs[wave] = mass;
    is[wave] = cnt; is[16 + wave] = (int)below; is[32 + wave] = (int)above; is[48 + wave] = low_most; is[64 + wave] = high_most;
  }
  __syncthreads();
  mass = fs[0]; cnt = is[0]; below = (uint32_t)is[16]; above = (uint32_t)is[32]; low_most = is[48]; high_most = is[64];
  for (int w = 1; w < kSampleThreads / 64; ++w) {
    mass += fs[w]; cnt += is[w];
    below = max(below, (uint32_t)is[16 + w]); above = min(above, (uint32_t)is[32 + w]);
    low_most = max(low_most, is[48 + w]); high_most = max(high_most, is[64 + w]);
  }
}

// Exclusive prefix of one float per thread in thread order, and the total; fixed order of additions.
__device__ __forceinline__ float block_exclusive_scan(float v, float* fs, float& total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float incl = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float up = __shfl_up(incl, o, 64);
    if (lane >= o) incl += up;
  }
  __syncthreads();
  if (lane == 63) fs[wave] = incl;
  __syncthreads();
  float before = 0.f, all = 0.f;
  for (int w = 0; w < kSampleThreads / 64; ++w) {
    if (w < wave) before += fs[w];
    all += fs[w];
  }
  total = all;
  return before + (incl - v);
}

// f(value, index) for every element of the calling thread, in its fixed order; the visitor goes in and comes back by
// value, so that what it gathers stays in registers.
template <bool IN_REGS, bool VEC, int HELD, class F>
__device__ __forceinline__ F for_each_element(const float (&held)[HELD], const float* __restrict__ z, int units, int tid, F f) {
  constexpr int kPer = VEC ? 4 : 1;
  constexpr int kFlight = 8;                                     // requests under way per thread in a pass over memory
  if constexpr (IN_REGS) {
#pragma unroll
    for (int s = 0; s < HELD; ++s) {
      if ((s / kPer) * kSampleThreads >= units) break;           // (the same for every thread: the slots from here on are empty)
      const int u = (s / kPer) * kSampleThreads + tid, i = u * kPer + (s % kPer);
      if (u < units) f(held[s], i);
    }
  } else {
    for (int u0 = 0; u0 < units; u0 += kFlight * kSampleThreads) {
      float v[kFlight][kPer];
#pragma unroll
      for (int q = 0; q < kFlight; ++q) {
        const int u = u0 + q * kSampleThreads + tid;
        if constexpr (VEC) {
          const float4 t = u < units ? reinterpret_cast<const float4*>(z)[u] : make_float4(0.f, 0.f, 0.f, 0.f);
          v[q][0] = t.x; v[q][1] = t.y; v[q][2] = t.z; v[q][3] = t.w;
        } else {
          v[q][0] = u < units ? z[u] : 0.f;
        }
      }
#pragma unroll
      for (int q = 0; q < kFlight; ++q) {
        const int u = u0 + q * kSampleThreads + tid;
        if (u >= units) continue;
#pragma unroll
        for (int e = 0; e < kPer; ++e) f(v[q][e], u * kPer + e);
      }
    }
  }
  return f;
}

// weight of a token (unnormalised probability): 2^((v - max) / T * log2 e), at most 1
struct Weigh {
  float zmax, rate;
  __device__ __forceinline__ float operator()(float v) const { return __builtin_amdgcn_exp2f((v - zmax) * rate); }
};
struct Extremes {                      // the maximum (first index) and the minimum
  ArgMax best; float lowest;
  __device__ __forceinline__ void operator()(float v, int i) { ArgMax c; c.v = v; c.i = i; best = better(best, c); lowest = fminf(lowest, v); }
};
struct SumOfWeights {
  Weigh w; float sum;
  __device__ __forceinline__ void operator()(float v, int) { sum += w(v); }
};
struct AroundPivot {                   // what lies above the pivot, and the nearest tokens on both sides inside [lo, hi]
  Weigh w; uint32_t lo, hi, mid;
  float mass; int cnt, low_mine, high_mine; uint32_t below, above;
  __device__ __forceinline__ void look(uint32_t key, float weight) {
    const bool up = key > mid, in_hi = up && key <= hi, in_lo = !up && key >= lo;
    cnt += up ? 1 : 0;
    mass += up ? weight : 0.f;
    above = in_hi ? min(above, key) : above;
    below = in_lo ? max(below, key) : below;
    high_mine += in_hi ? 1 : 0;
    low_mine += in_lo ? 1 : 0;
  }
  __device__ __forceinline__ void operator()(float v, int) {
    const uint32_t key = float_key(v);
    // (under branches: late passes have their pivot far up and a narrow interval, and whole wavefronts pass these by)
    if (key > mid) {
      cnt += 1;
      mass += w(v);
    }
    if (key - lo <= hi - lo) {                                   // inside [lo, hi]
      if (key > mid) { above = min(above, key); high_mine += 1; }
      else { below = max(below, key); low_mine += 1; }
    }
  }
};
template <int SLOTS>
struct FirstLook {                     // the first pass: the sum of all weights, as AroundPivot, and the tokens above the pivot taken along
  AroundPivot ap;
  uint32_t key[SLOTS]; float weight[SLOTS]; int n; float sum;
  __device__ __forceinline__ void operator()(float v, int) {
    const uint32_t k = float_key(v);
    const float wt = ap.w(v);
    sum += wt;
    if (k > ap.mid) {                                            // (few, in the usual row)
      ap.cnt += 1;
      ap.mass += wt;
#pragma unroll
      for (int s = 0; s < SLOTS; ++s) {
        const bool here = n == s;
        key[s] = here ? k : key[s];
        weight[s] = here ? wt : weight[s];
      }
      n += 1;
    }
    if (k - ap.lo <= ap.hi - ap.lo) {
      if (k > ap.mid) { ap.above = min(ap.above, k); ap.high_mine += 1; }
      else { ap.below = max(ap.below, k); ap.low_mine += 1; }
    }
  }
};
template <int SLOTS>
struct IntoWindow {                    // this thread's tokens inside [lo, hi] into registers, what lies above summed
  Weigh w; uint32_t lo, hi;
  uint32_t key[SLOTS]; float weight[SLOTS];
  int n, cnt_up; float mass_up;
  __device__ __forceinline__ void operator()(float v, int) {
    const uint32_t k = float_key(v);
    float wt = 0.f;
    if (k >= lo) wt = w(v);
    const bool up = k > hi, in = !up && k >= lo;
    cnt_up += up ? 1 : 0;
    mass_up += up ? wt : 0.f;
    if (in) {                                                    // (few tokens are: most wavefronts pass this by)
#pragma unroll
      for (int s = 0; s < SLOTS; ++s) {
        const bool here = n == s;
        key[s] = here ? k : key[s];
        weight[s] = here ? wt : weight[s];
      }
      n += 1;
    }
  }
};
struct KeptSum {
  Weigh w; uint32_t threshold; float sum;
  __device__ __forceinline__ void operator()(float v, int) { if (float_key(v) >= threshold) sum += w(v); }
};
struct Pick {                          // the first kept token at which the running sum passes the target
  Weigh w; uint32_t threshold; float run, target; int pick, last;
  __device__ __forceinline__ void operator()(float v, int i) {
    if (pick < 0 && float_key(v) >= threshold) {
      run += w(v);
      last = i;
      if (run > target) pick = i;
    }
  }
};

// ---------------------------------------------------------------------------------------------
// Candidates of a row: see the head of the file.  A row of `vocab` logits is cut into `chunks` chunks of `chunk` logits.
constexpr int kCandThreads = 256;
constexpr int kChunkPerThread = 16;          // logits of a chunk per thread (held in registers)
constexpr int kChunkMost = kCandThreads * kChunkPerThread;
constexpr int kMaxChunks = 64;               // (vocabularies of up to 262,144)
constexpr int kChunkCap = 192;               // candidates a chunk may hand on (about 90 are expected at the largest top_k)
constexpr int kCandTopK = 64;                // largest top_k that goes this way
constexpr int kMaxCandidates = kMaxChunks * kChunkCap;
static_assert(kMaxChunks <= 64, "a lane per chunk");
static_assert(kCandThreads == 256 && kCandTopK <= kCandThreads, "four wavefronts, each with at least k / 4 threads");

struct Candidates {                          // per row and chunk; null `count`: no candidates in this launch
  int* count;                                // candidates of the chunk; -1: the row goes the long way
  float* top;                                // the chunk's largest logit
  float* sum;                                // sum over the chunk of 2^((v - top) * rate)
  float* value;                              // [kChunkCap] per chunk
  int* index;                                // their places in the row
  int chunks, chunk;
};

constexpr int kCandMassVocab = 65536;        // rows at least this long that are cut by their mass alone try the candidates too

// The top_k with which a row's candidates are chosen; 0: the row is walked whole.  A row with a top_k of its own of at
// most kCandTopK takes that.  A long row that is cut by its mass (top_p < 1) under no top_k, or a larger one, takes
// kCandTopK: where few tokens carry the mass, the tokens that stay are among the kCandTopK largest, and the row's
// workgroup sees that they are when fewer than kCandTopK stay (the next token then went by its mass, as it would
// under any larger top_k); else it walks the row after all (a row of noise pays the detour, 20 us on 190).
__device__ __forceinline__ int candidates_top_k(float temp, int k, float p, int vocab) {
  if (temp < 1e-5f) return 0;
  if (k > 0 && k <= kCandTopK) return k < vocab ? k : 0;
  return (p < 1.f && vocab >= kCandMassVocab) ? kCandTopK : 0;
}

__global__ __launch_bounds__(kCandThreads) void sample_candidates_kernel(const float* __restrict__ logits, int vocab,
                                                                         const float* __restrict__ temperature,
                                                                         const int* __restrict__ top_k, const float* __restrict__ top_p,
                                                                         const Candidates cd) {
  __shared__ float fscratch[16];
  __shared__ float taus[kCandThreads / 64];
  __shared__ int wave_counts[kCandThreads / 64];
  const int row = blockIdx.y, c = blockIdx.x, tid = threadIdx.x;
  const size_t slot = (size_t)row * cd.chunks + c;
  const float temp = temperature[row];
  const int k = candidates_top_k(temp, top_k[row], top_p[row], vocab);
  if (k == 0) {
    if (tid == 0) cd.count[slot] = -1;
    return;
  }
  const float* z = logits + (size_t)row * vocab;
  const int begin = c * cd.chunk, end = min(vocab, begin + cd.chunk);
  // The chunk into registers (all loads under way at once), then this thread's largest and the chunk's largest.
  float v[kChunkPerThread];
#pragma unroll
  for (int j = 0; j < kChunkPerThread; ++j) {
    const int i = begin + j * kCandThreads + tid;
    v[j] = i < end ? z[i] : -INFINITY;
  }
  float mine = -INFINITY;
#pragma unroll
  for (int j = 0; j < kChunkPerThread; ++j) mine = fmaxf(mine, v[j]);
  const float top = block_max(mine, fscratch);
  // A bound from below on the chunk's k-th largest logit: each of the four wavefronts sorts its threads' largest (a
  // bitonic network over the lanes) and takes the ceil(k / 4)-th; at least k logits of the chunk are as large as the
  // smallest of those four, so the chunk's own k largest, and with them every logit of the chunk that may be among
  // the row's k largest, are at or above it.
  const int lane = tid & 63, wave = tid >> 6;
  float sorted = mine;
#pragma unroll
  for (int size = 2; size <= 64; size <<= 1) {
#pragma unroll
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      const float other = __shfl_xor(sorted, stride, 64);
      const bool larger_here = ((lane & stride) == 0) == ((lane & size) == 0);     // (descending over the lanes in the end)
      sorted = larger_here ? fmaxf(sorted, other) : fminf(sorted, other);
    }
  }
  const float of_wave = __shfl(sorted, (k + 3) / 4 - 1, 64);
  if (lane == 0) taus[wave] = of_wave;
  __syncthreads();
  const float tau = fminf(fminf(taus[0], taus[1]), fminf(taus[2], taus[3]));
  // the chunk's share of the sum of weights, and how many of this thread's logits go on
  const float rate = 1.4426950408889634f / fmaxf(temp, 1e-5f);
  float sum = 0.f;
  int n = 0;
#pragma unroll
  for (int j = 0; j < kChunkPerThread; ++j) {
    const bool there = begin + j * kCandThreads + tid < end;
    sum += there ? __builtin_amdgcn_exp2f((v[j] - top) * rate) : 0.f;
    n += there && v[j] >= tau ? 1 : 0;
  }
  sum = block_sum(sum, fscratch);
  // places in thread order: the wavefront's prefix, then the wavefronts before it
  int incl = n;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int up = __shfl_up(incl, o, 64);
    if (lane >= o) incl += up;
  }
  if (lane == 63) wave_counts[wave] = incl;
  __syncthreads();
  int before = incl - n, all = 0;
  for (int w = 0; w < kCandThreads / 64; ++w) {
    if (w < wave) before += wave_counts[w];
    all += wave_counts[w];
  }
  if (tid == 0) {
    cd.count[slot] = all <= kChunkCap ? all : -1;
    cd.top[slot] = top;
    cd.sum[slot] = sum;
  }
  if (all > kChunkCap) return;
#pragma unroll
  for (int j = 0; j < kChunkPerThread; ++j) {
    const int i = begin + j * kCandThreads + tid;
    if (i < end && v[j] >= tau) {
      cd.value[slot * kChunkCap + before] = v[j];
      cd.index[slot * kChunkCap + before] = i;
      ++before;
    }
  }
}

// Whether a row's candidates are there (every chunk handed its own on); the same answer in both kernels below and in
// every wavefront (a lane looks at one chunk: at most 64 of them).
__device__ __forceinline__ bool has_candidates(const Candidates& cd, int row) {
  const int lane = threadIdx.x & 63;
  const int n = lane < cd.chunks ? cd.count[(size_t)row * cd.chunks + lane] : 0;
  return __all(n >= 0);
}

// One row's token.  CAND: over the row's candidates (false: they do not settle it, the row has to be walked); else over
// the whole row.
template <bool IN_REGS, bool VEC, bool CAND>
__device__ __forceinline__ bool sample_row(const float* __restrict__ logits, int vocab, const float* __restrict__ temperature,
                                           const int* __restrict__ top_k, const float* __restrict__ top_p,
                                           const long long* __restrict__ request_key, const int* __restrict__ step,
                                           unsigned long long seed, int* __restrict__ out, const Candidates& cd) {
  static_assert(!CAND || (IN_REGS && !VEC), "candidates are few and of any number");
  __shared__ float fscratch[16];
  __shared__ int iscratch[80];
  __shared__ ArgMax ascratch[16];
  __shared__ int chosen, chooser;
  __shared__ int starts[65];                                     // CAND: where each chunk's candidates begin (a lane per chunk), and their number
  const int row = blockIdx.x, tid = threadIdx.x;
  const float* z = logits + (size_t)row * vocab;
  int units = VEC ? vocab >> 2 : vocab;                          // pieces of four, or single elements
  constexpr int kPer = VEC ? 4 : 1;
  float total_of_row = 0.f;                                      // CAND: the sum of the whole row's weights
  if constexpr (CAND) {
    // The chunks' candidates side by side in LDS, in the order of the chunks; the row's sum of weights from the
    // chunks' shares (relative to the row's largest logit, in the order of the chunks).
    __shared__ float gathered[kMaxCandidates];
    __shared__ float total_s;
    // (the first wavefront, a lane per chunk: where each chunk's candidates begin, the row's largest logit and its sum
    //  of weights; sums over lanes in the fixed order of wave_sum)
    if (tid < 64) {
      const bool there = tid < cd.chunks;
      const int n = there ? cd.count[(size_t)row * cd.chunks + tid] : 0;
      const float chunk_top = there ? cd.top[(size_t)row * cd.chunks + tid] : -INFINITY;
      const float chunk_sum = there ? cd.sum[(size_t)row * cd.chunks + tid] : 0.f;
      int incl = n;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(incl, o, 64);
        if (tid >= o) incl += up;
      }
      starts[tid] = incl - n;
      if (tid == 63) starts[64] = incl;
      const float top = wave_max(chunk_top);
      const float rate = 1.4426950408889634f / fmaxf(temperature[row], 1e-5f);
      const float sum = wave_sum(there ? chunk_sum * __builtin_amdgcn_exp2f((chunk_top - top) * rate) : 0.f);
      if (tid == 0) total_s = sum;
    }
    __syncthreads();
    // Wavefront w gathers chunks w, w + 8, ...: all of a wavefront's loads are requested before the first is stored.
    {
      const int lane = tid & 63, wave = tid >> 6;
      constexpr int kTurns = kMaxChunks / (kSampleThreads / 64), kPieces = kChunkCap / 64;
      float got[kTurns][kPieces];
#pragma unroll
      for (int turn = 0; turn < kTurns; ++turn) {
        const int c = wave + turn * (kSampleThreads / 64);
        const int n = c < cd.chunks ? starts[c + 1] - starts[c] : 0;
#pragma unroll
        for (int q = 0; q < kPieces; ++q)
          got[turn][q] = lane + q * 64 < n ? cd.value[((size_t)row * cd.chunks + c) * kChunkCap + lane + q * 64] : 0.f;
      }
#pragma unroll
      for (int turn = 0; turn < kTurns; ++turn) {
        const int c = wave + turn * (kSampleThreads / 64);
        const int n = c < cd.chunks ? starts[c + 1] - starts[c] : 0;
#pragma unroll
        for (int q = 0; q < kPieces; ++q)
          if (lane + q * 64 < n) gathered[starts[c] + lane + q * 64] = got[turn][q];
      }
    }
    __syncthreads();
    units = starts[64];
    total_of_row = total_s;
    z = gathered;
  }
  const int num_elements = CAND ? units : vocab;

  constexpr int kHeld = !IN_REGS ? 1 : (CAND ? kMaxCandidates / kSampleThreads : kSlots);      // elements of a thread in registers
  float held[kHeld];
  if constexpr (IN_REGS) {
#pragma unroll
    for (int s = 0; s < kHeld; s += kPer) {
      const int u = (s / kPer) * kSampleThreads + tid;
      if constexpr (VEC) {
        const float4 t = u < units ? reinterpret_cast<const float4*>(z)[u] : make_float4(0.f, 0.f, 0.f, 0.f);
        held[s] = t.x; held[s + 1] = t.y; held[s + 2] = t.z; held[s + 3] = t.w;
      } else {
        held[s] = u < units ? z[u] : 0.f;
      }
    }
  }
#define PLLM_WALK(visitor) for_each_element<IN_REGS, VEC, kHeld>(held, z, units, tid, visitor)

  Extremes ex; ex.best.v = -INFINITY; ex.best.i = 0x7fffffff; ex.lowest = INFINITY;
  ex = PLLM_WALK(ex);
  const ArgMax best = block_argmax(ex.best, ascratch);
  const float temp = temperature[row];
  if (temp < 1e-5f) {
    if (tid == 0) out[row] = best.i;
    return true;
  }
  Weigh weigh; weigh.zmax = best.v; weigh.rate = 1.4426950408889634f / fmaxf(temp, 1e-5f);

  int k = top_k[row];
  const float p = top_p[row];
  bool capped = false;                                           // CAND: the candidates were chosen under a smaller top_k than the row's own
  if constexpr (CAND) {
    const int own = k;
    k = candidates_top_k(temp, own, p, vocab);
    capped = k != own;
  }
  if (k <= 0 || k > num_elements) k = num_elements;
  const bool filtered = k < num_elements || p < 1.f;
  // The sum of all weights: a pass of its own where nothing is filtered, else part of the search's first pass.
  SumOfWeights sw; sw.w = weigh; sw.sum = 0.f;
  float total = 0.f;
  if (!filtered) {
    sw = PLLM_WALK(sw);
    total = block_sum(sw.sum, fscratch);
  }
  uint32_t threshold = 0;                                        // tokens whose key >= threshold stay; 0 keeps all
  constexpr int kSlotsHere = kWindowSlots<IN_REGS>;
  IntoWindow<kSlotsHere> win; win.n = 0; win.mass_up = 0.f;
  bool windowed = false;
  if constexpr (CAND) {
    if (filtered) {
      // Few candidates, all in registers: first the k-th largest key, by histograms of 256 bins over the range of keys that
      // still holds it (at first from the smallest to the largest candidate; the bin in which the k-th falls is the
      // next range: three passes for keys a few million apart), then the fewer than k candidates above it, each with
      // the weight of those above it, and the group at the k-th key as one.
      __shared__ int hist[256];
      __shared__ uint32_t lo_s, hi_s;
      __shared__ int rank_s;
      __shared__ uint32_t up_key[kCandTopK];
      __shared__ float up_weight[kCandTopK];
      __shared__ int up_counts[kSampleThreads / 64];
      total = total_of_row;
      const float lowest = -block_max(-ex.lowest, fscratch);
      uint32_t lo = float_key(lowest), hi = float_key(best.v);
      int rank = k;                                              // the key looked for is the rank-th largest of those in [lo, hi]
      for (;;) {
        const uint32_t span = hi - lo;
        const int shift = span < 256u ? 0 : 24 - __clz(span);    // (span >> shift) < 256
        if (tid < 256) hist[tid] = 0;
        __syncthreads();
#pragma unroll
        for (int s2 = 0; s2 < kHeld; ++s2) {
          if (s2 * kSampleThreads >= units) break;
          if (s2 * kSampleThreads + tid < units) {
            const uint32_t key = float_key(held[s2]);
            if (key - lo <= span) atomicAdd(&hist[(key - lo) >> shift], 1);
          }
        }
        __syncthreads();
        if (tid < 64) {                                          // lane l: bins 255 - 4 l down to 252 - 4 l
          int mine[4], sum = 0;
#pragma unroll
          for (int j = 0; j < 4; ++j) { mine[j] = hist[255 - 4 * tid - j]; sum += mine[j]; }
          int incl = sum;
#pragma unroll
          for (int o = 1; o < 64; o <<= 1) {
            const int up = __shfl_up(incl, o, 64);
            if (tid >= o) incl += up;
          }
          const unsigned long long reached = __ballot(incl >= rank);
          const int first = reached ? __ffsll((long long)reached) - 1 : 63;       // (the range holds at least rank candidates)
          if (tid == first) {
            int before = incl - sum, j = 0;
            while (j < 3 && before + mine[j] < rank) { before += mine[j]; ++j; }
            const uint32_t bin = 255 - 4 * tid - j;
            const unsigned long long top_of_bin = (unsigned long long)lo + ((unsigned long long)bin << shift) + ((1ull << shift) - 1);
            lo_s = lo + (bin << shift);
            hi_s = top_of_bin < hi ? (uint32_t)top_of_bin : hi;
            rank_s = rank - before;
          }
        }
        __syncthreads();
        lo = lo_s; hi = hi_s; rank = rank_s;
        if (shift == 0) break;                                   // (a bin was one key)
      }
      const uint32_t found = lo;
      const uint32_t kth = found;                                // k - rank candidates lie above it
      // the candidates above the k-th key, in the order of the threads
      int mine_up = 0;
#pragma unroll
      for (int s2 = 0; s2 < kHeld; ++s2) {
        if (s2 * kSampleThreads >= units) break;
        mine_up += (s2 * kSampleThreads + tid < units && float_key(held[s2]) > kth) ? 1 : 0;
      }
      const int lane = tid & 63, wave = tid >> 6;
      int incl = mine_up;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(incl, o, 64);
        if (lane >= o) incl += up;
      }
      if (lane == 63) up_counts[wave] = incl;
      __syncthreads();
      int at = incl - mine_up, num_up = 0;
      for (int w = 0; w < kSampleThreads / 64; ++w) {
        if (w < wave) at += up_counts[w];
        num_up += up_counts[w];
      }
#pragma unroll
      for (int s2 = 0; s2 < kHeld; ++s2) {
        if (s2 * kSampleThreads >= units) break;
        if (s2 * kSampleThreads + tid < units && float_key(held[s2]) > kth) {
          up_key[at] = float_key(held[s2]);
          up_weight[at] = weigh(held[s2]);
          ++at;
        }
      }
      __syncthreads();
      // Thread i < num_up: candidate i above the k-th key stays if what lies above it weighs at most p of the row;
      // thread num_up: the group at the k-th key, above which all of them lie.  (Fewer than k lie above each.)
      uint32_t dropped = 0, my_key = 0;
      if (tid <= num_up) {
        my_key = tid < num_up ? up_key[tid] : kth;
        float above = 0.f;
#pragma unroll 8
        for (int j = 0; j < num_up; ++j) above += up_key[j] > my_key ? up_weight[j] : 0.f;
        if (!(above <= p * total)) dropped = my_key;
      }
      // the largest key that goes; what stays is what lies above it
      const uint32_t cut = float_as_uint_max(dropped, fscratch);
      uint32_t lowest_kept = 0xffffffffu;
      if (tid <= num_up && my_key > cut) lowest_kept = my_key;
      threshold = float_as_uint_min(lowest_kept, fscratch);
      if (capped) {
        // Fewer than k stay: the next token went by its mass, and would under the row's own top_k.  Else the row's
        // own rule may keep more than these candidates hold.
        int staying = 0;
#pragma unroll
        for (int s2 = 0; s2 < kHeld; ++s2) {
          if (s2 * kSampleThreads >= units) break;
          staying += (s2 * kSampleThreads + tid < units && float_key(held[s2]) >= threshold) ? 1 : 0;
        }
        if ((int)block_sum((float)staying, fscratch) >= k) return false;
      }
    }
  } else if (filtered) {
    // kept(c)  <=>  count(key > c) < k  and  mass(key > c) <= p * total  is monotone in c; the threshold is the
    // smallest key of a token that stays.  [lo, hi]: kept(hi) holds, kept(lo - 1) does not, and both ends are keys of
    // tokens of the row (at the start its minimum, which cannot stay, and its maximum, which always does).  A pass takes
    // a pivot between them (the middle of the two values; of the two keys where that gives nothing new), counts and
    // weighs what lies above it, and moves one end to the nearest token's key on the pivot's side: the interval loses
    // the pivot's side and all the empty room next to it, so about a dozen passes are left where 32 halvings of all
    // keys were.  Once every thread has at most kWindowSlots of its tokens inside the interval it keeps those in
    // registers and the row is not read again.
    const float lowest = -block_max(-ex.lowest, fscratch);
    uint32_t lo = float_key(lowest), hi = float_key(best.v);
    float mass_above = 0.f;                                      // of the tokens above the interval, once windowed
    int cnt_above = 0;
    // The first pivot: the logit whose weight is 2^-13 of the largest.  Where a few tokens carry the mass (the usual
    // row) nearly all of it lies above that pivot, so the first pass already leaves an interval with few tokens in it.
    // That pass also takes the tokens above its pivot along, as many as the registers for the interval's tokens hold:
    // if the threshold does lie above the pivot they are the interval's tokens, and the pass that would fetch them is saved.
    bool first = true;
    while (lo < hi) {
      const float vmid = first ? best.v - 13.f / weigh.rate : 0.5f * key_value(lo) + 0.5f * key_value(hi);
      uint32_t mid = float_key(vmid);
      if (!(mid >= lo && mid < hi)) mid = lo + ((hi - lo) >> 1);
      AroundPivot ap; ap.w = weigh; ap.lo = lo; ap.hi = hi; ap.mid = mid;
      ap.mass = 0.f; ap.cnt = 0; ap.low_mine = 0; ap.high_mine = 0; ap.below = lo; ap.above = hi;
      if (windowed) {
#pragma unroll
        for (int s = 0; s < kSlotsHere; ++s) ap.look(win.key[s], win.weight[s]);     // (unused slots hold key 0: below every interval)
        ap.cnt += cnt_above; ap.mass += mass_above;
      } else if (first) {
        FirstLook<kSlotsHere> fl; fl.ap = ap; fl.n = 0; fl.sum = 0.f;
#pragma unroll
        for (int s = 0; s < kSlotsHere; ++s) { fl.key[s] = 0u; fl.weight[s] = 0.f; }
        fl = PLLM_WALK(fl);
        ap = fl.ap;
        total = block_sum(fl.sum, fscratch);
#pragma unroll
        for (int s = 0; s < kSlotsHere; ++s) { win.key[s] = fl.key[s]; win.weight[s] = fl.weight[s]; }
      } else {
        ap = PLLM_WALK(ap);
      }
      int low_most = ap.low_mine, high_most = ap.high_mine;
      block_reduce_pass(ap.mass, ap.cnt, ap.below, ap.above, low_most, high_most, fscratch, iscratch);
      const bool kept = ap.cnt < k && ap.mass <= p * total;
      if (kept) hi = ap.below; else lo = ap.above;
      if (first && !kept && high_most <= kSlotsHere) {
        // (the interval is what lay above the first pivot: its tokens are in the registers already, nothing lies above it)
        win.mass_up = 0.f;
        windowed = true;
      }
      first = false;
      if (!windowed && lo < hi && (kept ? low_most : high_most) <= kSlotsHere) {
        win.w = weigh; win.lo = lo; win.hi = hi; win.n = 0; win.cnt_up = 0; win.mass_up = 0.f;
#pragma unroll
        for (int s = 0; s < kSlotsHere; ++s) { win.key[s] = 0u; win.weight[s] = 0.f; }
        win = PLLM_WALK(win);
        mass_above = block_sum(win.mass_up, fscratch);
        cnt_above = (int)block_sum((float)win.cnt_up, fscratch);       // (exact: below 2^24)
        windowed = true;
      }
    }
    threshold = hi;
  }

  // ---- the draw: inverse CDF over the tokens that stay, in the order thread by thread, each thread's tokens in its own order
  KeptSum ks; ks.w = weigh; ks.threshold = threshold; ks.sum = sw.sum;
  if (windowed) {
    // (what this thread had above the interval when it took its tokens inside it into registers, and those of them that stay)
    ks.sum = win.mass_up;
#pragma unroll
    for (int s = 0; s < kSlotsHere; ++s) ks.sum += win.key[s] >= threshold ? win.weight[s] : 0.f;
  } else if (threshold != 0u) {                                  // (without a threshold every token stays: the sums above)
    ks.sum = 0.f;
    ks = PLLM_WALK(ks);
  }
  float kept_total;
  const float before = block_exclusive_scan(ks.sum, fscratch, kept_total);
  if (tid == 0) { chosen = -1; chooser = -1; }
  __syncthreads();
  const long long rkey = request_key[row];
  const uint32_t bits = philox_first_word((uint32_t)step[row], 0u, (uint32_t)rkey, (uint32_t)(rkey >> 32),
                                          (uint32_t)seed, (uint32_t)(seed >> 32));
  const float u01 = (float)(bits >> 8) * (1.0f / 16777216.0f);   // [0, 1)
  const float target = u01 * kept_total;
  // The token is taken by the last thread, in thread order, that has tokens that stay and whose share of the line starts at
  // or before the target.  The starts come out of a prefix sum and may be an ulp off each other's ends; "the last one that
  // starts at or before" names exactly one thread whatever the rounding (a test of each thread's own interval could name
  // two, or none), so a row's token depends on the row, the seed, the request and the step alone.
  if (ks.sum > 0.f && before <= target) atomicMax(&chooser, tid);
  __syncthreads();
  if (chooser == tid) {
    Pick pk; pk.w = weigh; pk.threshold = threshold; pk.run = before; pk.target = target; pk.pick = -1; pk.last = -1;
    pk = PLLM_WALK(pk);
    chosen = pk.pick >= 0 ? pk.pick : pk.last;               // (the target at or past the end of this share: its last token)
  }
  __syncthreads();
  // (a row without a finite weight: the maximum)
  if (tid == 0) {
    int token = chosen >= 0 ? chosen : best.i;
    if constexpr (CAND) {                                          // the candidate's place in the row
      int c = 0;
      while (c + 1 < cd.chunks && token >= starts[c + 1]) ++c;
      token = cd.index[((size_t)row * cd.chunks + c) * kChunkCap + (token - starts[c])];
    }
    out[row] = token;
  }
  return true;
#undef PLLM_WALK
}

// A workgroup per row: by the row's candidates where every chunk handed its own on, else over the whole row.
template <bool IN_REGS, bool VEC>
__global__ __launch_bounds__(kSampleThreads) void sample_kernel(const float* __restrict__ logits, int vocab, const float* __restrict__ temperature,
                                                                const int* __restrict__ top_k, const float* __restrict__ top_p,
                                                                const long long* __restrict__ request_key, const int* __restrict__ step,
                                                                unsigned long long seed, int* __restrict__ out, const Candidates cd) {
  if (cd.count && has_candidates(cd, blockIdx.x) &&
      sample_row<true, false, true>(logits, vocab, temperature, top_k, top_p, request_key, step, seed, out, cd))
    return;
  __syncthreads();                                               // (what the candidates' part left in LDS is done with)
  sample_row<IN_REGS, VEC, false>(logits, vocab, temperature, top_k, top_p, request_key, step, seed, out, cd);
}

// Bytes of workspace with which pllm_sample sends rows with a small top_k by their candidates; 0: it would not (many
// rows keep the GPU busy by themselves, a short row is walked quickly).
static int candidate_chunks(int rows, int vocab, int* chunk) {
  if (rows > 128 || vocab < 8192 || vocab > kMaxChunks * kChunkMost) return 0;
  int chunks = (vocab + 2047) / 2048;
  if (chunks > kMaxChunks) chunks = kMaxChunks;
  *chunk = ((vocab + chunks - 1) / chunks + kCandThreads - 1) / kCandThreads * kCandThreads;      // at most kChunkMost
  return (vocab + *chunk - 1) / *chunk;
}
PLLM_API long pllm_sample_workspace_bytes(int rows, int vocab) {
  int chunk = 0;
  const long slots = (long)rows * candidate_chunks(rows, vocab, &chunk);
  return slots * (3 + 2 * kChunkCap) * 4;
}

// workspace: null, or pllm_sample_workspace_bytes(rows, vocab) bytes (16-byte aligned) that the call may use.
PLLM_API int pllm_sample(const float* logits, int rows, int vocab, const float* temperature, const int* top_k,
                         const float* top_p, const long long* request_key, const int* step, unsigned long long seed,
                         int* out, void* workspace, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (vocab <= 0) return -2;
  const bool vec = (vocab & 3) == 0 && (reinterpret_cast<uintptr_t>(logits) & 15) == 0;
  const bool in_regs = vocab <= kSlots * kSampleThreads;
  Candidates cd = {};
  int chunk = 0;
  const int chunks = workspace ? candidate_chunks(rows, vocab, &chunk) : 0;
  if (chunks > 0) {
    const size_t slots = (size_t)rows * chunks;
    cd.count = (int*)workspace;
    cd.top = (float*)workspace + slots;
    cd.sum = (float*)workspace + 2 * slots;
    cd.value = (float*)workspace + 3 * slots;
    cd.index = (int*)workspace + (3 + kChunkCap) * slots;
    cd.chunks = chunks;
    cd.chunk = chunk;
    hipLaunchKernelGGL(sample_candidates_kernel, dim3(chunks, rows), dim3(kCandThreads), 0, stream, logits, vocab, temperature, top_k, top_p, cd);
  }
#define PLLM_SAMPLE(IN_REGS_, VEC_)                                                                                          \
  hipLaunchKernelGGL((sample_kernel<IN_REGS_, VEC_>), dim3(rows), dim3(kSampleThreads), 0, stream, logits, vocab, temperature, top_k, \
                     top_p, request_key, step, seed, out, cd)
  if (in_regs && vec) PLLM_SAMPLE(true, true);
  else if (in_regs) PLLM_SAMPLE(true, false);
  else if (vec) PLLM_SAMPLE(false, true);
  else PLLM_SAMPLE(false, false);
#undef PLLM_SAMPLE
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
