// Partitioned decode attention for callers that cannot allocate device memory.
//
// This entry point has no counterpart in the reference (xiyiji/paged-llm allocates its attention
// workspace through its tensor library at every call).  It is for callers that cannot call
// hipMalloc: code under HIP graph capture, tight serving loops, harnesses that forbid allocation.
//
// It does what pllm_paged_attention_mfma does with partition_size > 0 (the keys of every
// (sequence, kv head) cut into aligned partitions, one workgroup each, merged by a second kernel),
// but the partitions' partial results live in a fixed array inside the library instead of a
// workspace argument: PLLM_NOALLOC_SCRATCH_BYTES per GPU the library runs on, held until the
// process ends.  The call allocates and frees nothing, on the device or through any library.
//
//   needs   total_q * num_heads * num_partitions * (head size + 2) * 4 bytes <= PLLM_NOALLOC_SCRATCH_BYTES,
//           partition_size a positive multiple of 64, waves in {1, 4, 8}, max_q_len * group <= 64
//   returns 0, a hipError_t of a launch, or a PLLM_NOALLOC_* code; pllm_attention_noalloc_error()
//           gives the text of the calling thread's last refusal
//
// Every call on a GPU shares that GPU's array, which keeps what the last call left in it.  Nothing in
// it has to start at zero (every partial result that the merge counts is written by the same call
// first; what it does not count is dropped by a select), so nothing is cleared.  Calls that overlap
// on one GPU (two streams, two threads) race on the array: run them one after the other.
#pragma once
#include <hip/hip_runtime.h>

#define PLLM_NOALLOC_SCRATCH_BYTES (8u << 20)

enum {
  PLLM_NOALLOC_TOO_LARGE = -20,     // the partial results do not fit the array
  PLLM_NOALLOC_BAD_ARGUMENT = -21,  // a shape or launch parameter the kernels do not take
  PLLM_NOALLOC_NO_SYMBOL = -22,     // the array's device address could not be obtained
};

extern "C" __attribute__((visibility("default"))) int pllm_paged_attention_decode_noalloc(
    const void* q, int q_stride, const void* k_pages, const void* v_pages, void* out, int out_stride,
    const int* block_tables, int bt_stride, const int* cu_seqlens_q, const int* seq_lens_k, int num_seqs, int total_q,
    int max_q_len, int num_heads, int num_kv_heads, int block_size, float scale, int window, int partition_size,
    int num_partitions, int waves, hipStream_t stream);

extern "C" __attribute__((visibility("default"))) const char* pllm_attention_noalloc_error();
