// Partitioned decode attention for callers that cannot allocate device memory.
//
// This entry point has no counterpart in the reference (xiyiji/paged-llm allocates its attention
// workspace through its tensor library at every call).  It is for callers that cannot call
// hipMalloc: code under HIP graph capture, tight serving loops, harnesses that forbid allocation.
//
// It does what pllm_paged_attention_mfma (attention_mfma.hip, one library per head size) does with
// partition_size > 0: the keys of every (sequence, kv head) are cut into aligned partitions, one workgroup
// each, merged by a second kernel.  The partitions' partial results live in a fixed array inside the library
// of attention_noalloc.hip instead of a workspace argument: PLLM_NOALLOC_SCRATCH_BYTES per GPU that library
// runs on, held until the process ends, one array for all head sizes.  The call allocates and frees nothing,
// on the device or through any library.
//
//   set-up  pllm_attention_noalloc_prepare(api), once per head size and per device, with that device current and
//           OUTSIDE any stream capture: `api` is what the head size's attention library returns from
//           pllm_attention_mfma_api().  It asks for the array's address on this device and makes the device
//           queries of the launch code, so that the calls afterwards only launch kernels.
//   needs   total_q * num_heads * num_partitions * (head size + 2) * 4 bytes <= PLLM_NOALLOC_SCRATCH_BYTES;
//           partition_size a positive multiple of 64 with num_partitions * partition_size >= the longest
//           context of the batch (the lengths are on the device, so the call cannot check this: keys beyond
//           the last partition would be left out); waves in {1, 4, 8}; max_q_len * group <= 64
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
  PLLM_NOALLOC_NOT_PREPARED = -23,  // pllm_attention_noalloc_prepare has not run for this head size on this device
};

// What one attention library (attention_mfma.hip compiled for one head size) hands out.
struct pllm_attention_api {
  int head_dim;
  int (*paged_attention)(const void* q, int q_stride, const void* k_pages, const void* v_pages, void* out, int out_stride,
                         const int* block_tables, int bt_stride, const int* cu_seqlens_q, const int* seq_lens_k, int num_seqs,
                         int total_q, int max_q_len, int num_heads, int num_kv_heads, int block_size, float scale, int window,
                         int partition_size, int num_partitions, float* partials, int waves, int column_blocks,
                         const int* work_list, int num_work, hipStream_t stream);
  int (*warm_up)(void);             // makes the launch code's device queries now; 0 when they succeeded
};

extern "C" __attribute__((visibility("default"))) const pllm_attention_api* pllm_attention_mfma_api();   // in each attention library

extern "C" __attribute__((visibility("default"))) int pllm_attention_noalloc_prepare(const pllm_attention_api* api);

extern "C" __attribute__((visibility("default"))) int pllm_paged_attention_decode_noalloc(
    int head_dim, const void* q, int q_stride, const void* k_pages, const void* v_pages, void* out, int out_stride,
    const int* block_tables, int bt_stride, const int* cu_seqlens_q, const int* seq_lens_k, int num_seqs, int total_q,
    int max_q_len, int num_heads, int num_kv_heads, int block_size, float scale, int window, int partition_size,
    int num_partitions, int waves, hipStream_t stream);

extern "C" __attribute__((visibility("default"))) const char* pllm_attention_noalloc_error();
