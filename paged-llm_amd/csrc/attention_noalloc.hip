// The partitioned decode attention for callers that cannot allocate (see attention_noalloc.h): the partitions'
// partial results go to an array of this library instead of a workspace argument.  The kernels are those of the
// attention library of the head size (attention_mfma.hip), reached through the entry point that library hands out;
// they take the array's address as they take the workspace.  In host code the array's name is only a stand-in for the
// symbol, so its device address is asked for once per device (each GPU holds its own copy at its own address), in
// pllm_attention_noalloc_prepare, and only that address is used afterwards.
#include "attention_noalloc.h"
#include <mutex>
#include <stdio.h>

static __device__ __align__(256) float scratch[PLLM_NOALLOC_SCRATCH_BYTES / sizeof(float)];

constexpr int kMaxDevices = 64;
constexpr int kMaxHeadDim = 256;
static float* scratch_of_device[kMaxDevices];
static const pllm_attention_api* api_of_head_dim[kMaxHeadDim / 16 + 1];
static bool warmed[kMaxDevices][kMaxHeadDim / 16 + 1];
static std::mutex lock;
static thread_local char noalloc_error[320];

extern "C" __attribute__((visibility("default"))) const char* pllm_attention_noalloc_error() { return noalloc_error; }

static int current_device(int* dev) {
  hipError_t e = hipGetDevice(dev);
  if (e != hipSuccess || *dev < 0 || *dev >= kMaxDevices) {
    snprintf(noalloc_error, sizeof noalloc_error, "no current device, or device %d beyond the %d this library keeps addresses for", *dev, kMaxDevices);
    return PLLM_NOALLOC_NO_SYMBOL;
  }
  return 0;
}

extern "C" __attribute__((visibility("default"))) int pllm_attention_noalloc_prepare(const pllm_attention_api* api) {
  noalloc_error[0] = 0;
  if (!api || !api->paged_attention || !api->warm_up || api->head_dim < 16 || api->head_dim > kMaxHeadDim || api->head_dim % 16) {
    snprintf(noalloc_error, sizeof noalloc_error, "prepare takes what an attention library's pllm_attention_mfma_api() returns (head sizes 16..%d in steps of 16)", kMaxHeadDim);
    return PLLM_NOALLOC_BAD_ARGUMENT;
  }
  int dev = -1;
  if (int err = current_device(&dev)) return err;
  std::lock_guard<std::mutex> hold(lock);
  if (!scratch_of_device[dev]) {
    void* address = nullptr;
    hipError_t e = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !address) {
      snprintf(noalloc_error, sizeof noalloc_error, "hipGetSymbolAddress of the partials array failed on device %d: %s", dev, hipGetErrorString(e));
      return PLLM_NOALLOC_NO_SYMBOL;
    }
    scratch_of_device[dev] = static_cast<float*>(address);
  }
  if (api->warm_up() != 0) {
    snprintf(noalloc_error, sizeof noalloc_error, "the attention library for head size %d could not query device %d", api->head_dim, dev);
    return PLLM_NOALLOC_NO_SYMBOL;
  }
  api_of_head_dim[api->head_dim / 16] = api;
  warmed[dev][api->head_dim / 16] = true;
  return 0;
}

extern "C" __attribute__((visibility("default"))) int pllm_paged_attention_decode_noalloc(
    int head_dim, const void* q, int q_stride, const void* k_pages, const void* v_pages, void* out, int out_stride,
    const int* block_tables, int bt_stride, const int* cu_seqlens_q, const int* seq_lens_k, int num_seqs, int total_q,
    int max_q_len, int num_heads, int num_kv_heads, int block_size, float scale, int window, int partition_size,
    int num_partitions, int waves, hipStream_t stream) {
  noalloc_error[0] = 0;
  if (total_q <= 0 || num_seqs <= 0) return 0;
  if (!q || !k_pages || !v_pages || !out || !block_tables || !cu_seqlens_q || !seq_lens_k || num_heads <= 0 || num_kv_heads <= 0 ||
      num_heads % num_kv_heads || max_q_len < 1 || head_dim < 16 || head_dim > kMaxHeadDim || head_dim % 16) {
    snprintf(noalloc_error, sizeof noalloc_error, "null operand, head size %d outside 16..%d in steps of 16, or %d heads that are no multiple of %d kv heads",
             head_dim, kMaxHeadDim, num_heads, num_kv_heads);
    return PLLM_NOALLOC_BAD_ARGUMENT;
  }
  if (partition_size <= 0 || (partition_size & 63) || num_partitions < 1 || (long)max_q_len * (num_heads / num_kv_heads) > 64) {
    snprintf(noalloc_error, sizeof noalloc_error,
             "this entry point is the partitioned form: partition_size must be a positive multiple of 64 (got %d), num_partitions >= 1 "
             "(got %d) and queries x heads per kv head at most 64 (got %ld)", partition_size, num_partitions,
             (long)max_q_len * (num_heads / num_kv_heads));
    return PLLM_NOALLOC_BAD_ARGUMENT;
  }
  const unsigned long long need = (unsigned long long)total_q * num_heads * num_partitions * (head_dim + 2) * sizeof(float);
  if (need > PLLM_NOALLOC_SCRATCH_BYTES) {
    snprintf(noalloc_error, sizeof noalloc_error,
             "%d query rows x %d heads x %d partitions x (%d + 2) floats = %llu bytes of partial results; the library's array holds %u",
             total_q, num_heads, num_partitions, head_dim, need, (unsigned)PLLM_NOALLOC_SCRATCH_BYTES);
    return PLLM_NOALLOC_TOO_LARGE;
  }
  int dev = -1;
  if (int err = current_device(&dev)) return err;
  // (read without the lock: prepare has returned before the first call for its head size and device, and entries are only ever set)
  float* partials = scratch_of_device[dev];
  const pllm_attention_api* api = api_of_head_dim[head_dim / 16];
  if (!partials || !api || !warmed[dev][head_dim / 16]) {
    snprintf(noalloc_error, sizeof noalloc_error, "pllm_attention_noalloc_prepare has not run for head size %d on device %d", head_dim, dev);
    return PLLM_NOALLOC_NOT_PREPARED;
  }
  const int rc = api->paged_attention(q, q_stride, k_pages, v_pages, out, out_stride, block_tables, bt_stride, cu_seqlens_q, seq_lens_k,
                                      num_seqs, total_q, max_q_len, num_heads, num_kv_heads, block_size, scale, window, partition_size,
                                      num_partitions, partials, waves, 0, nullptr, 0, stream);
  if (rc == -2) {
    snprintf(noalloc_error, sizeof noalloc_error, "the attention kernels refuse this shape (pages of %d positions, %d wavefronts, %d/%d heads)",
             block_size, waves, num_heads, num_kv_heads);
    return PLLM_NOALLOC_BAD_ARGUMENT;
  }
  return rc;
}
