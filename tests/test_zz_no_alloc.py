"""The entry point that allocates nothing: partitioned decode attention with the partitions' partial
results in an array of the library itself (csrc/attention_noalloc.h), called through ctypes and
compared with the existing entry point, which takes the same buffer as a workspace argument, and with
a float reference of the attention itself."""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_void_p

import pytest
import torch

from tests.test_kernels_gpu import dense_attention, paged_case

pytestmark = pytest.mark.gpu

HEADS, KV_HEADS, D, BS = 8, 2, 64, 16
SIGNATURE = [c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int,
             c_int, c_int, c_int, c_float, c_int, c_int, c_int, c_int, c_void_p]
SCRATCH_BYTES = 8 << 20
NOT_PREPARED = -23


def libraries(head_dim=D):
    """(the library with the array and the entry point, what the head size's attention library hands out for it)"""
    from paged_llm_amd.csrc import build
    lib = build.load_library("attention_noalloc.hip")
    lib.pllm_paged_attention_decode_noalloc.argtypes = SIGNATURE
    lib.pllm_paged_attention_decode_noalloc.restype = c_int
    lib.pllm_attention_noalloc_prepare.argtypes = [c_void_p]
    lib.pllm_attention_noalloc_prepare.restype = c_int
    lib.pllm_attention_noalloc_error.argtypes = []
    lib.pllm_attention_noalloc_error.restype = ctypes.c_char_p
    kernels = build.load_library("attention_mfma.hip", {"HEAD_DIM": head_dim})
    kernels.pllm_attention_mfma_api.argtypes = []
    kernels.pllm_attention_mfma_api.restype = c_void_p
    return lib, kernels.pllm_attention_mfma_api()


def call(lib, q, kp, vp, tables, cu, sl, out, partition_size, parts, waves, head_dim=D):
    stream = torch.cuda.current_stream().cuda_stream
    return lib.pllm_paged_attention_decode_noalloc(
        head_dim, q.data_ptr(), q.stride(0), kp.data_ptr(), vp.data_ptr(), out.data_ptr(), out.stride(0), tables.data_ptr(),
        tables.stride(0), cu.data_ptr(), sl.data_ptr(), sl.numel(), q.shape[0], 1, HEADS, KV_HEADS, BS, c_float(head_dim ** -0.5), 0,
        partition_size, parts, waves, stream)


def case(lens, seed, head_dim=D):
    return paged_case(lens, [1] * len(lens), HEADS, KV_HEADS, head_dim, BS, torch.bfloat16, seed=seed)


def test_a_call_before_prepare_is_refused():
    lib, _ = libraries()
    on_gpu = [t.cuda() for t in case([64, 64], 3, head_dim=32)]
    out = torch.zeros(2, HEADS * 32, dtype=torch.bfloat16, device="cuda")
    assert call(lib, *on_gpu, out, 64, 1, 4, head_dim=32) == NOT_PREPARED      # (no test prepares head size 32)
    assert "prepare" in lib.pllm_attention_noalloc_error().decode()
    torch.cuda.synchronize()
    assert out.float().abs().sum().item() == 0


def test_two_calls_in_a_row_equal_the_entry_point_with_a_workspace():
    from paged_llm_amd.csrc import ops
    lib, api = libraries()
    assert lib.pllm_attention_noalloc_prepare(api) == 0, lib.pllm_attention_noalloc_error()
    # one call to have the code objects of both libraries on the device before free memory is read
    warm = [t.cuda() for t in case([200, 70], 4)]
    assert call(lib, *warm, torch.empty(2, HEADS * D, dtype=torch.bfloat16, device="cuda"), 128, 2, 4) == 0
    torch.cuda.synchronize()
    # the second call is smaller (fewer sequences, fewer partitions): what the first left in the array must not show
    for lens, partition_size, waves, seed in (([1500, 700, 1027, 64, 333], 256, 4, 5), ([130, 515], 128, 8, 6)):
        host = case(lens, seed)
        q, kp, vp, tables, cu, sl = [t.cuda() for t in host]
        parts = (max(lens) + partition_size - 1) // partition_size
        want = ops.paged_attention_mfma(q, kp, vp, tables, cu, sl, HEADS, KV_HEADS, D, D ** -0.5, 0, 1, partition_size, parts, waves)
        out = torch.full_like(want, float("nan"))
        torch.cuda.synchronize()
        # Free bytes of the device itself: an allocation by the runtime inside the call would lower it, which the
        # tensor library's own count (below) would not see.
        free_before, held_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
        rc = call(lib, q, kp, vp, tables, cu, sl, out, partition_size, parts, waves)
        torch.cuda.synchronize()
        assert rc == 0, lib.pllm_attention_noalloc_error()
        assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_allocated() == held_before
        assert torch.equal(out, want), (lens, (out.float() - want.float()).abs().max())
        # ... and both are the attention: against the float reference over the same pages
        ref = dense_attention(*host, HEADS, KV_HEADS, D, D ** -0.5)
        assert (out.float().cpu() - ref).abs().max().item() <= 2e-2 * max(1.0, ref.abs().max().item())


def test_sizes_beyond_the_array_are_refused_with_a_message():
    lib, api = libraries()
    assert lib.pllm_attention_noalloc_prepare(api) == 0, lib.pllm_attention_noalloc_error()
    q, kp, vp, tables, cu, sl = [t.cuda() for t in case([64, 64], 7)]
    out = torch.zeros(2, HEADS * D, dtype=torch.bfloat16, device="cuda")
    parts = SCRATCH_BYTES // (2 * HEADS * (D + 2) * 4) + 1          # one partition more than the array holds for two rows
    assert call(lib, q, kp, vp, tables, cu, sl, out, 64, parts, 4) == -20
    text = lib.pllm_attention_noalloc_error().decode()
    assert "partial results" in text and str(SCRATCH_BYTES) in text
    assert call(lib, q, kp, vp, tables, cu, sl, out, 100, 1, 4) == -21   # no multiple of 64
    assert "multiple of 64" in lib.pllm_attention_noalloc_error().decode()
    assert lib.pllm_attention_noalloc_prepare(None) == -21
    torch.cuda.synchronize()
    assert out.float().abs().sum().item() == 0                       # a refused call launches nothing
