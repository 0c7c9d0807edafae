"""How many pages the cache pool gets when the caller names no number: what the GPU's free memory
holds beside the activations of the largest step (the reference sizes its pool by the same kind of
probing step, pagedllm/engine.py:141-185)."""

from __future__ import annotations

import torch

from .batch import StepEntry
from .loading import build_runtime


def _probe_step(model, block_size: int, num_tokens: int, wanted_rows: int) -> None:
    """One step of ``num_tokens`` tokens of one request against a throw-away pool, so that the
    allocator's peak shows what a step's activations take.  No more tokens than the model has positions."""
    num_tokens = max(1, min(num_tokens, model.max_positions))
    manager, _, runner = build_runtime(model, block_size, -(-num_tokens // block_size), 1, enable_prefix_caching=False)
    if not manager.allocate("probe", 0, num_tokens):
        raise RuntimeError("the probing step could not get its own pages")
    tables = {g: manager.block_table("probe", g) for g in manager.groups}
    runner.step([StepEntry("probe", [0] * num_tokens, 0, tables, manager.state_slot("probe"), list(range(min(num_tokens, wanted_rows))))])
    torch.cuda.synchronize(model.device)


def pages_that_fit(model, config) -> int:
    """Pages per cache group such that weights, the largest step's activations and the pages of all groups
    stay within ``gpu_memory_utilization`` of the device, but never more than ``max_num_seqs`` requests of
    ``max_model_len`` positions could hold."""
    device, bs = model.device, config.block_size
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats(device)
    resting = torch.cuda.memory_allocated(device)
    _probe_step(model, bs, config.max_num_batched_tokens, config.max_num_seqs)
    step_peak = max(0, torch.cuda.max_memory_allocated(device) - resting)
    torch.cuda.empty_cache()
    free_now, total = torch.cuda.mem_get_info(device)
    # free memory, less the share of the device that is to stay unused, less room for a step's activations
    room = free_now - int(total * (1.0 - config.gpu_memory_utilization)) - step_peak
    page_bytes = sum(g.bytes_per_page(bs, model.dtype) for g in model.cache_groups().values())
    pages = room // max(1, page_bytes)
    ceiling = config.max_num_seqs * -(-config.max_model_len // bs)
    pages = min(pages, ceiling)
    if pages < 16:
        raise RuntimeError(f"not enough GPU memory for the KV cache: {max(pages, 0)} pages of {bs} positions fit "
                           f"({room / 2**20:.0f} MiB left for them); lower max_num_batched_tokens or raise "
                           "gpu_memory_utilization")
    return int(pages)
