"""Next-token choice: greedy, temperature, top-k and top-p (pagedllm/sampler.py:10-35), on the GPU.

All rows of a step go through one kernel launch.  Randomness is counter-based: the uniform number
of a row depends on (engine seed, request id, number of tokens the request has generated), not on
a generator shared by the batch, so a request draws the same tokens whatever runs beside it.
"""

from __future__ import annotations

import torch

from ..csrc import ops


class Sampler:
    def __init__(self, seed: int = 0, device="cuda"):
        self.seed = int(seed)
        self.device = torch.device(device)

    @torch.no_grad()
    def sample(self, logits: torch.Tensor, params: list, request_keys: list, steps: list) -> list:
        """logits float32 [n, vocab]; params: SamplingParams per row; returns n token ids."""
        n = logits.shape[0]
        assert n == len(params) == len(request_keys) == len(steps)
        if n == 0:
            return []
        if all(p.temperature < 1e-5 for p in params):
            return ops.argmax(logits).tolist()
        dev = logits.device
        temperature = torch.tensor([float(p.temperature) for p in params], dtype=torch.float32, device=dev)
        top_k = torch.tensor([int(p.top_k) for p in params], dtype=torch.int32, device=dev)
        top_p = torch.tensor([float(p.top_p) for p in params], dtype=torch.float32, device=dev)
        keys = torch.tensor([int(k) for k in request_keys], dtype=torch.int64, device=dev)
        step = torch.tensor([int(s) for s in steps], dtype=torch.int32, device=dev)
        return ops.sample(logits, temperature, top_k, top_p, keys, step, self.seed).tolist()
