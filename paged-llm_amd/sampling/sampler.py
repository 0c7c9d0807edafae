"""Next-token choice: greedy, temperature, top-k and top-p (pagedllm/sampler.py:10-35), on the GPU.

All rows of a step go through one kernel launch.  Randomness is counter-based: the uniform number
of a row depends on (engine seed, request id, number of tokens the request has generated), not on
a generator shared by the batch, so a request draws the same tokens whatever runs beside it.
"""

from __future__ import annotations

import torch

from ..csrc import ops


class PendingTokens:
    """Token ids on their way from the GPU: the kernel and the copy to pinned host memory are queued, ``result()``
    waits for them.  Host work done between the two overlaps the GPU's."""

    def __init__(self, staged: torch.Tensor | None, count: int, copied, on_device: torch.Tensor | None = None):
        self._staged, self._count, self._copied = staged, count, copied
        # The same ids as the sampling kernel left them on the GPU (int32 [count]): a step that is launched before
        # the host has seen them takes them from here.
        self.on_device = on_device

    def result(self) -> list:
        if self._count == 0:
            return []
        if self._copied is not None:
            self._copied.synchronize()
        return self._staged[: self._count].tolist()


class Sampler:
    def __init__(self, seed: int = 0, device="cuda"):
        self.seed = int(seed)
        self.device = torch.device(device)
        self._pinned = None
        self._copied = None

    def _to_host(self, tokens: torch.Tensor) -> PendingTokens:
        n = tokens.numel()
        if self._pinned is None or self._pinned.numel() < n:
            self._pinned = torch.empty(max(n, 256), dtype=torch.int32, pin_memory=True)
            self._copied = torch.cuda.Event()
        self._pinned[:n].copy_(tokens, non_blocking=True)
        self._copied.record()
        return PendingTokens(self._pinned, n, self._copied, tokens)

    @torch.no_grad()
    def launch(self, logits: torch.Tensor, params: list, request_keys: list, steps: list) -> PendingTokens:
        """logits float32 [n, vocab]; params: SamplingParams per row.  Queues the kernel and the copy of the n token
        ids to the host.  One result may be outstanding at a time (its buffer is reused by the next call)."""
        n = logits.shape[0]
        assert n == len(params) == len(request_keys) == len(steps)
        if n == 0:
            return PendingTokens(None, 0, None)
        if all(p.temperature < 1e-5 for p in params):
            return self._to_host(ops.argmax(logits))
        dev = logits.device
        temperature = torch.tensor([float(p.temperature) for p in params], dtype=torch.float32, device=dev)
        top_k = torch.tensor([int(p.top_k) for p in params], dtype=torch.int32, device=dev)
        top_p = torch.tensor([float(p.top_p) for p in params], dtype=torch.float32, device=dev)
        keys = torch.tensor([int(k) for k in request_keys], dtype=torch.int64, device=dev)
        step = torch.tensor([int(s) for s in steps], dtype=torch.int32, device=dev)
        return self._to_host(ops.sample(logits, temperature, top_k, top_p, keys, step, self.seed))

    def sample(self, logits: torch.Tensor, params: list, request_keys: list, steps: list) -> list:
        """The n token ids, waited for."""
        return self.launch(logits, params, request_keys, steps).result()
