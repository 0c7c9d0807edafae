"""Next-token choice: greedy, temperature, top-k and top-p (pagedllm/sampler.py:10-35), on the GPU.

All rows of a step go through one kernel launch.  Randomness is counter-based: the uniform number
of a row depends on (engine seed, request id, number of tokens the request has generated), not on
a generator shared by the batch, so a request draws the same tokens whatever runs beside it.
"""

from __future__ import annotations

import numpy as np
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
        self._rows_pinned = self._rows_device = self._rows_copied = None

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
        temperature, top_k, top_p, keys, step = self._rows_to_device(params, request_keys, steps, logits.device)
        # (the kernel that picks a row's candidates is launched only when some row's settings can use them)
        some = any(ops.sample_candidates_apply(p.temperature, p.top_k, p.top_p, logits.shape[1]) for p in params)
        return self._to_host(ops.sample(logits, temperature, top_k, top_p, keys, step, self.seed, candidates=some))

    def _rows_to_device(self, params: list, request_keys: list, steps: list, device):
        """The rows' settings as device tensors.  They travel as one piece of pinned memory with one queued copy: five
        small tensors made from lists would be five copies from pageable memory, each of which the host waits for
        behind whatever the stream still has to do."""
        n = len(params)
        if self._rows_pinned is None or self._rows_pinned.numel() < 6 * n:
            cap = max(6 * n, 6 * 64)
            self._rows_pinned = torch.empty(cap, dtype=torch.int32, pin_memory=True)
            self._rows_device = torch.empty(cap, dtype=torch.int32, device=device)
            self._rows_copied = torch.cuda.Event()
        else:
            self._rows_copied.synchronize()                    # the copy before has read the pinned piece (long ago)
        host = self._rows_pinned.numpy()
        host[:2 * n].view(np.int64)[:] = request_keys          # (first: 8-byte aligned)
        host[2 * n:3 * n].view(np.float32)[:] = [p.temperature for p in params]
        host[3 * n:4 * n].view(np.float32)[:] = [p.top_p for p in params]
        host[4 * n:5 * n] = [p.top_k for p in params]
        host[5 * n:6 * n] = steps
        dev = self._rows_device
        dev[:6 * n].copy_(self._rows_pinned[:6 * n], non_blocking=True)
        self._rows_copied.record()
        return (dev[2 * n:3 * n].view(torch.float32), dev[4 * n:5 * n], dev[3 * n:4 * n].view(torch.float32),
                dev[:2 * n].view(torch.int64), dev[5 * n:6 * n])

    def sample(self, logits: torch.Tensor, params: list, request_keys: list, steps: list) -> list:
        """The n token ids, waited for."""
        return self.launch(logits, params, request_keys, steps).result()
