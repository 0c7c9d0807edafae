"""Continuous batching with a token budget, prompt portions and recompute preemption.

The decisions follow pagedllm/scheduler.py:53-187:

* One step has ``max_num_batched_tokens`` tokens to give.  Running requests come first, in the
  order they were admitted: a decoding request takes one token, a request in the middle of its
  prompt takes as much of the rest as the budget allows (if portions are enabled; otherwise it
  waits for a step with room).
* **When pages run out** for a running request, the request admitted last is preempted: its
  pages and state slot are given back, its generated tokens are kept, and it returns to the
  head of the waiting queue to be recomputed as a longer prompt.  Victims are always at or
  behind the current request, so nothing already scheduled in this step is undone.  If the
  victim is the request itself, it simply does not run this step.
* Then waiting requests are admitted first-in first-out while budget, request slots and pages
  last; a reusable prefix is looked up first.  The first request that does not fit stops
  admission (no skipping ahead).
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

from ..cache.block_manager import CacheManager
from ..config.engine_config import EngineConfig
from .request import Request, RequestStatus


@dataclass
class ScheduledRequest:
    request: Request
    num_new_tokens: int
    # Decided when scheduled: this step computes the last known token, so its logits are sampled.
    needs_sampling: bool = field(init=False)

    def __post_init__(self) -> None:
        self.needs_sampling = self.request.num_computed_tokens + self.num_new_tokens == self.request.num_tokens

    @property
    def seq(self) -> Request:        # the reference's name
        return self.request


@dataclass
class SchedulerOutput:
    scheduled: list = field(default_factory=list)
    preempted: list = field(default_factory=list)
    num_prefill_tokens: int = 0
    num_decode_tokens: int = 0

    @property
    def is_empty(self) -> bool:
        return not self.scheduled

    @property
    def total_tokens(self) -> int:
        return self.num_prefill_tokens + self.num_decode_tokens


class Scheduler:
    def __init__(self, config: EngineConfig, cache_manager: CacheManager, eos_token_id=None):
        self.config = config
        self.cm = cache_manager
        if eos_token_id is None:
            self.eos_ids: frozenset = frozenset()
        elif isinstance(eos_token_id, (list, tuple, set, frozenset)):
            self.eos_ids = frozenset(int(t) for t in eos_token_id)
        else:
            self.eos_ids = frozenset([int(eos_token_id)])
        self.waiting: deque = deque()
        self.running: list = []
        self.finished: list = []
        self.num_preemptions = 0

    # ------------------------------------------------------------------ queues
    def add(self, req: Request) -> None:
        cfg = self.config
        if req.num_prompt_tokens >= cfg.max_model_len:
            raise ValueError(f"prompt has {req.num_prompt_tokens} tokens, max_model_len={cfg.max_model_len}")
        if not cfg.enable_chunked_prefill and req.num_prompt_tokens > cfg.max_num_batched_tokens:
            raise ValueError("prompt longer than max_num_batched_tokens; enable chunked prefill")
        if req.num_prompt_tokens + req.max_tokens > cfg.max_model_len:
            req.max_tokens = max(1, cfg.max_model_len - req.num_prompt_tokens)
        req.status = RequestStatus.WAITING
        self.waiting.append(req)

    def abort(self, request_id: int) -> None:
        for queue in (self.waiting, self.running):
            for req in list(queue):
                if req.request_id == request_id:
                    queue.remove(req)
                    self.cm.free(req.request_id)
                    req.status = RequestStatus.FINISHED_ABORTED
                    self.finished.append(req)
                    return

    @property
    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    @property
    def num_unfinished(self) -> int:
        return len(self.waiting) + len(self.running)

    # ------------------------------------------------------------------ one step's plan
    def _preempt(self, victim: Request, out: SchedulerOutput) -> None:
        self.running.remove(victim)
        self.cm.free(victim.request_id)
        victim.reset_for_recompute()
        self.waiting.appendleft(victim)
        out.preempted.append(victim)
        self.num_preemptions += 1

    def schedule(self) -> SchedulerOutput:
        out = SchedulerOutput()
        budget = self.config.max_num_batched_tokens
        portions = self.config.enable_chunked_prefill

        for req in list(self.running):
            if budget == 0:
                break
            if req.status is not RequestStatus.RUNNING:      # preempted earlier in this step
                continue
            n = req.num_uncomputed_tokens
            assert n >= 1
            if n > budget:
                if not portions:
                    continue
                n = budget
            while not self.cm.allocate(req.request_id, req.num_computed_tokens, n):
                victim = self.running[-1]
                self._preempt(victim, out)
                if victim is req:
                    break
            if req.status is not RequestStatus.RUNNING:
                continue
            budget -= n
            out.scheduled.append(ScheduledRequest(req, n))
            if req.is_prefill_done:
                out.num_decode_tokens += n
            else:
                out.num_prefill_tokens += n

        while self.waiting and budget > 0 and len(self.running) < self.config.max_num_seqs:
            req = self.waiting[0]
            hits, num_cached = self.cm.find_cached_prefix(req.token_ids)
            n = req.num_tokens - num_cached
            assert n >= 1
            if n > budget:
                if not portions:
                    break
                n = budget
            if not self.cm.allocate(req.request_id, num_cached, n, hits):
                break
            self.waiting.popleft()
            req.num_computed_tokens = num_cached
            req.num_cached_tokens = num_cached
            req.status = RequestStatus.RUNNING
            self.running.append(req)
            budget -= n
            out.scheduled.append(ScheduledRequest(req, n))
            out.num_prefill_tokens += n
        return out

    # ------------------------------------------------------------------ after the forward pass
    def update(self, out: SchedulerOutput, sampled: dict) -> list:
        """Advance what is computed, append sampled tokens, retire finished requests
        (pagedllm/scheduler.py:161-187).  ``sampled`` maps request id -> token for every
        scheduled request with ``needs_sampling``."""
        done = []
        for item in out.scheduled:
            req = item.request
            before = req.num_computed_tokens
            req.num_computed_tokens += item.num_new_tokens
            self.cm.note_computed(req.request_id, req.token_ids, before, req.num_computed_tokens)
            if not item.needs_sampling:
                continue
            token = int(sampled[req.request_id])
            req.token_ids.append(token)
            sp = req.sampling_params
            if (not sp.ignore_eos and token in self.eos_ids) or token in sp.stop_token_ids:
                req.status = RequestStatus.FINISHED_STOPPED
            elif req.num_generated_tokens >= req.max_tokens or req.num_tokens >= self.config.max_model_len:
                req.status = RequestStatus.FINISHED_LENGTH
            if req.is_finished:
                self.running.remove(req)
                self.cm.free(req.request_id)
                done.append(req)
        self.finished.extend(done)
        return done
