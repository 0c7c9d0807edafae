"""Sampling options of a request and the request's own bookkeeping.

``SamplingParams`` keeps the reference's option names and meanings (pagedllm/sequence.py:9-20), since
they are what a caller writes.  ``Request`` is this engine's record of one request: one growing token
list with the prompt's length beside it, a count of the tokens whose keys and values are in the cache,
and a life cycle of three stages with the reason of the end kept apart.
"""

from __future__ import annotations

import threading
import time
from dataclasses import dataclass
from enum import Enum


@dataclass
class SamplingParams:
    temperature: float = 1.0
    top_p: float = 1.0
    top_k: int = -1
    max_tokens: int = 128
    ignore_eos: bool = False
    stop_token_ids: tuple = ()

    @property
    def greedy(self) -> bool:
        return self.temperature < 1e-5


class Stage(Enum):
    QUEUED = "queued"        # waits for admission (new, or preempted and to be recomputed)
    ACTIVE = "active"        # holds pages; runs whenever the budget reaches it
    ENDED = "ended"


class EndReason(Enum):
    """Why a request ended; the values are what ``RequestOutput.finish_reason`` shows."""
    STOP = "stop"            # end-of-sequence or one of its stop tokens
    LENGTH = "length"        # its own limit of new tokens, or the engine's limit of positions
    ABORT = "abort"


class _Serial:
    """Request ids: consecutive integers, safe to draw from several threads."""

    def __init__(self):
        self._next, self._lock = 0, threading.Lock()

    def draw(self) -> int:
        with self._lock:
            self._next += 1
            return self._next - 1


_serial = _Serial()


class Request:
    """One request from arrival to its end.

    ``tokens`` holds the prompt followed by what has been generated; the first ``computed`` of them have
    their keys and values in the cache.  A decoding request therefore has exactly one token to run
    (the one sampled last), a request in the middle of its prompt has more, and a preempted one starts
    again from zero with its generated tokens as part of a longer prompt.
    """

    __slots__ = ("id", "params", "tokens", "prompt_len", "computed", "reused_prefix", "times_preempted", "new_token_limit",
                 "stage", "end_reason", "arrived")

    def __init__(self, prompt, params: SamplingParams | None = None, request_id: int | None = None):
        tokens = [int(t) for t in prompt]
        if not tokens:
            raise ValueError("a request needs at least one prompt token")
        self.id = _serial.draw() if request_id is None else request_id
        self.params = params or SamplingParams()
        self.tokens = tokens
        self.prompt_len = len(tokens)
        self.computed = 0
        self.reused_prefix = 0                  # tokens found in the prefix index at the last admission
        self.times_preempted = 0
        # The limit in force may be lowered at admission; it lives here because callers share SamplingParams objects.
        self.new_token_limit = self.params.max_tokens
        self.stage = Stage.QUEUED
        self.end_reason: EndReason | None = None
        self.arrived = time.perf_counter()

    # ---- what it holds
    @property
    def prompt(self) -> list:
        return self.tokens[: self.prompt_len]

    @property
    def generated(self) -> list:
        return self.tokens[self.prompt_len:]

    @property
    def num_generated(self) -> int:
        return len(self.tokens) - self.prompt_len

    @property
    def backlog(self) -> int:
        """Known tokens that have not been run yet."""
        return len(self.tokens) - self.computed

    @property
    def decoding(self) -> bool:
        """Its prompt is in the cache; what it runs now are generated tokens."""
        return self.computed >= self.prompt_len

    @property
    def ended(self) -> bool:
        return self.stage is Stage.ENDED

    # ---- transitions
    def admit(self, reused_prefix: int) -> None:
        self.stage = Stage.ACTIVE
        self.computed = self.reused_prefix = reused_prefix

    def back_to_queue(self) -> None:
        """Preempted: what it had in the cache is gone, what it generated stays, so it will be
        recomputed as a longer prompt (recompute preemption, pagedllm/sequence.py:101-106)."""
        self.stage = Stage.QUEUED
        self.computed = 0
        self.times_preempted += 1

    def end(self, reason: EndReason) -> None:
        self.stage = Stage.ENDED
        self.end_reason = reason

    def __repr__(self) -> str:
        return (f"Request(id={self.id}, {self.stage.value}, prompt={self.prompt_len}, generated={self.num_generated}, "
                f"computed={self.computed})")
