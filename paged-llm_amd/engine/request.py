"""A request and its sampling options (names and meanings as in pagedllm/sequence.py:9-112)."""

from __future__ import annotations

import itertools
import time
from dataclasses import dataclass, field
from enum import Enum, auto


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


class RequestStatus(Enum):
    WAITING = auto()
    RUNNING = auto()
    FINISHED_STOPPED = auto()   # end-of-sequence or a stop token
    FINISHED_LENGTH = auto()    # max_tokens or max_model_len reached
    FINISHED_ABORTED = auto()

    @property
    def finished(self) -> bool:
        return self in (RequestStatus.FINISHED_STOPPED, RequestStatus.FINISHED_LENGTH, RequestStatus.FINISHED_ABORTED)


_ids = itertools.count()


@dataclass(eq=False)
class Request:
    """``token_ids`` = prompt + generated so far; the first ``num_computed_tokens`` of them have
    their keys and values in the cache.  A fresh request has 0 there (or the length of a reused
    prefix); a decoding one has len(token_ids) - 1."""

    prompt_token_ids: list
    sampling_params: SamplingParams = field(default_factory=SamplingParams)
    request_id: int = field(default_factory=lambda: next(_ids))
    token_ids: list = field(init=False)
    status: RequestStatus = RequestStatus.WAITING
    num_computed_tokens: int = 0
    arrival_time: float = field(default_factory=time.perf_counter)
    # The effective output limit lives here, not in the (possibly shared) SamplingParams object.
    max_tokens: int = field(init=False)
    num_cached_tokens: int = 0      # prefix reuse at the last admission
    num_preemptions: int = 0

    def __post_init__(self) -> None:
        if not self.prompt_token_ids:
            raise ValueError("empty prompt")
        self.prompt_token_ids = [int(t) for t in self.prompt_token_ids]
        self.token_ids = list(self.prompt_token_ids)
        self.max_tokens = self.sampling_params.max_tokens

    @property
    def seq_id(self) -> int:          # the reference's name for the id
        return self.request_id

    @property
    def num_prompt_tokens(self) -> int:
        return len(self.prompt_token_ids)

    @property
    def num_tokens(self) -> int:
        return len(self.token_ids)

    @property
    def num_generated_tokens(self) -> int:
        return len(self.token_ids) - len(self.prompt_token_ids)

    @property
    def num_uncomputed_tokens(self) -> int:
        return len(self.token_ids) - self.num_computed_tokens

    @property
    def output_token_ids(self) -> list:
        return self.token_ids[len(self.prompt_token_ids):]

    @property
    def is_finished(self) -> bool:
        return self.status.finished

    @property
    def is_prefill_done(self) -> bool:
        return self.num_computed_tokens >= self.num_prompt_tokens

    def reset_for_recompute(self) -> None:
        """Preempted: the cache content is dropped, generated tokens stay, so the request comes
        back as a longer prompt (pagedllm/sequence.py:101-106)."""
        self.num_computed_tokens = 0
        self.status = RequestStatus.WAITING
        self.num_preemptions += 1
