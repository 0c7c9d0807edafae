"""Continuous batching: which requests run how many tokens in the next step.

The policy is the reference's (pagedllm/scheduler.py:53-187); the shape is this engine's: a step's plan
is made in two passes over one token budget, each pass a method of its own, and committed after the
forward pass.

1. **Active requests**, in the order they were admitted.  A decoding request asks for one token, a
   request inside its prompt for the rest of it; a request that asks for more than the budget has
   left takes what is left (a *portion*) if portions are enabled, else it sits this step out.
2. **Queued requests**, first in first out, while budget, request slots, pages and state slots last.
   The prefix index is asked first, so a request may start behind tokens that are already cached.
   The first request that does not fit ends the pass: nobody overtakes it.

**When pages run out** for an active request, the request admitted last gives up everything it holds
and goes back to the *front* of the queue with its generated tokens kept; it is recomputed later as a
longer prompt.  Victims are at or behind the asking request in admission order, so nothing planned
earlier in the same step is undone; a request that is its own victim just does not run this step.

A preempted request may have grown beyond the whole budget of a step.  With portions disabled it could
then never run again, so a request that exceeds the *whole* budget is always split, whatever the option
says (the option still keeps every prompt that fits in one step in one step).
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

from ..cache.block_manager import CacheManager
from ..config.engine_config import EngineConfig
from .request import EndReason, Request, Stage


@dataclass
class Grant:
    """One request's share of a step: its next ``count`` tokens."""
    request: Request
    count: int
    # Known when granted: the step reaches the request's last known token, so its logits are sampled from.
    samples: bool


@dataclass
class StepPlan:
    grants: list = field(default_factory=list)
    preempted: list = field(default_factory=list)
    prompt_tokens: int = 0
    decode_tokens: int = 0

    def __bool__(self) -> bool:
        return bool(self.grants)

    def add(self, request: Request, count: int) -> None:
        self.grants.append(Grant(request, count, request.computed + count == len(request.tokens)))
        if request.decoding:
            self.decode_tokens += count
        else:
            self.prompt_tokens += count


def _as_id_set(eos) -> frozenset:
    if eos is None:
        return frozenset()
    if isinstance(eos, (list, tuple, set, frozenset)):
        return frozenset(int(t) for t in eos)
    return frozenset((int(eos),))


class Scheduler:
    def __init__(self, config: EngineConfig, cache: CacheManager, eos_token_id=None):
        self.step_budget = config.max_num_batched_tokens
        self.max_active = config.max_num_seqs
        self.max_positions = config.max_model_len
        self.portions = config.enable_chunked_prefill
        self.cache = cache
        self.eos_ids = _as_id_set(eos_token_id)
        self.queue: deque = deque()          # Stage.QUEUED, the next to admit at the left
        self.active: list = []               # Stage.ACTIVE, in admission order
        self.num_preemptions = 0

    # ------------------------------------------------------------------ arrivals and departures
    def submit(self, request: Request) -> None:
        """Checks a new request against the engine's limits and queues it."""
        if request.prompt_len >= self.max_positions:
            raise ValueError(f"a prompt of {request.prompt_len} tokens leaves no room to generate within "
                             f"max_model_len={self.max_positions}")
        if not self.portions and request.prompt_len > self.step_budget:
            raise ValueError(f"a prompt of {request.prompt_len} tokens does not fit one step of max_num_batched_tokens="
                             f"{self.step_budget}, and enable_chunked_prefill is off")
        room = self.max_positions - request.prompt_len
        if request.new_token_limit > room:
            request.new_token_limit = max(1, room)
        request.stage = Stage.QUEUED
        self.queue.append(request)

    def cancel(self, request_id) -> Request | None:
        """Ends a queued or active request at once; returns it, or None if it is not here."""
        for request in (*self.queue, *self.active):
            if request.id == request_id:
                (self.queue if request.stage is Stage.QUEUED else self.active).remove(request)
                self._retire(request, EndReason.ABORT)
                return request
        return None

    @property
    def idle(self) -> bool:
        return not self.queue and not self.active

    def __len__(self) -> int:
        return len(self.queue) + len(self.active)

    def _retire(self, request: Request, reason: EndReason) -> None:
        self.cache.free(request.id)
        request.end(reason)

    # ------------------------------------------------------------------ planning a step
    def plan(self) -> StepPlan:
        plan = StepPlan()
        left = self._serve_active(plan, self.step_budget)
        self._admit_queued(plan, left)
        return plan

    def _share(self, wanted: int, left: int) -> int:
        """How many of ``wanted`` tokens a request gets from a budget with ``left`` tokens: all of
        them, a portion, or none (0)."""
        if wanted <= left:
            return wanted
        if self.portions or wanted > self.step_budget:
            return left
        return 0

    def _serve_active(self, plan: StepPlan, left: int) -> int:
        for request in list(self.active):
            if left == 0:
                break
            if request.stage is not Stage.ACTIVE:            # gave way to an earlier request in this pass
                continue
            count = self._share(request.backlog, left)
            if count == 0:
                continue
            if not self._pages_or_preempt(request, count, plan):
                continue
            left -= count
            plan.add(request, count)
        return left

    def _pages_or_preempt(self, request: Request, count: int, plan: StepPlan) -> bool:
        """Pages for the request's next ``count`` tokens, taken from the requests admitted last if need
        be.  False when the request itself had to give way."""
        while not self.cache.allocate(request.id, request.computed, count):
            victim = self.active.pop()
            self.cache.free(victim.id)
            victim.back_to_queue()
            self.queue.appendleft(victim)
            plan.preempted.append(victim)
            self.num_preemptions += 1
            if victim is request:
                return False
        return True

    def _admit_queued(self, plan: StepPlan, left: int) -> int:
        while self.queue and left > 0 and len(self.active) < self.max_active:
            request = self.queue[0]
            pages, reused = self.cache.find_cached_prefix(request.tokens)
            count = self._share(len(request.tokens) - reused, left)
            if count == 0 or not self.cache.allocate(request.id, reused, count, pages):
                break
            self.queue.popleft()
            request.admit(reused)
            self.active.append(request)
            left -= count
            plan.add(request, count)
        return left

    def plan_ahead(self, plan: StepPlan) -> StepPlan | None:
        """The plan of the step after ``plan``, made while ``plan`` still runs (its sampled tokens are not known yet), so
        that the step after can be launched before the host has seen them.  Only the steady state is foreseen: every
        active request is in ``plan`` and reaches its last known token there, nobody waits in the queue (or every
        place stays taken, so that nobody can be admitted: a place that an end-of-sequence token frees in ``plan``
        is then filled one step later than it could be), and a page for everybody's next token is there without
        taking anybody's.  Then the next plan is one token for each of
        them, in the same order, but for those that reach their limit of new tokens or of positions in ``plan``: they
        end there, whatever they sample.  None otherwise, or when nobody is left.  A request that ends in ``plan`` for
        another reason (an end-of-sequence token) is passed over when the plan made here is committed."""
        if plan.preempted or len(plan.grants) != len(self.active) or len(self.active) > self.step_budget:
            return None
        if not all(grant.samples for grant in plan.grants):
            return None
        most = self.max_positions
        ends = [r.num_generated + 1 >= r.new_token_limit or len(r.tokens) + 1 >= most for r in (grant.request for grant in plan.grants)]
        if self.queue and len(ends) - sum(ends) < self.max_active:
            return None                       # a place comes free (or is free): the next plan may admit somebody
        ahead = StepPlan()
        for grant, at_limit in zip(plan.grants, ends):
            request = grant.request
            if at_limit:
                continue                      # its last token comes from ``plan``
            if not self.cache.allocate(request.id, request.computed + grant.count, 1):
                return None                   # (pages taken for the others so far are the ones their next step takes anyway)
            ahead.grants.append(Grant(request, 1, True))
        ahead.decode_tokens = len(ahead.grants)
        return ahead if ahead.grants else None

    def why_stuck(self) -> str:
        """Says why an empty plan came out although requests remain (for the caller's error)."""
        if not self.queue:
            return "no request is queued"
        request = self.queue[0]
        need = self.cache.pages_for(min(len(request.tokens), self.step_budget))
        have = self.cache.num_pages()
        if need > have:
            return (f"request {request.id} needs {need} pages of {self.cache.block_size} positions for its next "
                    f"{min(len(request.tokens), self.step_budget)} tokens, the pool holds {have}")
        if self.cache.uses_state and self.cache.slots.num_slots == 0:
            return "the model keeps per-request state and there are no state slots"
        return (f"request {request.id} ({len(request.tokens)} tokens) cannot be admitted with {self.cache.num_free_pages()} "
                f"free pages of {have} and {len(self.active)} active requests")

    # ------------------------------------------------------------------ after the forward pass
    def commit(self, plan: StepPlan, sampled: dict) -> list:
        """Counts the step's tokens as computed, appends the sampled tokens (``sampled``: request id ->
        token for every grant with ``samples``) and ends the requests that are done; returns those.  A grant
        whose request is no longer active (it ended in the step before, which was still running when this one
        was launched, or it was cancelled) is passed over: what the step computed for it is dropped."""
        ended = []
        for grant in plan.grants:
            request = grant.request
            if request.stage is not Stage.ACTIVE:               # ended or cancelled after the step was launched
                continue
            before = request.computed
            request.computed = before + grant.count
            self.cache.note_computed(request.id, request.tokens, before, request.computed)
            if not grant.samples:
                continue
            token = int(sampled[request.id])
            request.tokens.append(token)
            reason = self._end_reason(request, token)
            if reason is not None:
                self.active.remove(request)
                self._retire(request, reason)
                ended.append(request)
        return ended

    def _end_reason(self, request: Request, token: int) -> EndReason | None:
        params = request.params
        if token in params.stop_token_ids or (token in self.eos_ids and not params.ignore_eos):
            return EndReason.STOP
        if request.num_generated >= request.new_token_limit or len(request.tokens) >= self.max_positions:
            return EndReason.LENGTH
        return None
