"""LLMEngine: the entry point.  A model folder in, generated tokens out.

The public face is the reference's (pagedllm/engine.py:105-234): ``LLMEngine(model, config, **overrides)``,
``generate``, ``add_request``, ``step``, ``abort_request``, ``has_unfinished_requests``, ``stats``, and the
fields of ``RequestOutput`` / ``StepOutput`` / ``EngineStats``.  Behind it one step is: the scheduler's plan
-> entries for the step function -> logits of the rows to sample from -> the sampler -> the plan committed.
"""

from __future__ import annotations

import gc
import logging
import os
import time
from dataclasses import dataclass, field

from ..config.engine_config import EngineConfig
from ..config.registry import read_config_json
from ..sampling.sampler import Sampler
from .batch import StepEntry
from .loading import build_model, build_runtime, load_model, require_gpu
from .pool_sizing import pages_that_fit
from .request import Request, SamplingParams
from .scheduler import Scheduler, StepPlan

log = logging.getLogger("paged_llm_amd")


@dataclass
class StepOutput:
    seq_id: int
    new_token: int | None
    finished: bool


@dataclass
class RequestOutput:
    seq_id: int
    prompt_token_ids: list
    token_ids: list            # generated tokens only
    text: str
    finish_reason: str
    num_cached_tokens: int
    num_preemptions: int


@dataclass
class EngineStats:
    num_steps: int = 0
    num_prefill_tokens: int = 0
    num_decode_tokens: int = 0
    num_preemptions: int = 0
    num_dropped_tokens: int = 0        # computed in a step that ran ahead for requests that had ended meanwhile
    step_times: list = field(default_factory=list)

    def count(self, plan: StepPlan, seconds: float, dropped: int = 0) -> None:
        """``dropped``: decoded tokens of the plan that were computed for requests that had ended meanwhile."""
        self.num_steps += 1
        self.num_prefill_tokens += plan.prompt_tokens
        self.num_decode_tokens += plan.decode_tokens - dropped
        self.num_dropped_tokens += dropped
        self.num_preemptions += len(plan.preempted)
        self.step_times.append(seconds)


def _tokenizer_of(folder: str):
    """The folder's tokenizer.json, if it has one; prompts given as token ids need none."""
    path = os.path.join(folder, "tokenizer.json")
    if not os.path.isfile(path):
        return None
    from tokenizers import Tokenizer
    return Tokenizer.from_file(path)


_static_heap_frozen = False


def _freeze_static_heap() -> None:
    """What exists before the first engine of a process is built (the tensor library and everything else that was
    imported: a million objects or so) lives as long as the process does.  Taken out of the garbage collector's
    generations, it is no longer walked by every full collection; such a collection then costs what the engine's and the
    live requests' objects cost (at 512 requests a pause of 50 ms every few dozen steps became one of 5 ms: 7.9 -> 6.6 ms a
    step on average).  Once per process, and before the engine's own objects exist: an engine that is dropped later is
    collected as ever."""
    global _static_heap_frozen
    if not _static_heap_frozen:
        gc.collect()
        gc.freeze()
        _static_heap_frozen = True


def _shared_model(held, hf_config: dict, cfg: EngineConfig, device):
    """``held`` (another engine's model) if it is the model that ``hf_config`` and ``cfg`` ask for; else one error
    that says what differs."""
    from ..config.dtypes import resolve_dtype
    from ..config.registry import lookup_architecture
    arch = lookup_architecture(hf_config)
    spec = arch.build_spec(arch.read_config(hf_config))
    problems = []
    if spec != held.spec:
        problems.append("the folder's config.json describes another model")
    else:
        wanted = resolve_dtype(cfg.dtype, spec.stored_dtype)
        if wanted != held.dtype:
            problems.append(f"it computes in {held.dtype}, this engine is to compute in {wanted}")
        if max(spec.max_positions, cfg.max_model_len or 0) > held.max_positions:
            problems.append(f"it covers {held.max_positions} positions, this engine needs {max(spec.max_positions, cfg.max_model_len or 0)}")
    if held.device != device:
        problems.append(f"it lives on {held.device}, this engine on {device}")
    if problems:
        raise ValueError("the other engine's weights cannot be shared: " + "; ".join(problems))
    return held


class LLMEngine:
    freeze_static_heap = True          # False: the garbage collector keeps walking everything that was imported
    def __init__(self, model: str, config: EngineConfig | None = None, **overrides):
        """``model``: a folder with config.json and *.safetensors.  ``random_weights=SEED`` among
        the overrides fills the model of that folder's config.json with seeded random weights
        instead of reading tensors.  ``weights_of=ENGINE`` runs on the weights that another engine of the same
        config.json, compute type and device holds already (a second cache, scheduler and set of graphs over one
        model in memory); that engine's model must cover this one's positions."""
        seed_for_weights = overrides.pop("random_weights", None)
        weights_of = overrides.pop("weights_of", None)
        self.config = cfg = config or EngineConfig(**overrides)
        self.device = require_gpu(cfg.device)
        if self.freeze_static_heap:
            _freeze_static_heap()
        if not os.path.isdir(model):
            raise FileNotFoundError(f"{model!r} is no folder (models are not downloaded)")
        self.tokenizer = _tokenizer_of(model)
        started = time.perf_counter()
        if weights_of is not None:
            self.model = _shared_model(weights_of.model, read_config_json(model), cfg, self.device)
        elif seed_for_weights is None:
            self.model = load_model(model, cfg.dtype, self.device, cfg.max_model_len)
        else:
            from ..weights.random_init import fill_random
            self.model = build_model(read_config_json(model), cfg.dtype, self.device, cfg.max_model_len)
            fill_random(self.model, int(seed_for_weights))
        self.dtype = self.model.dtype
        self.attention_backend = "hip"       # the one there is; shown where the reference shows its backend's name
        log.info("model %s ready after %.1f s, computing in %s", model, time.perf_counter() - started, self.dtype)

        pages = cfg.num_gpu_blocks or pages_that_fit(self.model, cfg)
        self.cache_manager, self.kv_cache, self.runner = build_runtime(
            self.model, cfg.block_size, pages, cfg.max_num_seqs, cfg.enable_prefix_caching, use_graphs=cfg.enable_hip_graphs)
        self.groups = list(self.cache_manager.groups)
        self.scheduler = Scheduler(cfg, self.cache_manager, self.model.spec.eos_token_id)
        self.sampler = Sampler(cfg.seed, self.device)
        self.stats = EngineStats()
        self._live: dict[int, Request] = {}          # requests that have not ended
        # Called, if set, before every sampling with (requests, logits): the requests whose next token is about
        # to be drawn, in the order of the float logits' rows [n, vocab]; row i is the distribution behind
        # position len(requests[i].tokens) - 1.  The tensor is only valid during the call.
        self.on_logits = None
        # A step that is launched and sampled but not committed yet: (plan, requests of the sampled rows, pending tokens).
        self._flight = None
        # Launch the step after the one under way before waiting for its tokens (see ``_advance``); off: one step at a time.
        self.run_ahead = True
        # Prompt portions of at least this many tokens have the digests of their pages made while the GPU computes them.
        self.digests_ahead_from = 4 * cfg.block_size
        log.info("cache: %d pages of %d positions per group (%d positions, %.2f GiB)", pages, cfg.block_size,
                 pages * cfg.block_size, self.kv_cache.total_bytes() / 2**30)

    # ------------------------------------------------------------------ requests
    def _token_ids(self, prompt) -> list:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("text prompts need a tokenizer.json in the model folder; pass token ids instead")
            return self.tokenizer.encode(prompt).ids
        ids = [int(t) for t in prompt]
        vocab = self.model.spec.vocab_size
        if any(not 0 <= t < vocab for t in ids):
            raise ValueError(f"prompt holds a token id outside [0, {vocab})")
        return ids

    def _new_request(self, prompt, sampling_params: SamplingParams | None) -> Request:
        request = Request(self._token_ids(prompt), sampling_params)
        self.scheduler.submit(request)
        self._live[request.id] = request
        return request

    def add_request(self, prompt, sampling_params: SamplingParams | None = None) -> int:
        return self._new_request(prompt, sampling_params).id

    def abort_request(self, seq_id: int) -> None:
        if self.scheduler.cancel(seq_id) is not None:
            self._live.pop(seq_id, None)

    @property
    def has_unfinished_requests(self) -> bool:
        return not self.scheduler.idle

    @property
    def step_in_flight(self) -> bool:
        """A step has been launched beyond the last committed one (see ``_advance``): the next ``step()`` commits it,
        whatever has arrived or been cancelled since."""
        return self._flight is not None and not all(g.request.ended for g in self._flight[0].grants)

    # ------------------------------------------------------------------ one step
    def _entry(self, grant) -> StepEntry:
        request = grant.request
        first = request.computed
        tables, slot, version = self.cache_manager.step_fields(request.id)
        if len(tables) != len(self.groups):                      # (groups in the order the step function knows them)
            tables = {g: tables[g] for g in self.groups}
        return StepEntry(request.id, request.tokens[first:first + grant.count], first, tables, slot,
                         [grant.count - 1] if grant.samples else [], version)

    def _sample(self, logits, grants: list):
        """Queues the sampling of the grants whose last row was asked for; (requests in the order of the rows, pending
        tokens).  Rows of requests that ended while the step was already running are sampled with the others and
        dropped when the step is committed; the ``on_logits`` hook does not see them."""
        chosen = [g.request for g in grants if g.samples]
        rows = logits[: len(chosen)]
        if self.on_logits is not None and chosen:
            live = [i for i, r in enumerate(chosen) if not r.ended]
            if len(live) == len(chosen):
                self.on_logits(chosen, rows)
            elif live:
                self.on_logits([chosen[i] for i in live], rows[live])
        pending = self.sampler.launch(rows, [r.params for r in chosen], [r.id for r in chosen], [r.num_generated for r in chosen])
        return chosen, pending

    def _launch(self, plan: StepPlan):
        """Queues the step of ``plan`` from the tokens the requests hold; the step's logits."""
        cm = self.cache_manager
        state_copies = cm.take_pending_state_copies() if cm.uses_state else None
        return self.runner.step([self._entry(g) for g in plan.grants], cm.take_pending_copies(), borrow=True, state_copies=state_copies)

    def _launch_ahead(self, plan: StepPlan, pending):
        """While the GPU runs ``plan`` and its sampling: the step after it, queued behind them with the sampled ids
        taken where the sampling kernel leaves them on the GPU, so that the GPU goes from one step into the next
        without waiting for the host to see the tokens (see ``Scheduler.plan_ahead`` for when that is possible;
        the step's graph must exist already).  (the next plan, its logits), or None."""
        if not self.run_ahead or pending.on_device is None:
            return None
        ahead = self.scheduler.plan_ahead(plan)
        if ahead is None:
            return None
        cm = self.cache_manager
        # (the grants of ``ahead`` are those of ``plan`` in the same order, without the requests that reach their limit: one
        #  walk over both; with hundreds of requests this loop is most of the host's part of a step, so it is kept lean.
        #  A request's state of fixed size moves once per step, in the order of the steps on the stream, whoever launched
        #  them; the state of a request that ends in ``plan`` is moved once more in its freed slot, which the next owner's
        #  first step clears.)
        entries, rows = [], []
        fields, groups = cm.step_fields, self.groups
        source = iter(enumerate(plan.grants))                  # every grant of ``plan`` samples: row i
        for then in ahead.grants:
            request = then.request
            for row, grant in source:
                if grant.request is request:
                    break
            tables, slot, version = fields(request.id)
            if len(tables) != len(groups):                       # (groups in the order the step function knows them)
                tables = {g: tables[g] for g in groups}
            rows.append(row)
            entries.append(StepEntry(request.id, [0], request.computed + grant.count, tables, slot, [0], version))
        staged = self.runner.prepare(entries)
        if staged is None:
            return None                                      # (the pages taken for the next tokens stay with their requests)
        take = None if len(rows) == len(plan.grants) else rows    # (some reach their limit in ``plan``: their rows are left out)
        return ahead, self.runner.run_prepared(staged, pending.on_device, cm.take_pending_copies(), borrow=True, take=take)

    def _advance(self):
        """Commits one step.  (the grants it commits, sampled tokens by request id, requests that ended); no grants
        when there is nothing to do.

        One step may be under way beyond the committed one: a step is launched together with its sampling, and
        before the host waits for the sampled ids it launches the step after, if that one can be foreseen.  When the
        ids arrive the step is committed; a request that ends there (an end-of-sequence token, a cancellation) is
        dropped from the step that is already running, whose other rows are as good as ever."""
        started = time.perf_counter()
        flight, self._flight = self._flight, None
        if flight is not None and all(g.request.ended for g in flight[0].grants):
            flight = None                                    # everybody in it was cancelled meanwhile: nothing to commit
        if flight is None:
            plan = self.scheduler.plan()
            if not plan:
                if not self.scheduler.idle:
                    raise RuntimeError("no request can run: " + self.scheduler.why_stuck())
                return [], {}, []
            # The sampler runs at once, so the step may hand out its graph's own logits buffer.
            chosen, pending = self._sample(self._launch(plan), plan.grants)
        else:
            plan, chosen, pending = flight
        ahead = self._launch_ahead(plan, pending)            # the GPU's next millisecond, queued before the host waits
        if plan.prompt_tokens >= self.digests_ahead_from:    # (page digests of long portions: made while the GPU runs)
            for g in plan.grants:
                if g.count >= self.digests_ahead_from:
                    self.cache_manager.digests_ahead(g.request.id, g.request.tokens, g.request.computed + g.count)
        sampled = {r.id: t for r, t in zip(chosen, pending.result())}
        committed = [g for g in plan.grants if not g.request.ended]      # (the others ended while this step already ran)
        ended = self.scheduler.commit(plan, sampled)
        for request in ended:
            self._live.pop(request.id, None)
        if ahead is not None:
            next_plan, logits = ahead
            if any(not g.request.ended for g in next_plan.grants):
                self._flight = (next_plan, *self._sample(logits, next_plan.grants))
        self.stats.count(plan, time.perf_counter() - started, dropped=len(plan.grants) - len(committed))
        return committed, sampled, ended

    def step(self) -> list:
        grants, sampled, ended = self._advance()
        done = {r.id for r in ended}
        return [StepOutput(g.request.id, sampled.get(g.request.id) if g.samples else None, g.request.id in done) for g in grants]

    # ------------------------------------------------------------------ whole requests
    def _output(self, request: Request) -> RequestOutput:
        generated = request.generated
        text = self.tokenizer.decode(generated, skip_special_tokens=True) if self.tokenizer is not None else ""
        return RequestOutput(request.id, request.prompt, generated, text, request.end_reason.value, request.reused_prefix,
                             request.times_preempted)

    def generate(self, prompts: list, sampling_params=None, use_tqdm: bool = False) -> list:
        """Runs the prompts to their ends; outputs in the order of the prompts."""
        if isinstance(sampling_params, list):
            if len(sampling_params) != len(prompts):
                raise ValueError(f"{len(sampling_params)} sampling_params for {len(prompts)} prompts")
            per_prompt = sampling_params
        else:
            per_prompt = [sampling_params or SamplingParams()] * len(prompts)
        mine = [self._new_request(p, sp) for p, sp in zip(prompts, per_prompt)]
        waiting_for = {r.id for r in mine}
        progress = None
        if use_tqdm:
            from tqdm import tqdm
            progress = tqdm(total=len(mine), desc="requests")
        while waiting_for:
            _, _, ended = self._advance()
            mine_ended = sum(1 for r in ended if r.id in waiting_for)
            waiting_for.difference_update(r.id for r in ended)
            if progress is not None and mine_ended:
                progress.update(mine_ended)
        if progress is not None:
            progress.close()
        return [self._output(r) for r in mine]
