"""LLMEngine: scheduler + step function + sampler in one loop (pagedllm/engine.py:105-234)."""

from __future__ import annotations

import logging
import os
import time
from dataclasses import dataclass, field

import torch

from ..config.engine_config import EngineConfig
from ..config.registry import read_config_json
from ..sampling.sampler import Sampler
from .batch import StepEntry
from .loading import build_model, build_runtime, load_model, require_gpu
from .request import Request, RequestStatus, SamplingParams
from .scheduler import Scheduler, SchedulerOutput

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
    step_times: list = field(default_factory=list)


def _load_tokenizer(path: str):
    """tokenizer.json of the model folder, if there is one; token-id prompts need none."""
    file = os.path.join(path, "tokenizer.json")
    if not os.path.isfile(file):
        return None
    from tokenizers import Tokenizer
    return Tokenizer.from_file(file)


class LLMEngine:
    def __init__(self, model: str, config: EngineConfig | None = None, **overrides):
        """``model``: a folder with config.json and *.safetensors.  ``random_weights=SEED`` among
        the overrides fills the model of that folder's config.json with seeded random weights
        instead of reading tensors."""
        random_seed = overrides.pop("random_weights", None)
        self.config = cfg = config or EngineConfig(**overrides)
        self.device = require_gpu(cfg.device)
        if not os.path.isdir(model):
            raise FileNotFoundError(f"{model!r} is no folder (models are not downloaded)")
        hf_cfg = read_config_json(model)
        self.tokenizer = _load_tokenizer(model)
        t0 = time.perf_counter()
        if random_seed is None:
            self.model = load_model(model, cfg.dtype, self.device, cfg.max_model_len)
        else:
            from ..weights.random_init import fill_random
            self.model = build_model(hf_cfg, cfg.dtype, self.device, cfg.max_model_len)
            fill_random(self.model, int(random_seed))
        self.dtype = self.model.dtype
        # What runs the attention (the reference reports its backend's name here, pagedllm/engine.py:117-118).
        self.attention_backend = "hip"
        log.info("loaded %s in %.1fs (dtype=%s)", model, time.perf_counter() - t0, self.dtype)

        num_pages = cfg.num_gpu_blocks or self._profile_num_pages()
        self.cache_manager, self.kv_cache, self.runner = build_runtime(
            self.model, cfg.block_size, num_pages, cfg.max_num_seqs, cfg.enable_prefix_caching,
            use_graphs=cfg.enable_hip_graphs)
        self.groups = list(self.cache_manager.groups)
        eos = self.model.spec.eos_token_id
        self.scheduler = Scheduler(cfg, self.cache_manager, eos)
        self.sampler = Sampler(cfg.seed, self.device)
        self.stats = EngineStats()
        self._requests: dict[int, Request] = {}
        log.info("KV cache: %d pages x %d tokens = %d tokens (%.2f GiB)", num_pages, cfg.block_size,
                 num_pages * cfg.block_size, self.kv_cache.total_bytes() / 2**30)

    # ------------------------------------------------------------------ sizing the page pool
    def _bytes_per_page(self) -> int:
        return sum(g.bytes_per_page(self.config.block_size, self.model.dtype) for g in self.model.cache_groups().values())

    def _dummy_forward(self, n_tok: int) -> None:
        """One forward of n_tok tokens against a throw-away cache, to measure the activation peak
        (pagedllm/engine.py:141-159).  Positions stay inside the model's range."""
        cfg = self.config
        n_tok = min(n_tok, self.model.max_positions)
        pages = (n_tok + cfg.block_size - 1) // cfg.block_size
        manager, storage, runner = build_runtime(self.model, cfg.block_size, pages, 1, False)
        assert manager.allocate("probe", 0, n_tok)
        entry = StepEntry("probe", [0] * n_tok, 0, {g: manager.block_table("probe", g) for g in manager.groups},
                          manager.state_slot("probe"), list(range(min(n_tok, cfg.max_num_seqs))))
        runner.step([entry])
        torch.cuda.synchronize(self.device)

    def _profile_num_pages(self) -> int:
        cfg = self.config
        torch.cuda.empty_cache()
        torch.cuda.reset_peak_memory_stats(self.device)
        before = torch.cuda.memory_allocated(self.device)
        self._dummy_forward(cfg.max_num_batched_tokens)
        peak = torch.cuda.max_memory_allocated(self.device)
        torch.cuda.empty_cache()
        free, total = torch.cuda.mem_get_info(self.device)
        held = torch.cuda.memory_allocated(self.device)
        used_by_others = total - free - held
        activation = max(0, peak - before)
        budget = int(total * cfg.gpu_memory_utilization) - used_by_others - held - activation
        pages = budget // max(1, self._bytes_per_page())
        # No request can use more than max_model_len positions; cap what max_num_seqs could ever hold.
        pages = min(pages, cfg.max_num_seqs * ((cfg.max_model_len + cfg.block_size - 1) // cfg.block_size))
        if pages < 16:
            raise RuntimeError(f"not enough GPU memory for the KV cache ({pages} pages); lower "
                               "max_num_batched_tokens or raise gpu_memory_utilization")
        return int(pages)

    # ------------------------------------------------------------------ requests
    def add_request(self, prompt, sampling_params: SamplingParams | None = None) -> int:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("text prompts need a tokenizer.json in the model folder; pass token ids instead")
            ids = self.tokenizer.encode(prompt).ids
        else:
            ids = [int(t) for t in prompt]
        vocab = self.model.spec.vocab_size
        if any(t < 0 or t >= vocab for t in ids):
            raise ValueError(f"prompt holds a token id outside [0, {vocab})")
        req = Request(ids, sampling_params or SamplingParams())
        self.scheduler.add(req)
        self._requests[req.request_id] = req
        return req.request_id

    def abort_request(self, seq_id: int) -> None:
        self.scheduler.abort(seq_id)

    @property
    def has_unfinished_requests(self) -> bool:
        return self.scheduler.has_unfinished

    # ------------------------------------------------------------------ one step
    def _run(self, out: SchedulerOutput) -> dict:
        entries, sampled_items = [], []
        for item in out.scheduled:
            req, n = item.request, item.num_new_tokens
            start = req.num_computed_tokens
            entries.append(StepEntry(
                req.request_id, req.token_ids[start:start + n], start,
                {g: self.cache_manager.block_table(req.request_id, g) for g in self.groups},
                self.cache_manager.state_slot(req.request_id), [n - 1] if item.needs_sampling else [],
                self.cache_manager.table_version(req.request_id)))
            if item.needs_sampling:
                sampled_items.append(req)
        logits = self.runner.step(entries, self.cache_manager.take_pending_copies(), borrow=True)    # sampled from at once
        if not sampled_items:
            return {}
        tokens = self.sampler.sample(logits, [r.sampling_params for r in sampled_items],
                                     [r.request_id for r in sampled_items],
                                     [r.num_generated_tokens for r in sampled_items])
        return {r.request_id: t for r, t in zip(sampled_items, tokens)}

    def step(self) -> list:
        t0 = time.perf_counter()
        out = self.scheduler.schedule()
        if out.is_empty:
            if self.scheduler.has_unfinished:
                raise RuntimeError("nothing can be scheduled: the page pool is too small for the oldest request")
            return []
        sampled = self._run(out)
        finished = {r.request_id for r in self.scheduler.update(out, sampled)}
        st = self.stats
        st.num_steps += 1
        st.num_prefill_tokens += out.num_prefill_tokens
        st.num_decode_tokens += out.num_decode_tokens
        st.num_preemptions += len(out.preempted)
        st.step_times.append(time.perf_counter() - t0)
        return [StepOutput(i.request.request_id, sampled.get(i.request.request_id), i.request.request_id in finished)
                for i in out.scheduled]

    def _to_output(self, req: Request) -> RequestOutput:
        reason = {RequestStatus.FINISHED_STOPPED: "stop", RequestStatus.FINISHED_LENGTH: "length",
                  RequestStatus.FINISHED_ABORTED: "abort"}[req.status]
        text = ""
        if self.tokenizer is not None:
            text = self.tokenizer.decode(req.output_token_ids, skip_special_tokens=True)
        return RequestOutput(req.request_id, req.prompt_token_ids, req.output_token_ids, text, reason,
                             req.num_cached_tokens, req.num_preemptions)

    def generate(self, prompts: list, sampling_params=None, use_tqdm: bool = False) -> list:
        """Outputs in the order of the prompts (pagedllm/engine.py:219-234)."""
        if not isinstance(sampling_params, list):
            sampling_params = [sampling_params or SamplingParams()] * len(prompts)
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, sampling_params)]
        bar = None
        if use_tqdm:
            from tqdm import tqdm
            bar = tqdm(total=len(ids), desc="requests")
        while self.has_unfinished_requests:
            for o in self.step():
                if o.finished and bar:
                    bar.update(1)
        if bar:
            bar.close()
        return [self._to_output(self._requests.pop(i)) for i in ids]
