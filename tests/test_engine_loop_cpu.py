"""The engine's step loop (one step launched ahead of the committed one) with the GPU replaced by a model of a
model, on the CPU.

The stand-in step function keeps a dictionary for the cache pages: the content of a slot is a digest of every token
up to its position, chained from the slot before it, which it reads through the block table it is given, as
attention would.  The "logits" of a position are that digest, and the stand-in sampler draws the next token from it.
So a request's tokens depend on everything the cache holds for it, and any mistake of the loop, the scheduler or the
cache manager (a stale slot, a wrong page, a step out of order, a row of an ended request that shows up, ids handed
on to the wrong row) changes them.  The oracle recomputes each request alone, without a cache.  Random arrivals,
stop tokens, cancellations, pools small enough to preempt, prefix reuse, and graphs that appear after a while.
"""

import random
import zlib

import pytest

from paged_llm_amd import EngineConfig, SamplingParams
from paged_llm_amd.cache import CacheManager, GroupSpec
from paged_llm_amd.engine import Scheduler
from paged_llm_amd.engine.llm_engine import EngineStats, LLMEngine

VOCAB = 50


def chain(prev: int, token: int) -> int:
    return zlib.crc32(f"{prev}:{token}".encode())


def next_token(digest: int) -> int:
    return digest % VOCAB


def alone(prompt: list, params: SamplingParams) -> list:
    """What the request generates by itself: no cache, no batch."""
    digest = 0
    for t in prompt:
        digest = chain(digest, t)
    out = []
    while True:
        token = next_token(digest)
        out.append(token)
        if token in params.stop_token_ids or len(out) >= params.max_tokens:
            return out
        digest = chain(digest, token)


class Pending:
    def __init__(self, tokens):
        self.on_device = list(tokens)

    def result(self):
        return list(self.on_device)


class StandInSampler:
    def launch(self, logits, params, request_keys, steps):
        assert len(logits) == len(params) == len(request_keys) == len(steps)
        return Pending(next_token(d) for d in logits)


class StandInRunner:
    """``step`` / ``prepare`` / ``run_prepared`` of the step function, over a dictionary of slots."""

    def __init__(self, block_size: int, graph_after: int, rng):
        self.bs, self.slots, self.sightings, self.graph_after, self.rng = block_size, {}, {}, graph_after, rng
        self.prepared = 0

    def _slot(self, entry, pos):
        table = entry.block_tables["full"]
        return table[pos // self.bs], pos % self.bs

    def _run(self, entries, token_lists):
        rows = []
        for entry, tokens in zip(entries, token_lists):
            digest = self.slots[self._slot(entry, entry.start - 1)] if entry.start else 0
            for i, t in enumerate(tokens):
                digest = chain(digest, t)
                self.slots[self._slot(entry, entry.start + i)] = digest
                if i in entry.want:
                    rows.append(digest)
        return rows

    def step(self, entries, copies=None, borrow=False, state_copies=None):
        self._copy(copies)
        key = (len(entries), all(len(e.tokens) == 1 for e in entries))
        self.sightings[key] = self.sightings.get(key, 0) + 1
        return self._run(entries, [e.tokens for e in entries])

    def prepare(self, entries):
        assert all(len(e.tokens) == 1 and e.want == [0] for e in entries)
        if self.sightings.get((len(entries), True), 0) < self.graph_after:
            return None                                        # no graph for this many rows yet
        return list(entries)

    def run_prepared(self, handle, token_ids, copies=None, borrow=False, take=None):
        self._copy(copies)
        if take is not None:
            token_ids = [token_ids[i] for i in take]
        assert len(token_ids) == len(handle)
        self.prepared += 1
        return self._run(handle, [[t] for t in token_ids])

    def _copy(self, copies):
        for ops in (copies or {}).values():
            for op in ops:
                for off in range(self.bs):
                    if (op.src, off) in self.slots:
                        self.slots[(op.dst, off)] = self.slots[(op.src, off)]


def stand_in_engine(num_pages, block_size, budget, max_seqs, prefix, run_ahead, graph_after, rng):
    cfg = EngineConfig(block_size=block_size, max_num_batched_tokens=budget, max_num_seqs=max_seqs, enable_prefix_caching=prefix,
                       max_model_len=512, num_gpu_blocks=num_pages)
    engine = object.__new__(LLMEngine)                         # the loop and the request bookkeeping, nothing of the GPU
    engine.config = cfg
    engine.cache_manager = CacheManager([GroupSpec("full")], num_pages, block_size, prefix)
    engine.groups = list(engine.cache_manager.groups)
    engine.scheduler = Scheduler(cfg, engine.cache_manager, None)
    engine.runner = StandInRunner(block_size, graph_after, rng)
    engine.sampler = StandInSampler()
    engine.stats = EngineStats()
    engine.tokenizer = None
    engine.on_logits = None
    engine._live, engine._flight, engine.run_ahead, engine.digests_ahead_from = {}, None, run_ahead, 2 * block_size
    engine._token_ids = lambda prompt: [int(t) for t in prompt]
    return engine


@pytest.mark.parametrize("seed", range(40))
def test_random_workloads_give_what_each_request_gives_alone(seed):
    rng = random.Random(seed)
    block_size = rng.choice([2, 4, 8])
    engine = stand_in_engine(num_pages=rng.choice([12, 24, 200]) * 8 // block_size, block_size=block_size, budget=rng.choice([16, 64]),
                             max_seqs=rng.choice([2, 4, 8]), prefix=rng.random() < 0.5, run_ahead=seed % 4 != 0,
                             graph_after=rng.choice([1, 2, 5]), rng=rng)
    shared = [rng.randrange(VOCAB) for _ in range(rng.choice([0, 9]))]
    todo = []
    for _ in range(rng.randrange(3, 12)):
        prompt = shared + [rng.randrange(VOCAB) for _ in range(rng.randrange(1, 30))]
        stops = tuple(rng.sample(range(VOCAB), rng.choice([0, 0, 3, 10])))
        todo.append((prompt, SamplingParams(temperature=0.0, max_tokens=rng.randrange(1, 40), stop_token_ids=stops)))
    want, got, cancelled, arrivals = {}, {}, set(), list(todo)
    steps = 0
    while arrivals or engine.has_unfinished_requests:
        for _ in range(rng.choice([0, 0, 1, 3]) if steps else 2):          # requests arrive while others run
            if arrivals:
                prompt, params = arrivals.pop()
                rid = engine.add_request(prompt, params)
                want[rid], got[rid] = alone(prompt, params), []
        if not engine.has_unfinished_requests:
            continue
        if rng.random() < 0.05 and engine._live:                           # somebody gives up, perhaps with a row under way
            rid = rng.choice(sorted(engine._live))
            engine.abort_request(rid)
            cancelled.add(rid)
        for out in engine.step():
            assert out.seq_id not in cancelled, "a cancelled request showed up"
            if out.new_token is not None:
                got[out.seq_id].append(out.new_token)
            assert out.finished == (got[out.seq_id] == want[out.seq_id]), (out.seq_id, got[out.seq_id], want[out.seq_id])
        engine.cache_manager.check_invariants()
        steps += 1
        assert steps < 5000, "the loop does not come to an end"
    assert not engine.step_in_flight and engine.scheduler.idle
    for rid in want:
        if rid in cancelled:
            assert got[rid] == want[rid][: len(got[rid])]
        else:
            assert got[rid] == want[rid], rid
    assert engine.cache_manager.num_free_pages() == engine.cache_manager.num_pages()
    if engine.run_ahead and engine.runner.graph_after == 1 and any(p.max_tokens > 6 for _, p in todo):
        assert engine.runner.prepared > 0, "no step was ever launched ahead"


def test_generate_drains_what_it_launched_ahead():
    rng = random.Random(1)
    engine = stand_in_engine(64, 4, 64, 8, False, True, 1, rng)
    prompts = [[rng.randrange(VOCAB) for _ in range(n)] for n in (3, 11, 6)]
    params = [SamplingParams(temperature=0.0, max_tokens=m, stop_token_ids=(7, 21)) for m in (9, 30, 17)]
    outs = engine.generate(prompts, params)
    assert [o.token_ids for o in outs] == [alone(p, sp) for p, sp in zip(prompts, params)]
    assert {o.finish_reason for o in outs} <= {"stop", "length"} and not engine.step_in_flight
    assert engine.cache_manager.num_free_pages() == 64 and engine.runner.prepared > 0
    # what the statistics count is what was handed out
    assert engine.stats.num_prefill_tokens == sum(map(len, prompts))
    assert engine.stats.num_decode_tokens == sum(len(o.token_ids) - 1 for o in outs)


def test_a_newcomer_is_admitted_at_once_although_steps_run_ahead():
    rng = random.Random(2)
    engine = stand_in_engine(200, 4, 64, 8, False, True, 1, rng)
    long = SamplingParams(temperature=0.0, max_tokens=200)
    for n in (5, 9, 7):
        engine.add_request([rng.randrange(VOCAB) for _ in range(n)], long)
    for _ in range(6):
        engine.step()
    assert engine.step_in_flight                                 # the steady state: one step under way beyond the committed one
    late = engine.add_request([1, 2, 3], SamplingParams(temperature=0.0, max_tokens=5))
    first = engine.step()                                        # commits the step that was under way when it arrived
    assert late not in [o.seq_id for o in first] and not engine.step_in_flight
    second = engine.step()                                       # the next one is planned afresh and takes it in
    assert late in [o.seq_id for o in second] and len(second) == 4


def test_the_static_heap_is_frozen_once():
    """What was imported before the first engine is taken out of the garbage collector's generations once per process;
    objects made afterwards (an engine's own, the requests') are collected as ever."""
    import gc
    from paged_llm_amd.engine import llm_engine
    llm_engine._freeze_static_heap()
    frozen = gc.get_freeze_count()
    assert llm_engine._static_heap_frozen and frozen > 0

    class Node:
        pass
    a, b = Node(), Node()
    a.other, b.other = b, a                                       # a cycle made after the freeze
    import weakref
    seen = weakref.ref(a)
    del a, b
    llm_engine._freeze_static_heap()                              # (a second call freezes nothing more)
    assert gc.get_freeze_count() == frozen
    gc.collect()
    assert seen() is None

