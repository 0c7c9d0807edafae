"""The scheduler's decisions with the model replaced by a constant token (the vectors of the
reference's tests/test_scheduler.py:24-132, plus what happens when pages or state slots run out)."""

import pytest

from paged_llm_amd import EngineConfig, SamplingParams
from paged_llm_amd.cache import CacheManager, GroupSpec
from paged_llm_amd.engine import Request, RequestStatus, Scheduler

EOS = 2


def make(num_blocks=64, block_size=4, budget=32, max_seqs=8, chunked=True, prefix=True, max_len=256, state_slots=0, eos=EOS):
    cfg = EngineConfig(block_size=block_size, max_num_batched_tokens=budget, max_num_seqs=max_seqs,
                       enable_chunked_prefill=chunked, enable_prefix_caching=prefix, max_model_len=max_len,
                       num_gpu_blocks=num_blocks)
    cm = CacheManager([GroupSpec("full")], num_blocks, block_size, prefix, num_state_slots=state_slots)
    return cfg, cm, Scheduler(cfg, cm, eos)


def run_step(sched, next_token=7):
    out = sched.schedule()
    sampled = {s.request.request_id: next_token for s in out.scheduled if s.needs_sampling}
    finished = sched.update(out, sampled)
    sched.cm.check_invariants()
    return out, finished


def test_prefill_then_decode_then_finish():
    _, _, sched = make()
    req = Request(list(range(10, 20)), SamplingParams(max_tokens=3))
    sched.add(req)
    out, _ = run_step(sched)
    assert out.num_prefill_tokens == 10 and out.num_decode_tokens == 0
    assert req.status is RequestStatus.RUNNING and req.num_generated_tokens == 1
    out, _ = run_step(sched)
    assert out.num_decode_tokens == 1
    out, finished = run_step(sched)
    assert finished == [req] and req.status is RequestStatus.FINISHED_LENGTH
    assert req.output_token_ids == [7, 7, 7] and not sched.has_unfinished


def test_eos_and_stop_tokens():
    _, cm, sched = make()
    req = Request([5, 6, 7], SamplingParams(max_tokens=10))
    sched.add(req)
    sched.update(out := sched.schedule(), {req.request_id: EOS})
    assert req.status is RequestStatus.FINISHED_STOPPED and cm.num_free_pages() == 64
    assert req.output_token_ids == [EOS]                        # the stop token stays in the output
    ignoring = Request([5, 6, 7], SamplingParams(max_tokens=2, ignore_eos=True))
    sched.add(ignoring)
    sched.update(out := sched.schedule(), {ignoring.request_id: EOS})
    assert ignoring.status is RequestStatus.RUNNING
    stopper = Request([5, 6, 7], SamplingParams(max_tokens=9, stop_token_ids=(42,)))
    sched.add(stopper)
    out = sched.schedule()
    sched.update(out, {ignoring.request_id: 1, stopper.request_id: 42})
    assert stopper.status is RequestStatus.FINISHED_STOPPED and ignoring.status is RequestStatus.FINISHED_LENGTH


def test_several_eos_ids_from_config_json():
    _, _, sched = make(eos=[2, 9])
    req = Request([5], SamplingParams(max_tokens=10))
    sched.add(req)
    sched.update(out := sched.schedule(), {req.request_id: 9})
    assert req.status is RequestStatus.FINISHED_STOPPED


def test_prompt_portions_respect_the_budget():
    _, _, sched = make(budget=8)
    req = Request(list(range(100, 120)), SamplingParams(max_tokens=2))
    sched.add(req)
    out, _ = run_step(sched)
    assert out.scheduled[0].num_new_tokens == 8 and req.num_computed_tokens == 8
    assert req.num_generated_tokens == 0 and not out.scheduled[0].needs_sampling
    run_step(sched)
    assert req.num_computed_tokens == 16
    run_step(sched)
    assert req.num_computed_tokens == 20 and req.num_generated_tokens == 1


def test_decode_and_prompt_portion_share_a_step():
    _, _, sched = make(budget=16)
    a = Request(list(range(4)), SamplingParams(max_tokens=10))
    sched.add(a)
    run_step(sched)
    b = Request(list(range(40)), SamplingParams(max_tokens=10))
    sched.add(b)
    out, _ = run_step(sched)
    assert out.num_decode_tokens == 1 and out.num_prefill_tokens == 15
    assert [s.request for s in out.scheduled] == [a, b]


def test_first_in_first_out_and_max_num_seqs():
    _, _, sched = make(max_seqs=2, budget=1000)
    reqs = [Request([1, 2, 3], SamplingParams(max_tokens=5)) for _ in range(3)]
    for r in reqs:
        sched.add(r)
    out, _ = run_step(sched)
    assert [x.request for x in out.scheduled] == reqs[:2] and reqs[2].status is RequestStatus.WAITING


def test_when_pages_run_out_the_last_admitted_is_preempted_and_recomputed():
    # 6 pages of 4: two prompts of 8 fill 4; each needs a 3rd page at token 8 and a 4th at token 12.
    _, cm, sched = make(num_blocks=6, block_size=4, budget=1000)
    a = Request(list(range(8)), SamplingParams(max_tokens=8))
    b = Request(list(range(8, 16)), SamplingParams(max_tokens=8))
    sched.add(a)
    sched.add(b)
    run_step(sched)
    assert cm.num_free_pages() == 2
    run_step(sched)
    assert cm.num_free_pages() == 0
    for _ in range(3):
        out, _ = run_step(sched)
    assert cm.num_free_pages() == 0 and not out.preempted
    out, _ = run_step(sched)
    assert b in out.preempted and b.status is RequestStatus.WAITING and not cm.holds(b.request_id)
    assert a.status is RequestStatus.RUNNING and sched.num_preemptions >= 1 and sched.waiting[0] is b
    generated_before = b.num_generated_tokens
    while a.status is RequestStatus.RUNNING:
        run_step(sched)
    assert a.output_token_ids == [7] * 8
    while sched.has_unfinished:
        run_step(sched)
    assert b.status is RequestStatus.FINISHED_LENGTH and b.num_generated_tokens == 8
    assert b.num_preemptions >= 1 and generated_before >= 1 and cm.num_free_pages() == 6


def test_a_request_that_cannot_get_a_page_alone_just_waits_this_step():
    # one running request needs a page that does not exist: it is its own victim and returns to waiting
    _, cm, sched = make(num_blocks=2, block_size=4, budget=1000, prefix=False)
    a = Request(list(range(8)), SamplingParams(max_tokens=4))
    sched.add(a)
    run_step(sched)                                             # 8 tokens fill both pages
    out = sched.schedule()
    assert out.is_empty and out.preempted == [a] and a.status is RequestStatus.WAITING and cm.num_free_pages() == 2


def test_admission_stops_at_the_first_request_that_does_not_fit():
    _, cm, sched = make(num_blocks=4, block_size=4, budget=1000)
    big, small = Request(list(range(30)), SamplingParams()), Request([1, 2], SamplingParams())
    sched.add(big)
    sched.add(small)
    out = sched.schedule()
    assert out.is_empty and list(sched.waiting) == [big, small]    # no skipping ahead
    assert cm.num_free_pages() == 4


def test_prefix_reuse_across_requests():
    _, cm, sched = make(block_size=4, budget=1000)
    shared = list(range(50, 66))
    a = Request(shared + [1, 2], SamplingParams(max_tokens=1))
    sched.add(a)
    while sched.has_unfinished:
        run_step(sched)
    b = Request(shared + [3, 4, 5], SamplingParams(max_tokens=1))
    sched.add(b)
    out, _ = run_step(sched)
    assert b.num_cached_tokens == 16 and out.scheduled[0].num_new_tokens == 3 and cm.num_cache_hits == 1


def test_no_portions_when_disabled():
    _, _, sched = make(budget=8, chunked=False)
    small = Request(list(range(8)), SamplingParams(max_tokens=1))
    sched.add(small)
    out, _ = run_step(sched)
    assert out.scheduled[0].num_new_tokens == 8
    with pytest.raises(ValueError, match="chunked"):
        sched.add(Request(list(range(9)), SamplingParams()))


def test_length_checks_and_clamp_do_not_touch_shared_params():
    _, _, sched = make(max_len=32)
    with pytest.raises(ValueError, match="max_model_len"):
        sched.add(Request(list(range(32)), SamplingParams()))
    shared = SamplingParams(max_tokens=100)
    a, b = Request(list(range(20)), shared), Request(list(range(5)), shared)
    sched.add(a)
    sched.add(b)
    assert a.max_tokens == 12 and b.max_tokens == 27 and shared.max_tokens == 100
    with pytest.raises(ValueError, match="empty"):
        Request([], SamplingParams())


def test_abort_gives_everything_back():
    _, cm, sched = make()
    a, b = Request(list(range(9)), SamplingParams()), Request(list(range(5)), SamplingParams())
    sched.add(a)
    run_step(sched)
    sched.add(b)
    sched.abort(a.request_id)
    sched.abort(b.request_id)
    assert a.status is b.status is RequestStatus.FINISHED_ABORTED and not sched.has_unfinished
    assert cm.num_free_pages() == 64


def test_state_slots_limit_admission():
    _, cm, sched = make(state_slots=1, budget=1000)
    a, b = Request([1, 2, 3], SamplingParams(max_tokens=2)), Request([4, 5], SamplingParams(max_tokens=2))
    sched.add(a)
    sched.add(b)
    out, _ = run_step(sched)
    assert [s.request for s in out.scheduled] == [a] and b.status is RequestStatus.WAITING
    run_step(sched)                                             # a finishes, its slot comes back
    out, _ = run_step(sched)
    assert [s.request for s in out.scheduled] == [b] and cm.state_slot(b.request_id) == 0
