"""The scheduler's decisions with the model replaced by a constant token (the vectors of the
reference's tests/test_scheduler.py:24-132, plus what happens when pages or state slots run out)."""

import pytest

from paged_llm_amd import EngineConfig, SamplingParams
from paged_llm_amd.cache import CacheManager, GroupSpec
from paged_llm_amd.engine import EndReason, Request, Scheduler, Stage

EOS = 2


def make(num_blocks=64, block_size=4, budget=32, max_seqs=8, chunked=True, prefix=True, max_len=256, state_slots=0, eos=EOS):
    cfg = EngineConfig(block_size=block_size, max_num_batched_tokens=budget, max_num_seqs=max_seqs,
                       enable_chunked_prefill=chunked, enable_prefix_caching=prefix, max_model_len=max_len,
                       num_gpu_blocks=num_blocks)
    cm = CacheManager([GroupSpec("full")], num_blocks, block_size, prefix, num_state_slots=state_slots)
    return cfg, cm, Scheduler(cfg, cm, eos)


def run_step(sched, next_token=7):
    plan = sched.plan()
    sampled = {g.request.id: next_token for g in plan.grants if g.samples}
    ended = sched.commit(plan, sampled)
    sched.cache.check_invariants()
    return plan, ended


def test_prefill_then_decode_then_finish():
    _, _, sched = make()
    req = Request(list(range(10, 20)), SamplingParams(max_tokens=3))
    sched.submit(req)
    out, _ = run_step(sched)
    assert out.prompt_tokens == 10 and out.decode_tokens == 0
    assert req.stage is Stage.ACTIVE and req.num_generated == 1
    out, _ = run_step(sched)
    assert out.decode_tokens == 1
    out, finished = run_step(sched)
    assert finished == [req] and req.end_reason is EndReason.LENGTH
    assert req.generated == [7, 7, 7] and sched.idle


def test_eos_and_stop_tokens():
    _, cm, sched = make()
    req = Request([5, 6, 7], SamplingParams(max_tokens=10))
    sched.submit(req)
    sched.commit(out := sched.plan(), {req.id: EOS})
    assert req.end_reason is EndReason.STOP and cm.num_free_pages() == 64
    assert req.generated == [EOS]                        # the stop token stays in the output
    ignoring = Request([5, 6, 7], SamplingParams(max_tokens=2, ignore_eos=True))
    sched.submit(ignoring)
    sched.commit(out := sched.plan(), {ignoring.id: EOS})
    assert ignoring.stage is Stage.ACTIVE
    stopper = Request([5, 6, 7], SamplingParams(max_tokens=9, stop_token_ids=(42,)))
    sched.submit(stopper)
    out = sched.plan()
    sched.commit(out, {ignoring.id: 1, stopper.id: 42})
    assert stopper.end_reason is EndReason.STOP and ignoring.end_reason is EndReason.LENGTH


def test_several_eos_ids_from_config_json():
    _, _, sched = make(eos=[2, 9])
    req = Request([5], SamplingParams(max_tokens=10))
    sched.submit(req)
    sched.commit(out := sched.plan(), {req.id: 9})
    assert req.end_reason is EndReason.STOP


def test_prompt_portions_respect_the_budget():
    _, _, sched = make(budget=8)
    req = Request(list(range(100, 120)), SamplingParams(max_tokens=2))
    sched.submit(req)
    out, _ = run_step(sched)
    assert out.grants[0].count == 8 and req.computed == 8
    assert req.num_generated == 0 and not out.grants[0].samples
    run_step(sched)
    assert req.computed == 16
    run_step(sched)
    assert req.computed == 20 and req.num_generated == 1


def test_decode_and_prompt_portion_share_a_step():
    _, _, sched = make(budget=16)
    a = Request(list(range(4)), SamplingParams(max_tokens=10))
    sched.submit(a)
    run_step(sched)
    b = Request(list(range(40)), SamplingParams(max_tokens=10))
    sched.submit(b)
    out, _ = run_step(sched)
    assert out.decode_tokens == 1 and out.prompt_tokens == 15
    assert [g.request for g in out.grants] == [a, b]


def test_first_in_first_out_and_max_num_seqs():
    _, _, sched = make(max_seqs=2, budget=1000)
    reqs = [Request([1, 2, 3], SamplingParams(max_tokens=5)) for _ in range(3)]
    for r in reqs:
        sched.submit(r)
    out, _ = run_step(sched)
    assert [g.request for g in out.grants] == reqs[:2] and reqs[2].stage is Stage.QUEUED


def test_when_pages_run_out_the_last_admitted_is_preempted_and_recomputed():
    # 6 pages of 4: two prompts of 8 fill 4; each needs a 3rd page at token 8 and a 4th at token 12.
    _, cm, sched = make(num_blocks=6, block_size=4, budget=1000)
    a = Request(list(range(8)), SamplingParams(max_tokens=8))
    b = Request(list(range(8, 16)), SamplingParams(max_tokens=8))
    sched.submit(a)
    sched.submit(b)
    run_step(sched)
    assert cm.num_free_pages() == 2
    run_step(sched)
    assert cm.num_free_pages() == 0
    for _ in range(3):
        out, _ = run_step(sched)
    assert cm.num_free_pages() == 0 and not out.preempted
    out, _ = run_step(sched)
    assert b in out.preempted and b.stage is Stage.QUEUED and not cm.holds(b.id)
    assert a.stage is Stage.ACTIVE and sched.num_preemptions >= 1 and sched.queue[0] is b
    generated_before = b.num_generated
    while a.stage is Stage.ACTIVE:
        run_step(sched)
    assert a.generated == [7] * 8
    while not sched.idle:
        run_step(sched)
    assert b.end_reason is EndReason.LENGTH and b.num_generated == 8
    assert b.times_preempted >= 1 and generated_before >= 1 and cm.num_free_pages() == 6


def test_a_request_that_cannot_get_a_page_alone_just_waits_this_step():
    # one running request needs a page that does not exist: it is its own victim and returns to waiting
    _, cm, sched = make(num_blocks=2, block_size=4, budget=1000, prefix=False)
    a = Request(list(range(8)), SamplingParams(max_tokens=4))
    sched.submit(a)
    run_step(sched)                                             # 8 tokens fill both pages
    out = sched.plan()
    assert not out and out.preempted == [a] and a.stage is Stage.QUEUED and cm.num_free_pages() == 2


def test_admission_stops_at_the_first_request_that_does_not_fit():
    _, cm, sched = make(num_blocks=4, block_size=4, budget=1000)
    big, small = Request(list(range(30)), SamplingParams()), Request([1, 2], SamplingParams())
    sched.submit(big)
    sched.submit(small)
    out = sched.plan()
    assert not out and list(sched.queue) == [big, small]    # no skipping ahead
    assert cm.num_free_pages() == 4


def test_prefix_reuse_across_requests():
    _, cm, sched = make(block_size=4, budget=1000)
    shared = list(range(50, 66))
    a = Request(shared + [1, 2], SamplingParams(max_tokens=1))
    sched.submit(a)
    while not sched.idle:
        run_step(sched)
    b = Request(shared + [3, 4, 5], SamplingParams(max_tokens=1))
    sched.submit(b)
    out, _ = run_step(sched)
    assert b.reused_prefix == 16 and out.grants[0].count == 3 and cm.num_cache_hits == 1


def test_no_portions_when_disabled():
    _, _, sched = make(budget=8, chunked=False)
    small = Request(list(range(8)), SamplingParams(max_tokens=1))
    sched.submit(small)
    out, _ = run_step(sched)
    assert out.grants[0].count == 8
    with pytest.raises(ValueError, match="enable_chunked_prefill"):
        sched.submit(Request(list(range(9)), SamplingParams()))


def test_length_checks_and_clamp_do_not_touch_shared_params():
    _, _, sched = make(max_len=32)
    with pytest.raises(ValueError, match="max_model_len"):
        sched.submit(Request(list(range(32)), SamplingParams()))
    shared = SamplingParams(max_tokens=100)
    a, b = Request(list(range(20)), shared), Request(list(range(5)), shared)
    sched.submit(a)
    sched.submit(b)
    assert a.new_token_limit == 12 and b.new_token_limit == 27 and shared.max_tokens == 100
    with pytest.raises(ValueError, match="at least one prompt token"):
        Request([], SamplingParams())


def test_abort_gives_everything_back():
    _, cm, sched = make()
    a, b = Request(list(range(9)), SamplingParams()), Request(list(range(5)), SamplingParams())
    sched.submit(a)
    run_step(sched)
    sched.submit(b)
    sched.cancel(a.id)
    sched.cancel(b.id)
    assert a.end_reason is b.end_reason is EndReason.ABORT and sched.idle
    assert cm.num_free_pages() == 64


def test_state_slots_limit_admission():
    _, cm, sched = make(state_slots=1, budget=1000)
    a, b = Request([1, 2, 3], SamplingParams(max_tokens=2)), Request([4, 5], SamplingParams(max_tokens=2))
    sched.submit(a)
    sched.submit(b)
    out, _ = run_step(sched)
    assert [g.request for g in out.grants] == [a] and b.stage is Stage.QUEUED
    run_step(sched)                                             # a finishes, its slot comes back
    out, _ = run_step(sched)
    assert [g.request for g in out.grants] == [b] and cm.state_slot(b.id) == 0


def test_a_preempted_request_beyond_the_whole_budget_is_recomputed_in_portions_even_when_portions_are_off():
    """Portions disabled, budget 8: a request admitted with 8 tokens grows, loses its pages to an earlier
    request, and is then longer than any step may hold.  It must still come back (in portions), not
    block the queue for ever."""
    _, cm, sched = make(num_blocks=5, block_size=4, budget=8, chunked=False, prefix=False)
    a, b = Request(list(range(4)), SamplingParams(max_tokens=10)), Request(list(range(8, 12)), SamplingParams(max_tokens=10))
    sched.submit(a)
    sched.submit(b)
    steps, longest_backlog = 0, 0
    while not sched.idle:
        plan, _ = run_step(sched)
        assert plan or sched.idle, "an empty plan although requests remain"
        longest_backlog = max([longest_backlog] + [len(r.tokens) for r in plan.preempted])
        steps += 1
        assert steps < 200
    assert b.times_preempted >= 1 and longest_backlog > 8          # it came back longer than a step's whole budget
    assert a.end_reason is b.end_reason is EndReason.LENGTH
    assert a.generated == b.generated == [7] * 10 and cm.num_free_pages() == 5


def test_why_stuck_names_the_pool_when_one_request_cannot_fit():
    _, _, sched = make(num_blocks=2, block_size=4, budget=1000)
    sched.submit(Request(list(range(30)), SamplingParams()))
    assert not sched.plan()
    assert "pages" in sched.why_stuck() and "the pool holds 2" in sched.why_stuck()


def test_a_finished_request_is_no_longer_held_by_the_scheduler():
    _, _, sched = make()
    req = Request([1, 2, 3], SamplingParams(max_tokens=1))
    sched.submit(req)
    _, ended = run_step(sched)
    assert ended == [req] and sched.idle and len(sched) == 0


def test_the_step_after_can_be_planned_while_this_one_runs_only_in_the_steady_state():
    """``plan_ahead`` foresees one more token for everybody who does not reach a limit in the step under way, in the
    same order, and nothing else: not while somebody waits in the queue, is still inside its prompt, or would need
    somebody else's pages."""
    _, cm, sched = make(num_blocks=12, block_size=4, budget=16)
    a, b = Request([1] * 6, SamplingParams(max_tokens=5, ignore_eos=True)), Request([2] * 3, SamplingParams(max_tokens=19, ignore_eos=True))
    sched.submit(a), sched.submit(b)
    plan = sched.plan()                                              # both prompts whole
    ahead = sched.plan_ahead(plan)
    assert [g.request for g in ahead.grants] == [a, b] and all(g.count == 1 and g.samples for g in ahead.grants) and ahead.decode_tokens == 2
    sched.commit(plan, {a.id: 7, b.id: 7})
    after = sched.plan_ahead(ahead)                                  # and the one after that, from the plan that is under way
    assert [g.request for g in after.grants] == [a, b]
    sched.commit(ahead, {a.id: 7, b.id: 7})
    sched.commit(after, {a.id: 7, b.id: 7})
    cm.check_invariants()
    assert a.num_generated == 3 and a.computed == 8 and len(cm.block_table(a.id, "full")) == 2
    plan = sched.plan()                                              # a's fourth token of five
    sched.commit(plan, {a.id: 7, b.id: 7})
    plan = sched.plan()                                              # a's fifth: it ends by length in this step, whatever it samples
    ahead = sched.plan_ahead(plan)
    assert [g.request for g in ahead.grants] == [b]                  # so the step after is foreseen without it
    sched.commit(plan, {a.id: 7, b.id: 7})
    assert a.ended and not b.ended
    sched.commit(ahead, {b.id: 7})
    only = Request([9] * 3, SamplingParams(max_tokens=1))
    sched.submit(only)
    plan = sched.plan()
    assert len(plan.grants) == 2 and sched.plan_ahead(plan).grants[0].request is b and len(sched.plan_ahead(plan).grants) == 1
    sched.commit(plan, {b.id: 7, only.id: 7})
    assert only.ended
    late = Request([3] * 40, SamplingParams(max_tokens=2))
    sched.submit(late)
    plan = sched.plan()                                              # a portion of the newcomer beside b
    assert len(plan.grants) == 2 and not plan.grants[1].samples and sched.plan_ahead(plan) is None
    sched.cancel(late.id)
    sched.commit(plan, {b.id: 7})                                    # (the cancelled request's grant is passed over)
    plan = sched.plan()
    assert [g.request for g in plan.grants] == [b] and sched.plan_ahead(plan) is not None
    cm.check_invariants()


def test_a_request_that_ended_is_passed_over_by_the_step_that_already_ran_for_it():
    _, cm, sched = make()
    a, b = Request([1] * 5, SamplingParams(max_tokens=9, stop_token_ids=(42,))), Request([2] * 5, SamplingParams(max_tokens=9, ignore_eos=True))
    sched.submit(a), sched.submit(b)
    sched.commit(sched.plan(), {a.id: 7, b.id: 7})
    plan = sched.plan()
    ahead = sched.plan_ahead(plan)
    assert sched.commit(plan, {a.id: 42, b.id: 7}) == [a]            # a stops; the step after is under way with a row for it
    free = cm.num_free_pages()
    assert sched.commit(ahead, {a.id: 9, b.id: 8}) == []
    assert a.generated == [7, 42] and b.generated == [7, 7, 8] and cm.num_free_pages() == free
    assert sched.plan_ahead(ahead) is None                           # two grants, one active request: plan afresh
    cm.check_invariants()


def test_no_plan_ahead_when_the_next_token_needs_a_page_that_somebody_would_have_to_give():
    _, cm, sched = make(num_blocks=4, block_size=4, budget=16)
    a, b = Request([1] * 8, SamplingParams(max_tokens=9, ignore_eos=True)), Request([2] * 7, SamplingParams(max_tokens=9, ignore_eos=True))
    sched.submit(a), sched.submit(b)
    plan = sched.plan()                                              # 2 + 2 pages: the pool is full
    assert cm.num_free_pages() == 0 and len(plan.grants) == 2
    assert sched.plan_ahead(plan) is None                            # a's next token needs a third page
    sched.commit(plan, {a.id: 7, b.id: 7})
    plan = sched.plan()                                              # decided the ordinary way: the last admitted gives way
    assert plan.preempted == [b] and [g.request for g in plan.grants] == [a]
    cm.check_invariants()


def test_plan_ahead_goes_on_while_others_wait_for_a_place_that_stays_taken():
    _, cm, sched = make(max_seqs=2)
    a, b = Request([1] * 4, SamplingParams(max_tokens=3, ignore_eos=True)), Request([2] * 4, SamplingParams(max_tokens=9, ignore_eos=True))
    waiting = Request([3] * 4, SamplingParams(max_tokens=2))
    for r in (a, b, waiting):
        sched.submit(r)
    plan = sched.plan()
    assert [g.request for g in plan.grants] == [a, b] and len(sched.queue) == 1
    ahead = sched.plan_ahead(plan)                                   # both stay: nobody can be admitted in the step after
    assert [g.request for g in ahead.grants] == [a, b]
    sched.commit(plan, {a.id: 7, b.id: 7})
    sched.commit(ahead, {a.id: 7, b.id: 7})
    plan = sched.plan()                                              # a's third token, its last
    assert sched.plan_ahead(plan) is None                            # its place comes free: the step after may admit the one that waits
    sched.commit(plan, {a.id: 7, b.id: 7})
    assert a.ended
    plan = sched.plan()
    assert [g.request for g in plan.grants] == [b, waiting]
    cm.check_invariants()
