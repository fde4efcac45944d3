"""The scheduler's decisions, with a stand-in for the model: a ``Driver`` plans a step, pretends
it ran and hands a fixed token back for every request whose slice reached its end.  The worked
cases are the reference's (tests/test_scheduler.py:28-134 of the reference: what is planned for
which budget, who is preempted, who waits); the decisions about runs of decode steps and
``commit`` are this engine's own."""

from __future__ import annotations

import pytest

from kvforge_amd.cache import CacheGroup, CacheManager
from kvforge_amd.config import SchedulerConfig
from kvforge_amd.engine.request import FinishReason, Request, RequestStatus
from kvforge_amd.engine.scheduler import RequestRejectedError, Scheduler
from kvforge_amd.sampling import SamplingParams


class Driver:
    def __init__(self, num_blocks=64, block_size=4, run_steps=1, run_ahead=False, device_runs=None,
                 **limits):
        cache = CacheManager(block_size, [CacheGroup((0,))], num_blocks)
        self.sched = Scheduler(SchedulerConfig(**limits), cache, run_steps, run_ahead,
                               device_runs=device_runs)
        self.cache = cache

    def add(self, rid, prompt_len, arrival, max_tokens=8, priority=0, **params):
        req = Request(rid, range(1, prompt_len + 1), SamplingParams(max_tokens=max_tokens, **params),
                      arrival_time=arrival, priority=priority)
        self.sched.add_request(req)
        return req

    def plan(self, **kw):
        return self.sched.schedule(**kw)

    def ran(self, plan, token=0):
        """The plan's step(s) ran: one token per step for every slice that reached the end."""
        sampled = {s.request.request_id: [token] * plan.run_steps for s in plan.slices if s.samples}
        return self.sched.commit(plan, sampled)

    def step(self, **kw):
        plan = self.plan(**kw)
        self.ran(plan)
        return plan


def shares(plan):
    return [(s.request.request_id, s.count) for s in plan.slices]


def test_priority_policy_orders_the_line_by_priority_then_arrival():
    """src/tokenvault/scheduler.py:85-88: with the priority policy a smaller priority is served
    sooner, arrival decides within one priority; without it the priority is not looked at."""
    from kvforge_amd.config.engine import SchedulingPolicy
    for policy, want in ((SchedulingPolicy.PRIORITY, ["late-urgent", "early-urgent", "early"]),
                         (SchedulingPolicy.FCFS, ["early", "early-urgent", "late-urgent"])):
        d = Driver(max_num_seqs=3, policy=policy)
        d.add("early", 4, 1.0, priority=5)
        d.add("early-urgent", 4, 2.0, priority=1)
        d.add("late-urgent", 4, 3.0, priority=0)
        assert [s.request.request_id for s in d.plan().slices] == want


def test_priority_policy_preempts_the_least_urgent_and_readmits_it_behind_the_urgent():
    """When pages run out the last in line gives way (src/tokenvault/scheduler.py:178-190): under
    the priority policy that is the least urgent request, however early it came, and it goes back
    in line at its place, behind a more urgent request that arrived meanwhile."""
    from kvforge_amd.config.engine import SchedulingPolicy
    d = Driver(num_blocks=4, block_size=4, max_num_seqs=4, policy=SchedulingPolicy.PRIORITY)
    d.add("bulk", 7, 1.0, priority=9, max_tokens=6)
    d.add("urgent", 7, 2.0, priority=0, max_tokens=6)
    d.step()                                   # both prompts: two pages each, the pool is full
    d.step()                                   # token 8 of each still fits its second page
    plan = d.plan()                            # token 9 needs a third page
    assert [r.request_id for r in plan.preempted] == ["bulk"] and shares(plan) == [("urgent", 1)]
    d.ran(plan)
    d.add("urgent-2", 3, 5.0, priority=1, max_tokens=2)
    assert [r.request_id for r in d.sched._waiting] == ["urgent-2", "bulk"]


def test_admission_follows_arrival_and_stops_at_max_num_seqs():
    d = Driver(max_num_seqs=2)
    for name, arrival in (("r0", 3.0), ("r1", 1.0), ("r2", 2.0)):
        d.add(name, 4, arrival)
    plan = d.plan()
    assert shares(plan) == [("r1", 4), ("r2", 4)] and not any(s.decode for s in plan.slices)
    assert (d.sched.num_running, d.sched.num_waiting) == (2, 1)
    assert [r.request_id for r in d.sched.running] == ["r1", "r2"]


def test_a_prompt_is_fed_whole_then_one_token_a_step():
    d = Driver()
    d.add("a", 6, 0.0)
    first = d.step()
    assert shares(first) == [("a", 6)] and first.slices[0].samples and not first.slices[0].decode
    second = d.plan()
    assert shares(second) == [("a", 1)] and second.slices[0].decode and second.slices[0].start == 6


def test_budget_cuts_a_prompt_into_portions():
    d = Driver(max_num_batched_tokens=8, enable_chunked_prefill=True)
    req = d.add("a", 20, 0.0)
    portions = []
    while req.num_output_tokens == 0:
        plan = d.step()
        assert plan.num_tokens <= 8
        portions.append((plan.slices[0].start, plan.slices[0].count, plan.slices[0].samples))
    assert portions == [(0, 8, False), (8, 8, False), (16, 4, True)]


def test_running_requests_are_planned_before_arrivals():
    d = Driver(max_num_batched_tokens=10)
    d.add("a", 4, 0.0)
    d.step()
    d.add("b", 30, 1.0)
    plan = d.plan()
    assert shares(plan) == [("a", 1), ("b", 9)]
    assert [s.decode for s in plan.slices] == [True, False]


def test_without_chunking_a_prompt_waits_for_a_step_it_fits_in():
    d = Driver(max_num_batched_tokens=10, enable_chunked_prefill=False)
    d.add("a", 4, 0.0)
    d.step()
    d.add("b", 10, 1.0)
    assert shares(d.plan()) == [("a", 1)]          # 9 tokens of budget are left, b brings 10
    d.sched.abort_request("a")
    assert shares(d.plan()) == [("b", 10)]


def test_without_chunking_a_preempted_request_that_outgrew_the_budget_is_fed_in_portions():
    """The reference refuses at the door what exceeds the budget by its prompt alone
    (src/tokenvault/scheduler.py:109-129) but looks at prompt plus outputs when a preempted
    request comes back (:206-207): a request that was preempted after it had grown past the
    budget would then stand at the head of the line for ever.  Here it is fed again in portions.
    5 pages of 4 tokens, 8 tokens a step, two prompts of 7 tokens with 12 new tokens each."""
    d = Driver(num_blocks=5, block_size=4, max_num_batched_tokens=8, enable_chunked_prefill=False)
    a = d.add("a", 7, 0.0, max_tokens=12)
    b = d.add("b", 7, 1.0, max_tokens=12)
    preempted_at, fed_again = None, []
    for step in range(80):
        if not d.sched.has_unfinished():
            break
        plan = d.step()
        assert not plan.is_empty or plan.preempted, f"nothing planned at step {step}"
        assert plan.num_tokens <= 8
        if plan.preempted:
            assert [r.request_id for r in plan.preempted] == ["b"]
            preempted_at = (step, b.num_tokens)
        elif preempted_at and len(fed_again) < 2:
            fed_again += [(s.start, s.count, s.samples) for s in plan.slices if s.request is b]
    assert preempted_at is not None and preempted_at[1] > 8          # it had outgrown a step
    assert fed_again == [(0, 8, False), (8, preempted_at[1] - 8, True)]
    assert a.finish_reason is FinishReason.LENGTH and b.finish_reason is FinishReason.LENGTH
    assert a.num_output_tokens == b.num_output_tokens == 12
    assert d.cache.num_free_blocks == 5


def test_without_chunking_a_preempted_request_that_still_fits_a_step_comes_back_whole():
    d = Driver(num_blocks=5, block_size=4, max_num_batched_tokens=16, enable_chunked_prefill=False)
    d.add("a", 7, 0.0, max_tokens=12)
    b = d.add("b", 7, 1.0, max_tokens=12)
    whole = None
    for _ in range(80):
        if not d.sched.has_unfinished():
            break
        plan = d.step()
        for s in plan.slices:
            if s.request is b and b.num_preemptions and not s.decode and whole is None:
                whole = (s.start, s.count, s.samples)
    assert b.num_preemptions == 1 and whole == (0, whole[1], True) and whole[1] > 7
    assert d.cache.num_free_blocks == 5


def test_a_step_without_admission_leaves_arrivals_in_line():
    """``schedule(admit=False)`` and ``schedule(queued_steps=n)``: only what runs is planned."""
    d = Driver()
    d.add("a", 4, 1.0)
    d.step()
    d.add("b", 4, 2.0)
    plan = d.plan(admit=False)
    assert shares(plan) == [("a", 1)] and (d.sched.num_waiting, d.sched.num_running) == (1, 1)
    d.ran(plan)
    plan = d.plan(queued_steps=3)
    assert shares(plan) == [("a", 1)] and plan.run_steps == 3 and d.sched.num_waiting == 1
    d.ran(plan)
    assert shares(d.plan()) == [("a", 1), ("b", 4)] and d.sched.num_waiting == 0


def test_what_can_never_be_served_is_refused():
    d = Driver(max_num_batched_tokens=8, enable_chunked_prefill=False)
    with pytest.raises(RequestRejectedError, match="chunked"):
        d.add("big", 9, 0.0)
    d = Driver(num_blocks=2, block_size=4)
    with pytest.raises(RequestRejectedError, match="never fit"):
        d.add("a", 6, 0.0, max_tokens=8)
    d = Driver(max_model_len=16)
    with pytest.raises(RequestRejectedError, match="max_model_len"):
        d.add("long", 16, 0.0)
    with pytest.raises(RequestRejectedError, match="empty"):
        d.add("e", 0, 0.0)
    d.add("a", 3, 0.0)
    with pytest.raises(RequestRejectedError, match="duplicate"):
        d.add("a", 3, 1.0)
    assert issubclass(RequestRejectedError, ValueError)


def test_when_pages_run_out_the_latest_arrival_goes_back_in_line():
    d = Driver(num_blocks=4, block_size=4, max_num_seqs=4)
    d.add("old", 7, 0.0, max_tokens=4)
    new = d.add("new", 7, 1.0, max_tokens=4)
    d.step()
    d.step()
    plan = d.plan()                      # both need a third page and none is free
    assert [r.request_id for r in plan.preempted] == ["new"] and shares(plan) == [("old", 1)]
    assert new.status == RequestStatus.WAITING and new.computed == 0 and new.num_tokens == 9
    assert (new.num_preemptions, d.sched.num_preemptions) == (1, 1)
    assert not d.cache.has_request("new") and d.sched.num_waiting == 1
    d.ran(plan)
    # "new" keeps its place in line: a later arrival does not overtake it
    d.add("later", 2, 2.0)
    d.sched.finish_request(d.sched.running[0], FinishReason.LENGTH)
    plan = d.plan()
    # it is fed again from its first token: prompt and what it generated
    assert shares(plan)[0] == ("new", 9) and plan.slices[0].start == 0 and not plan.slices[0].decode
    assert plan.slices[0].samples


def test_a_request_takes_pages_from_a_later_one_and_then_nobody_is_admitted():
    d = Driver(num_blocks=2, block_size=4, max_num_seqs=2)
    d.add("a", 4, 0.0, max_tokens=4)          # worst case 8 tokens = 2 pages
    d.add("b", 4, 1.0, max_tokens=4)
    d.step()                                   # each holds one page, the pool is full
    plan = d.plan()
    assert [r.request_id for r in plan.preempted] == ["b"] and shares(plan) == [("a", 1)]
    assert d.sched.num_waiting == 1            # b was not admitted again in the same step


def test_the_last_request_standing_gives_up_its_own_pages():
    d = Driver(num_blocks=2, block_size=4, max_num_seqs=2)
    a = d.add("a", 4, 0.0, max_tokens=4)
    d.step()
    d.cache.allocate("elsewhere", 4)           # the other page is taken by someone the scheduler does not know
    plan = d.plan()
    assert plan.is_empty and plan.preempted == [a] and a.status == RequestStatus.WAITING
    assert d.sched.has_unfinished() and not d.cache.has_request("a")


def test_the_head_of_the_line_is_not_overtaken():
    d = Driver(num_blocks=4, block_size=4, max_num_seqs=4)
    d.add("big", 13, 0.0, max_tokens=2)       # needs all four pages
    d.add("small", 2, 1.0, max_tokens=2)
    d.cache.allocate("elsewhere", 4)
    assert d.plan().is_empty
    d.cache.free("elsewhere")
    assert shares(d.plan()) == [("big", 13)]


def test_the_watermark_keeps_nobody_out_of_an_empty_pool():
    cache = CacheManager(4, [CacheGroup((0,))], 8, watermark=0.25)
    sched = Scheduler(SchedulerConfig(), cache)
    sched.add_request(Request("fills", range(30), SamplingParams(max_tokens=2), arrival_time=0.0))
    sched.add_request(Request("next", range(4), SamplingParams(max_tokens=2), arrival_time=1.0))
    plan = sched.schedule()
    # 8 pages for the first although 2 are to be kept free: nothing runs that could need them;
    # the second meets the watermark
    assert [(s.request.request_id, s.count) for s in plan.slices] == [("fills", 30)]


def test_abort_of_a_waiting_and_of_a_running_request():
    d = Driver(max_num_seqs=1)
    d.add("a", 4, 0.0)
    d.add("b", 4, 1.0)
    d.plan()
    gone = d.sched.abort_request("b")
    assert gone.status == RequestStatus.ABORTED and d.sched.num_waiting == 0
    gone = d.sched.abort_request("a")
    assert gone.finish_reason == FinishReason.ABORT and gone.clock.finished is not None
    assert not d.sched.has_unfinished() and d.cache.num_free_blocks == d.cache.num_blocks
    assert d.sched.abort_request("a") is None and d.sched.abort_request("nobody") is None


def test_commit_ends_requests_and_frees_their_pages():
    d = Driver()
    a = d.add("a", 3, 0.0, max_tokens=2)
    b = d.add("b", 3, 1.0, max_tokens=9, stop_token_ids=[7])
    done = d.ran(d.plan(), token=5)
    assert [(r.request_id, t) for r, t in done] == [("a", [5]), ("b", [5])]
    done = d.ran(d.plan(), token=7)
    assert a.finish_reason == FinishReason.LENGTH and b.finish_reason == FinishReason.STOP
    assert a.output_token_ids == [5, 7] and a.is_finished and b.is_finished
    assert not d.sched.has_unfinished() and d.cache.num_free_blocks == d.cache.num_blocks


# ---------------------------------------------------------------------- runs of decode steps
def test_runs_are_planned_only_for_decoding_requests_and_allocate_their_pages():
    d = Driver(num_blocks=64, block_size=4, run_steps=8, device_runs=lambda n: True)
    a = d.add("a", 5, 0.0, max_tokens=40)
    first = d.step()
    assert first.run_steps == 1                          # a prompt is in the step
    plan = d.plan()
    assert plan.run_steps == 8 and not plan.run_ahead
    assert len(d.cache.block_table("a")) == 4           # positions 5..12 need pages up to 13 tokens
    done = d.ran(plan, token=3)
    assert a.num_output_tokens == 9 and a.computed == 13 and done[0][1] == [3] * 8
    assert a.pending == 1 and a.decoding


def test_a_run_is_no_longer_than_the_longest_remainder_and_tokens_past_an_end_are_dropped():
    d = Driver(run_steps=8, device_runs=lambda n: True)
    a = d.add("a", 4, 0.0, max_tokens=4)
    b = d.add("b", 4, 1.0, max_tokens=6)
    d.step()
    plan = d.plan()
    assert plan.run_steps == 5           # b has five tokens left, a three
    d.ran(plan, token=1)
    assert a.finish_reason == FinishReason.LENGTH and a.num_output_tokens == 4
    assert b.finish_reason == FinishReason.LENGTH and b.num_output_tokens == 6
    assert d.cache.num_free_blocks == d.cache.num_blocks


def test_while_somebody_waits_a_run_ends_with_the_first_certain_end():
    d = Driver(run_steps=8, max_num_seqs=2, device_runs=lambda n: True)
    d.add("a", 4, 0.0, max_tokens=4)
    d.add("b", 4, 1.0, max_tokens=20)
    d.add("c", 4, 2.0, max_tokens=20)        # no sequence slot for c
    d.step()
    plan = d.plan()
    assert plan.run_steps == 3 and d.sched.num_waiting == 1
    d.ran(plan)
    assert shares(d.plan()) == [("b", 1), ("c", 4)]


def test_the_models_length_bounds_a_run_and_ends_the_request_at_the_right_token():
    d = Driver(run_steps=8, max_model_len=12, device_runs=lambda n: True)
    a = d.add("a", 6, 0.0, max_tokens=50)
    d.step()                                  # 7 tokens
    plan = d.plan()
    assert plan.run_steps == 5                # room for 12 - 7 tokens
    d.ran(plan)
    assert a.finish_reason == FinishReason.LENGTH and a.num_tokens == 12


def test_no_run_without_pages_for_all_of_it_or_when_the_device_cannot():
    d = Driver(num_blocks=3, block_size=4, run_steps=8, device_runs=lambda n: True)
    d.add("a", 7, 0.0, max_tokens=5)          # 12 tokens at most: fits the pool
    d.cache.allocate("elsewhere", 4)
    d.step()
    assert d.plan().run_steps == 1            # 8 positions more would need a third page, which is taken
    d = Driver(run_steps=8, device_runs=lambda n: False)
    d.add("a", 4, 0.0, max_tokens=30)
    d.step()
    assert d.plan().run_steps == 1
    d = Driver(run_steps=8)                   # no device to run by itself at all
    d.add("a", 4, 0.0, max_tokens=30)
    d.step()
    assert d.plan().run_steps == 1


def test_the_following_run_is_allowed_early_only_with_room_tokens_and_pages_for_both():
    d = Driver(num_blocks=64, block_size=4, run_steps=4, run_ahead=True, device_runs=lambda n: True)
    a = d.add("a", 4, 0.0, max_tokens=40)
    d.step()
    plan = d.plan()
    assert plan.run_steps == 4 and plan.run_ahead
    assert len(d.cache.block_table("a")) == 3          # positions 4..11 of both runs: 12 tokens
    d.ran(plan)
    d.add("b", 4, 1.0)                                  # somebody waits: no run ahead, and no admission
    plan = d.plan(queued_steps=4)
    assert plan.run_steps == 4 and not plan.run_ahead and d.sched.num_waiting == 1
    d.ran(plan)
    d.sched.abort_request("b")
    a.sampling_params.max_tokens = a.num_output_tokens + 4      # exactly one run left
    plan = d.plan()
    assert plan.run_steps == 4 and not plan.run_ahead


# ---------------------------------------------------------------------- the request itself
def test_when_a_request_stops():
    r = Request("a", [1, 2], SamplingParams(max_tokens=3, stop_token_ids=[9]), eos_token_id=5)
    assert r.reason_to_stop(100) is None
    r.accept(4)
    assert r.reason_to_stop(100) is None
    r.accept(5)
    assert r.reason_to_stop(100) == FinishReason.STOP           # the end-of-sequence id
    r.sampling_params.ignore_eos = True
    assert r.reason_to_stop(100) is None
    r.accept(7)
    assert r.reason_to_stop(100) == FinishReason.LENGTH         # max_tokens
    r = Request("b", [1, 2, 3], SamplingParams(max_tokens=50, stop_token_ids=[9]))
    r.accept(1)
    assert r.reason_to_stop(4) == FinishReason.LENGTH and r.reason_to_stop(5) is None
    r.accept(9)
    assert r.reason_to_stop(100) == FinishReason.STOP           # a stop token of its own


def test_the_cursor_and_what_is_pending():
    r = Request("a", [1, 2, 3], SamplingParams(max_tokens=5))
    assert (r.pending, r.decoding, r.next_tokens(2)) == (3, False, [1, 2])
    r.advance(3)
    r.accept(8)
    assert (r.pending, r.decoding, r.next_tokens(1)) == (1, True, [8])
    assert r.prompt_token_ids == [1, 2, 3] and r.output_token_ids == [8]
    r.advance(1)
    r.accept(9)
    r.rewind()
    assert (r.pending, r.decoding, r.computed) == (5, False, 0)      # all five are fed again
    assert r.next_tokens(5) == [1, 2, 3, 8, 9]
    with pytest.raises(ValueError):
        r.advance(6)
    out = r.output([9])
    assert (out.prompt_token_ids, out.output_token_ids, out.new_token_ids, out.finished) == (
        [1, 2, 3], [8, 9], [9], False)


def test_times_of_a_request():
    r = Request("a", [1], arrival_time=10.0)
    assert r.clock.time_to_first_token is None and r.clock.time_per_output_token is None
    r.accept(1, now=10.5)
    assert r.clock.time_to_first_token == 0.5 and r.clock.time_per_output_token is None
    r.accept(1, now=10.7)
    r.accept(1, now=11.1)
    assert r.clock.time_per_output_token == pytest.approx(0.3)
    r.close(FinishReason.LENGTH, now=11.5)
    assert r.clock.end_to_end == 1.5 and r.status == RequestStatus.FINISHED
