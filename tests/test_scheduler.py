"""The scheduler's decisions, driven with a stand-in for "the model ran" as the reference's own
tests do (tests/test_scheduler.py of the reference); every vector below is one of theirs."""

from __future__ import annotations

import pytest

from kvforge_amd.cache import CacheGroup, CacheManager
from kvforge_amd.config import SchedulerConfig
from kvforge_amd.engine.request import FinishReason, Request, RequestStatus
from kvforge_amd.engine.scheduler import RequestRejectedError, Scheduler
from kvforge_amd.sampling import SamplingParams


def make(num_blocks=64, block_size=4, **cfg) -> Scheduler:
    cache = CacheManager(block_size, [CacheGroup((0,), 1, 16, None)], num_blocks)
    return Scheduler(SchedulerConfig(**cfg), cache)


def req(rid, n, arrival, max_tokens=8) -> Request:
    return Request(rid, list(range(1, n + 1)), SamplingParams(max_tokens=max_tokens),
                   arrival_time=arrival)


def complete(out) -> None:
    for s in out.scheduled:
        r = s.request
        r.num_computed_tokens += s.num_new_tokens
        if r.num_computed_tokens == r.num_tokens:
            r.append_token(0)


def test_fcfs_admission_order_and_max_seqs():      # :28-35
    s = make(max_num_seqs=2)
    for i, t in enumerate([3.0, 1.0, 2.0]):
        s.add_request(req(f"r{i}", 4, t))
    out = s.schedule()
    assert [x.request.request_id for x in out.scheduled] == ["r1", "r2"]
    assert all(x.is_prefill for x in out.scheduled)
    assert s.num_running == 2 and s.num_waiting == 1


def test_prefill_then_decode_phases():             # :45-52
    s = make()
    s.add_request(req("a", 6, 0.0))
    out = s.schedule()
    assert out.scheduled[0].is_prefill and out.scheduled[0].num_new_tokens == 6
    complete(out)
    out = s.schedule()
    assert not out.scheduled[0].is_prefill and out.scheduled[0].num_new_tokens == 1


def test_token_budget_and_chunked_prefill():       # :55-67
    s = make(max_num_batched_tokens=8, enable_chunked_prefill=True)
    s.add_request(req("a", 20, 0.0))
    chunks = []
    while True:
        out = s.schedule()
        x = out.scheduled[0]
        chunks.append(x.num_new_tokens)
        complete(out)
        if not x.is_prefill or x.request.num_output_tokens:
            break
    assert chunks == [8, 8, 4] and out.num_batched_tokens <= 8


def test_decodes_are_scheduled_before_new_prefills():   # :70-77
    s = make(max_num_batched_tokens=10)
    s.add_request(req("a", 4, 0.0))
    complete(s.schedule())
    s.add_request(req("b", 30, 1.0))
    out = s.schedule()
    assert [(x.request.request_id, x.num_new_tokens) for x in out.scheduled] == [("a", 1), ("b", 9)]
    assert [x.request.request_id for x in out.decodes] == ["a"]
    assert [x.request.request_id for x in out.prefills] == ["b"]


def test_a_step_without_admission_leaves_arrivals_waiting():
    """``schedule(admit=False)`` (the engine's step that reads decode steps already queued on the
    device): the running request decodes, the arrival waits one step and is admitted the next."""
    s = make()
    s.add_request(req("a", 4, 1.0))
    complete(s.schedule())
    s.add_request(req("b", 4, 2.0))
    out = s.schedule(admit=False)
    assert [(x.request.request_id, x.num_new_tokens, x.is_prefill) for x in out.scheduled] == [("a", 1, False)]
    assert s.num_waiting == 1 and s.num_running == 1
    complete(out)
    out = s.schedule()
    assert [(x.request.request_id, x.is_prefill) for x in out.scheduled] == [("a", False), ("b", True)]
    assert s.num_waiting == 0


def test_rejections():                             # :80-89 and scheduler.py:109-129
    s = make(max_num_batched_tokens=8, enable_chunked_prefill=False)
    with pytest.raises(RequestRejectedError):
        s.add_request(req("big", 9, 0.0))
    s = make(num_blocks=2, block_size=4)
    with pytest.raises(RequestRejectedError, match="never fit"):
        s.add_request(req("a", 6, 0.0, max_tokens=8))
    s = make(max_model_len=16)
    with pytest.raises(RequestRejectedError, match="max_model_len"):
        s.add_request(req("long", 16, 0.0))
    with pytest.raises(RequestRejectedError, match="empty"):
        s.add_request(Request("e", []))
    s.add_request(req("a", 3, 0.0))
    with pytest.raises(RequestRejectedError, match="duplicate"):
        s.add_request(req("a", 3, 1.0))


def test_pages_run_out_latest_arrival_is_preempted_and_recomputes():   # :92-111
    s = make(num_blocks=4, block_size=4, max_num_seqs=4)
    s.add_request(req("old", 7, 0.0, max_tokens=4))
    s.add_request(req("new", 7, 1.0, max_tokens=4))
    complete(s.schedule())
    complete(s.schedule())
    out = s.schedule()                      # both need a third page, none is free
    assert [r.request_id for r in out.preempted] == ["new"]
    assert [x.request.request_id for x in out.scheduled] == ["old"]
    victim = out.preempted[0]
    assert victim.status == RequestStatus.WAITING and victim.num_computed_tokens == 0
    assert victim.num_preemptions == 1 and s.num_preemptions == 1
    assert not s.cache.has_request("new")
    complete(out)
    # nothing is admitted in a step that preempted; afterwards "new" waits for room
    s.finish_request(s.running[0], FinishReason.LENGTH)
    out = s.schedule()
    assert out.scheduled[0].request is victim
    assert out.scheduled[0].num_new_tokens == victim.num_tokens == 9   # prompt + generated
    assert out.scheduled[0].is_prefill


def test_a_lone_request_that_cannot_grow_preempts_itself():
    s = make(num_blocks=2, block_size=4, max_num_seqs=2)
    s.add_request(req("a", 4, 0.0, max_tokens=4))       # worst case 8 tokens = 2 pages
    s.add_request(req("b", 4, 1.0, max_tokens=4))
    complete(s.schedule())                               # each holds one page, pool is full
    out = s.schedule()
    # "a" grows by preempting "b"; then "b" cannot be admitted in the same step
    assert [r.request_id for r in out.preempted] == ["b"]
    assert [x.request.request_id for x in out.scheduled] == ["a"]


def test_head_of_line_blocking():
    s = make(num_blocks=4, block_size=4, max_num_seqs=4)
    s.add_request(req("big", 13, 0.0, max_tokens=2))    # needs 4 pages
    s.add_request(req("small", 2, 1.0, max_tokens=2))
    s.cache.allocate("other", 4)                         # one page is taken elsewhere
    out = s.schedule()
    assert out.is_empty                                  # "small" may not overtake "big"
    s.cache.free("other")
    assert [x.request.request_id for x in s.schedule().scheduled] == ["big"]


def test_abort_waiting_and_running():              # :125-134
    s = make(max_num_seqs=1)
    s.add_request(req("a", 4, 0.0))
    s.add_request(req("b", 4, 1.0))
    s.schedule()
    assert s.abort_request("b").status == RequestStatus.ABORTED
    assert s.abort_request("a").finish_reason == FinishReason.ABORT
    assert not s.has_unfinished()
    assert s.cache.num_free_blocks == s.cache.num_blocks
    assert s.abort_request("a") is None


def test_request_stop_rules():                     # batching/request.py:99-110
    r = Request("a", [1, 2], SamplingParams(max_tokens=3, stop_token_ids=[9]), eos_token_id=5)
    r.append_token(4)
    assert r.check_stop(100) is None
    r.append_token(5)
    assert r.check_stop(100) == FinishReason.STOP
    r.sampling_params.ignore_eos = True
    assert r.check_stop(100) is None
    r.append_token(7)
    assert r.check_stop(100) == FinishReason.LENGTH
    r2 = Request("b", [1, 2, 3], SamplingParams(max_tokens=50))
    r2.append_token(1)
    assert r2.check_stop(4) == FinishReason.LENGTH and r2.check_stop(5) is None
    assert r2.token_slice(2, 2) == [3, 1] and r2.token_slice(0, 2) == [1, 2] and r2.token_slice(3, 1) == [1]
