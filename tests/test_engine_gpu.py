"""Generation through the entry point (``InferenceEngine.generate`` / ``step``) against the plain
model: the reference's end-to-end tests (tests/test_continuous_batching.py:42-169 of the
reference) on this engine, plus sampling that does not depend on batching."""

from __future__ import annotations

import random

import pytest
import torch

import kvforge_amd
from kvforge_amd import (CacheConfig, EngineConfig, InferenceEngine, RequestStatus, SamplingParams,
                         SchedulerConfig)
from tests.plain import llama as plain
from tests.plain import sampling as plain_sampling

pytestmark = pytest.mark.gpu
GREEDY = SamplingParams(max_tokens=10, temperature=0.0)


class Oracle:
    """Plain greedy continuation that also reports how safe each choice was."""

    def __init__(self, folder):
        self.folder = folder
        self.w = plain.read_weights(folder)
        self.cfg = plain.read_config(folder)
        self._twins = {}

    def of(self, dtype):
        """The oracle of the same model as a ``dtype`` engine is given it (``engine_for``)."""
        from tests.replay_util import stored_as
        twin = stored_as(self.folder, dtype)
        if twin == self.folder:
            return self
        if dtype not in self._twins:
            self._twins[dtype] = Oracle(twin)
        return self._twins[dtype]

    def greedy(self, prompt, n):
        ids, out, gaps = list(prompt), [], []
        for _ in range(n):
            logits = plain.forward(self.w, self.cfg, ids)[-1]
            top = torch.topk(logits, 2).values
            gaps.append(float(top[0] - top[1]))
            out.append(int(logits.argmax()))
            ids.append(out[-1])
        return out, gaps

    def logits(self, ids):
        return plain.forward(self.w, self.cfg, ids)

    def check_choices(self, prompt, out, margin):
        """Every generated token is the plain model's argmax, given the engine's own history, up
        to ``margin`` in the logits (one plain forward covers all places, by causality)."""
        logits = self.logits(list(prompt) + list(out))
        for i, tok in enumerate(out):
            row = logits[len(prompt) - 1 + i]
            assert float(row.max() - row[tok]) <= margin, (
                f"token {i} = {tok}: plain logit {row[tok]:.5f}, best {row.max():.5f} "
                f"at {int(row.argmax())}")


def assert_greedy_equal(got, want, gaps, margin=1e-4):
    """Tokens must agree up to the first place where the plain model's top two logits are closer
    than ``margin`` (there rounding may choose either and the continuations part ways)."""
    for i, (g, w, gap) in enumerate(zip(got, want, gaps)):
        if gap < margin:
            return
        assert g == w, f"token {i}: engine {g}, plain {w} (gap {gap:.2e}); got {got}, want {want}"
    assert len(got) == len(want)


@pytest.fixture(scope="module")
def model_a_flat(tmp_path_factory):
    """Tiny A exactly as the baseline configuration words it: N(0, 0.02) weights, tied head.
    Its greedy output repeats the prompt's last token whatever the context, so only the test of
    that configuration uses it."""
    folder = str(tmp_path_factory.mktemp("tiny_a_flat"))
    kvforge_amd.write_random_model(folder, kvforge_amd.preset_dict("tiny-a"), seed=0, dtype="float32")
    return folder, Oracle(folder)


@pytest.fixture(scope="module")
def model_a(tmp_path_factory):
    """Tiny A with peaked attention and layer outputs that outweigh the embedding: its next
    token depends on what the cache holds (checked here for the kinds of prompt the tests use),
    so a test of generated tokens fails on a broken cache."""
    from tests.replay_util import context_matters, liven
    folder = str(tmp_path_factory.mktemp("tiny_a"))
    kvforge_amd.write_random_model(folder, kvforge_amd.preset_dict("tiny-a"), seed=0, dtype="float32")
    liven(folder)
    assert context_matters(folder, prompts_for(256, 6, 2) + prompts_for(256, 4, 1)
                           + [list(range(1, 60)), list(range(100, 140)), [7, 7, 7], [5, 17, 3]])
    return folder, Oracle(folder)


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    folder = str(tmp_path_factory.mktemp("tiny_b"))
    kvforge_amd.write_random_model(folder, kvforge_amd.preset_dict("tiny-b"), seed=1, dtype="float32")
    return folder, Oracle(folder)


def engine_for(folder, dtype="float32", block_size=4, num_blocks=256, max_num_seqs=8,
               max_num_batched_tokens=256, **kw):
    cfg = EngineConfig(cache=CacheConfig(block_size=block_size, num_blocks=num_blocks),
                       scheduler=SchedulerConfig(max_num_seqs=max_num_seqs,
                                                 max_num_batched_tokens=max_num_batched_tokens),
                       dtype=dtype, **kw)
    # the fixtures' folders store 32-bit weights, which a float32 engine is to meet; a bfloat16
    # engine gets the same model stored in bfloat16 (``Oracle.of`` gives the oracle of that)
    from tests.replay_util import stored_as
    return InferenceEngine.from_folder(stored_as(folder, dtype), cfg)


def prompts_for(vocab, n, seed, lo=2, hi=30):
    rng = random.Random(seed)
    return [[rng.randrange(1, vocab) for _ in range(rng.randint(lo, hi))] for _ in range(n)]


def test_baseline_config_a(model_a_flat):
    """Tiny Llama A, fp32, seed 0, block 16: prompts of 5/17/33 tokens, greedy, 16 new each."""
    folder, oracle = model_a_flat
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, 256, (n,), generator=g).tolist() for n in (5, 17, 33)]
    engine = engine_for(folder, block_size=16, num_blocks=64)
    outs = engine.generate(prompts, SamplingParams(max_tokens=16, temperature=0.0))
    for p, o in zip(prompts, outs):
        want, gaps = oracle.greedy(p, 16)
        assert_greedy_equal(o.output_token_ids, want, gaps)
        assert o.finish_reason.value == "length" and o.prompt_token_ids == p


def test_baseline_config_b_chunked_temperature(model_b):
    """Tiny Llama B, fp32, seed 1, block 8: prompts of 1/9/40/70 tokens, chunk 24 mixed with
    decodes, temperature 0.8, 12 new.  Every sampled token must be the plain rule's draw from the
    plain model's logits of the engine's own token history."""
    folder, oracle = model_b
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, 384, (n,), generator=g).tolist() for n in (1, 9, 40, 70)]
    engine = engine_for(folder, block_size=8, num_blocks=64, max_num_batched_tokens=24, seed=1)
    params = SamplingParams(max_tokens=12, temperature=0.8)
    outs = engine.generate(prompts, params)
    assert max(engine.metrics.batch_sizes) >= 2 and max(engine.metrics.batched_tokens) <= 24
    for stream, (p, o) in enumerate(zip(prompts, outs)):
        assert len(o.output_token_ids) == 12
        logits = oracle.logits(p + o.output_token_ids)
        for i, tok in enumerate(o.output_token_ids):
            probs = plain_sampling.processed_probs(logits[len(p) - 1 + i], 0.8)
            u = plain_sampling.uniform(1, stream, i)
            assert plain_sampling.draw_margin(probs, u, tok) < 1e-4, (stream, i, tok)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batched_output_equals_isolated_greedy(model_a, dtype):
    folder, oracle = model_a
    prompts = prompts_for(256, 6, 0)
    engine = engine_for(folder, dtype)
    outs = engine.generate(prompts, GREEDY)
    for p, o in zip(prompts, outs):
        assert len(o.output_token_ids) == 10
        if dtype == "float32":
            want, gaps = oracle.greedy(p, 10)
            assert_greedy_equal(o.output_token_ids, want, gaps)
            oracle.check_choices(p, o.output_token_ids, 1e-4)
        else:
            oracle.of("bfloat16").check_choices(p, o.output_token_ids, 3e-2)


def test_requests_join_running_batch(model_a):
    folder, oracle = model_a
    prompts = prompts_for(256, 4, 1)
    engine = engine_for(folder, decode_run_steps=1)   # the test counts steps of one token
    engine.add_request(prompts[0], GREEDY, request_id="r0")
    engine.add_request(prompts[1], GREEDY, request_id="r1")
    done, step = {}, 0
    while engine.has_unfinished_requests():
        if step == 3:
            engine.add_request(prompts[2], GREEDY, request_id="r2")
        if step == 5:
            engine.add_request(prompts[3], GREEDY, request_id="r3")
        if step == 4:
            assert engine.scheduler.num_running == 3
        for out in engine.step():
            if out.finished:
                done[out.request_id] = out.output_token_ids
        step += 1
    for i, p in enumerate(prompts):
        want, gaps = oracle.greedy(p, 10)
        assert_greedy_equal(done[f"r{i}"], want, gaps)
    assert max(engine.metrics.batch_sizes) >= 3


def test_short_requests_leave_early_and_free_pages(model_a):
    folder, _ = model_a
    engine = engine_for(folder)
    engine.add_request([1, 2, 3], SamplingParams(max_tokens=2, temperature=0), request_id="short")
    engine.add_request([4, 5, 6], SamplingParams(max_tokens=12, temperature=0), request_id="long")
    finished_at, step = {}, 0
    while engine.has_unfinished_requests():
        for o in engine.step():
            if o.finished:
                finished_at[o.request_id] = step
        step += 1
    assert finished_at["short"] < finished_at["long"]
    assert engine.cache.num_free_blocks == engine.cache.num_blocks


def test_pages_run_out_preemption_preserves_outputs(model_a):
    folder, oracle = model_a
    prompts = prompts_for(256, 6, 2)
    engine = engine_for(folder, num_blocks=14, max_num_seqs=6, max_num_batched_tokens=64)
    outs = engine.generate(prompts, GREEDY)
    assert engine.scheduler.num_preemptions > 0
    for p, o in zip(prompts, outs):
        want, gaps = oracle.greedy(p, 10)
        assert_greedy_equal(o.output_token_ids, want, gaps)
        oracle.check_choices(p, o.output_token_ids, 1e-4)
    assert engine.cache.num_free_blocks == engine.cache.num_blocks


def test_a_preempted_request_is_fed_again_into_pages_others_have_used(model_a):
    """Two requests outgrow a pool of six pages: the later one loses its pages in the middle of
    decoding, the earlier one grows into them, and the later one comes back under its own id,
    is fed prompt and generated tokens again into pages that held the other's keys, and goes
    on.  Every token of both is the plain model's choice."""
    folder, oracle = model_a
    prompts = [[9, 200, 31, 77, 5, 150, 42], [120, 8, 66, 201, 13, 90, 3]]
    params = SamplingParams(max_tokens=12, temperature=0.0)
    engine = engine_for(folder, block_size=4, num_blocks=6, max_num_seqs=2, decode_run_steps=1)
    ids = [engine.add_request(p, params) for p in prompts]
    second = engine.scheduler.requests[ids[1]]
    outs, seen_back = {}, False
    while engine.has_unfinished_requests():
        for o in engine.step():
            outs[o.request_id] = o
        if second.num_preemptions and second.status == RequestStatus.RUNNING and not second.is_finished:
            seen_back = True
    assert second.num_preemptions >= 1 and seen_back
    for rid, p in zip(ids, prompts):
        assert len(outs[rid].output_token_ids) == 12
        oracle.check_choices(p, outs[rid].output_token_ids, 1e-4)
        want, gaps = oracle.greedy(p, 12)
        assert_greedy_equal(outs[rid].output_token_ids, want, gaps)
    assert engine.cache.num_free_blocks == engine.cache.num_blocks


def test_without_chunked_prefill_a_preempted_request_that_outgrew_the_budget_goes_on(model_a):
    """Chunked prefill off, eight tokens a step, five pages of four: the second of two 7-token
    prompts loses its pages after it has grown past eight tokens, so what it has to be fed again
    no longer fits a step.  It is fed in portions (the reference would leave it at the head of
    the line for ever, src/tokenvault/scheduler.py:109-129 against :206-207), ``generate``
    returns, and every token of both requests is the plain model's choice."""
    folder, oracle = model_a
    prompts = [[9, 200, 31, 77, 5, 150, 42], [120, 8, 66, 201, 13, 90, 3]]
    cfg = EngineConfig(cache=CacheConfig(block_size=4, num_blocks=5),
                       scheduler=SchedulerConfig(max_num_seqs=2, max_num_batched_tokens=8,
                                                 enable_chunked_prefill=False),
                       dtype="float32", decode_run_steps=1)
    engine = InferenceEngine.from_folder(folder, cfg)
    outs = engine.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0))
    assert engine.scheduler.num_preemptions >= 1 and max(engine.metrics.batched_tokens) <= 8
    assert [len(o.output_token_ids) for o in outs] == [12, 12]
    for p, o in zip(prompts, outs):
        oracle.check_choices(p, o.output_token_ids, 1e-4)
        want, gaps = oracle.greedy(p, 12)
        assert_greedy_equal(o.output_token_ids, want, gaps)
    assert engine.cache.num_free_blocks == engine.cache.num_blocks


def test_generate_raises_when_nothing_can_be_planned(model_a, monkeypatch):
    """A scheduler that plans nothing while requests wait would make ``generate`` ask for ever;
    it raises instead (forced here by a scheduler that refuses to admit)."""
    folder, _ = model_a
    engine = engine_for(folder)
    monkeypatch.setattr(engine.scheduler, "_admit", lambda plan, budget: None)
    with pytest.raises(RuntimeError, match="stuck"):
        engine.generate([[5, 17, 3]], GREEDY)


@pytest.mark.parametrize("budget", [16, 24])
def test_chunked_prefill_preserves_outputs(model_a, budget):
    folder, oracle = model_a
    prompts = [list(range(1, 60)), list(range(100, 140))]
    engine = engine_for(folder, max_num_batched_tokens=budget)
    outs = engine.generate(prompts, GREEDY)
    assert max(engine.metrics.batched_tokens) <= budget
    for p, o in zip(prompts, outs):
        want, gaps = oracle.greedy(p, 10)
        assert_greedy_equal(o.output_token_ids, want, gaps)


def test_abort_mid_generation(model_a):
    folder, _ = model_a
    engine = engine_for(folder)
    rid = engine.add_request([1, 2, 3], SamplingParams(max_tokens=50))
    engine.step()
    engine.step()
    req = engine.scheduler.requests[rid]
    assert req.status == RequestStatus.RUNNING and req.num_output_tokens >= 2
    assert engine.abort_request(rid)
    assert req.status == RequestStatus.ABORTED and not engine.has_unfinished_requests()
    assert engine.stats()["metrics"]["requests_aborted"] == 1
    assert engine.cache.num_free_blocks == engine.cache.num_blocks
    assert not engine.abort_request(rid)


def test_stop_token_and_metrics(model_a):
    folder, oracle = model_a
    want, gaps = oracle.greedy([7, 7, 7], 10)
    # a token that first appears some way into the output, so that stopping there is an event
    at = next(i for i in range(2, 10) if want[i] not in want[:i])
    assert min(gaps[:at + 1]) > 1e-4
    stop = want[at]
    engine = engine_for(folder)
    out = engine.generate([[7, 7, 7]], SamplingParams(max_tokens=10, temperature=0,
                                                      stop_token_ids=[stop]))[0]
    assert out.output_token_ids == want[:at + 1] and len(out.output_token_ids) >= 3
    assert out.finish_reason.value == "stop"
    stats = engine.stats()
    m = stats["metrics"]
    assert m["requests_finished"] == 1 and m["output_tokens_per_s"] > 0 and m["ttft_p50_ms"] > 0
    assert stats["forward_passes"] == engine.runner.num_forward_passes > 0
    assert stats["kv_cache"]["num_free_blocks"] == stats["kv_cache"]["num_blocks"]
    # what a decode step reads: every tensor of the checkpoint once (fp32 here), except an
    # embedding table that no head shares (only the batch's rows of it are read)
    tensors = plain.read_weights(folder)
    every = sum(t.numel() * 4 for t in tensors.values())
    untied = sum(t.numel() * 4 for n, t in tensors.items() if n.endswith("embed_tokens.weight")
                 and "lm_head.weight" in tensors)
    assert stats["weights_bytes"] == every - untied
    assert stats["weights_bytes_resident"] == every       # fp32: one copy of every tensor


def test_sampling_does_not_depend_on_batching(model_b):
    """The same request, alone and inside a busy chunked batch, draws the same tokens: the
    uniform numbers are keyed by (seed, request stream, output index), not by batch order."""
    folder, _ = model_b
    target = list(range(3, 40))
    params = SamplingParams(max_tokens=12, temperature=0.8, top_k=50, top_p=0.9, seed=77)
    alone = engine_for(folder, block_size=8, seed=5).generate([target], params)[0].output_token_ids
    others = prompts_for(384, 5, 9, 10, 60)
    busy = engine_for(folder, block_size=8, seed=5, max_num_batched_tokens=24)
    outs = busy.generate(others[:3] + [target] + others[3:],
                         [SamplingParams(max_tokens=9, temperature=1.0)] * 3 + [params]
                         + [SamplingParams(max_tokens=20, temperature=0.0)] * 2)
    assert outs[3].output_token_ids == alone
    again = engine_for(folder, block_size=8, seed=5).generate([target], params)[0].output_token_ids
    other_seed = engine_for(folder, block_size=8, seed=6).generate([target], params)[0].output_token_ids
    assert again == alone and other_seed != alone


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_runs_of_decode_steps_on_the_device_equal_single_steps(model_b, dtype):
    """With nothing waiting the device takes several decode steps before the host looks (each
    sampled token becomes the next input there).  Tokens, stop handling, lengths that are no
    multiple of the run, pages that begin inside a run and freed pages must all be what single
    steps give, for greedy and for drawn tokens."""
    folder, oracle = model_b
    prompts = prompts_for(384, 4, 21, 3, 40)
    params = [SamplingParams(max_tokens=21, temperature=0.0),
              SamplingParams(max_tokens=13, temperature=0.9, top_k=40, top_p=0.95, seed=3),
              SamplingParams(max_tokens=30, temperature=0.0),
              SamplingParams(max_tokens=5, temperature=1.0, seed=4)]
    single = engine_for(folder, dtype, decode_run_steps=1, seed=2)
    want = single.generate(prompts, params)
    for run in (2, 8, 16):
        engine = engine_for(folder, dtype, decode_run_steps=run, seed=2)
        got = engine.generate(prompts, params)
        for g, w in zip(got, want):
            assert g.output_token_ids == w.output_token_ids and g.finish_reason == w.finish_reason
        assert engine.runner.num_forward_passes < single.runner.num_forward_passes + 4 * run
        assert engine.cache.num_free_blocks == engine.cache.num_blocks
    if dtype == "float32":
        oracle.check_choices(prompts[0], want[0].output_token_ids, 1e-4)
        oracle.check_choices(prompts[2], want[2].output_token_ids, 1e-4)
    # a stop token inside a run: what the device sampled after it is dropped
    stop = want[2].output_token_ids[10]
    first = want[2].output_token_ids.index(stop)
    engine = engine_for(folder, dtype, decode_run_steps=8, seed=2)
    out = engine.generate([prompts[2]], SamplingParams(max_tokens=30, temperature=0.0,
                                                      stop_token_ids=[stop]))[0]
    assert out.output_token_ids == want[2].output_token_ids[:first + 1]
    assert out.finish_reason == "stop"
    assert engine.cache.num_free_blocks == engine.cache.num_blocks


def test_runs_go_on_while_blocked_requests_wait(model_a):
    """Six requests over two sequence slots: those that wait cannot be admitted before a running
    one ends, so the device keeps taking steps by itself up to the first end that is certain (the
    fewest tokens left), and the slot is filled in the very next step, as with single steps:
    same tokens, same number of model steps, far fewer looks of the host."""
    folder, oracle = model_a
    prompts = prompts_for(256, 6, 8, 3, 12)
    params = [SamplingParams(max_tokens=n, temperature=0.0) for n in (20, 9, 17, 12, 25, 6)]

    def run(steps):
        engine = engine_for(folder, "float32", max_num_seqs=2, decode_run_steps=steps)
        ids = [engine.add_request(p, sp) for p, sp in zip(prompts, params)]
        outs, looks = {}, 0
        while engine.has_unfinished_requests():
            for o in engine.step():
                outs[o.request_id] = o.output_token_ids
            looks += 1
        assert engine.cache.num_free_blocks == engine.cache.num_blocks
        return [outs[i] for i in ids], looks, engine

    want, single_looks, single = run(1)
    got, looks, engine = run(8)
    assert got == want and [len(t) for t in got] == [20, 9, 17, 12, 25, 6]
    assert engine.runner.num_forward_passes == single.runner.num_forward_passes
    assert looks < single_looks // 2
    oracle.check_choices(prompts[4], got[4], 1e-4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_runs_queued_ahead_give_the_same_tokens(model_b, dtype):
    """While decode runs follow each other for the same requests the next run is queued before
    the current one is read.  Whatever ends that (a length reached, a stop token, a request that
    arrives, one that is aborted), the tokens are those of an engine that never queues ahead, no
    page is lost, and runs were in fact queued and read."""
    folder, _ = model_b
    prompts = prompts_for(384, 4, 33, 3, 40)
    params = [SamplingParams(max_tokens=70, temperature=0.0),
              SamplingParams(max_tokens=41, temperature=0.9, top_k=40, top_p=0.95, seed=3),
              SamplingParams(max_tokens=64, temperature=0.0),
              SamplingParams(max_tokens=23, temperature=1.0, seed=4)]

    # In fp32 a token does not depend on what else is in its batch, so requests may arrive while
    # others decode (with runs queued ahead they are admitted one run later); in bf16 the
    # batches have to be the same with and without queueing, so all requests are there at once.
    arrivals = dtype == "float32"

    def scenario(engine, stop=None):
        """Two requests; a third arrives after a few steps, a fourth later and is aborted."""
        ps = list(params)
        if stop is not None:
            ps[0] = SamplingParams(max_tokens=70, temperature=0.0, stop_token_ids=[stop])
        ids = [engine.add_request(prompts[0], ps[0]), engine.add_request(prompts[1], ps[1])]
        if not arrivals:
            ids += [engine.add_request(prompts[2], ps[2]), engine.add_request(prompts[3], ps[3])]
        outs, steps = {}, 0
        while engine.has_unfinished_requests():
            for o in engine.step():
                outs[o.request_id] = o
            steps += 1
            if steps == 3 and arrivals:
                ids.append(engine.add_request(prompts[2], ps[2]))
            if steps == 5 and arrivals:
                ids.append(engine.add_request(prompts[3], ps[3]))
            if steps == 7:
                engine.abort_request(ids[3])
        assert engine.cache.num_free_blocks == engine.cache.num_blocks
        return [(outs[i].output_token_ids, outs[i].finish_reason) for i in ids[:3]]

    for run in (4, 8):
        plain_engine = engine_for(folder, dtype, decode_run_steps=run, decode_run_ahead=False, seed=2)
        want = scenario(plain_engine)
        assert plain_engine.runner.num_runs_queued_ahead == 0
        engine = engine_for(folder, dtype, decode_run_steps=run, decode_run_ahead=True, seed=2)
        got = scenario(engine)
        assert got == want
        # every queued run was read: by all of its requests, or by those that were left
        assert engine.runner.num_runs_read_ahead == engine.runner.num_runs_queued_ahead >= 3
    # a stop token met while the next run is queued already
    stop = want[0][0][37]
    cut = want[0][0].index(stop)
    engine = engine_for(folder, dtype, decode_run_steps=8, decode_run_ahead=True, seed=2)
    got = scenario(engine, stop)
    assert got[0] == (want[0][0][:cut + 1], "stop")
    plain_stop = scenario(engine_for(folder, dtype, decode_run_steps=8, decode_run_ahead=False, seed=2), stop)
    assert got == plain_stop
    # more steps in a run than half the ring holds: nothing is queued ahead
    engine = engine_for(folder, dtype, decode_run_steps=16, decode_run_ahead=True, seed=2)
    scenario(engine)
    assert engine.runner.num_runs_queued_ahead == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_layers_give_pages_back_while_runs_go_on(tmp_path, dtype):
    """Two kinds of layer (all keys; the last 24): pages behind the window go back to the pool
    while the request lives, also when the device takes runs of steps by itself and the next run
    is queued before the host has read the current one.  Tokens are the plain model's choices
    (fp32) and the same however the steps are run."""
    from tests.replay_util import TINY_C, sharpen
    folder = str(tmp_path / "c")
    kvforge_amd.write_random_model(folder, TINY_C, seed=3, dtype="float32")
    sharpen(folder, 6.0)
    oracle = Oracle(folder)
    prompts = prompts_for(200, 3, 8, 20, 60)
    params = SamplingParams(max_tokens=90, temperature=0.0)
    results = []
    for kw in (dict(decode_run_steps=1), dict(decode_run_steps=8, decode_run_ahead=False),
               dict(decode_run_steps=8, decode_run_ahead=True)):
        engine = engine_for(folder, dtype, block_size=4, num_blocks=160, **kw)
        ids = [engine.add_request(p, params) for p in prompts]
        windowed = [g.window is not None for g in engine.cache.groups]
        assert sorted(windowed) == [False, True]
        outs, peak = {}, [0, 0]
        while engine.has_unfinished_requests():
            for o in engine.step():
                outs[o.request_id] = o
            peak = [max(p, pool.num_used) for p, pool in zip(peak, engine.cache.pools)]
        # the group that keeps every key grows with the requests, the other stays near its window
        assert peak[windowed.index(True)] < peak[windowed.index(False)] // 2
        assert engine.cache.num_free_blocks == engine.cache.num_blocks
        results.append([outs[i].output_token_ids for i in ids])
        if kw.get("decode_run_ahead"):
            assert engine.runner.num_runs_read_ahead > 0
    assert results[1] == results[0] and results[2] == results[0]
    if dtype == "float32":
        for p, out in zip(prompts, results[0]):
            oracle.check_choices(p, out, 1e-4)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_traffic_gives_the_same_tokens_however_it_is_run(model_a, seed):
    """Requests of random lengths arrive at random steps into a pool so small that some are
    preempted; some carry stop tokens, two are aborted.  In fp32 a token does not depend on its
    batch as long as the step's rows stay on one side of the 32 rows at which the 32-bit product
    changes its order of summation (they do here: at most 8 sequences), so every way of running (single steps, runs, runs queued ahead) must give every
    request the same tokens and the same end, and give every page back."""
    folder, oracle = model_a
    rng = random.Random(seed)
    n = 12
    prompts = prompts_for(256, n, 100 + seed, 1, 30)
    params = [SamplingParams(max_tokens=rng.randint(1, 40), temperature=rng.choice([0.0, 0.0, 0.8]),
                             top_k=rng.choice([0, 20]), seed=7,
                             stop_token_ids=rng.sample(range(256), rng.choice([0, 0, 12])))
              for _ in range(n)]
    arrive = sorted(rng.randint(0, 25) for _ in range(n))
    aborted = {rng.randrange(n): rng.randint(3, 30), rng.randrange(n): rng.randint(3, 30)}

    def run(**kw):
        engine = engine_for(folder, "float32", block_size=4, num_blocks=26, max_num_seqs=6,
                            max_num_batched_tokens=32, seed=5, **kw)
        ids, outs, step = {}, {}, 0
        while len(ids) < n or engine.has_unfinished_requests():
            for i in range(n):
                if i not in ids and arrive[i] <= step:
                    ids[i] = engine.add_request(prompts[i], params[i])
            for i, when in aborted.items():
                if when == step and i in ids:
                    engine.abort_request(ids[i])
            for o in engine.step():
                outs[o.request_id] = o
            step += 1
            assert step < 2000
        assert engine.cache.num_free_blocks == engine.cache.num_blocks
        return ({i: (outs[ids[i]].output_token_ids, outs[ids[i]].finish_reason)
                 for i in range(n) if i not in aborted and ids[i] in outs}, engine)

    want, single = run(decode_run_steps=1)
    assert len(want) >= n - 2
    # the single-step run is held to the plain model: greedy requests by their choices, drawn
    # ones by the plain sampling rule on the plain logits of their own history
    for i, (tokens, _) in want.items():
        if params[i].greedy:
            oracle.check_choices(prompts[i], tokens, 1e-4)
        else:
            logits = oracle.logits(prompts[i] + tokens)
            for j, tok in enumerate(tokens):
                probs = plain_sampling.processed_probs(logits[len(prompts[i]) - 1 + j],
                                                       params[i].temperature, params[i].top_k)
                u = plain_sampling.uniform(5, 7, j)
                assert plain_sampling.draw_margin(probs, u, tok) < 1e-4, (i, j, tok)
    saw_ahead = 0
    for kw in (dict(decode_run_steps=8, decode_run_ahead=False), dict(decode_run_steps=8, decode_run_ahead=True),
               dict(decode_run_steps=3, decode_run_ahead=True)):
        got, engine = run(**kw)
        assert got == want, kw
        saw_ahead += engine.runner.num_runs_read_ahead
    assert single.scheduler.num_preemptions > 0 or seed != 0   # the pool is meant to run out
    assert saw_ahead > 0                                        # and runs are meant to be queued ahead


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_the_heads_greedy_pick_gives_the_tokens_of_logits_and_argmax(model_a, seed):
    """Captured steps whose rows are all greedy end in the head's own kernel: no logits, the
    next inputs and embeddings made there.  The product's sums are those of the kernel that
    stores logits, so every token must be the one that the stored logits' largest entry names:
    random traffic in bf16 (requests of random lengths arriving while others decode, long
    prompts that make the workspace grow, token limits and stop tokens that cut runs short, a
    pool that runs out) through an engine with the pick and one without it."""
    folder, oracle = model_a
    rng = random.Random(40 + seed)
    n = 10
    prompts = [prompts_for(256, 1, 300 + seed * 20 + i, lo, hi)[0]
               for i, (lo, hi) in enumerate([(1, 12)] * 6 + [(60, 110)] * 2 + [(1, 30)] * 2)]
    rng.shuffle(prompts)
    params = [SamplingParams(max_tokens=rng.randint(1, 45), temperature=0.0,
                             stop_token_ids=rng.sample(range(256), rng.choice([0, 0, 10])))
              for _ in range(n)]
    arrive = sorted(rng.randint(0, 14) for _ in range(n))

    def run(with_pick):
        engine = engine_for(folder, "bfloat16", block_size=4, num_blocks=80, max_num_seqs=4,
                            max_num_batched_tokens=128, seed=5)
        assert engine.runner._tail is not None
        if not with_pick:
            engine.runner._tail = None
        ids, outs, step = {}, {}, 0
        while len(ids) < n or engine.has_unfinished_requests():
            for i in range(n):
                if i not in ids and arrive[i] <= step:
                    ids[i] = engine.add_request(prompts[i], params[i])
            for o in engine.step():
                outs[o.request_id] = o
            step += 1
            assert step < 2000
        assert engine.cache.num_free_blocks == engine.cache.num_blocks
        return [(outs[ids[i]].output_token_ids, outs[ids[i]].finish_reason) for i in range(n)], engine

    want, plain_engine = run(False)
    got, engine = run(True)
    assert engine.runner.num_greedy_tails > 20 and plain_engine.runner.num_greedy_tails == 0
    assert got == want
    for i, (tokens, _) in enumerate(got):
        oracle.of("bfloat16").check_choices(prompts[i], tokens, 3e-2)


@pytest.mark.parametrize("use_graphs", [True, False])
def test_an_id_used_again_brings_its_own_sampling_parameters(model_b, use_graphs):
    """Request "a" runs greedy to its end; then "a" again, alone, with a temperature, then once
    more greedy.  Each must be what a fresh engine gives for those parameters: the rows of
    sampling parameters that the captured decode path keeps on the device are keyed by who sits
    in them, not by the id's string."""
    folder, oracle = model_b
    prompt = [3, 14, 15, 92, 65, 35]
    greedy = SamplingParams(max_tokens=9, temperature=0.0)
    drawn = SamplingParams(max_tokens=9, temperature=0.8, seed=11)

    def run_a(engine, params):
        engine.add_request(prompt, params, request_id="a")
        final = None
        while engine.has_unfinished_requests():
            for o in engine.step():
                final = o
        assert final.request_id == "a" and final.finished
        return final.output_token_ids

    def fresh():
        return engine_for(folder, block_size=8, seed=4, use_graphs=use_graphs)

    want_greedy, want_drawn = run_a(fresh(), greedy), run_a(fresh(), drawn)
    assert want_greedy != want_drawn
    oracle.check_choices(prompt, want_greedy, 1e-4)
    engine = fresh()
    for params, want in ((greedy, want_greedy), (drawn, want_drawn), (greedy, want_greedy),
                         (drawn, want_drawn)):
        assert run_a(engine, params) == want, params


@pytest.mark.parametrize("run", [1, 8])
def test_the_models_length_ends_a_request_inside_a_run(model_b, run):
    """``max_model_len`` 40: a request of 29 prompt tokens that asks for 50 more ends with
    ``length`` after the 11th, whether the device takes its decode steps one by one or in runs
    (the last run is cut to the room that is left)."""
    folder, oracle = model_b
    prompt = prompts_for(384, 1, 77, 29, 29)[0]
    cfg = EngineConfig(cache=CacheConfig(block_size=8, num_blocks=32),
                       scheduler=SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=64, max_model_len=40),
                       dtype="float32", decode_run_steps=run)
    engine = InferenceEngine.from_folder(folder, cfg)
    out = engine.generate([prompt], SamplingParams(max_tokens=50, temperature=0.0))[0]
    assert out.finish_reason.value == "length" and len(prompt) + len(out.output_token_ids) == 40
    oracle.check_choices(prompt, out.output_token_ids, 1e-4)
    assert engine.cache.num_free_blocks == engine.cache.num_blocks
    if run > 1:
        assert engine.runner.num_graph_replays > 0


def test_more_requests_than_the_captured_decode_path_takes(model_b):
    """140 requests decode together: beyond the largest captured batch (128) every step is
    launched kernel by kernel; as requests end the batch falls below it and the captured path
    takes over.  All tokens are the plain model's choices within bf16 rounding."""
    from kvforge_amd.engine.runner import GRAPH_MAX_BATCH
    folder, oracle = model_b
    n = GRAPH_MAX_BATCH + 12
    prompts = prompts_for(384, n, 31, 2, 12)
    params = [SamplingParams(max_tokens=4 + (i % 9), temperature=0.0) for i in range(n)]
    cfg = EngineConfig(cache=CacheConfig(block_size=8, num_blocks=1024),
                       scheduler=SchedulerConfig(max_num_seqs=n, max_num_batched_tokens=2048),
                       dtype="bfloat16")
    from tests.replay_util import stored_as
    engine = InferenceEngine.from_folder(stored_as(folder, "bfloat16"), cfg)
    outs = engine.generate(prompts, params)
    assert max(engine.metrics.batch_sizes) == n and engine.runner.num_graph_replays > 0
    assert [len(o.output_token_ids) for o in outs] == [p.max_tokens for p in params]
    for i in range(0, n, 7):
        oracle.of("bfloat16").check_choices(prompts[i], outs[i].output_token_ids, 3e-2)
    assert engine.cache.num_free_blocks == engine.cache.num_blocks


def test_a_model_stored_in_two_files_generates_the_same_tokens(model_b, tmp_path):
    import shutil
    from kvforge_amd.weights import write_safetensors
    folder, oracle = model_b
    sharded = str(tmp_path / "sharded")
    shutil.copytree(folder, sharded)
    write_safetensors(sharded, plain.read_weights(folder), shards=2)
    prompts = prompts_for(384, 3, 5, 4, 30)
    want = [o.output_token_ids for o in engine_for(folder, block_size=8).generate(prompts, GREEDY)]
    got = [o.output_token_ids for o in engine_for(sharded, block_size=8).generate(prompts, GREEDY)]
    assert got == want
    oracle.check_choices(prompts[2], got[2], 1e-4)


def test_rejections_at_the_entry_point(model_a):
    folder, _ = model_a
    engine = engine_for(folder)
    with pytest.raises(ValueError, match="vocabulary"):
        engine.add_request([1, 999])
    with pytest.raises(ValueError, match="tokenizer"):
        engine.add_request("text")
    with pytest.raises(ValueError):
        engine.add_request([])
    with pytest.raises(ValueError, match="max_model_len"):
        engine.add_request(list(range(128)))     # max_position_embeddings of tiny-a


def test_long_decoding(model_b):
    """200 tokens decoded from a short prompt in bfloat16 and float32 stay on the plain model's
    greedy path wherever that path is safe."""
    folder, oracle = model_b
    prompt = [11, 45, 200, 3]
    want, gaps = oracle.greedy(prompt, 200)
    for dtype, margin in (("float32", 1e-4), ("bfloat16", 3e-2)):
        engine = engine_for(folder, dtype, block_size=8)
        out = engine.generate([prompt], SamplingParams(max_tokens=200, temperature=0.0))[0]
        assert len(out.output_token_ids) == 200
        oracle.of(dtype).check_choices(prompt, out.output_token_ids, margin)
        if dtype == "float32":
            assert_greedy_equal(out.output_token_ids, want, gaps, margin)


def test_captured_greedy_steps_after_the_workspace_has_grown(model_a):
    """A captured step that ends in the head's greedy pick finds its first embeddings where the
    step before left them, or where the host's embedding of a new run's first token put them:
    both must be the memory the graph was recorded with, also after a long prompt has made the
    workspace's buffers grow.  One request decodes alone (the graph is recorded while the buffers
    are small), a long prompt passes through, and another request decodes alone through the
    same graph."""
    folder, oracle = model_a
    greedy = SamplingParams(max_tokens=14, temperature=0.0)

    def run(long_prompt_between):
        engine = engine_for(folder, "bfloat16", num_blocks=128, max_num_seqs=4, max_num_batched_tokens=256)
        assert engine.runner.use_graphs and engine.model.can_pick(1)
        first = engine.generate([[5, 17, 3, 11, 2, 40]], greedy)[0].output_token_ids
        tails = engine.runner.num_greedy_tails
        assert tails > 0
        if long_prompt_between:
            engine.generate([prompts_for(256, 1, 9, 100, 100)[0]], SamplingParams(max_tokens=1, temperature=0.0))
        second = engine.generate([[9, 8, 7, 6]], greedy)[0].output_token_ids    # no longer than the first
        assert engine.runner.num_greedy_tails > tails and len(engine.runner.graphs) == 1
        return first, second

    # the same kernels either way: the same tokens, whatever passed through in between
    assert run(True) == run(False)
    for prompt, out in zip(([5, 17, 3, 11, 2, 40], [9, 8, 7, 6]), run(True)):
        oracle.of("bfloat16").check_choices(prompt, out, 3e-2)
        assert out != [prompt[-1]] * 14


def test_command_line(model_a, capsys):
    from kvforge_amd import generate
    folder, oracle = model_a
    rc = generate.main(["--model", folder, "--prompt-ids", "5,17,3", "--prompt-ids", "9 8 7 6",
                        "--max-tokens", "6", "--temperature", "0", "--block-size", "4",
                        "--num-blocks", "32", "--json"])
    assert rc == 0
    import json
    rec = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    for p, o in zip(([5, 17, 3], [9, 8, 7, 6]), rec["outputs"]):
        want, gaps = oracle.greedy(p, 6)
        assert_greedy_equal(o["output_token_ids"], want, gaps)
        oracle.check_choices(p, o["output_token_ids"], 1e-4)
        assert o["output_token_ids"] != [p[-1]] * 6
    assert rec["stats"]["kv_cache"]["num_blocks"] == 32


def test_command_line_with_text_and_the_folders_own_tokenizer(model_a, capsys, tmp_path):
    """``--prompt`` goes through the model folder's tokenizer.json when it has one: the same
    tokens as the ids given directly, and the output comes back as text."""
    import json
    import shutil
    tokenizers = pytest.importorskip("tokenizers")
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import Whitespace
    from kvforge_amd import generate
    folder, oracle = model_a
    mine = str(tmp_path / "with_tokenizer")
    shutil.copytree(folder, mine)
    words = ["<unk>"] + [f"w{i}" for i in range(1, 60)]
    tok = tokenizers.Tokenizer(WordLevel({w: i for i, w in enumerate(words)}, unk_token="<unk>"))
    tok.pre_tokenizer = Whitespace()
    tok.save(mine + "/tokenizer.json")
    rc = generate.main(["--model", mine, "--prompt", "w5 w17 w3", "--max-tokens", "6", "--temperature", "0",
                        "--block-size", "4", "--num-blocks", "32", "--ignore-eos", "--json"])
    assert rc == 0
    out = json.loads(capsys.readouterr().out.strip().splitlines()[-1])["outputs"][0]
    assert out["prompt_token_ids"] == [5, 17, 3]
    want, gaps = oracle.greedy([5, 17, 3], 6)
    assert_greedy_equal(out["output_token_ids"], want, gaps)
    assert out["text"] == tok.decode(out["output_token_ids"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replay_equals_eager_steps(model_b, dtype):
    """Decode steps replayed from captured HIP graphs give the tokens of the same steps launched
    one kernel at a time: requests join and leave (the padded batch size and the context bucket
    change, so several graphs are captured and each is replayed many times, with eager prefill
    steps and synchronisations in between)."""
    folder, _ = model_b
    prompts = prompts_for(384, 7, 3, 3, 50)
    params = [SamplingParams(max_tokens=n, temperature=t, top_k=k, top_p=p)
              for n, t, k, p in ((40, 0.0, 0, 1.0), (25, 0.8, 0, 1.0), (60, 1.0, 40, 0.9),
                                 (12, 0.0, 0, 1.0), (33, 0.7, 0, 0.8), (50, 0.0, 0, 1.0),
                                 (45, 1.2, 10, 1.0))]

    def run(use_graphs):
        # one token per step in both runs: the same steps then hold the same requests, and bf16
        # logits (hence drawn tokens) are compared bit for bit
        engine = engine_for(folder, dtype, block_size=8, max_num_seqs=5, max_num_batched_tokens=32,
                            seed=11, use_graphs=use_graphs, decode_run_steps=1)
        done, step = {}, 0
        pending = list(zip(prompts, params))
        for p, sp in pending[:3]:
            engine.add_request(p, sp)
        pending = pending[3:]
        while engine.has_unfinished_requests() or pending:
            if pending and step % 9 == 4:
                engine.add_request(*pending.pop(0))
            for o in engine.step():
                if o.finished:
                    done[o.request_id] = o.output_token_ids
            step += 1
        return done, engine

    eager, _ = run(False)
    graphed, engine = run(True)
    assert len(engine.runner.graphs) >= 3 and engine.runner.num_graph_replays > 50
    assert graphed == eager


def test_graph_replay_of_library_products_at_the_served_width(tmp_path):
    """64 requests decode through layers of the Llama 3.2 1B shape (two of them, and a small
    vocabulary, to keep the folder small): a padded batch of 64 rows sends every product to the
    library, whose kernels for these widths (up to 16,384 columns, K up to 8,192) are others than
    the tiny models meet and may bring a workspace along.  Replays of the captured graph, with
    eager prefill steps and synchronisations around them, give the tokens of eager launches."""
    cfg = kvforge_amd.preset_dict("llama-1b")
    cfg.update(num_hidden_layers=2, vocab_size=4096)
    folder = str(tmp_path / "served")
    kvforge_amd.write_random_model(folder, cfg, seed=0)
    prompts = prompts_for(4096, 64, 5, 8, 40)
    params = SamplingParams(max_tokens=24, temperature=0.0, ignore_eos=True)

    def run(use_graphs):
        engine = engine_for(folder, "bfloat16", block_size=16, num_blocks=512, max_num_seqs=64,
                            max_num_batched_tokens=4096, use_graphs=use_graphs)
        return [o.output_token_ids for o in engine.generate(prompts, params)], engine

    eager, _ = run(False)
    graphed, engine = run(True)
    assert any(b == 64 for b, *_ in engine.runner.graphs) and engine.runner.num_graph_replays >= 16
    assert graphed == eager
    again, _ = run(True)
    assert again == graphed


def test_one_long_context_among_short_ones(tmp_path):
    """Twelve requests decode together, one of them past 2,300 tokens: the decode kernel then
    cuts the key range although the sequences alone would fill the chip, in eager steps and in
    captured ones (a cell of graphs of its own).  Every token is the plain model's choice within
    bf16 rounding, for the long request and for short ones beside it."""
    from tests.replay_util import TINY_C, sharpen
    cfg = dict(TINY_C, max_position_embeddings=4096)
    folder = str(tmp_path / "skew")
    kvforge_amd.write_random_model(folder, cfg, seed=8)
    sharpen(folder, 6.0)
    oracle = Oracle(folder)
    rng = random.Random(4)
    prompts = [[rng.randrange(1, 200) for _ in range(2310)]] + prompts_for(200, 11, 9, 5, 40)
    params = SamplingParams(max_tokens=18, temperature=0.0)
    for use_graphs in (False, True):
        config = EngineConfig(cache=CacheConfig(block_size=16, num_blocks=400),
                              scheduler=SchedulerConfig(max_num_seqs=16, max_num_batched_tokens=1024,
                                                        max_model_len=4096),
                              dtype="bfloat16", use_graphs=use_graphs)
        engine = InferenceEngine.from_folder(folder, config)
        outs = [o.output_token_ids for o in engine.generate(prompts, params)]
        if use_graphs:
            assert any(skew > 1 for _, keys, _ in engine.runner.graphs for _, skew in keys)
        for i in (0, 1, 7):
            oracle.of("bfloat16").check_choices(prompts[i], outs[i], 3e-2)
        assert engine.cache.num_free_blocks == engine.cache.num_blocks


def test_wide_layers_through_graphs_and_queued_runs(tmp_path):
    """A model whose layers are wide enough for the kernels a real model is served with (the down
    projection in two halves of K, one of them owed from layer to layer; two groups of columns
    per wave in gate/up; head size 64 on the matrix cores): six requests in bf16 through captured
    graphs, runs of steps on the device and runs queued ahead give the tokens of single captured
    steps, and every token, theirs and that of eager steps, is the plain model's choice within
    bf16 rounding."""
    from tests.replay_util import WIDE, sharpen
    folder = str(tmp_path / "wide")
    kvforge_amd.write_random_model(folder, dict(WIDE), seed=4)
    sharpen(folder, 4.0)
    oracle = Oracle(folder)
    prompts = prompts_for(1000, 6, 17, 5, 60)
    params = SamplingParams(max_tokens=40, temperature=0.0)

    def run(**kw):
        engine = engine_for(folder, "bfloat16", block_size=16, num_blocks=128, max_num_seqs=8,
                            max_num_batched_tokens=512, **kw)
        return [o.output_token_ids for o in engine.generate(prompts, params)], engine

    eager, _ = run(use_graphs=False, decode_run_steps=1)
    single, _ = run(use_graphs=True, decode_run_steps=1)
    served, engine = run(use_graphs=True, decode_run_steps=8, decode_run_ahead=True)
    assert engine.runner.num_graph_replays > 0 and engine.runner.num_runs_queued_ahead >= 1
    # captured steps end in the head's greedy pick (no logits, the norm inside the product):
    # the same kernels whether the device takes one step or runs of them
    assert engine.runner.num_greedy_tails > 0
    assert served == single
    # eager steps make logits and pick from them; the two round differently, so where the plain
    # model's two best logits lie within bf16 rounding they may part ways: each is held to the
    # plain model on its own history
    for p, a, b in zip(prompts, served, eager):
        oracle.of("bfloat16").check_choices(p, a, 3e-2)
        oracle.of("bfloat16").check_choices(p, b, 3e-2)


@pytest.mark.parametrize("count,bucket", [(24, 32), (40, 64)])
def test_graph_replay_with_many_requests(model_a, count, bucket):
    """Many requests decode together.  A padded batch of 32 is two row tiles of the hand-written
    matrix product; one of 64 is past what it takes, so the captured graph holds the library's
    products.  Replays must give the tokens of eager launches either way."""
    folder, oracle = model_a
    prompts = prompts_for(256, count, 12, 4, 20)
    params = SamplingParams(max_tokens=14, temperature=0.0)

    def run(use_graphs):
        engine = engine_for(folder, "bfloat16", block_size=8, max_num_seqs=64, num_blocks=512,
                            max_num_batched_tokens=256, use_graphs=use_graphs)
        outs = engine.generate(prompts, params)
        return [o.output_token_ids for o in outs], engine

    eager, _ = run(False)
    graphed, engine = run(True)
    assert any(b == bucket for b, *_ in engine.runner.graphs) and engine.runner.num_graph_replays >= 8
    assert graphed == eager
    for p, out in zip(prompts, graphed):
        oracle.of("bfloat16").check_choices(p, out, 3e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_weights_drawn_on_the_device(dtype):
    """``Transformer.from_random`` (what the benchmark's large models are made with) hands the
    parts tensors that never pass through a file or the loader's checks.  The tensors it drew,
    given to the plain model, must explain every token the engine generates; in float32 they
    are 32-bit numbers that bfloat16 cannot hold."""
    from kvforge_amd.models.transformer import Transformer
    cfg = kvforge_amd.preset_dict("tiny-b")
    drawn = {}
    model = Transformer.from_random(cfg, 5, kvforge_amd.EngineConfig(dtype=dtype).dtype, "cuda", drawn=drawn)
    w = {k: v.cpu() for k, v in drawn.items()}
    floating = [t for t in w.values() if t.is_floating_point()]
    if dtype == "float32":
        assert all(t.dtype == torch.float32 for t in floating)
        assert not any(torch.equal(t.bfloat16().float(), t) for t in floating)
    else:
        assert all(t.dtype == torch.bfloat16 for t in floating)
    engine = InferenceEngine(model, EngineConfig(
        cache=CacheConfig(block_size=8, num_blocks=64),
        scheduler=SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=64), dtype=dtype))
    prompts = prompts_for(384, 5, 3, 1, 50)
    outs = engine.generate(prompts, SamplingParams(max_tokens=8, temperature=0.0))
    plain_cfg = dict(cfg)
    plain_cfg.setdefault("num_key_value_heads", cfg["num_attention_heads"])
    margin = 1e-4 if dtype == "float32" else 3e-2
    for p, o in zip(prompts, outs):
        logits = plain.forward(w, plain_cfg, p + o.output_token_ids)
        for i, tok in enumerate(o.output_token_ids):
            row = logits[len(p) - 1 + i]
            assert float(row.max() - row[tok]) <= margin, (i, tok)
    # and the logits of a step themselves, so that a flat model cannot hide a wrong tensor
    from kvforge_amd.engine.batch import StepEntry
    ids = prompts[1] + outs[1].output_token_ids
    engine.cache.allocate("probe", len(ids))
    got = engine.runner.step([StepEntry("probe", ids, 0, "all")]).cpu()
    engine.cache.free("probe")
    t = dict(atol=2e-5, rtol=1e-4) if dtype == "float32" else dict(atol=1.5e-2, rtol=1.5e-2)
    torch.testing.assert_close(got, plain.forward(w, plain_cfg, ids), **t)


def test_float32_steps_on_both_sides_of_the_streaming_kernels_row_limit(model_a):
    """The 32-bit product sums along K in another order for up to 32 rows (lanes side by side,
    then a tree) than for more (one term after the other), so a token's float32 logits differ
    by rounding between a step of 32 rows and one of 33.  Forty requests decode together and
    end one by one: steps of 40 down to 1 rows, every token the plain model's choice within
    1e-4."""
    folder, oracle = model_a
    prompts = prompts_for(256, 40, 41, 2, 24)
    params = [SamplingParams(max_tokens=3 + (i % 12), temperature=0.0) for i in range(40)]
    engine = engine_for(folder, "float32", block_size=8, num_blocks=512, max_num_seqs=40,
                        max_num_batched_tokens=512)
    outs = engine.generate(prompts, params)
    assert max(engine.metrics.batch_sizes) == 40
    assert [len(o.output_token_ids) for o in outs] == [p.max_tokens for p in params]
    for i in range(0, 40, 3):
        oracle.check_choices(prompts[i], outs[i].output_token_ids, 1e-4)
