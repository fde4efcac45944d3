"""InferenceEngine: model, cache, scheduler and sampler behind one ``step()`` loop
(src/tokenvault/engine.py:39-297, without speculative decoding and quantization).

One ``step()`` = one scheduler decision, one forward over the flat batch (prompt portions beside
single decode tokens), one sampling launch for the requests whose last token was in the batch.
The engine is synchronous and single-threaded, as the reference's.
"""

from __future__ import annotations

import itertools
import os
import tempfile
import time
from typing import Any, Sequence

import torch

from kvforge_amd import registry
from kvforge_amd.config.engine import EngineConfig
from kvforge_amd.engine.batch import StepEntry
from kvforge_amd.engine.metrics import CostModel, MetricsCollector
from kvforge_amd.engine.request import FinishReason, Request, RequestOutput
from kvforge_amd.engine.runner import ModelRunner
from kvforge_amd.engine.scheduler import ScheduledRequest, Scheduler
from kvforge_amd.models.transformer import Transformer
from kvforge_amd.sampling.params import SamplingParams
from kvforge_amd.sampling.sampler import Sampler
from kvforge_amd.weights.random_init import write_random_model


class InferenceEngine:
    def __init__(self, model: Transformer, config: EngineConfig | None = None,
                 tokenizer: Any = None) -> None:
        self.config = config = config or EngineConfig()
        self.model = model
        self.tokenizer = tokenizer
        if model.dtype != config.dtype:
            raise ValueError(f"model holds {model.dtype} tensors, engine dtype is {config.dtype}")
        config.clamp_to_model(model.config.max_position_embeddings)
        sc, cc = config.scheduler, config.cache
        num_blocks = cc.resolve_num_blocks(ModelRunner.bytes_per_block(model, cc.block_size))
        self.runner = ModelRunner(model, cc.block_size, num_blocks, sc.max_num_seqs,
                                  sc.max_num_batched_tokens, sc.max_model_len, cc.watermark,
                                  use_graphs=config.use_graphs)
        self.cache = self.runner.cache
        self.sampler = Sampler(config.seed, model.device)
        self.scheduler = Scheduler(sc, self.cache)
        self.metrics = MetricsCollector()
        self._ids = itertools.count()
        self._arrivals = itertools.count()

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_folder(cls, folder: str, config: EngineConfig | None = None,
                    tokenizer: Any = None) -> "InferenceEngine":
        config = config or EngineConfig()
        model = Transformer.from_folder(folder, config.dtype, config.device)
        return cls(model, config, tokenizer)

    @classmethod
    def from_config(cls, model_config: "dict[str, Any] | str", config: EngineConfig | None = None,
                    tokenizer: Any = None, seed: int | None = None) -> "InferenceEngine":
        """Random weights: ``model_config`` is a config.json dictionary or a preset name; the
        model folder is written to a temporary place and loaded like any other."""
        from kvforge_amd.config.presets import preset_dict

        config = config or EngineConfig()
        d = preset_dict(model_config) if isinstance(model_config, str) else model_config
        with tempfile.TemporaryDirectory(prefix="kvforge_amd_model_") as tmp:
            write_random_model(tmp, d, config.seed if seed is None else seed)
            return cls.from_folder(tmp, config, tokenizer)

    # ------------------------------------------------------------------ API
    def add_request(self, prompt: "str | Sequence[int]", sampling_params: SamplingParams | None = None,
                    request_id: str | None = None, priority: int = 0,
                    arrival_time: float | None = None) -> str:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("string prompts need a tokenizer")
            token_ids = self.tokenizer.encode(prompt)
        else:
            token_ids = [int(t) for t in prompt]
        vocab = self.model.config.vocab_size
        if any(t < 0 or t >= vocab for t in token_ids):
            raise ValueError("prompt contains out-of-vocabulary token ids")
        request_id = request_id or f"req-{next(self._ids)}"
        eos = self.tokenizer.eos_token_id if self.tokenizer else self.model.config.eos_token_id
        params = sampling_params or SamplingParams()
        arrival = next(self._arrivals)
        req = Request(request_id=request_id, prompt_token_ids=token_ids, sampling_params=params,
                      priority=priority, eos_token_id=eos,
                      sample_stream=params.seed if params.seed is not None else arrival)
        if arrival_time is not None:
            req.arrival_time = arrival_time
        self.scheduler.add_request(req)
        return request_id

    def abort_request(self, request_id: str) -> bool:
        req = self.scheduler.abort_request(request_id)
        if req is not None:
            self.metrics.record_finished(req)
        return req is not None

    def has_unfinished_requests(self) -> bool:
        return self.scheduler.has_unfinished()

    def generate(self, prompts: Sequence["str | Sequence[int]"],
                 sampling_params: "SamplingParams | Sequence[SamplingParams] | None" = None
                 ) -> list[RequestOutput]:
        """Offline batch generation; outputs in prompt order."""
        if sampling_params is None or isinstance(sampling_params, SamplingParams):
            sampling_params = [sampling_params or SamplingParams()] * len(prompts)
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, sampling_params)]
        done: dict[str, RequestOutput] = {}
        while self.has_unfinished_requests():
            for out in self.step():
                if out.finished:
                    done[out.request_id] = out
        return [done[i] for i in ids if i in done]

    # ----------------------------------------------------------------- step
    def step(self) -> list[RequestOutput]:
        t0 = time.perf_counter()
        # A run that is queued on the device for the running requests is read before anybody new
        # is admitted: arrivals wait for at most one run, and no queued work is thrown away.
        running = sorted(self.scheduler.running, key=self.scheduler._key)
        queued = self.runner.queued_run_steps([(r.request_id, r.num_computed_tokens) for r in running])
        sched = self.scheduler.schedule(admit=not queued)
        if sched.is_empty:
            return []
        run, ahead = self._decode_run_length(sched, queued)
        new_tokens = self._run(sched.scheduled, run, ahead)
        outputs = self._postprocess(sched.scheduled, new_tokens)
        # a run of decode steps counts as that many steps of the batch, each with its share of the time
        dt = (time.perf_counter() - t0) / run
        used = 1.0 - self.cache.num_free_blocks / max(1, self.cache.num_blocks)
        for _ in range(run):
            self.metrics.record_step(len(sched.scheduled), sched.num_batched_tokens, dt, used)
        return outputs

    def _decode_run_length(self, sched, queued: int = 0) -> tuple[int, bool]:
        """How many decode steps the device takes before the host looks again: more than one
        only while every scheduled request decodes, no request can reach the model's length
        inside the run, and the pages of the run's positions are free.  While requests wait
        that the scheduler could not admit beside these (no sequence slot, no pages), nothing
        changes for them before a running request ends: the run then goes up to the first end
        that is certain, the smallest number of tokens a request has left (one that meets a
        stop token earlier keeps its slot until the run is read).
        ``queued``: the steps of a run that is queued for these requests already (its room and
        pages were made sure of then).
        The second value says that all of this also holds for the run after it, whose pages are
        then allocated as well, so that the runner may queue that run before this one is read
        (``EngineConfig.decode_run_ahead``)."""
        limit = self.config.decode_run_steps
        group = sched.scheduled
        decoding = not (sched.preempted or any(s.is_prefill or s.num_new_tokens != 1 for s in group))
        if queued and not decoding:
            queued = 0  # cannot be: a queued run is for requests that decode
        if not queued and (limit <= 1 or not decoding):
            return 1, False
        # A request that reaches its number of tokens inside a run is cut there when the run is
        # read, like one that meets a stop token; only the model's length is a hard limit.  No
        # run is longer than the longest remainder.
        max_len = self.config.scheduler.max_model_len
        room = min(max_len - s.request.num_tokens for s in group)
        left = [s.request.sampling_params.max_tokens - s.request.num_output_tokens for s in group]
        longest = max(left)
        if queued:
            limit = queued
        else:
            limit = min(limit, room, min(left) if self.scheduler.num_waiting else longest)
            if limit <= 1:
                return 1, False
            entries = [StepEntry(s.request.request_id, [0], s.request.num_computed_tokens, "last")
                       for s in group]
            if not self.runner.graph_takes(entries, len(entries)):
                return 1, False
        wanted = [(s.request.request_id, s.request.num_computed_tokens + limit) for s in group]
        if not queued and not self.cache.can_append_all(wanted):
            return 1, False
        ahead = (self.config.decode_run_ahead and not self.scheduler.num_waiting
                 and limit == self.config.decode_run_steps and room >= 2 * limit and longest > limit)
        if ahead:
            further = [(rid, total + limit) for rid, total in wanted]
            ahead = self.cache.can_append_all(further)
            if ahead:
                wanted = further
        for s, (rid, total) in zip(group, wanted):
            self.cache.append_slots(rid, total, s.request.num_computed_tokens)
        return limit, ahead

    def _run(self, group: list[ScheduledRequest], run: int = 1, ahead: bool = False
             ) -> dict[str, list[int]]:
        if run > 1:
            reqs = [s.request for s in group]
            entries = [StepEntry(r.request_id, r.token_slice(r.num_computed_tokens, 1),
                                 r.num_computed_tokens, "last") for r in reqs]
            steps = self.runner.decode_run(entries, self.sampler.seed,
                                           [r.sampling_params for r in reqs],
                                           [r.sample_stream for r in reqs],
                                           [r.num_output_tokens for r in reqs], run, ahead)
            for r in reqs:
                r.num_computed_tokens += 1
            return {r.request_id: [step[i] for step in steps] for i, r in enumerate(reqs)}
        entries: list[StepEntry] = []
        sampled: list[Request] = []
        for s in group:
            r = s.request
            start = r.num_computed_tokens
            completes = start + s.num_new_tokens == r.num_tokens
            entries.append(StepEntry(r.request_id, r.token_slice(start, s.num_new_tokens), start,
                                     "last" if completes else "none"))
            if completes:
                sampled.append(r)
        tokens = self.runner.step_and_sample(entries, self.sampler,
                                             [r.sampling_params for r in sampled],
                                             [r.sample_stream for r in sampled],
                                             [r.num_output_tokens for r in sampled])
        for s in group:
            s.request.num_computed_tokens += s.num_new_tokens
        return {r.request_id: [t] for r, t in zip(sampled, tokens)}

    def _postprocess(self, scheduled: list[ScheduledRequest], new_tokens: dict[str, list[int]]
                     ) -> list[RequestOutput]:
        now = time.perf_counter()
        max_len = self.config.scheduler.max_model_len
        outputs: list[RequestOutput] = []
        for s in scheduled:
            r = s.request
            emitted: list[int] = []
            reason: FinishReason | None = None
            for j, t in enumerate(new_tokens.get(r.request_id, ())):
                if j > 0:
                    r.num_computed_tokens += 1  # the step that took the token before as its input
                r.append_token(t, now)
                emitted.append(t)
                reason = r.check_stop(max_len)
                if reason is not None:
                    break  # what the device sampled past a stop is dropped
            if reason is not None:
                self.scheduler.finish_request(r, reason)
                self.metrics.record_finished(r)
            else:
                self.cache.mark_computed(r.request_id, r.num_computed_tokens)
                self.cache.release_behind(r.request_id, r.num_computed_tokens)
            if emitted or r.is_finished:
                out = RequestOutput.from_request(r, emitted)
                if self.tokenizer is not None:
                    out.text = self.tokenizer.decode(out.output_token_ids)
                outputs.append(out)
        return outputs

    # ---------------------------------------------------------------- stats
    def stats(self, cost: CostModel | None = None) -> dict[str, Any]:
        cs = self.cache.stats()
        bpb = ModelRunner.bytes_per_block(self.model, self.cache.block_size)
        return {
            "metrics": self.metrics.summary(cost),
            "kv_cache": {
                "num_blocks": cs.num_blocks, "block_size": self.cache.block_size,
                "num_used_blocks": cs.num_used_blocks, "num_free_blocks": cs.num_free_blocks,
                "num_tokens": cs.num_tokens, "utilization": cs.utilization,
                "internal_fragmentation": cs.internal_fragmentation,
                "bytes_total": self.runner.storage.memory_bytes, "bytes_per_block": bpb,
                "bytes_in_use": cs.num_used_blocks * bpb,
            },
            "scheduler": {
                "num_running": self.scheduler.num_running,
                "num_waiting": self.scheduler.num_waiting,
                "num_preemptions": self.scheduler.num_preemptions,
            },
            "weights_bytes": self.model.weight_bytes,
            "forward_passes": self.runner.num_forward_passes,
        }
