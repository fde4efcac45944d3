"""``InferenceEngine``: a model, its cache, the scheduler and the sampler behind ``generate`` and
``step``, with the entry points of the reference's engine (src/tokenvault/engine.py:105-194:
``add_request``, ``step``, ``generate``, ``abort_request``, ``has_unfinished_requests``,
``stats``; no speculative decoding, no quantization).

A call of ``step`` is: ask the scheduler for a plan, run it (one forward over the flat batch and
one sampling launch, or a run of decode steps that the device takes by itself), hand the sampled
tokens back to the scheduler, report.  Single-threaded and synchronous, like the reference's.
"""

from __future__ import annotations

import tempfile
import time
from typing import Any, Sequence

from kvforge_amd.config.engine import EngineConfig
from kvforge_amd.engine.batch import StepEntry
from kvforge_amd.engine.metrics import CostModel, MetricsCollector
from kvforge_amd.engine.request import Request, RequestOutput
from kvforge_amd.engine.runner import ModelRunner
from kvforge_amd.engine.scheduler import Plan, Scheduler
from kvforge_amd.models.transformer import Transformer
from kvforge_amd.sampling.params import SamplingParams
from kvforge_amd.sampling.sampler import Sampler
from kvforge_amd.weights.random_init import write_random_model

Prompt = "str | Sequence[int]"


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
        self.scheduler = Scheduler(sc, self.cache, run_steps=config.decode_run_steps,
                                   run_ahead=config.decode_run_ahead,
                                   device_runs=self.runner.takes_runs)
        self.metrics = MetricsCollector()
        self._num_added = 0
        self.stalled = False      # the last step found requests but nothing to plan

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_folder(cls, folder: str, config: EngineConfig | None = None,
                    tokenizer: Any = None) -> "InferenceEngine":
        config = config or EngineConfig()
        model = Transformer.from_folder(folder, config.dtype, config.device)
        return cls(model, config, tokenizer)

    @classmethod
    def from_config(cls, model_config: "dict[str, Any] | str", config: EngineConfig | None = None,
                    tokenizer: Any = None, seed: int | None = None,
                    on_device: bool = False) -> "InferenceEngine":
        """Random weights: ``model_config`` is a config.json dictionary or a preset name; the
        model folder is written to a temporary place, stored in the engine's type (a float32
        engine gets 32-bit weights), and loaded like any other.  With
        ``on_device`` the tensors are drawn on the GPU instead and no file is written (for
        models of many gigabytes; other numbers than the folder's for the same seed)."""
        from kvforge_amd.config.presets import preset_dict

        config = config or EngineConfig()
        d = preset_dict(model_config) if isinstance(model_config, str) else model_config
        if on_device:
            model = Transformer.from_random(d, config.seed if seed is None else seed, config.dtype,
                                            config.device)
            return cls(model, config, tokenizer)
        with tempfile.TemporaryDirectory(prefix="kvforge_amd_model_") as tmp:
            write_random_model(tmp, d, config.seed if seed is None else seed, dtype=config.dtype)
            return cls.from_folder(tmp, config, tokenizer)

    # ------------------------------------------------------------------ requests in
    def _token_ids(self, prompt: Prompt) -> list[int]:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("a text prompt needs a tokenizer; pass token ids instead")
            ids = list(self.tokenizer.encode(prompt))
        else:
            ids = [int(t) for t in prompt]
        vocab = self.model.config.vocab_size
        bad = next((t for t in ids if not 0 <= t < vocab), None)
        if bad is not None:
            raise ValueError(f"token id {bad} is outside the model's vocabulary of {vocab}")
        return ids

    def add_request(self, prompt: Prompt, sampling_params: SamplingParams | None = None,
                    request_id: str | None = None, priority: int = 0,
                    arrival_time: float | None = None) -> str:
        """Queue a prompt (text, with a tokenizer, or token ids); returns the request's id.
        Raises ``ValueError`` for what can never be served (the scheduler's rejections are
        ``ValueError`` too)."""
        params = sampling_params if sampling_params is not None else SamplingParams()
        index = self._num_added
        rid = request_id if request_id is not None else f"req-{index}"
        eos = getattr(self.tokenizer, "eos_token_id", None) if self.tokenizer is not None \
            else self.model.config.eos_token_id
        req = Request(rid, self._token_ids(prompt), params, priority=priority,
                      arrival_time=arrival_time, eos_token_id=eos,
                      sample_stream=index if params.seed is None else params.seed)
        self.scheduler.add_request(req)
        self._num_added += 1
        return rid

    def abort_request(self, request_id: str) -> bool:
        gone = self.scheduler.abort_request(request_id)
        if gone is None:
            return False
        self.metrics.record_finished(gone)
        return True

    def has_unfinished_requests(self) -> bool:
        return self.scheduler.has_unfinished()

    def generate(self, prompts: Sequence[Prompt],
                 sampling_params: "SamplingParams | Sequence[SamplingParams] | None" = None
                 ) -> list[RequestOutput]:
        """Run the prompts to their ends; one output per prompt, in the prompts' order."""
        if sampling_params is None or isinstance(sampling_params, SamplingParams):
            each = [sampling_params] * len(prompts)
        else:
            each = list(sampling_params)
            if len(each) != len(prompts):
                raise ValueError("one SamplingParams per prompt, or one for all")
        order = [self.add_request(p, sp) for p, sp in zip(prompts, each)]
        final: dict[str, RequestOutput] = {}
        while self.has_unfinished_requests() and len(final) < len(order):
            final.update((o.request_id, o) for o in self.step() if o.finished)
            if self.stalled:
                raise RuntimeError(
                    f"nothing can be planned although {self.scheduler.num_waiting} request(s) "
                    f"wait and {self.scheduler.num_running} run: the scheduler is stuck")
        return [final[rid] for rid in order if rid in final]

    # ------------------------------------------------------------------ one step
    def step(self) -> list[RequestOutput]:
        began = time.perf_counter()
        # A run that is queued on the device for the running requests is read before anybody
        # new is admitted: arrivals wait for at most one run and no queued work is thrown away.
        queued = self.runner.queued_run_steps(
            [(r.request_id, r.computed) for r in self.scheduler.running])
        plan = self.scheduler.schedule(queued_steps=queued)
        # A plan without tokens that took nobody's pages either changes nothing: the next one
        # would be the same.  ``generate`` raises on it instead of asking for ever.
        self.stalled = (plan.is_empty and not plan.preempted
                        and self.scheduler.has_unfinished())
        if plan.is_empty:
            return []
        sampled = self._execute(plan)
        outputs = []
        for req, accepted in self.scheduler.commit(plan, sampled):
            if req.is_finished:
                self.metrics.record_finished(req)
            text = self.tokenizer.decode(req.output_token_ids) if self.tokenizer is not None else None
            outputs.append(req.output(accepted, text))
        # a run of decode steps counts as that many steps of the batch, each with its share
        share = (time.perf_counter() - began) / plan.run_steps
        used = 1.0 - self.cache.num_free_blocks / max(1, self.cache.num_blocks)
        for _ in range(plan.run_steps):
            self.metrics.record_step(len(plan.slices), plan.num_tokens, share, used)
        return outputs

    def _execute(self, plan: Plan) -> dict[str, list[int]]:
        """Run the plan's step(s); the tokens sampled for each request whose slice reached the
        end of its sequence, one per step."""
        ending = [s.request for s in plan.slices if s.samples]
        params = [r.sampling_params for r in ending]
        streams = [r.sample_stream for r in ending]
        drawn = [r.num_output_tokens for r in ending]
        if plan.run_steps > 1:
            entries = [StepEntry(s.request.request_id, s.request.next_tokens(1), s.start, "last")
                       for s in plan.slices]
            steps = self.runner.decode_run(entries, self.sampler.seed, params, streams, drawn,
                                           plan.run_steps, plan.run_ahead)
            return {r.request_id: [tokens[i] for tokens in steps] for i, r in enumerate(ending)}
        entries = [StepEntry(s.request.request_id, s.request.next_tokens(s.count), s.start,
                             "last" if s.samples else "none") for s in plan.slices]
        tokens = self.runner.step_and_sample(entries, self.sampler, params, streams, drawn)
        return {r.request_id: [t] for r, t in zip(ending, tokens)}

    # ------------------------------------------------------------------ figures
    def stats(self, cost: CostModel | None = None) -> dict[str, Any]:
        """Serving metrics, the cache's state, the scheduler's queues and what the weights
        weigh: ``weights_bytes`` is what one decode step reads, ``weights_bytes_resident`` what
        they occupy on the device (matrices that are streamed for few rows are also kept in
        tiles, so they count twice there)."""
        pool = self.cache.stats()
        per_block = ModelRunner.bytes_per_block(self.model, self.cache.block_size)
        cache = {name: getattr(pool, name) for name in (
            "num_blocks", "num_used_blocks", "num_free_blocks", "num_tokens", "utilization",
            "internal_fragmentation")}
        cache.update(block_size=self.cache.block_size, bytes_per_block=per_block,
                     bytes_total=self.runner.storage.memory_bytes,
                     bytes_in_use=pool.num_used_blocks * per_block)
        sched = self.scheduler
        return {
            "metrics": self.metrics.summary(cost),
            "kv_cache": cache,
            "scheduler": {"num_running": sched.num_running, "num_waiting": sched.num_waiting,
                          "num_preemptions": sched.num_preemptions},
            "weights_bytes": self.model.weight_bytes,
            "weights_bytes_resident": self.model.resident_bytes,
            "forward_passes": self.runner.num_forward_passes,
        }
