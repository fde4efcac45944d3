"""The step function: a batch of (request, its next tokens), portions of prompts beside single
decoded tokens, cut anywhere, run as one batch from the cache; logits come back for the wanted
places.  The counterpart of the reference's ``ModelRunner.execute``
(src/tokenvault/batching/continuous.py:90-117).

Preconditions, as in the reference: the request's block tables already cover
``start_pos + len(tokens)`` (the scheduler or the replay program asked the cache manager), and
positions below ``start_pos`` are in the cache.
"""

from __future__ import annotations

from typing import Sequence

import torch

from kvforge_amd.cache.manager import CacheManager
from kvforge_amd.cache.storage import PagedStorage, StateStorage, bytes_per_block
from kvforge_amd.engine.batch import (DecodeShape, DecodeTail, MetaBuffers, Step, StepEntry,
                                      Workspace, extend_tables, fill_step)
from kvforge_amd.kernels import ops
from kvforge_amd.sampling.rng import uniform
from kvforge_amd.kernels import library
from kvforge_amd.models.transformer import Transformer


class ModelRunner:
    def __init__(self, model: Transformer, block_size: int, num_blocks: "int | list[int]",
                 max_num_seqs: int, max_num_batched_tokens: int, max_model_len: int,
                 watermark: float = 0.0, use_graphs: bool = True) -> None:
        if torch.device(model.device).type != "cuda":
            raise RuntimeError("the engine runs on the GPU only; there is no CPU path")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible to this process")
        library.ensure(model.kernel_modules())
        self.model = model
        self.device = model.device
        self.block_size = int(block_size)
        self.max_model_len = int(max_model_len)
        groups = model.cache_groups
        counts = [num_blocks] * len(groups) if isinstance(num_blocks, int) else list(num_blocks)
        self.cache = CacheManager(block_size, groups, counts,
                                  num_state_slots=max_num_seqs if model.state_specs else 0,
                                  watermark=watermark)
        self.storage = PagedStorage(groups, counts, block_size, model.dtype, self.device)
        self.states = StateStorage(model.state_specs, max_num_seqs, self.device)
        model.attach(self.storage, self.states)
        model.prepare(self.max_model_len)
        width = -(-self.max_model_len // self.block_size)
        self.meta = MetaBuffers(max(max_num_batched_tokens, max_num_seqs), max_num_seqs,
                                [width] * len(groups), self.device)
        self.ws = Workspace(self.device)
        # The residual stream is where a captured step that ends in the head's greedy pick finds
        # its first embeddings, written either by the step before it or by the host's embedding
        # of a run's first tokens: one piece of memory for every step there will be, made at its
        # full size now, so that no later, longer step makes the workspace move it.
        self.ws.buf("residual", (self.meta.max_tokens, model.spec.embedding.hidden), torch.float32)
        self._windowed = [g.window is not None for g in groups]
        self.num_forward_passes = 0
        self.num_tokens_processed = 0
        # decode steps replayed from HIP graphs: (padded batch, the parts' launch keys) -> graph;
        # only if every part's launches may be replayed for another batch
        self.use_graphs = bool(use_graphs) and all(p.replayable for p in model.spec.all_parts())
        self.graphs: dict[tuple[int, tuple], _DecodeGraph] = {}
        self.num_graph_replays = 0
        cap = self.meta.max_seqs
        # floats: temperatures, top-p, then MAX_DECODE_RUN rows of uniform numbers; ints: top-k,
        # the sampled tokens, then the counter of steps in a run and the ring of their tokens
        nf = (2 + MAX_DECODE_RUN) * cap
        self._sample_f = torch.zeros(nf, dtype=torch.float32, device=self.device)
        self._sample_i = torch.zeros(2 * cap, dtype=torch.int32, device=self.device)
        self._run_counter = torch.zeros(1, dtype=torch.int32, device=self.device)
        # tickets and chunk results of greedy rows read by several workgroups (zero between launches)
        self._sample_work = torch.zeros(ops.sample_work_size(cap), dtype=torch.int32, device=self.device)
        self._run_ring = torch.zeros(MAX_DECODE_RUN, cap, dtype=torch.int32, device=self.device)
        self._ring_host = torch.zeros(MAX_DECODE_RUN, cap, dtype=torch.int32, pin_memory=True)
        self._ring_host_np = self._ring_host.numpy()
        self._queued: _QueuedRun | None = None   # a run queued ahead of the call that will read it
        self.num_runs_queued_ahead = 0
        self.num_runs_read_ahead = 0
        self._sample_f_host = torch.zeros(nf, dtype=torch.float32, pin_memory=True)
        self._sample_i_host = torch.zeros(cap, dtype=torch.int32, pin_memory=True)
        self._sample_f_np, self._sample_i_np = self._sample_f_host.numpy(), self._sample_i_host.numpy()
        self._sample_rows: list[tuple] = []
        self._sample_bucket = 0
        self._sample_drawn: list[int] = []
        # Steps whose rows are all picked greedily end in the head's own kernel (no logits, no
        # sampling, advance or embedding kernels) where the model allows it.
        self.num_greedy_tails = 0
        self._tail: DecodeTail | None = None
        if self.use_graphs and model.can_pick(1):
            self._tail = DecodeTail(self._sample_i[cap:2 * cap], self._run_ring, self._run_counter,
                                    model.spec.embedding.pick_table(),
                                    ops.pick_workspace(16, model.config.vocab_size, self.device))

    @staticmethod
    def bytes_per_block(model: Transformer, block_size: int) -> int:
        return bytes_per_block(model.cache_groups, block_size, model.dtype)

    def _slot_of(self, request_id: str) -> int:
        return self.cache.slots.slot(request_id) if self.cache.slots.num_slots else -1

    def build_step(self, entries: Sequence[StepEntry], pad_to: int | None = None,
                   lookahead: int = 0) -> tuple[Step, list[int]]:
        for e in entries:
            if e.start_pos + len(e.token_ids) + lookahead > self.max_model_len:
                raise ValueError(f"request {e.request_id} would pass max_model_len "
                                 f"{self.max_model_len}")
        step = Step()
        step.ws, step.act_dtype, step.device = self.ws, self.model.dtype, self.device
        counts = fill_step(step, self.meta, entries, self.cache.block_table, self._slot_of,
                           self.block_size, pad_to, self._windowed, self.cache.serial, lookahead)
        return step, counts

    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """One forward over the entries; fp32 logits ``[sum of wanted places, vocab]``, rows in
        entry order then place order.  The tensor is a view of memory the next step reuses."""
        self._queued = None  # whatever is queued ahead is not what comes next
        step, _ = self.build_step(entries)
        logits = self.model.forward(step)
        self.num_forward_passes += 1
        self.num_tokens_processed += step.n_tokens
        return logits

    def takes_runs(self, num_requests: int) -> bool:
        """Whether runs of decode steps on the device are possible for so many requests."""
        return self.use_graphs and 0 < num_requests <= GRAPH_MAX_BATCH

    def graph_takes(self, entries: Sequence[StepEntry], num_params: int) -> bool:
        """Whether a step goes through the captured decode path: single tokens that each want
        their logits, within the largest captured batch."""
        b = len(entries)
        return (self.use_graphs and b == num_params and b <= GRAPH_MAX_BATCH
                and all(len(e.token_ids) == 1 and e.want == "last" for e in entries))

    @torch.inference_mode()
    def step_and_sample(self, entries: Sequence[StepEntry], sampler, params, streams, counters
                        ) -> list[int]:
        """One forward, then one token for every wanted place (in row order)."""
        if self.graph_takes(entries, len(params)):
            return self.decode_run(entries, sampler.seed, params, streams, counters, 1)[0]
        logits = self.step(entries)
        if logits.shape[0] != len(params):
            raise ValueError("one SamplingParams per wanted place")
        return sampler(logits, params, streams, counters)

    # ------------------------------------------------------------------ decode through graphs
    @torch.inference_mode()
    def decode_run(self, entries, seed, params, streams, counters, num_steps: int = 1,
                   ahead: bool = False) -> list[list[int]]:
        """``num_steps`` decode steps of single tokens with one wait for the device at the end;
        returns the tokens of every step, ``[step][entry]``.

        The batch is padded to a bucket of sizes so that its launches are captured once in a HIP
        graph and replayed: metadata and sampling parameters live at fixed device addresses and
        are refreshed by two copies before the run.  The graph ends with a kernel that turns each
        sampled token into the sequence's next input, so further steps need nothing from the
        host; the pages of their positions must be in the requests' tables already.

        ``ahead``: the caller expects to come back for the same requests, ``num_steps`` further
        on, with the pages of those positions allocated already (twice ``num_steps`` from here).
        The runner then queues that next run before it waits for this one, so the device goes on
        while the host looks at the tokens; a next call that is this continuation finds its run
        queued.  Any other call simply leaves the queued run to finish unread: its launches only
        rewrite cache positions that the next real step computes again, in stream order before
        it.  (Not for models with per-request state, which a discarded run would advance.)"""
        b = len(entries)
        k = int(num_steps)
        if not 1 <= k <= MAX_DECODE_RUN:
            raise ValueError(f"a run holds 1 to {MAX_DECODE_RUN} steps")
        if not self.graph_takes(entries, len(params)):
            raise ValueError("a decode run takes single tokens that each want their logits")
        queued, self._queued = self._queued, None
        rows = self._rows_in(queued, [(e.request_id, e.start_pos) for e in entries], k)
        if rows is not None:
            run = queued
            self.num_runs_read_ahead += 1
        else:
            run = self._launch_run(entries, seed, params, streams, counters, k,
                                   lookahead=(2 * k if ahead else k) - 1)
            rows = list(range(b))
        # Only the whole batch is carried on: rows of requests that have left meanwhile would go
        # on writing into pages that are no longer theirs.
        whole = rows == list(range(len(run.ids)))
        if ahead and whole and 2 * k <= MAX_DECODE_RUN and not self.model.state_specs:
            self._queued = self._continue_run(run, entries, seed, streams, counters)
            self.num_runs_queued_ahead += self._queued is not None
        run.event.synchronize()
        tokens = self._ring_host_np[run.base:run.base + k][:, rows].tolist()
        self.num_graph_replays += run.replays
        self.num_forward_passes += k
        self.num_tokens_processed += b * k
        return tokens

    @staticmethod
    def _rows_in(queued: "_QueuedRun | None", wanted: list[tuple[str, int]], k: int
                 ) -> list[int] | None:
        """The rows of a queued run that hold the tokens of ``wanted`` (request id, position it
        begins at), in that order; ``None`` unless every one of them is in the run, in the run's
        order, at that position, for ``k`` steps.  Requests of the run that are not wanted any
        more (finished, aborted) are simply not read."""
        if queued is None or queued.k != k or not wanted:
            return None
        place = {rid: i for i, rid in enumerate(queued.ids)}
        rows = [place.get(rid, -1) for rid, _ in wanted]
        if any(r < 0 for r in rows) or rows != sorted(rows):
            return None
        if any(queued.begins[r] != pos for r, (_, pos) in zip(rows, wanted)):
            return None
        return rows

    def queued_run_steps(self, wanted: list[tuple[str, int]]) -> int:
        """How many steps a run that is queued ahead holds for exactly these requests at these
        positions (0 if none is queued for them)."""
        q = self._queued
        return q.k if q is not None and self._rows_in(q, wanted, q.k) is not None else 0

    def _launch_run(self, entries, seed, params, streams, counters, k: int, lookahead: int
                    ) -> "_QueuedRun":
        """Upload the batch and queue ``k`` decode steps for it (ring rows ``0..k-1``)."""
        b = len(entries)
        bucket = 1
        while bucket < b:
            bucket *= 2
        bucket = min(bucket, self.meta.max_seqs)
        step, _ = self.build_step(entries, pad_to=bucket, lookahead=lookahead)
        # The contexts' lengths enter the captured launches only through what the parts make of
        # them (a mixer's cuts of the key range, say): graphs are kept per such key.
        launch_key = self.model.launch_key(step.decode_shape)
        cap = self.meta.max_seqs
        fh, ih = self._sample_f_np, self._sample_i_np
        ids = [e.request_id for e in entries]
        # who sits in which row, with what parameters: an id that was freed and is used again
        # (another serial) or comes with other parameters is another occupant
        rows = [(e.request_id, self.cache.serial(e.request_id), p.temperature, p.top_p, p.top_k)
                for e, p in zip(entries, params)]
        if rows != self._sample_rows or bucket != self._sample_bucket:
            # the batch changed: rewrite the per-row parameters (padding rows are greedy)
            fh[:bucket] = 0.0
            fh[cap:cap + bucket] = 1.0
            fh[2 * cap:] = 0.0
            ih[:bucket] = 0
            for i, p in enumerate(params):
                fh[i], fh[cap + i], ih[i] = p.temperature, p.top_p, p.top_k
            self._sample_rows, self._sample_bucket = rows, bucket
            self._sample_drawn = [i for i, p in enumerate(params) if not p.greedy]
            self._sample_i[:cap].copy_(self._sample_i_host, non_blocking=True)
            dirty = True
        else:
            dirty = bool(self._sample_drawn)
        for i in self._sample_drawn:
            for j in range(k):
                fh[(2 + j) * cap + i] = uniform(seed, streams[i], counters[i] + j)
        if dirty:
            self._sample_f.copy_(self._sample_f_host, non_blocking=True)
        self._run_counter.zero_()
        greedy = self._tail is not None and not self._sample_drawn and self.model.can_pick(bucket)
        key = (bucket, launch_key, greedy)
        graph = self.graphs.get(key)
        replays = k
        if greedy:
            # the run's first residual stream; every later one is left there by the step before
            self.model.embed(step)
            self.num_greedy_tails += k
        if graph is None:
            self._forward_and_sample(step, bucket, greedy)  # the first step, and a warm-up
            graph = self.graphs[key] = self._capture(step, bucket, greedy)
            replays -= 1
        for _ in range(replays):
            graph.graph.replay()
        return self._queue_read(ids, [e.start_pos for e in entries], k, 0, bucket, replays, greedy)

    def _queue_read(self, ids, begins, k: int, base: int, bucket: int, replays: int,
                    greedy: bool = False) -> "_QueuedRun":
        """Queue the copy of ring rows ``base..base+k-1`` to the host behind the run's launches."""
        self._ring_host[base:base + k].copy_(self._run_ring[base:base + k], non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        return _QueuedRun(ids, begins, k, base, bucket, replays, event, greedy)

    def _continue_run(self, run: "_QueuedRun", entries, seed, streams, counters
                      ) -> "_QueuedRun | None":
        """Queue the run that follows ``run`` for the same batch, whose inputs the device holds
        already; ``None`` where its launches are not captured yet or its pages are missing."""
        k, cap = run.k, self.meta.max_seqs
        starts = [p + k for p in run.begins]     # where the following run begins
        if any(s + k > self.max_model_len for s in starts):
            return None
        shape = DecodeShape(len(starts), max(starts) + 1, sum(s + 1 for s in starts))
        graph = self.graphs.get((run.bucket, self.model.launch_key(shape), run.greedy))
        if graph is None:
            return None
        base = k if run.base == 0 else 0
        # its pages have to be in the requests' tables by now; they travel behind the launches
        # that are queued already
        groups = range(len(self.model.cache_groups))
        for e, s in zip(entries, starts):
            if any(len(self.cache.block_table(e.request_id, g)) * self.block_size < s + k for g in groups):
                return None
        extend_tables(self.meta, entries, run.bucket, [s + k for s in starts], self.cache.block_table,
                      self.block_size, self._windowed, self.cache.serial)
        if self._sample_drawn:
            fh = self._sample_f_np
            lo = (2 + base) * cap
            for i in self._sample_drawn:
                for j in range(k):
                    fh[lo + j * cap + i] = uniform(seed, streams[i], counters[i] + k + j)
            self._sample_f[lo:lo + k * cap].copy_(self._sample_f_host[lo:lo + k * cap], non_blocking=True)
        if base == 0:
            self._run_counter.zero_()
        for _ in range(k):
            graph.graph.replay()
        self.num_greedy_tails += k if run.greedy else 0
        return self._queue_read(run.ids, starts, k, base, run.bucket, k, run.greedy)

    def _forward_and_sample(self, step: Step, rows: int, greedy: bool = False) -> torch.Tensor | None:
        """One decode step of a padded batch with everything up to its next inputs.  ``greedy``:
        all rows take the largest logit and the residual stream is in place already: the head's
        kernel does the whole tail."""
        if greedy:
            return self.model.forward(step, tail=self._tail, embedded=True)
        cap = self.meta.max_seqs
        logits = self.model.forward(step)
        sampled = self._sample_i[cap:cap + rows]
        ops.sample(logits, self._sample_f[:rows], self._sample_i[:rows],
                   self._sample_f[cap:cap + rows], self._sample_f[2 * cap:].view(MAX_DECODE_RUN, cap),
                   sampled, self._run_counter, self._sample_work)
        ops.decode_advance(sampled, step.token_ids, step.positions, step.ctx_lens, self._run_ring,
                           self._run_counter)
        return logits

    def _capture(self, step: Step, rows: int, greedy: bool = False) -> "_DecodeGraph":
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        self.ws.frozen = True
        try:
            with torch.cuda.graph(graph):
                logits = self._forward_and_sample(step, rows, greedy)
        finally:
            self.ws.frozen = False
        # the graph keeps the workspace it was recorded with alive, whatever grows later
        return _DecodeGraph(graph, logits, self.ws.snapshot())


GRAPH_MAX_BATCH = 128  # beyond this the matrix products leave the weight-streaming kernel
MAX_DECODE_RUN = 16    # decode steps the device can take by itself before the host looks


class _QueuedRun:
    """Decode steps that are queued on the device: whose they are, the position each request
    begins them at, which ring rows hold their tokens, and the event behind the copy of those
    rows."""

    def __init__(self, ids, begins, k, base, bucket, replays, event, greedy=False) -> None:
        self.ids, self.begins, self.k, self.base = ids, begins, k, base
        self.bucket, self.replays, self.event, self.greedy = bucket, replays, event, greedy


class _DecodeGraph:
    def __init__(self, graph, logits, keep) -> None:
        self.graph, self.logits, self.keep = graph, logits, keep
