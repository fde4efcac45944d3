"""The runnable model: a ``ModelSpec`` (parts chosen by the registry's builder) with its weights
on the device, its cache groups worked out, and one ``forward`` over a flat batch
(src/tokenvault/model.py:175-191)."""

from __future__ import annotations

import torch

from kvforge_amd import registry
from kvforge_amd.cache.manager import CacheGroup
from kvforge_amd.kernels import library
from kvforge_amd.parts.base import Block, CacheSpec, LayerState, ModelSpec, Positions, StateSpec
from kvforge_amd.weights.loader import load_model_weights


class Transformer:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device: torch.device | str) -> None:
        self.spec, self.config = spec, spec.config
        self.dtype, self.device = dtype, device
        self.order = spec.run_order()
        n, calls = len(spec.blocks), len(self.order)
        for c in self.order:
            if not 0 <= c.layer < n:
                raise ValueError(f"run order names a layer outside 0..{n - 1}: {c}")
        # Pages and state belong to a *call* (an entry of the run order), not to a block: a block
        # named twice shares its weights, and each of its calls keeps a cache of its own.
        owners = [i for i, c in enumerate(self.order) if c.cache_of is None
                  and spec.blocks[c.layer].mixer.cache_spec is not None]
        for i, c in enumerate(self.order):
            if c.cache_of is None:
                continue
            if not 0 <= c.cache_of < calls or c.cache_of not in owners:
                raise ValueError(f"call {i} reads the cache of call {c.cache_of}, which owns none")
            if c.cache_of >= i:
                raise ValueError(f"call {i} reads the cache of a later call ({c.cache_of})")
            a = spec.blocks[c.layer].mixer.cache_spec
            b = spec.blocks[self.order[c.cache_of].layer].mixer.cache_spec
            if a != b:
                raise ValueError(f"call {i} and call {c.cache_of} need different caches: {a} / {b}")
        by_spec: dict[CacheSpec, list[int]] = {}
        for i in owners:
            by_spec.setdefault(spec.blocks[self.order[i].layer].mixer.cache_spec, []).append(i)
        self.cache_groups = [CacheGroup(tuple(ix), cs.pages, cs.window)
                             for cs, ix in by_spec.items()]
        self.state_specs: dict[int, StateSpec] = {
            i: spec.blocks[c.layer].mixer.state_spec for i, c in enumerate(self.order)
            if spec.blocks[c.layer].mixer.state_spec is not None}
        self.layer_states: list[LayerState] = []
        self._loaded = False

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_folder(cls, folder: str, dtype: torch.dtype, device: torch.device | str = "cuda"
                    ) -> "Transformer":
        cfg = registry.config_from_folder(folder)
        model = cls(registry.build_spec(cfg), dtype, device)
        model.load_folder(folder)
        return model

    @classmethod
    def from_random(cls, config, seed: int, dtype: torch.dtype, device: torch.device | str = "cuda",
                    drawn: "dict[str, torch.Tensor] | None" = None) -> "Transformer":
        """Random weights drawn on the device, no files (``config``: a config.json dictionary or
        a typed configuration).  ``drawn``, if given, is filled with the tensors by checkpoint
        name as they were drawn, for whoever wants to compute the same model another way."""
        from kvforge_amd.weights.random_init import load_random_weights

        cfg = registry.config_from_dict(config) if isinstance(config, dict) else config
        model = cls(registry.build_spec(cfg), dtype, device)
        tensors = load_random_weights(model.spec, seed, dtype, device)
        if drawn is not None:
            drawn.update(tensors)
        del tensors
        model._seal()
        return model

    def load_folder(self, folder: str) -> None:
        load_model_weights(self.spec, folder, self.dtype, self.device)
        self._seal()

    def _seal(self) -> None:
        for p in self.spec.all_parts():
            p.seal()
        self._loaded = True

    def kernel_modules(self) -> list[str]:
        mods: set[str] = {"elementwise", "sampling"}
        for p in self.spec.all_parts():
            mods |= p.kernel_modules(self.dtype)
        return sorted(m for m in mods if m in library.available_modules())

    def prepare(self, max_positions: int) -> None:
        for p in self.spec.positions:
            p.prepare(max_positions, self.device)

    def attach(self, storage, states) -> None:
        """Bind every call of the run order to its pages and state tensor."""
        self.layer_states = []
        for i, c in enumerate(self.order):
            src = i if c.cache_of is None else c.cache_of
            ls = LayerState(owns_cache=c.cache_of is None)
            if src in storage.pages:
                ls.group, ls.pages = storage.group_of[src], storage.pages[src]
            if states is not None and i in states.tensors:
                ls.state = states.tensors[i]
            self.layer_states.append(ls)

    @property
    def weight_bytes(self) -> int:
        """Bytes of weights one decode step reads: what every part says it reads (``num_bytes``),
        a block once for each time the run order names it.  An embedding table counts only where
        a head reads it whole."""
        spec = self.spec
        total = sum(p.num_bytes() for p in (spec.embedding, spec.final_norm, spec.head, *spec.positions))
        return total + sum(spec.blocks[c.layer].num_bytes() for c in self.order)

    def launch_key(self, shape) -> tuple:
        """The distinct launch keys of the model's parts for a step of single tokens (see
        ``Part.launch_key``): what captured decode steps are kept by, beside the batch size."""
        keys = []
        for top in self.spec.all_parts():
            for p in (top, *(top.parts() if isinstance(top, Block) else ())):
                k = p.launch_key(shape)
                if k is not None and k not in keys:
                    keys.append(k)
        return tuple(keys)

    @property
    def resident_bytes(self) -> int:
        """Bytes the weights occupy on the device, every copy and layout counted (a tensor that
        two parts share counts once)."""
        seen: dict[int, int] = {}
        for p in self.spec.all_parts():
            for t in p.held_tensors():
                seen[t.data_ptr()] = t.numel() * t.element_size()
        return sum(seen.values())

    # ------------------------------------------------------------------ forward
    def can_pick(self, rows: int) -> bool:
        """Whether a decode step of ``rows`` sequences can end in the head's greedy pick
        (``forward(step, tail=...)``): the parts say so themselves.  The embedding names a bf16
        table that holds its outputs (``Embedding.pick_table``), no position encoding touches
        the embedding output, and the head takes so many rows (``Head.can_pick``)."""
        spec = self.spec
        untouched = all(type(p).on_embedding is Positions.on_embedding for p in spec.positions)
        return (self.dtype == torch.bfloat16 and untouched
                and spec.embedding.pick_table() is not None and spec.head.can_pick(rows))

    def embed(self, step) -> torch.Tensor:
        """The step's residual stream, filled from the embedding."""
        spec = self.spec
        residual = step.ws.buf("residual", (step.n_tokens, spec.embedding.hidden), torch.float32)
        spec.embedding.forward(step.token_ids, residual)
        for p in spec.positions:
            p.on_embedding(residual, step)
        return residual

    def forward(self, step, tail=None, embedded: bool = False) -> torch.Tensor | None:
        """Runs the step's tokens from the cache; returns fp32 logits ``[n_logits, vocab]`` (a
        view of workspace memory, valid until the next forward).

        ``tail`` (a ``DecodeTail``, for a step of single tokens that all want their logits and
        are picked greedily, where ``can_pick`` allows it): no logits are made; the head's
        kernel picks the tokens, makes them the sequences' next inputs and leaves their
        embeddings in the residual stream, so that the next such step runs with ``embedded``
        (the stream is there already) and returns ``None`` again."""
        spec = self.spec
        cfg = self.config
        hidden = spec.embedding.hidden
        if embedded:
            residual = step.ws.buf("residual", (step.n_tokens, hidden), torch.float32)
        else:
            residual = self.embed(step)
        for call, ls in zip(self.order, self.layer_states):
            spec.blocks[call.layer].forward(residual, step, ls)
        r = step.n_logits
        if tail is not None and (r != step.n_tokens or not self.can_pick(r)):
            raise ValueError("the greedy tail is for steps of single tokens that all want their "
                             "logits, on a model that can_pick")
        if r == 0:
            step.owed = None
            return torch.empty((0, cfg.vocab_size), dtype=torch.float32, device=residual.device)
        x = step.ws.buf("final_normed", (r, hidden), step.act_dtype)
        # only the wanted rows matter now: what is still owed to the stream is added to them alone
        spec.final_norm.forward(residual, x, step.logits_rows, add=step.take_owed(residual))
        if tail is not None:
            spec.head.pick(x, residual, step, tail)
            return None
        logits = step.ws.buf("logits", (r, cfg.vocab_size), torch.float32)
        spec.head.forward(x, logits)
        return logits
