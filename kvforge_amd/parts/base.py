"""What every part of a model is made of.

A *part* (norm, position encoding, mixer, feed-forward, embedding, head) takes its sizes and
constants as constructor arguments, names the checkpoint tensors it needs, and knows nothing of
the model it sits in.  A *block* arranges parts around the fp32 residual stream.  A model is a
list of blocks plus the order in which they run (``LayerCall``), which is data: a block may be
named twice, and a call may use another block's cache.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import TYPE_CHECKING

import torch

if TYPE_CHECKING:  # pragma: no cover
    from kvforge_amd.engine.batch import Step


@dataclass(frozen=True)
class WeightSpec:
    """One checkpoint tensor a part expects.

    ``init`` drives the random-weights mode: ``"normal"`` draws N(0, std), ``"norm"`` draws
    1 + N(0, std), ``"zeros"`` is zero.  ``integer`` tensors are tables of int32."""

    shape: tuple[int, ...]
    init: str = "normal"
    std: float = 0.02
    integer: bool = False


BLOCK = "block"   # stands for the page size (tokens per page) in a ``PageTensor``'s shape


@dataclass(frozen=True)
class PageTensor:
    """One tensor of a mixer's pages: ``name`` is what the mixer finds it under in
    ``LayerState.pages``, ``shape`` the shape of one page, in which ``BLOCK`` stands for the
    number of tokens a page holds (so the mixer chooses where the token index lies), ``dtype``
    the element type (``None``: the engine's)."""

    name: str
    shape: tuple
    dtype: torch.dtype | None = None

    def page_shape(self, block_size: int) -> tuple[int, ...]:
        return tuple(block_size if s == BLOCK else int(s) for s in self.shape)

    def page_bytes(self, block_size: int, engine_dtype: torch.dtype) -> int:
        n = 1
        for s in self.page_shape(block_size):
            n *= s
        return n * torch.tensor([], dtype=self.dtype or engine_dtype).element_size()


def attention_pages(num_kv_heads: int, head_dim: int) -> tuple[PageTensor, PageTensor]:
    """Keys ``[kv heads, block, head size]`` (a key's elements side by side) and values
    transposed, ``[kv heads, head size, block]`` (an element's keys side by side, the order in
    which the matrix cores contract ``P * V``)."""
    return (PageTensor("k", (num_kv_heads, BLOCK, head_dim)),
            PageTensor("v", (num_kv_heads, head_dim, BLOCK)))


@dataclass(frozen=True)
class CacheSpec:
    """A mixer's need for per-token memory that grows with the sequence: the tensors its pages
    consist of (keys and values for attention; any others for another mixer, one latent vector
    per token, say).

    ``window``: ``None`` keeps every position; ``w`` keeps the last ``w`` positions, and pages
    wholly behind the window are given back while the request is live.  Layers with equal specs
    form one cache group with pages and block tables of its own."""

    pages: tuple[PageTensor, ...]
    window: int | None = None


@dataclass(frozen=True)
class StateSpec:
    """A mixer's per-request state of fixed size: one slot of ``shape`` per live request."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class LayerState:
    """What a mixer call is handed besides activations: the cache pages it reads and writes
    (possibly another block's), the group whose block tables address them, and its state slots."""

    group: int | None = None
    pages: dict[str, torch.Tensor] = field(default_factory=dict)   # by ``PageTensor.name``
    owns_cache: bool = True
    state: torch.Tensor | None = None

    @property
    def k_pages(self) -> torch.Tensor | None:
        return self.pages.get("k")

    @property
    def v_pages(self) -> torch.Tensor | None:
        return self.pages.get("v")


class Part:
    """Base of all parts.  ``prefix`` is the part's place in the checkpoint's name space."""

    prefix: str = ""

    # Whether ``forward`` only launches device work whose arguments live in the step's device
    # buffers, so that a launch captured for one batch may be replayed for another.  A part that
    # looks at the step's host-side fields (lengths, slot numbers) or waits for the device is
    # not; one such part keeps the whole model out of the captured decode path.
    replayable: bool = False

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        """Take the named tensors (already on the device, already in their run-time dtype)."""

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return set()

    def num_bytes(self) -> int:
        """Bytes of weights this part reads in one step."""
        return 0

    def held_tensors(self) -> list[torch.Tensor]:
        """The device tensors this part keeps for its weights, every copy and layout of them
        (what the weights occupy, as opposed to what a step reads)."""
        return []

    def launch_key(self, shape):
        """What this part's launches for a step of single tokens depend on besides the padded
        batch size, worked out from ``shape`` (``n`` sequences with a context, ``max_ctx``,
        ``sum_ctx``): any hashable value.  Captured launches are replayed only for steps whose
        parts all give the keys they were captured with.  ``None``: nothing (the default)."""
        return None

    def seal(self) -> None:
        """Called once after ``load`` (and any ``absorb_norm``), before the first forward: the
        place for the last re-layout of weights, such as tiles for the weight-streaming kernel."""

    def absorb_norm(self, norm: "Norm") -> bool:
        """Offer the norm that feeds this part.  A part that can apply it inside its own first
        kernel takes what it needs from ``norm`` and returns True; from then on its ``forward``
        is handed the fp32 residual stream instead of normalised activations."""
        return False

    def _name(self, local: str) -> str:
        return f"{self.prefix}.{local}" if self.prefix else local


class Norm(Part):
    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: torch.Tensor | None = None,
                add: torch.Tensor | None = None) -> None:
        """``out[m] = norm(x[rows[m] or m])``; ``x`` is the fp32 residual stream.  ``add`` is a
        product still owed to ``x`` (same shape): the norm is taken of ``x + add``, and without
        ``rows`` the sum is left in ``x``."""
        raise NotImplementedError


class Positions(Part):
    """Position encoding.  Two hooks, both optional: one on the embedding output (absolute
    encodings) and tables a mixer applies to queries and keys (rotary encodings)."""

    def prepare(self, max_positions: int, device: torch.device | str) -> None:
        """Build per-position tables for positions ``0..max_positions-1``."""

    def on_embedding(self, residual: torch.Tensor, step: "Step") -> None:
        """Modify the embedding output in place (default: nothing)."""


class Mixer(Part):
    """Mixes information across the tokens of a sequence (attention, recurrences, ...).

    ``settles_residual``: a part that sets this looks after ``step.owed`` itself (it takes the
    owed product into its norm kernel); every other part is handed a residual stream that is
    up to date."""

    settles_residual = False

    cache_spec: CacheSpec | None = None
    state_spec: StateSpec | None = None

    def forward(self, x: torch.Tensor, step: "Step", layer: LayerState,
                residual: torch.Tensor) -> None:
        """Add the mixer's output for activations ``x [N, hidden]`` into ``residual`` (fp32)."""
        raise NotImplementedError


class FeedForward(Part):
    settles_residual = False

    def forward(self, x: torch.Tensor, step: "Step", residual: torch.Tensor) -> None:
        """Add the feed-forward output for ``x [N, hidden]`` into ``residual`` (fp32)."""
        raise NotImplementedError


class Embedding(Part):
    """Turns token ids into the first residual stream.  ``hidden``: the stream's width."""

    hidden: int

    def forward(self, ids: torch.Tensor, out: torch.Tensor) -> None:
        """``out[m]`` (fp32 ``[N, hidden]``) = the embedding of token ``ids[m]``."""
        raise NotImplementedError

    def pick_table(self) -> torch.Tensor | None:
        """A bf16 table ``[vocab, hidden]`` whose row ``t``, widened to fp32, *is* what
        ``forward`` gives for token ``t``, or ``None`` (the default) when no such table
        exists.  A head whose kernel chooses the next token itself (``Head.pick``) gathers the
        next step's residual rows from it; an embedding that says ``None`` keeps its model on
        the path that samples from stored logits and embeds in a kernel of its own."""
        return None


class Head(Part):
    """Turns normalised rows into logits over the vocabulary."""

    def forward(self, x: torch.Tensor, logits: torch.Tensor) -> None:
        """``logits`` (fp32 ``[R, vocab]``) for the rows ``x [R, hidden]``."""
        raise NotImplementedError

    def can_pick(self, rows: int) -> bool:
        """Whether ``pick`` takes ``rows`` rows (default: never)."""
        return False

    def pick(self, x: torch.Tensor, residual: torch.Tensor, step: "Step", tail) -> None:
        """The tail of a greedy step of single tokens without stored logits: choose every row's
        best token (the lowest index among equals), make it the sequence's next input in the
        step's device buffers and leave its embedding (``tail.embed_table``) in ``residual``.
        Only called where ``can_pick`` said yes."""
        raise NotImplementedError


class Block(Part):
    """An arrangement of parts around the residual stream."""

    mixer: Mixer

    def parts(self) -> list[Part]:
        raise NotImplementedError

    def forward(self, residual: torch.Tensor, step: "Step", layer: LayerState) -> None:
        raise NotImplementedError

    def weight_specs(self) -> dict[str, WeightSpec]:
        out: dict[str, WeightSpec] = {}
        for p in self.parts():
            out.update(p.weight_specs())
        return out

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        for p in self.parts():
            p.load(tensors)

    def seal(self) -> None:
        for p in self.parts():
            p.seal()

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        out: set[str] = set()
        for p in self.parts():
            out |= p.kernel_modules(dtype)
        return out

    def num_bytes(self) -> int:
        return sum(p.num_bytes() for p in self.parts())

    def held_tensors(self) -> list[torch.Tensor]:
        return [t for p in self.parts() for t in p.held_tensors()]

    @property
    def replayable(self) -> bool:
        return all(p.replayable for p in self.parts())


def add_product(step: "Step", a: torch.Tensor, w: torch.Tensor, residual: torch.Tensor,
                owed: torch.Tensor | None = None) -> None:
    """``residual += a @ w.T``, the last product of a mixer or feed-forward.  With few rows (or in
    fp32) the product kernel adds in its epilogue.  Many bf16 rows go to the library, whose
    product is left owed to the stream (``step.owe``) so that the next norm adds it on its way
    instead of an add kernel of its own.  One tile of rows over a deep weight with few columns
    is cut into two halves of K so that every compute unit pulls on the weight: the first half
    is added here, the second is left owed (rounded to bf16, as a stored product is).
    ``owed``: a sum the caller took from the step (``step.take_owed``) and has not added yet;
    it is added here, in the same kernel where that is possible."""
    from kvforge_amd.kernels import ops

    if ops.is_library_product(a, w):
        if owed is not None:
            ops.add_rows(residual, owed)
        product = step.ws.buf("owed_product", (a.shape[0], w.shape[0]), a.dtype)
        ops.gemm(a, w, product)
        step.owe(residual, product)
    elif ops.k_halves_pay(a, w) and residual.is_contiguous():
        half = step.ws.buf("owed_half", tuple(residual.shape), torch.bfloat16)
        if owed is not None and owed.data_ptr() == half.data_ptr():
            # what the caller took from the step is the half the product before this one left
            # there: this product's workgroups read it while others write their half, so the
            # new half goes to the other of two buffers
            half = step.ws.buf("owed_half_other", tuple(residual.shape), torch.bfloat16)
        ops.gemm(a, w, residual, accumulate=True, owed=owed, half_out=half)
        step.owe(residual, half)
    else:
        ops.gemm(a, w, residual, accumulate=True, owed=owed)


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order: run block ``layer``.  ``cache_of``: ``None`` gives the call a
    cache of its own, which it writes and reads; an index into the run order (of an earlier
    call) makes it read that call's cache and write none."""

    layer: int
    cache_of: int | None = None


@dataclass
class ModelSpec:
    """Everything the registry's builder decides for one architecture."""

    config: object
    embedding: Embedding
    blocks: list[Block]
    final_norm: Norm
    head: Head
    positions: list[Positions] = field(default_factory=list)
    schedule: list[LayerCall] | None = None
    # checkpoint names that may be present and are not loaded (regular expressions)
    ignored_weights: tuple[str, ...] = ()

    def run_order(self) -> list[LayerCall]:
        return self.schedule if self.schedule is not None else [
            LayerCall(i) for i in range(len(self.blocks))]

    def all_parts(self) -> list[Part]:
        return [self.embedding, *self.positions, *self.blocks, self.final_norm, self.head]

    def weight_specs(self) -> dict[str, WeightSpec]:
        out: dict[str, WeightSpec] = {}
        for p in self.all_parts():
            for name, spec in p.weight_specs().items():
                if name in out and out[name] != spec:
                    raise ValueError(f"two parts expect {name} with different shapes")
                out[name] = spec
        return out
