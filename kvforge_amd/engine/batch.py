"""The flat batch of one step: entries (request, its next tokens, where they start, which logits
are wanted) become int32 arrays in one fixed-address device buffer.

This is the reference's ``BatchItem`` / ``prepare_inputs`` (src/tokenvault/batching/continuous.py:
27-87) with two differences: there is no per-token slot list (kernels compute a token's slot from
its sequence's block-table row and its position), and sequences are told apart into query runs
(more than one token, prefill kernel) and single tokens (decode kernel) while the matrix products
still see one ``[N, hidden]`` matrix.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Sequence

import numpy as np
import torch



@dataclass(frozen=True)
class DecodeShape:
    """What the single-token sequences of a step look like, as far as a part's launches may
    depend on it besides the padded batch size: how many hold a context, the longest context
    and the sum of all.  Parts turn it into a launch key (``Part.launch_key``); steps with equal
    keys may replay the same captured launches."""

    n: int
    max_ctx: int
    sum_ctx: int


@dataclass
class DecodeTail:
    """What the head's greedy pick needs besides the step to do the tail of a decode step by
    itself (``Transformer.forward(step, tail=...)``): where the picked tokens go, the ring and
    the counter of the run's steps, the embedding table for the next step's residual stream,
    and the pick's scratch."""

    tokens: torch.Tensor
    ring: torch.Tensor
    run_counter: torch.Tensor
    embed_table: torch.Tensor
    work: tuple


@dataclass
class StepEntry:
    """``want``: places among ``token_ids`` whose logits are returned, or ``"last"`` / ``"all"``
    / ``"none"`` (the reference's ``LogitsMode``)."""

    request_id: str
    token_ids: Sequence[int]
    start_pos: int
    want: "Sequence[int] | str" = "last"

    def wanted(self) -> list[int]:
        n = len(self.token_ids)
        if isinstance(self.want, str):
            if self.want == "last":
                return [n - 1]
            if self.want == "all":
                return list(range(n))
            if self.want == "none":
                return []
            raise ValueError(f"unknown logits mode {self.want!r}")
        out = [int(i) for i in self.want]
        for i in out:
            if not 0 <= i < n:
                raise ValueError(f"wanted place {i} outside the entry's {n} tokens")
        return out


class Workspace:
    """Named scratch tensors that live across steps and grow on demand."""

    def __init__(self, device: torch.device | str) -> None:
        self.device = device
        self._bufs: dict[tuple[str, torch.dtype], torch.Tensor] = {}
        # views handed out before, by (name, dtype, shape): a step asks for the same ones again
        self._views: dict[tuple, torch.Tensor] = {}
        self.frozen = False

    def buf(self, name: str, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        view = self._views.get((name, dtype, shape))
        if view is not None:
            return view
        n = 1
        for s in shape:
            n *= int(s)
        key = (name, dtype)
        flat = self._bufs.get(key)
        if flat is None or flat.numel() < n:
            if self.frozen:
                raise RuntimeError(f"workspace buffer {name} would grow during graph capture")
            flat = torch.empty(max(n, 1), dtype=dtype, device=self.device)
            self._bufs[key] = flat
            for k in [k for k in self._views if k[0] == name and k[1] == dtype]:
                del self._views[k]           # they show the memory that was let go
        view = flat[:n].view(shape)
        if len(self._views) < 4096:
            self._views[(name, dtype, shape)] = view
        return view

    def zeros(self, name: str, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        """Like ``buf`` for memory whose users leave it zero: cleared once, when it is made."""
        n = 1
        for s in shape:
            n *= int(s)
        key = (name, dtype)
        flat = self._bufs.get(key)
        if flat is None or flat.numel() < n:
            if self.frozen:
                raise RuntimeError(f"workspace buffer {name} would grow during graph capture")
            flat = torch.zeros(max(n, 1), dtype=dtype, device=self.device)
            self._bufs[key] = flat
            for k in [k for k in self._views if k[0] == name and k[1] == dtype]:
                del self._views[k]
        return flat[:n].view(shape)

    def snapshot(self) -> list[torch.Tensor]:
        return list(self._bufs.values())


class MetaBuffers:
    """Fixed-address int32 device memory for batch metadata, filled through pinned staging."""

    def __init__(self, max_tokens: int, max_seqs: int, table_widths: list[int],
                 device: torch.device | str) -> None:
        self.max_tokens, self.max_seqs, self.table_widths = max_tokens, max_seqs, list(table_widths)
        off = 0
        self.off: dict[str, int] = {}
        for name, size in (("cu_q", max_seqs + 1), ("ctx_lens", max_seqs), ("slot_ids", max_seqs),
                           ("decode_seq_ids", max_seqs), ("token_ids", max_tokens),
                           ("positions", max_tokens), ("seq_of_token", max_tokens),
                           ("logits_rows", max_tokens)):
            self.off[name] = off
            off += (size + 3) // 4 * 4
        self.table_off: list[int] = []
        for w in self.table_widths:
            self.table_off.append(off)
            off += max_seqs * w
        # room behind the batch's own fields for what parts send along with a step
        # (``Step.upload_ints``)
        self.extra_off, self.extra_size = off, max(4096, 4 * max_tokens)
        off += self.extra_size
        self.total = off
        self.device_buf = torch.zeros(self.total, dtype=torch.int32, device=device)
        pin = torch.device(device).type == "cuda"
        self.staging = [torch.zeros(self.total, dtype=torch.int32, pin_memory=pin) for _ in range(2)]
        self.staging_np = [s.numpy() for s in self.staging]
        self.events: list[torch.cuda.Event | None] = [None, None]
        self.turn = 0
        # host mirror of the block tables: a row is rewritten only where it changed since the
        # step before (a request that keeps its row only appends pages)
        self.table_host = [np.full((max_seqs, w), -1, dtype=np.int32) for w in self.table_widths]
        self.row_owner: list[list[tuple | None]] = [[None] * max_seqs for _ in self.table_widths]
        self.row_filled = [np.zeros(max_seqs, dtype=np.int64) for _ in self.table_widths]

    def view(self, name: str, n: int) -> torch.Tensor:
        o = self.off[name]
        return self.device_buf[o:o + n]

    def table_view(self, g: int) -> torch.Tensor:
        o, w = self.table_off[g], self.table_widths[g]
        return self.device_buf[o:o + self.max_seqs * w].view(self.max_seqs, w)


class Step:
    """One step's batch on the device, plus the host-side facts parts may need."""

    def __init__(self) -> None:
        self.n_tokens = 0
        self.n_seqs = 0
        self.n_logits = 0
        self.n_decode = 0
        self.act_dtype: torch.dtype = torch.float32
        self.ws: Workspace = None  # type: ignore[assignment]
        self.token_ids = self.positions = self.seq_of_token = None
        self.cu_q = self.ctx_lens = self.slot_ids = self.logits_rows = None
        self.decode_seq_ids: torch.Tensor | None = None
        self.block_tables: list[torch.Tensor] = []
        # host copies
        self.request_ids: list[str] = []
        self.q_lens: list[int] = []
        self.start_pos: list[int] = []
        self.host_slot_ids: list[int] = []
        self.host_token_ids: np.ndarray | None = None
        self.prefill_seqs: list[int] = []
        self.decode_shape = DecodeShape(0, 0, 0)
        self.max_position = 0
        # What parts keep for the length of the step (work lists, launch plans, tables), under
        # keys of their own choosing: the step knows nothing of any part's tiling.
        self.scratch: dict = {}
        self.device: torch.device | str = "cuda"
        # A product still owed to the residual stream: (stream, product).  A part that ends in a
        # library product over many rows leaves it here instead of running an add kernel; the
        # next norm adds it on its way (``take_owed``), anything else calls ``settle`` first.
        self.owed: tuple[torch.Tensor, torch.Tensor] | None = None
        # the staging memory this step was filled from (``fill_step``), for ``upload_ints``
        self._meta: "MetaBuffers | None" = None
        self._turn = 0
        self._extra_used = 0

    def upload_ints(self, values) -> torch.Tensor:
        """An int32 device tensor holding ``values`` (a flat sequence or array), for what a part
        derives on the host for this step (a work list, a table): it travels through the same
        pinned staging memory as the batch itself, queued on the stream without waiting for
        the device, and stays valid until the next step is filled.  A step that was not filled
        from staging memory (or has no room left there) sends it the slow way."""
        arr = np.asarray(values, dtype=np.int32).reshape(-1)
        meta, n = self._meta, int(arr.shape[0])
        if meta is None or not meta.device_buf.is_cuda or self._extra_used + n > meta.extra_size:
            return torch.from_numpy(arr.copy()).to(self.device)
        lo = meta.extra_off + self._extra_used
        self._extra_used += (n + 3) // 4 * 4
        meta.staging_np[self._turn][lo:lo + n] = arr
        dst = meta.device_buf[lo:lo + n]
        dst.copy_(meta.staging[self._turn][lo:lo + n], non_blocking=True)
        meta.events[self._turn].record()     # the staging memory is free again after this copy
        return dst

    def owe(self, residual: torch.Tensor, product: torch.Tensor) -> None:
        self.settle()
        self.owed = (residual, product)

    def take_owed(self, residual: torch.Tensor) -> torch.Tensor | None:
        """The product owed to ``residual``, for a norm kernel that adds it itself."""
        if self.owed is None:
            return None
        if self.owed[0] is not residual:
            self.settle()
            return None
        product = self.owed[1]
        self.owed = None
        return product

    def settle(self) -> None:
        """Add what is owed to the residual stream now."""
        if self.owed is not None:
            from kvforge_amd.kernels import ops
            ops.add_rows(*self.owed)
            self.owed = None


def _fill_tables(meta: "MetaBuffers", host: np.ndarray, entries: Sequence[StepEntry], Bp: int,
                 need_tokens: Sequence[int], tables_of, block_size: int,
                 windowed_groups: Sequence[bool] | None, serial_of) -> int:
    """Bring the host mirror of the block tables up to date for ``entries`` (row ``b`` holds the
    pages of ``need_tokens[b]`` positions; rows ``len(entries)..Bp-1`` are empty) and write the
    rows into the staging memory ``host``.  Returns the end of the table region."""
    B = len(entries)
    end = 0
    for g, (to, w) in enumerate(zip(meta.table_off, meta.table_widths)):
        mirror, owner, filled = meta.table_host[g], meta.row_owner[g], meta.row_filled[g]
        windowed = windowed_groups is not None and windowed_groups[g]
        for b, e in enumerate(entries):
            t = tables_of(e.request_id, g)
            need = -(-need_tokens[b] // block_size)
            if need > w or need > len(t):
                raise ValueError(f"request {e.request_id} needs {need} pages in group {g}; "
                                 f"table holds {len(t)}, width {w}")
            have = int(filled[b])
            tag = (e.request_id, serial_of(e.request_id)) if serial_of is not None else None
            if tag is not None and owner[b] == tag and have <= need and not windowed:
                if have < need:
                    mirror[b, have:need] = t[have:need]
            else:
                mirror[b, :have] = -1
                mirror[b, :need] = t[:need]
                owner[b] = tag
            filled[b] = need
        for b in range(B, Bp):
            if filled[b]:
                mirror[b, :int(filled[b])] = -1
            owner[b], filled[b] = None, 0
        host[to:to + Bp * w].reshape(Bp, w)[:] = mirror[:Bp]
        end = to + Bp * w
    return end


def extend_tables(meta: "MetaBuffers", entries: Sequence[StepEntry], padded: int,
                  need_tokens: Sequence[int], tables_of, block_size: int,
                  windowed_groups: Sequence[bool] | None = None, serial_of=None) -> None:
    """For a batch that is on the device already (same entries, same rows): make its block
    tables hold the pages of ``need_tokens[b]`` positions.  Only the table region travels, in
    stream order, so launches queued before it still see the tables they were queued with (it
    only adds pages, or takes away pages that lie wholly behind a window)."""
    if not meta.table_off:
        return
    turn = meta.turn
    meta.turn ^= 1
    if meta.events[turn] is not None:
        meta.events[turn].synchronize()
    host = meta.staging_np[turn]
    end = _fill_tables(meta, host, entries, padded, need_tokens, tables_of, block_size,
                       windowed_groups, serial_of)
    start = meta.table_off[0]
    meta.device_buf[start:end].copy_(meta.staging[turn][start:end], non_blocking=True)
    if meta.device_buf.is_cuda:
        ev = meta.events[turn] or torch.cuda.Event()
        ev.record()
        meta.events[turn] = ev


def fill_step(step: Step, meta: MetaBuffers, entries: Sequence[StepEntry], tables_of, slot_of,
              block_size: int, pad_to: int | None = None,
              windowed_groups: Sequence[bool] | None = None, serial_of=None,
              lookahead: int = 0) -> list[int]:
    """Write the batch into ``meta`` (one host-to-device copy) and point ``step`` at it.
    ``tables_of(request_id, group) -> list[int]``; ``slot_of(request_id) -> int``.
    ``pad_to``: pad a pure-decode batch with empty sequences up to this many.
    ``windowed_groups[g]``: group ``g`` gives pages back while a request lives, so its rows are
    rewritten whole every step.  ``serial_of(request_id)`` tells a request id that was freed and
    allocated again from its former self (without it rows are always rewritten whole).
    ``lookahead``: the tables also carry the pages of this many positions past the step's, for
    further decode steps that the device advances to by itself.
    Returns how many logits rows each entry gets."""
    B = len(entries)
    q_lens = [len(e.token_ids) for e in entries]
    if B == 0 or min(q_lens) <= 0:
        raise ValueError("a step needs entries, each with at least one token")
    Bp = B if pad_to is None else int(pad_to)
    N = sum(q_lens) + (Bp - B)
    if Bp > meta.max_seqs or N > meta.max_tokens:
        raise ValueError(f"step of {N} tokens / {Bp} requests exceeds the runner's capacity "
                         f"({meta.max_tokens} tokens / {meta.max_seqs} requests)")
    turn = meta.turn
    meta.turn ^= 1
    if meta.events[turn] is not None:
        meta.events[turn].synchronize()
    host = meta.staging_np[turn]
    off = meta.off

    lens = np.asarray(q_lens + [1] * (Bp - B), dtype=np.int32)
    starts = np.asarray([e.start_pos for e in entries] + [0] * (Bp - B), dtype=np.int32)
    cu = np.zeros(Bp + 1, dtype=np.int32)
    np.cumsum(lens, out=cu[1:])
    host[off["cu_q"]:off["cu_q"] + Bp + 1] = cu
    ctx = starts + lens
    ctx[B:] = 0  # padding sequences hold nothing
    host[off["ctx_lens"]:off["ctx_lens"] + Bp] = ctx
    slots = [slot_of(e.request_id) for e in entries] + [-1] * (Bp - B)
    host[off["slot_ids"]:off["slot_ids"] + Bp] = slots
    tok = host[off["token_ids"]:off["token_ids"] + N]
    pos = host[off["positions"]:off["positions"] + N]
    p = 0
    for e, n, s in zip(entries, q_lens, starts[:B]):
        tok[p:p + n] = e.token_ids
        pos[p:p + n] = np.arange(s, s + n, dtype=np.int32)
        p += n
    tok[p:] = 0
    pos[p:] = 0
    host[off["seq_of_token"]:off["seq_of_token"] + N] = np.repeat(np.arange(Bp, dtype=np.int32), lens)

    counts, rows = [], []
    for b, e in enumerate(entries):
        w = e.wanted()
        counts.append(len(w))
        rows.extend(int(cu[b]) + i for i in w)
    if pad_to is not None:
        # a padded batch has a fixed shape: one wanted row per sequence, padding included
        if any(c != 1 for c in counts) or any(n != 1 for n in q_lens):
            raise ValueError("padding is for batches of single tokens that each want their logits")
        rows = list(range(Bp))
    R = len(rows)
    host[off["logits_rows"]:off["logits_rows"] + R] = rows

    decode = [b for b in range(Bp) if lens[b] == 1]
    prefill = [b for b in range(B) if lens[b] > 1]
    host[off["decode_seq_ids"]:off["decode_seq_ids"] + len(decode)] = decode

    end = off["logits_rows"] + max(R, 1)
    need_tokens = [int(ctx[b]) + lookahead for b in range(B)]
    end = max(end, _fill_tables(meta, host, entries, Bp, need_tokens, tables_of, block_size,
                                windowed_groups, serial_of))
    meta.device_buf[:end].copy_(meta.staging[turn][:end], non_blocking=True)
    if meta.device_buf.is_cuda:
        ev = meta.events[turn] or torch.cuda.Event()
        ev.record()
        meta.events[turn] = ev

    step.n_tokens, step.n_seqs, step.n_logits, step.n_decode = N, Bp, R, len(decode)
    step.token_ids = meta.view("token_ids", N)
    step.positions = meta.view("positions", N)
    step.seq_of_token = meta.view("seq_of_token", N)
    step.cu_q = meta.view("cu_q", Bp + 1)
    step.ctx_lens = meta.view("ctx_lens", Bp)
    step.slot_ids = meta.view("slot_ids", Bp)
    step.logits_rows = meta.view("logits_rows", max(R, 1))[:R]
    step.decode_seq_ids = None if len(decode) == Bp else meta.view("decode_seq_ids", len(decode))
    step.block_tables = [meta.table_view(g)[:Bp] for g in range(len(meta.table_widths))]
    step.request_ids = [e.request_id for e in entries]
    step.q_lens = [int(x) for x in lens]
    step.start_pos = [int(x) for x in starts]
    step.host_slot_ids = slots
    step.host_token_ids = tok.copy()
    step.prefill_seqs = prefill
    live = [int(ctx[b]) for b in decode if ctx[b] > 0]
    step.decode_shape = DecodeShape(len(live), max(live, default=0), sum(live))
    step.max_position = int(ctx.max()) if Bp else 0
    step.scratch = {}
    step._meta, step._turn, step._extra_used = meta, turn, 0
    return counts
