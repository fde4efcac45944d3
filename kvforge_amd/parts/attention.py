"""Grouped-query causal attention over the paged cache (src/tokenvault/model.py:64-92).

Order of work per call, as in the reference: project q, k, v; rotate q and k; write k and v into
the cache; attend from the cache (the current tokens' keys are read back from it); project out.
Query runs longer than one token go to the prefill kernel, single tokens to the decode kernel;
both read the same pages through the same block tables.
"""

from __future__ import annotations

import math

import torch

from kvforge_amd.kernels import ops
from kvforge_amd.parts.base import (CacheSpec, LayerState, Mixer, WeightSpec, add_product,
                                    attention_pages)
from kvforge_amd.parts.positions import RotaryPositions
from kvforge_amd.registry import register_mixer

# Launch planning of the decode kernels.  The key range of single-token queries is cut so that
# about one workgroup per compute unit pulls on the cache when the sequences alone do not fill
# the chip, each cut with at least KEYS_PER_CUT keys (below that the merge of the cuts costs more
# than they save), and further when contexts are uneven.  Everything the launches depend on
# besides the padded batch size is the pair (context cell, cuts for uneven contexts) that
# ``PagedAttention.launch_key`` returns, so that captured launches can be replayed for any step
# with the same pair.
KEYS_PER_CUT = 512
MAX_CUTS = 64            # what the merge kernels take
SKEW_MAX_CUTS = 8


def compute_units(device) -> int:
    return ops.compute_units(device)


def skew_cuts(max_ctx: int, sum_ctx: int, n: int) -> int:
    """Cuts of the key range that uneven contexts ask for, whatever the number of sequences: a
    sequence's keys are walked by the waves of one workgroup per kv head and cut, so one long
    context among short ones sets the step's time (measured at 32 sequences of 32 heads: 31
    contexts of 600 and one of 32,768 take 153 us with one cut, 60 with eight; one of 8,192
    takes 45 and 33).  The longest walk is brought down to about twice the mean one; a power of
    two, so that captured launches change seldom."""
    if n <= 1 or max_ctx < 4 * KEYS_PER_CUT or sum_ctx <= 0:
        return 1
    want = min(max_ctx * n / (2.0 * sum_ctx), max_ctx // KEYS_PER_CUT, SKEW_MAX_CUTS)
    cuts = 1
    while cuts * 2 <= want:
        cuts *= 2
    return cuts


def prefill_work_rows(q_lens, prefill_seqs, group_size: int, rows_per_item: int,
                      start_pos=None) -> list[tuple]:
    """Rows (sequence row, item, -1) for every query run longer than one token: a run of ``q``
    tokens has ``q * group_size`` rows per kv head, an item covers ``rows_per_item`` of them, and
    a workgroup takes one item.  Under the causal mask an item walks the keys up to its last
    row's position (``start_pos``: the keys before each run): the items of all runs are handed
    out longest walk first, so that the short ones fill the gaps the long ones leave as compute
    units come free.  (The kernels also take two items per row, an early one paired with a late
    one, which balances the workgroups among themselves; measured once the kv heads were spread
    over the XCDs it lost to this order, which keeps twice the workgroups in flight: 2,048
    queries of 32 heads of size 64 take 58 us in pairs and 47 us one by one, 2,048 at the end
    of 8,192 keys 398 and 301.)"""
    rows = []
    for b in prefill_seqs:
        n = -(-q_lens[b] * group_size // rows_per_item)
        before = start_pos[b] if start_pos is not None else 0
        rows += [(before + min(q_lens[b], -(-(i + 1) * rows_per_item // group_size)), b, i) for i in range(n)]
    rows.sort(key=lambda r: -r[0])        # stable: equal walks stay in sequence and item order
    return [(b, i, -1) for _, b, i in rows]


@register_mixer("attention")
class PagedAttention(Mixer):
    """``window``: ``None`` attends to every earlier position, ``w`` to the last ``w``.
    ``rotary``: the rotation of q and k, or ``None`` for none.  ``score_slopes``: one number per
    q head, or ``None``; the score of key ``j`` for a query at position ``p`` of head ``h`` then
    gets ``score_slopes[h] * (j - p)`` added, a position encoding by distance that lives in the
    scores instead of in q and k."""

    replayable = True
    settles_residual = True  # its norm kernel adds what is owed to the stream

    def __init__(self, prefix: str, hidden: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 rotary: RotaryPositions | None, scale: float | None = None,
                 window: int | None = None, score_slopes=None) -> None:
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if head_dim % 16 or head_dim > 256:
            raise ValueError(
                f"attention kernels take head sizes in steps of 16 up to 256, got {head_dim}")
        self.prefix = prefix
        self.hidden, self.H, self.KV, self.d = int(hidden), int(num_heads), int(num_kv_heads), int(head_dim)
        self.rotary = rotary
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.d)
        self.window = int(window) if window else None
        self.score_slopes = None if score_slopes is None else [float(v) for v in score_slopes]
        if self.score_slopes is not None and len(self.score_slopes) != self.H:
            raise ValueError(f"score_slopes needs one number per q head ({self.H}), got {len(self.score_slopes)}")
        self.slopes: torch.Tensor | None = None
        self.cache_spec = CacheSpec(attention_pages(self.KV, self.d), self.window)
        self.w_qkv: torch.Tensor | None = None
        self.w_o: torch.Tensor | None = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, H, KV, d = self.hidden, self.H, self.KV, self.d
        return {
            self._name("q_proj.weight"): WeightSpec((H * d, h)),
            self._name("k_proj.weight"): WeightSpec((KV * d, h)),
            self._name("v_proj.weight"): WeightSpec((KV * d, h)),
            self._name("o_proj.weight"): WeightSpec((h, H * d)),
        }

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        q, k, v = (tensors[self._name(f"{n}_proj.weight")] for n in "qkv")
        if not (q.dtype == k.dtype == v.dtype):
            q, k, v = q.float(), k.float(), v.float()
        # The kernels rotate neighbouring elements (2i, 2i+1); the checkpoint pairs element i
        # with i + rot/2.  Permuting the rows of the q and k projections inside each head moves
        # the checkpoint's pairs next to each other; q.k does not depend on the order, v and the
        # output projection keep theirs.
        perm = self.pair_permutation()
        q = q.view(self.H, self.d, -1)[:, perm].reshape(self.H * self.d, -1)
        k = k.view(self.KV, self.d, -1)[:, perm].reshape(self.KV * self.d, -1)
        # one product for the three projections: rows of q heads, then k heads, then v heads
        self.w_qkv = torch.cat([q, k, v], dim=0).contiguous()
        self.w_o = tensors[self._name("o_proj.weight")]
        self.norm_eps = None
        if self.score_slopes is not None:
            self.slopes = torch.tensor(self.score_slopes, dtype=torch.float32, device=self.w_o.device)

    def pair_permutation(self) -> torch.Tensor:
        """``perm[new] = old`` within a head: new elements 2i and 2i+1 are the checkpoint's
        elements i and i + rot/2; elements beyond the rotary width stay."""
        rot = self.rotary.rot_dim if self.rotary is not None else 0
        perm = torch.arange(self.d)
        for i in range(rot // 2):
            perm[2 * i], perm[2 * i + 1] = i, i + rot // 2
        return perm

    def after_projection(self, qkv: torch.Tensor, step) -> None:
        """A place for a variant to change the projected rows before they are rotated and
        written to the cache (a bias on the projections, a norm per head of q and k): ``qkv``
        is ``[N, (H + 2 KV) d]`` in the step's activation type, q heads, then k heads, then v
        heads, each head's rotary pairs as neighbouring elements (``pair_permutation``); it is
        changed in place.  The default does nothing.  A subclass that overrides it runs
        projection, this, and rotation + cache write as kernels of their own in every step
        (the kernel that fuses the three has no place for it) and keeps its norm a kernel."""

    def _hooked(self) -> bool:
        return type(self).after_projection is not PagedAttention.after_projection

    def absorb_norm(self, norm) -> bool:
        if self._hooked():
            return False
        if self.norm_eps is not None or not getattr(norm, "foldable_into", lambda m: False)(self.w_qkv):
            return False
        self.w_qkv = (self.w_qkv.float() * norm.weight.float()[None, :]).to(torch.bfloat16).contiguous()
        self.norm_eps = norm.eps
        return True

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        mods = {"elementwise", "gemm_generic", "attn_generic"}
        if dtype == torch.bfloat16:
            mods |= {"gemm_bf16", "attn_mfma"}
        return mods

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size()
                   for t in map(ops.plain_of, (self.w_qkv, self.w_o)) if t is not None)

    def held_tensors(self) -> list[torch.Tensor]:
        return ops.copies_of(self.w_qkv) + ops.copies_of(self.w_o)

    def seal(self) -> None:
        self.w_qkv, self.w_o = ops.streamed(ops.plain_of(self.w_qkv)), ops.streamed(ops.plain_of(self.w_o))

    # ------------------------------------------------------------------ launch planning
    def launch_key(self, shape) -> tuple[int, int]:
        """(context cell, cuts for uneven contexts): all that this part's decode launches depend
        on besides the padded batch size.  A cell is ``KEYS_PER_CUT`` keys of the longest
        context (of the window, for a windowed layer), and the plan is made for the cell's lower
        edge."""
        ctx = min(shape.max_ctx, self.window) if self.window else shape.max_ctx
        cell = min(ctx // KEYS_PER_CUT, MAX_CUTS)
        return cell, skew_cuts(max(cell * KEYS_PER_CUT, 1), shape.sum_ctx, shape.n)

    def _decode_cuts(self, step, on_matrix_cores: bool) -> int:
        cell, skew = self.launch_key(step.decode_shape)
        chunks = -(-(self.H // self.KV) // (16 if on_matrix_cores else 8))
        workgroups = max(1, step.n_decode * self.KV * chunks)
        # the vector-ALU kernel's waves take 64 keys at a time and its workgroups are light: it is
        # worth cutting down to one such block per cut and to two workgroups per compute unit
        # (measured in fp32 at the 1B shape, 600 keys: 2.48 to 2.37 ms a step at batch 8, 1.91 to
        # 1.77 at batch 1)
        finest = cell if on_matrix_cores else 8 * cell
        room = compute_units(step.device) * (1 if on_matrix_cores else 2)
        cuts = max(1, min(room // workgroups, finest, MAX_CUTS))
        return max(cuts, min(skew, max(1, cell)))

    def _prefill_work(self, step, act: torch.dtype, block_size: int):
        """(work rows on the device, rows per item) of the step's query runs, or ``(None, 0)``.
        Items of two row tiles per wave halve what a key block costs per row (its page lookups,
        staging and barrier) and halve the workgroups.  They are taken where the kernel has them
        and their workgroups alone are as many as the chip holds of the one-tile kernel at a
        time (so that short items are left to fill in behind the long ones), or give every
        compute unit two while every run starts at least its own length into its sequence (then
        all items walk long and nothing needs filling in).  Measured at 32 heads over 8 kv heads,
        one against two tiles: 2,048 queries from position 0, 47 against 55 us at head size 64
        and 70 against 82 at 128; 4,096 queries, 140 against 114 and 231 against 196; 2,048
        queries behind 2,048 keys, 106 against 100 and 209 against 151.  The layers of a model
        that agree on group size and item share the rows through the step's scratch."""
        if not step.prefill_seqs:
            return None, 0
        G = self.H // self.KV
        key = ("attention.prefill_work", G, self.KV, self.d, act, block_size)
        found = step.scratch.get(key)
        if found is None:
            units = compute_units(step.device)
            per_item = ops.prefill_rows_per_item(act, self.d, block_size, 2)
            rows = prefill_work_rows(step.q_lens, step.prefill_seqs, G, per_item, step.start_pos)
            groups = len(rows) * self.KV
            fills = groups >= ops.prefill_blocks_per_cu(act, self.d, block_size, 1) * units
            deep = groups >= 2 * units and all(step.start_pos[b] >= step.q_lens[b] for b in step.prefill_seqs)
            if not (fills or deep):
                per_item = ops.prefill_rows_per_item(act, self.d, block_size, 1)
                rows = prefill_work_rows(step.q_lens, step.prefill_seqs, G, per_item, step.start_pos)
            found = (step.upload_ints([x for row in rows for x in row]).view(-1, 3), per_item)
            step.scratch[key] = found
        return found

    def forward(self, x, step, layer: LayerState, residual) -> None:
        """``x``: normalised activations, or (after ``absorb_norm``) the fp32 residual stream."""
        n = x.shape[0]
        H, KV, d = self.H, self.KV, self.d
        ws = step.ws
        act = step.act_dtype
        table = step.block_tables[layer.group]
        cos, sin = (self.rotary.cos, self.rotary.sin) if self.rotary is not None else (None, None)
        rms = self.norm_eps
        owed = None
        if rms is not None and not ops.bf16_kernel_takes(x, self.w_qkv, True):
            # too many rows for the norm to ride in the projection: a norm kernel of its own,
            # which also adds what the layer before still owes the stream
            normed = ws.buf("normed", (n, self.hidden), act)
            ops.rmsnorm(x, None, rms, normed, add=step.take_owed(residual))
            x, rms = normed, None
        fused = (not self._hooked() and ops.bf16_kernel_takes(x, self.w_qkv, rms is not None, True)
                 and layer.k_pages.dtype == torch.bfloat16)
        if fused and rms is not None:
            # what the layer before owes the stream rides in this projection's loads and is
            # added to the stream by the output projection
            owed = step.take_owed(residual)
            if owed is not None and (owed.dtype != torch.bfloat16 or owed.stride() != x.stride()):
                ops.add_rows(residual, owed)
                owed = None
        else:
            step.settle()
        if fused:
            # one kernel: (norm,) projection, rotary, cache write
            qkv = ws.buf("q_rot", (n, H * d), act)
            ops.gemm_qkv_rope(x, self.w_qkv, qkv, step.positions, step.seq_of_token, cos, sin, table,
                              layer.k_pages, layer.v_pages, H, KV, d, write_kv=layer.owns_cache,
                              rms_eps=rms, a_owed=owed)
        else:
            qkv = ws.buf("qkv", (n, (H + 2 * KV) * d), act)
            ops.gemm(x, self.w_qkv, qkv)
            self.after_projection(qkv, step)
            ops.rope_kvwrite(qkv, step.positions, step.seq_of_token, cos, sin, table,
                             layer.k_pages, layer.v_pages, H, KV, d, write_kv=layer.owns_cache)
        out = ws.buf("attn_out", (n, H * d), act)
        window = self.window or 0
        bs = layer.k_pages.shape[2]
        work, rows_per_item = self._prefill_work(step, act, bs)
        if work is not None:
            ops.attn_prefill(qkv, layer.k_pages, layer.v_pages, table, step.cu_q, step.ctx_lens,
                             work, out, H, KV, d, self.scale, window, self.slopes, rows_per_item)
        if step.n_decode:
            splits = self._decode_cuts(step, ops.attention_on_matrix_cores(act, bs))
            workspace = None
            if splits > 1:
                workspace = (ws.buf("decode_part_acc", (step.n_decode * H * splits * d,), torch.float32),
                             ws.buf("decode_part_ml", (step.n_decode * H * splits * 2,), torch.float32))
            ops.attn_decode(qkv, layer.k_pages, layer.v_pages, table, step.decode_seq_ids,
                            step.n_decode, step.cu_q, step.ctx_lens, out, H, KV, d, self.scale,
                            window, splits, workspace,
                            token_is_seq=step.decode_seq_ids is None and work is None,
                            slopes=self.slopes)
        add_product(step, out, self.w_o, residual, owed=owed)
