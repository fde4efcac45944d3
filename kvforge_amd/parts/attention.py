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
from kvforge_amd.parts.base import CacheSpec, LayerState, Mixer, WeightSpec, add_product
from kvforge_amd.parts.positions import RotaryPositions
from kvforge_amd.registry import register_mixer


@register_mixer("attention")
class PagedAttention(Mixer):
    """``window``: ``None`` attends to every earlier position, ``w`` to the last ``w``."""

    replayable = True
    settles_residual = True  # its norm kernel adds what is owed to the stream

    def __init__(self, prefix: str, hidden: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 rotary: RotaryPositions | None, scale: float | None = None,
                 window: int | None = None) -> None:
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
        self.cache_spec = CacheSpec(self.KV, self.d, self.window)
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

    def pair_permutation(self) -> torch.Tensor:
        """``perm[new] = old`` within a head: new elements 2i and 2i+1 are the checkpoint's
        elements i and i + rot/2; elements beyond the rotary width stay."""
        rot = self.rotary.rot_dim if self.rotary is not None else 0
        perm = torch.arange(self.d)
        for i in range(rot // 2):
            perm[2 * i], perm[2 * i + 1] = i, i + rot // 2
        return perm

    def absorb_norm(self, norm) -> bool:
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

    def forward(self, x, step, layer: LayerState, residual) -> None:
        """``x``: normalised activations, or (after ``absorb_norm``) the fp32 residual stream."""
        n = x.shape[0]
        H, KV, d = self.H, self.KV, self.d
        ws = step.ws
        act = step.act_dtype
        table = step.block_tables[layer.group]
        cos, sin = (self.rotary.cos, self.rotary.sin) if self.rotary is not None else step.no_rotation()
        rms = self.norm_eps
        owed = None
        if rms is not None and not ops.bf16_kernel_takes(x, self.w_qkv, True):
            # too many rows for the norm to ride in the projection: a norm kernel of its own,
            # which also adds what the layer before still owes the stream
            normed = ws.buf("normed", (n, self.hidden), act)
            ops.rmsnorm(x, None, rms, normed, add=step.take_owed(residual))
            x, rms = normed, None
        fused = (ops.bf16_kernel_takes(x, self.w_qkv, rms is not None, True)
                 and layer.k_pages.dtype == torch.bfloat16)
        if fused and rms is not None:
            # what the layer before owes the stream in fp32 rides in this projection's loads and
            # is added to the stream by the output projection
            owed = step.take_owed(residual)
            if owed is not None and owed.dtype != torch.float32:
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
            ops.rope_kvwrite(qkv, step.positions, step.seq_of_token, cos, sin, table,
                             layer.k_pages, layer.v_pages, H, KV, d, write_kv=layer.owns_cache)
        out = ws.buf("attn_out", (n, H * d), act)
        window = self.window or 0
        bs = layer.k_pages.shape[2]
        work = step.prefill_work(H // KV, ops.prefill_rows_per_item(act, d, bs))
        if work is not None:
            ops.attn_prefill(qkv, layer.k_pages, layer.v_pages, table, step.cu_q, step.ctx_lens,
                             work, out, H, KV, d, self.scale, window)
        if step.n_decode:
            splits, workspace = step.decode_plan(H, KV, d, window)
            ops.attn_decode(qkv, layer.k_pages, layer.v_pages, table, step.decode_seq_ids,
                            step.n_decode, step.cu_q, step.ctx_lens, out, H, KV, d, self.scale,
                            window, splits, workspace,
                            token_is_seq=step.decode_seq_ids is None and work is None)
        add_product(step, out, self.w_o, residual, owed=owed)
