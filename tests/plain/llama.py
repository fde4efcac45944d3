"""A plain, slow Llama decoder: whole sequences, no cache, one function per part, 32-bit torch
on the CPU.  It is the oracle the engine is held to and shares no code with ``kvforge_amd``:
it parses ``config.json`` itself and takes weights as a ``{checkpoint name: tensor}`` dict.

Every function cites the lines of the reference (``/root/reference``) whose formula it follows.
The reference has no llama3 frequency scaling and no sliding window; those two follow the
parameter names of the model's ``config.json`` and are pinned by invariants in the tests
(``factor == 1`` is the identity, thresholds are continuous; a window as long as the sequence
is plain causal attention).
"""

from __future__ import annotations

import json
import math
import os
from typing import Any

import torch


# --------------------------------------------------------------------------- configuration
def read_config(folder: str) -> dict[str, Any]:
    with open(os.path.join(folder, "config.json")) as f:
        c = json.load(f)
    # defaults as in src/tokenvault/model_loader.py:64-86 and src/tokenvault/config.py:56-60
    c.setdefault("num_key_value_heads", c["num_attention_heads"])
    if c.get("head_dim") is None:
        c["head_dim"] = c["hidden_size"] // c["num_attention_heads"]
    c.setdefault("rope_theta", 10000.0)
    c.setdefault("tie_word_embeddings", False)
    return c


# --------------------------------------------------------------------------- parts
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """src/tokenvault/model.py:35-38 — eps inside the rsqrt, weight multiplied in fp32."""
    xf = x.float()
    xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return xf * weight.float()


def rope_inv_freq(head_dim: int, theta: float) -> torch.Tensor:
    """src/tokenvault/model.py:44."""
    return 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))


def llama3_scale_inv_freq(inv_freq: torch.Tensor, factor: float, low_freq_factor: float,
                          high_freq_factor: float, original_max_position: int) -> torch.Tensor:
    """Not in the reference.  Per frequency ``f`` with wavelength ``2*pi/f``: shorter than
    ``orig/high`` keeps ``f``; longer than ``orig/low`` gives ``f/factor``; between them
    ``(1-s)*f/factor + s*f`` with ``s = (orig/wavelength - low)/(high - low)``."""
    out = []
    low_wavelen = original_max_position / low_freq_factor
    high_wavelen = original_max_position / high_freq_factor
    for f in inv_freq.tolist():
        wavelen = 2 * math.pi / f
        if wavelen < high_wavelen:
            out.append(f)
        elif wavelen > low_wavelen:
            out.append(f / factor)
        else:
            s = (original_max_position / wavelen - low_freq_factor) / (
                high_freq_factor - low_freq_factor)
            out.append((1 - s) * f / factor + s * f)
    return torch.tensor(out, dtype=torch.float32)


def rope_cos_sin(positions: torch.Tensor, inv_freq: torch.Tensor):
    """src/tokenvault/model.py:47-50 — angles in fp32, the half-width table repeated twice."""
    freqs = positions.float()[..., None] * inv_freq.float()
    emb = torch.cat([freqs, freqs], dim=-1)
    return emb.cos(), emb.sin()


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """src/tokenvault/model.py:53-55 — element i pairs with i + d/2."""
    x1, x2 = x.chunk(2, dim=-1)
    return torch.cat([-x2, x1], dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """src/tokenvault/model.py:58-61 — ``x: [T, heads, d]``, ``cos/sin: [T, d]``."""
    cos, sin = cos.unsqueeze(-2), sin.unsqueeze(-2)
    return x.float() * cos + rotate_half(x.float()) * sin


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                     q_offset: int = 0, window: int | None = None) -> torch.Tensor:
    """src/tokenvault/cache/paged_attention.py:94-108 — ``q: [Q, H, d]``, ``k, v: [L, KV, d]``;
    query ``i`` sits at position ``q_offset + i`` and sees keys at or before it; q-head ``h``
    uses kv-head ``h // (H/KV)``.  Scores are scaled after the dot product, softmax in fp32.
    ``window`` (not in the reference): only the last ``window`` keys, the query's own included."""
    group = q.shape[1] // k.shape[1]
    kk = k.repeat_interleave(group, dim=1)
    vv = v.repeat_interleave(group, dim=1)
    scores = torch.einsum("qhd,lhd->hql", q.float(), kk.float()) * scale
    q_pos = torch.arange(q.shape[0])[:, None] + q_offset
    k_pos = torch.arange(k.shape[0])[None, :]
    visible = k_pos <= q_pos
    if window is not None:
        visible = visible & (k_pos > q_pos - window)
    scores = scores.masked_fill(~visible[None], float("-inf"))
    return torch.einsum("hql,lhd->qhd", torch.softmax(scores, -1), vv.float())


def swiglu(x: torch.Tensor, gate_w: torch.Tensor, up_w: torch.Tensor,
           down_w: torch.Tensor) -> torch.Tensor:
    """src/tokenvault/model.py:131-132 — ``down(silu(gate(x)) * up(x))``, weights ``[out, in]``."""
    g = x @ gate_w.float().T
    u = x @ up_w.float().T
    return (torch.nn.functional.silu(g) * u) @ down_w.float().T


def attention_block(x: torch.Tensor, w: dict[str, torch.Tensor], prefix: str, cfg: dict,
                    cos: torch.Tensor, sin: torch.Tensor, window: int | None) -> torch.Tensor:
    """src/tokenvault/model.py:77-92 without the cache: project, rotate q and k, attend,
    project out."""
    T = x.shape[0]
    H, KV, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = (x @ w[prefix + "q_proj.weight"].float().T).view(T, H, d)
    k = (x @ w[prefix + "k_proj.weight"].float().T).view(T, KV, d)
    v = (x @ w[prefix + "v_proj.weight"].float().T).view(T, KV, d)
    q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    out = causal_attention(q, k, v, 1.0 / math.sqrt(d), 0, window)
    return out.reshape(T, H * d) @ w[prefix + "o_proj.weight"].float().T


def inv_freq_for(cfg: dict) -> torch.Tensor:
    f = rope_inv_freq(cfg["head_dim"], cfg["rope_theta"])
    rs = cfg.get("rope_scaling")
    if rs and rs.get("rope_type", rs.get("type")) == "llama3":
        f = llama3_scale_inv_freq(f, rs["factor"], rs["low_freq_factor"], rs["high_freq_factor"],
                                  rs["original_max_position_embeddings"])
    return f


def layer_window(cfg: dict, i: int) -> int | None:
    types = cfg.get("layer_types")
    if types and types[i] == "sliding_attention":
        return int(cfg["sliding_window"])
    return None


def forward(w: dict[str, torch.Tensor], cfg: dict, token_ids: list[int],
            first_position: int = 0) -> torch.Tensor:
    """src/tokenvault/model.py:175-191 for one whole sequence: logits ``[T, vocab]`` in fp32.
    ``first_position`` shifts every position (only distances count under rotary)."""
    ids = torch.tensor(token_ids, dtype=torch.long)
    h = w["model.embed_tokens.weight"].float()[ids]                      # model.py:169-170
    pos = torch.arange(len(token_ids)) + first_position
    cos, sin = rope_cos_sin(pos, inv_freq_for(cfg))
    eps = cfg["rms_norm_eps"]
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        a = rms_norm(h, w[p + "input_layernorm.weight"], eps)
        h = h + attention_block(a, w, p + "self_attn.", cfg, cos, sin, layer_window(cfg, i))
        m = rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
        h = h + swiglu(m, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                       w[p + "mlp.down_proj.weight"])                     # model.py:186-187
    hidden = rms_norm(h, w["model.norm.weight"], eps)                    # model.py:188
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return hidden @ head.float().T                                       # model.py:157-158,190-191


def greedy(w: dict[str, torch.Tensor], cfg: dict, prompt: list[int], n: int) -> list[int]:
    """tests/conftest.py:22-32 of the reference: full recomputation for every new token."""
    ids, out = list(prompt), []
    for _ in range(n):
        tok = int(forward(w, cfg, ids)[-1].argmax())
        out.append(tok)
        ids.append(tok)
    return out
