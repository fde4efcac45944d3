"""A plain, slow Llama decoder: whole sequences, no cache, one function per part, 32-bit torch
on the CPU.  It is the oracle the engine is held to and shares no code with ``kvforge_amd``:
it parses ``config.json`` itself and reads a folder's tensors with the ``safetensors`` package
(``read_weights``), as a ``{checkpoint name: tensor}`` dict.

Every function cites the lines of the reference (``src/tokenvault/...``) whose formula it
follows.
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


def read_weights(folder: str) -> dict[str, torch.Tensor]:
    """Every tensor of every ``*.safetensors`` file in the folder, as stored, on the CPU."""
    from safetensors.torch import load_file
    out: dict[str, torch.Tensor] = {}
    for name in sorted(os.listdir(folder)):
        if name.endswith(".safetensors"):
            out.update(load_file(os.path.join(folder, name)))
    if not out:
        raise FileNotFoundError(f"no .safetensors file in {folder}")
    return out


# --------------------------------------------------------------------------- parts
def _wide(x: torch.Tensor) -> torch.Tensor:
    """``x.float()`` as the reference writes it; a float64 tensor stays float64, so that the same
    functions also give a reference that is all but free of rounding (``forward(..., dtype=
    torch.float64)``), against which the rounding of a 32-bit implementation can be measured."""
    return x if x.dtype == torch.float64 else x.float()


def _stored(x: torch.Tensor, store: torch.dtype | None) -> torch.Tensor:
    """What a tensor is after the reference has stored it in its model dtype ``store`` (rounded
    to bfloat16 and widened again), or unchanged for ``None``.  With ``store=torch.bfloat16``
    ``forward`` reproduces the arithmetic of the reference run with ``dtype=bfloat16``
    (src/tokenvault/config.py:143,150-151): every tensor between two operations, the residual
    stream included, holds bfloat16 values, while norms, rotation, scores and softmax are
    computed in 32-bit and rounded once (src/tokenvault/model.py:36-38,61;
    src/tokenvault/cache/paged_attention.py:85-89)."""
    return x if store is None else x.to(store).to(x.dtype)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """src/tokenvault/model.py:35-38 — eps inside the rsqrt, weight multiplied in fp32 (in the
    precision of ``x`` when that is float64)."""
    xf = _wide(x)
    xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return xf * weight.to(xf.dtype)


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
    x = _wide(x)
    return x * cos.to(x.dtype) + rotate_half(x) * sin.to(x.dtype)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                     q_offset: int = 0, window: int | None = None) -> torch.Tensor:
    """src/tokenvault/cache/paged_attention.py:94-108 — ``q: [Q, H, d]``, ``k, v: [L, KV, d]``;
    query ``i`` sits at position ``q_offset + i`` and sees keys at or before it; q-head ``h``
    uses kv-head ``h // (H/KV)``.  Scores are scaled after the dot product, softmax in fp32.
    ``window`` (not in the reference): only the last ``window`` keys, the query's own included."""
    group = q.shape[1] // k.shape[1]
    kk = k.repeat_interleave(group, dim=1)
    vv = v.repeat_interleave(group, dim=1)
    scores = torch.einsum("qhd,lhd->hql", _wide(q), _wide(kk)) * scale
    q_pos = torch.arange(q.shape[0])[:, None] + q_offset
    k_pos = torch.arange(k.shape[0])[None, :]
    visible = k_pos <= q_pos
    if window is not None:
        visible = visible & (k_pos > q_pos - window)
    scores = scores.masked_fill(~visible[None], float("-inf"))
    return torch.einsum("hql,lhd->qhd", torch.softmax(scores, -1), _wide(vv))


def swiglu(x: torch.Tensor, gate_w: torch.Tensor, up_w: torch.Tensor,
           down_w: torch.Tensor, store: torch.dtype | None = None,
           out_store: torch.dtype | None = None) -> torch.Tensor:
    """src/tokenvault/model.py:131-132 — ``down(silu(gate(x)) * up(x))``, weights ``[out, in]``."""
    g = _stored(x @ gate_w.to(x.dtype).T, store)
    u = _stored(x @ up_w.to(x.dtype).T, store)
    act = _stored(_stored(torch.nn.functional.silu(g), store) * u, store)
    return _stored(act @ down_w.to(x.dtype).T, out_store)


def attention_block(x: torch.Tensor, w: dict[str, torch.Tensor], prefix: str, cfg: dict,
                    cos: torch.Tensor, sin: torch.Tensor, window: int | None,
                    store: torch.dtype | None = None,
                    out_store: torch.dtype | None = None,
                    query_block: int | None = None) -> torch.Tensor:
    """src/tokenvault/model.py:77-92 without the cache: project, rotate q and k, attend,
    project out.  ``query_block``: attend that many queries at a time (each over the keys up to
    its block's end), so that the scores of a sequence of tens of thousands of tokens never
    exist all at once; the same numbers."""
    T = x.shape[0]
    H, KV, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = _stored(x @ w[prefix + "q_proj.weight"].to(x.dtype).T, store).view(T, H, d)
    k = _stored(x @ w[prefix + "k_proj.weight"].to(x.dtype).T, store).view(T, KV, d)
    v = _stored(x @ w[prefix + "v_proj.weight"].to(x.dtype).T, store).view(T, KV, d)
    q, k = _stored(apply_rope(q, cos, sin), store), _stored(apply_rope(k, cos, sin), store)
    if query_block is None:
        out = causal_attention(q, k, v, 1.0 / math.sqrt(d), 0, window)
    else:
        out = torch.cat([causal_attention(q[lo:lo + query_block], k[:lo + query_block], v[:lo + query_block],
                                          1.0 / math.sqrt(d), lo, window)
                         for lo in range(0, T, query_block)])
    out = _stored(out, store)
    return _stored(out.reshape(T, H * d) @ w[prefix + "o_proj.weight"].to(x.dtype).T, out_store)


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
            first_position: int = 0, dtype: torch.dtype = torch.float32,
            residual_in_fp32: bool = False, query_block: int | None = None,
            last: int | None = None) -> torch.Tensor:
    """src/tokenvault/model.py:175-191 for one whole sequence: logits ``[T, vocab]`` in fp32
    (of the last ``last`` positions only, if given; ``query_block``: see ``attention_block``).
    ``first_position`` shifts every position (only distances count under rotary).
    ``dtype=torch.float64`` computes everything but the rotary angles (which are 32-bit by
    definition) in double precision.  ``dtype=torch.bfloat16`` gives what the reference computes
    when it runs in bfloat16 (see ``_stored``), returned in fp32 like its logits
    (src/tokenvault/batching/continuous.py:117).  With ``residual_in_fp32`` only the tensors
    *between* operations are rounded (normalised rows, q, k, v, attention output, the gated
    feed-forward activation, the final normalised rows), while the residual stream, the products
    added to it and the logits stay 32-bit: the least rounding a bfloat16 engine with a 32-bit
    residual sum can do."""
    store = stream = None
    if dtype == torch.bfloat16:
        store, dtype = torch.bfloat16, torch.float32
        stream = None if residual_in_fp32 else store
    ids = torch.tensor(token_ids, dtype=torch.long)
    h = w["model.embed_tokens.weight"][ids].to(dtype)                    # model.py:169-170
    pos = torch.arange(len(token_ids)) + first_position
    cos, sin = rope_cos_sin(pos, inv_freq_for(cfg))
    eps = cfg["rms_norm_eps"]
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        a = _stored(rms_norm(h, w[p + "input_layernorm.weight"], eps), store)
        h = _stored(h + attention_block(a, w, p + "self_attn.", cfg, cos, sin,
                                        layer_window(cfg, i), store, stream, query_block), stream)
        m = _stored(rms_norm(h, w[p + "post_attention_layernorm.weight"], eps), store)
        h = _stored(h + swiglu(m, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                               w[p + "mlp.down_proj.weight"], store, stream), stream)   # model.py:186-187
    if last is not None:
        h = h[-last:]
    hidden = _stored(rms_norm(h, w["model.norm.weight"], eps), store)    # model.py:188
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return _stored(hidden @ head.to(hidden.dtype).T, stream)            # model.py:157-158,190-191


def greedy(w: dict[str, torch.Tensor], cfg: dict, prompt: list[int], n: int) -> list[int]:
    """tests/conftest.py:22-32 of the reference: full recomputation for every new token."""
    ids, out = list(prompt), []
    for _ in range(n):
        tok = int(forward(w, cfg, ids)[-1].argmax())
        out.append(tok)
        ids.append(tok)
    return out
