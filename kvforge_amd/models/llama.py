"""``LlamaForCausalLM``: how a Llama configuration becomes a list of parts.

Checkpoint names are the Hugging Face ones (``model.embed_tokens.weight``,
``model.layers.{i}.self_attn.q_proj.weight`` ...); the reference strips the ``model.`` prefix and
aliases a missing ``lm_head.weight`` to the embedding (src/tokenvault/model_loader.py:104-106).
"""

from __future__ import annotations

from kvforge_amd.config.model import LlamaConfig
from kvforge_amd.parts.base import ModelSpec
from kvforge_amd.parts.embedding import LMHead, TokenEmbedding
from kvforge_amd.registry import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, part_class,
                                  register_architecture)


def build_llama(cfg: LlamaConfig) -> ModelSpec:
    norm_cls = part_class(NORMS, "rmsnorm", "norm")
    attn_cls = part_class(MIXERS, "attention", "mixer")
    ffn_cls = part_class(FEED_FORWARDS, "swiglu", "feed-forward")
    block_cls = part_class(BLOCKS, "pre_norm", "block")
    rotary = part_class(POSITIONS, "rotary", "position encoding")(
        cfg.head_dim, cfg.rope_theta, cfg.rope_scaling)
    h = cfg.hidden_size
    blocks = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}"
        sliding = cfg.layer_types is not None and cfg.layer_types[i] == "sliding_attention"
        mixer = attn_cls(f"{p}.self_attn", h, cfg.num_attention_heads, cfg.num_key_value_heads,
                         cfg.head_dim, rotary, window=cfg.sliding_window if sliding else None)
        blocks.append(block_cls(
            norm_cls(f"{p}.input_layernorm", h, cfg.rms_norm_eps), mixer,
            norm_cls(f"{p}.post_attention_layernorm", h, cfg.rms_norm_eps),
            ffn_cls(f"{p}.mlp", h, cfg.intermediate_size)))
    embedding = TokenEmbedding("model.embed_tokens", cfg.vocab_size, h)
    head = LMHead("lm_head", cfg.vocab_size, h,
                  tied_to="model.embed_tokens.weight" if cfg.tie_word_embeddings else None)
    ignored = (r".*rotary_emb\.inv_freq",) + ((r"lm_head\.weight",) if cfg.tie_word_embeddings else ())
    return ModelSpec(config=cfg, embedding=embedding, blocks=blocks,
                     final_norm=norm_cls("model.norm", h, cfg.rms_norm_eps), head=head,
                     positions=[rotary], ignored_weights=ignored)


register_architecture("LlamaForCausalLM", LlamaConfig, build_llama)
