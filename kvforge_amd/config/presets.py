"""Named model shapes, each written exactly as its ``config.json`` would read.

The reference keeps ``PRESETS`` of ModelConfig objects (src/tokenvault/model_loader.py:17-39);
here a preset is the JSON dictionary itself, so a preset goes through the same
``from_dict`` path as a model folder and no size is held anywhere else.
"""

from __future__ import annotations

from typing import Any

_LLAMA3_32 = {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
              "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}
_LLAMA3_8 = dict(_LLAMA3_32, factor=8.0)


def _llama(**kw: Any) -> dict[str, Any]:
    base: dict[str, Any] = {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu",
        "attention_bias": False, "mlp_bias": False, "rope_scaling": None,
        "tie_word_embeddings": False, "bos_token_id": None, "eos_token_id": None,
    }
    base.update(kw)
    return base


PRESETS: dict[str, dict[str, Any]] = {
    "tiny-a": _llama(
        vocab_size=256, hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
        num_key_value_heads=2, head_dim=16, intermediate_size=176,
        max_position_embeddings=128, rope_theta=10000.0, rms_norm_eps=1e-5,
        tie_word_embeddings=True),
    "tiny-b": _llama(
        vocab_size=384, hidden_size=96, num_hidden_layers=3, num_attention_heads=3,
        num_key_value_heads=1, head_dim=32, intermediate_size=256,
        max_position_embeddings=256, rope_theta=500000.0, rms_norm_eps=1e-6,
        rope_scaling={"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0,
                      "high_freq_factor": 4.0, "original_max_position_embeddings": 64}),
    # the reference's unit-test and CPU-benchmark shapes (src/tokenvault/model_loader.py:19-27)
    "tiny": _llama(
        vocab_size=512, hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
        num_key_value_heads=2, head_dim=16, intermediate_size=172,
        max_position_embeddings=1024, rope_theta=10000.0, rms_norm_eps=1e-6),
    "small": _llama(
        vocab_size=8192, hidden_size=512, num_hidden_layers=6, num_attention_heads=8,
        num_key_value_heads=4, head_dim=64, intermediate_size=1408,
        max_position_embeddings=2048, rope_theta=10000.0, rms_norm_eps=1e-6),
    "llama-1b": _llama(
        vocab_size=128256, hidden_size=2048, num_hidden_layers=16, num_attention_heads=32,
        num_key_value_heads=8, head_dim=64, intermediate_size=8192,
        max_position_embeddings=131072, rope_theta=500000.0, rms_norm_eps=1e-5,
        rope_scaling=_LLAMA3_32, tie_word_embeddings=True),
    "llama-3b": _llama(
        vocab_size=128256, hidden_size=3072, num_hidden_layers=28, num_attention_heads=24,
        num_key_value_heads=8, head_dim=128, intermediate_size=8192,
        max_position_embeddings=131072, rope_theta=500000.0, rms_norm_eps=1e-5,
        rope_scaling=_LLAMA3_32, tie_word_embeddings=True),
    "llama-8b": _llama(
        vocab_size=128256, hidden_size=4096, num_hidden_layers=32, num_attention_heads=32,
        num_key_value_heads=8, head_dim=128, intermediate_size=14336,
        max_position_embeddings=131072, rope_theta=500000.0, rms_norm_eps=1e-5,
        rope_scaling=_LLAMA3_8),
}


def preset_dict(name: str) -> dict[str, Any]:
    try:
        return dict(PRESETS[name])
    except KeyError:
        raise KeyError(f"unknown preset {name!r}; known: {sorted(PRESETS)}") from None
