from __future__ import annotations

import json

import pytest
import torch

import kvforge_amd
from kvforge_amd import registry
from kvforge_amd.config import (CacheConfig, ConfigError, EngineConfig, LlamaConfig, PRESETS,
                                RopeScaling, SchedulerConfig, preset_dict)


def test_llama_config_from_its_own_keys():
    d = preset_dict("tiny-b")
    cfg = registry.config_from_dict(d)
    assert isinstance(cfg, LlamaConfig)
    assert (cfg.hidden_size, cfg.num_hidden_layers, cfg.num_attention_heads,
            cfg.num_key_value_heads, cfg.head_dim) == (96, 3, 3, 1, 32)
    assert cfg.rope_scaling == RopeScaling("llama3", 4.0, 1.0, 4.0, 64)
    assert cfg.rms_norm_eps == 1e-6 and cfg.rope_theta == 500000.0 and not cfg.tie_word_embeddings
    # defaults the reference applies (src/tokenvault/model_loader.py:74-78, config.py:57-60)
    d2 = {k: v for k, v in preset_dict("tiny-a").items()
          if k not in ("head_dim", "num_key_value_heads", "rope_theta")}
    c2 = registry.config_from_dict(d2)
    assert c2.head_dim == 16 and c2.num_key_value_heads == 4 and c2.rope_theta == 10000.0


def test_every_preset_round_trips(tmp_path):
    for name in PRESETS:
        cfg = registry.config_from_dict(preset_dict(name))
        cfg.save(str(tmp_path / name))
        again = registry.config_from_folder(str(tmp_path / name))
        assert again == cfg, name
    one_b = registry.config_from_dict(preset_dict("llama-1b"))
    assert one_b.num_params == 16 * (2048 * 64 * 80 + 3 * 2048 * 8192) + 128256 * 2048


@pytest.mark.parametrize("change,fragment", [
    ({"num_key_value_heads": 3}, "multiple of num_key_value_heads"),
    ({"hidden_size": None}, "hidden_size"),
    ({"rms_norm_eps": None}, "rms_norm_eps"),
    ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "rope_scaling"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 2.0}}, "low_freq_factor"),
    ({"head_dim": 15}, "head_dim"),
    ({"layer_types": ["sliding_attention", "full_attention"]}, "sliding_window"),
])
def test_config_errors(change, fragment):
    d = preset_dict("tiny-a")
    d.update(change)
    with pytest.raises(ConfigError, match=fragment):
        registry.config_from_dict(d)


def test_unknown_architecture_lists_known_ones():
    d = preset_dict("tiny-a")
    d["architectures"] = ["NopeForCausalLM"]
    with pytest.raises(ConfigError, match="LlamaForCausalLM"):
        registry.config_from_dict(d)
    with pytest.raises(ConfigError, match="architectures"):
        registry.config_from_dict({"hidden_size": 4})


def test_eos_list_takes_first_and_head_dim_divisibility():
    d = preset_dict("tiny-a")
    d["eos_token_id"] = [7, 9]
    assert registry.config_from_dict(d).eos_token_id == 7
    d = preset_dict("tiny-a")
    d.pop("head_dim")
    d["hidden_size"] = 66
    with pytest.raises(ConfigError, match="divisible"):
        registry.config_from_dict(d)


def test_engine_config_rules():
    ec = EngineConfig(dtype="bfloat16", scheduler=SchedulerConfig(max_model_len=4096))
    assert ec.dtype == torch.bfloat16 and ec.cache.dtype == torch.bfloat16
    ec.clamp_to_model(128)                       # src/tokenvault/config.py:146-149
    assert ec.scheduler.max_model_len == 128
    with pytest.raises(ValueError):
        EngineConfig(dtype="float16")
    cc = CacheConfig(num_blocks=None, kv_cache_memory_gb=1.0)
    assert cc.resolve_num_blocks(524288) == 2048  # 1B bf16: 2*16*16*8*64*2 bytes per block
    with pytest.raises(ValueError):
        CacheConfig(num_blocks=None).resolve_num_blocks(10)
    assert CacheConfig().block_size == 16 and CacheConfig().num_blocks == 256
    sc = SchedulerConfig()
    assert (sc.max_num_seqs, sc.max_num_batched_tokens, sc.max_model_len) == (32, 2048, 2048)


def test_model_spec_has_no_size_of_its_own():
    """Two different configurations give parts with exactly the configured sizes."""
    for name in ("tiny-a", "tiny-b"):
        d = preset_dict(name)
        spec = registry.build_spec(registry.config_from_dict(d))
        shapes = {k: v.shape for k, v in spec.weight_specs().items()}
        h, H, KV, hd, I, V = (d["hidden_size"], d["num_attention_heads"], d["num_key_value_heads"],
                              d["head_dim"], d["intermediate_size"], d["vocab_size"])
        assert shapes["model.embed_tokens.weight"] == (V, h)
        assert shapes["model.layers.0.self_attn.q_proj.weight"] == (H * hd, h)
        assert shapes["model.layers.0.self_attn.k_proj.weight"] == (KV * hd, h)
        assert shapes["model.layers.0.self_attn.o_proj.weight"] == (h, H * hd)
        assert shapes["model.layers.0.mlp.down_proj.weight"] == (h, I)
        assert ("lm_head.weight" in shapes) == (not d["tie_word_embeddings"])
        assert len([k for k in shapes if k.endswith("input_layernorm.weight")]) == d["num_hidden_layers"]
        blk = spec.blocks[0]
        assert blk.mixer_norm.eps == d["rms_norm_eps"] and blk.mixer.scale == pytest.approx(hd ** -0.5)


def test_bytes_per_block_follow_from_the_page_tensors_the_mixers_declare():
    """Llama 3.2 1B in bf16 with pages of 16 tokens: 2 * 16 layers * 16 * 8 heads * 64 * 2 bytes
    (src/tokenvault/config.py:91-95), worked out from what attention declares as its pages."""
    import torch
    from kvforge_amd import registry
    from kvforge_amd.cache.storage import bytes_per_block
    from kvforge_amd.models.transformer import Transformer
    model = Transformer(registry.build_spec(registry.config_from_dict(preset_dict("llama-1b"))),
                        torch.bfloat16, "cpu")
    assert [len(g.layers) for g in model.cache_groups] == [16]
    assert [t.name for t in model.cache_groups[0].pages] == ["k", "v"]
    assert bytes_per_block(model.cache_groups, 16, torch.bfloat16) == 524288
    assert bytes_per_block(model.cache_groups, 16, torch.float32) == 2 * 524288
