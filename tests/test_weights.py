from __future__ import annotations

import pytest
import torch

import kvforge_amd
from kvforge_amd import registry
from kvforge_amd.config import preset_dict
from kvforge_amd.models.transformer import Transformer
from kvforge_amd.weights import (WeightsError, read_safetensors_folder, runtime_dtype,
                                 write_random_model, write_safetensors)


def make(tmp_path, preset="tiny-a", seed=0, **kw):
    folder = str(tmp_path / f"{preset}-{seed}")
    write_random_model(folder, preset_dict(preset), seed=seed, **kw)
    return folder


def test_random_model_folder(tmp_path):
    folder = make(tmp_path, "tiny-b", 1)
    w = read_safetensors_folder(folder)
    cfg = registry.config_from_folder(folder)
    assert set(w) == set(registry.build_spec(cfg).weight_specs())
    assert all(t.dtype == torch.bfloat16 for t in w.values())
    q = w["model.layers.1.self_attn.q_proj.weight"].float()
    assert abs(q.std().item() - 0.02) < 0.003 and abs(q.mean().item()) < 0.002
    n = torch.cat([v.float() for k, v in w.items() if "norm" in k])
    assert abs(n.mean().item() - 1.0) < 0.03 and 0.07 < n.std().item() < 0.13   # 1 + N(0, 0.1)
    # the seed decides the tensors
    again = read_safetensors_folder(make(tmp_path / "x", "tiny-b", 1))
    other = read_safetensors_folder(make(tmp_path / "y", "tiny-b", 2))
    assert all(torch.equal(w[k], again[k]) for k in w)
    assert not torch.equal(w["model.norm.weight"], other["model.norm.weight"])
    f32 = read_safetensors_folder(make(tmp_path / "z", "tiny-b", 1, dtype="float32"))
    assert f32["model.norm.weight"].dtype == torch.float32


def test_loading_keeps_stored_precision(tmp_path):
    folder = make(tmp_path)
    w = read_safetensors_folder(folder)
    w["model.norm.weight"] = w["model.norm.weight"].float()        # one tensor stored in 32-bit
    write_safetensors(folder, w)
    m = Transformer.from_folder(folder, torch.bfloat16, "cpu")
    assert m.spec.final_norm.weight.dtype == torch.float32          # stays 32-bit
    assert m.spec.blocks[0].mixer.w_qkv.dtype == torch.bfloat16
    assert m.spec.head.weight is m.spec.embedding.table             # tied: one tensor
    m32 = Transformer.from_folder(folder, torch.float32, "cpu")
    assert m32.spec.blocks[0].mixer.w_qkv.dtype == torch.float32
    assert torch.equal(m32.spec.blocks[0].ffn.w_down, w["model.layers.0.mlp.down_proj.weight"].float())
    assert runtime_dtype(torch.int64, torch.bfloat16) == torch.int32
    assert runtime_dtype(torch.float16, torch.bfloat16) == torch.bfloat16
    assert runtime_dtype(torch.float16, torch.float32) == torch.float32
    # fused projections: q, k, v stacked with rotary pairs made neighbours inside each q and k
    # head; gate and up interleaved row by row
    blk = m32.spec.blocks[1]
    p = "model.layers.1."
    perm = blk.mixer.pair_permutation()
    assert perm.tolist() == [0, 8, 1, 9, 2, 10, 3, 11, 4, 12, 5, 13, 6, 14, 7, 15]
    q = w[p + "self_attn.q_proj.weight"].float().view(4, 16, 64)[:, perm].reshape(64, 64)
    k = w[p + "self_attn.k_proj.weight"].float().view(2, 16, 64)[:, perm].reshape(32, 64)
    assert torch.equal(blk.mixer.w_qkv, torch.cat([q, k, w[p + "self_attn.v_proj.weight"].float()]))
    assert torch.equal(blk.ffn.w_gate_up[0::2], w[p + "mlp.gate_proj.weight"].float())
    assert torch.equal(blk.ffn.w_gate_up[1::2], w[p + "mlp.up_proj.weight"].float())
    # under bf16 the norm in front of a projection is folded into its columns; fp32 keeps it apart
    blk16 = m.spec.blocks[1]
    assert blk16.mixer_takes_residual and blk16.ffn_takes_residual and blk16.mixer.norm_eps == 1e-5
    gamma = w[p + "post_attention_layernorm.weight"].float()
    want = (torch.stack([w[p + "mlp.gate_proj.weight"].float(), w[p + "mlp.up_proj.weight"].float()], 1)
            .reshape(352, 64) * gamma[None]).to(torch.bfloat16)
    assert torch.equal(blk16.ffn.w_gate_up, want)
    assert not blk.mixer_takes_residual and not m32.spec.blocks[0].ffn_takes_residual


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = make(tmp_path)
    w = read_safetensors_folder(folder)
    del w["model.layers.0.mlp.up_proj.weight"]
    del w["model.norm.weight"]
    w["model.layers.0.self_attn.q_bias"] = torch.zeros(3)
    w["model.layers.1.self_attn.k_proj.weight"] = torch.zeros(5, 64, dtype=torch.bfloat16)
    w["model.layers.1.mlp.down_proj.weight"] = torch.zeros(64, 176, dtype=torch.int32)
    write_safetensors(folder, w)
    with pytest.raises(WeightsError) as e:
        Transformer.from_folder(folder, torch.float32, "cpu")
    msg = str(e.value)
    assert "missing tensors (2)" in msg and "model.layers.0.mlp.up_proj.weight" in msg
    assert "model.norm.weight" in msg
    assert "unexpected tensors (1)" in msg and "model.layers.0.self_attn.q_bias" in msg
    assert "model.layers.1.self_attn.k_proj.weight: expected [32, 64], found [5, 64]" in msg
    assert "model.layers.1.mlp.down_proj.weight: expected a floating tensor" in msg


def test_tied_head_tolerates_a_stored_copy_and_untied_needs_it(tmp_path):
    folder = make(tmp_path, "tiny-a")
    w = read_safetensors_folder(folder)
    w["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    w["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    write_safetensors(folder, w)
    Transformer.from_folder(folder, torch.float32, "cpu")            # both are ignored
    folder_b = make(tmp_path, "tiny-b", 1)
    wb = read_safetensors_folder(folder_b)
    del wb["lm_head.weight"]
    write_safetensors(folder_b, wb)
    with pytest.raises(WeightsError, match="lm_head.weight"):
        Transformer.from_folder(folder_b, torch.float32, "cpu")


def test_a_model_in_several_files_named_by_the_index(tmp_path):
    """Two and three shards with ``model.safetensors.index.json``: the loader finds every tensor
    by name whichever file holds it, the model is bit for bit the one-file model, and an index
    that names a file that is not there is one clear error."""
    import json
    import os
    folder = make(tmp_path, "tiny-b", 1)
    w = read_safetensors_folder(folder)
    one = Transformer.from_folder(folder, torch.float32, "cpu")
    for shards in (2, 3):
        sharded = str(tmp_path / f"shards{shards}")
        registry.config_from_dict(preset_dict("tiny-b")).save(sharded)
        index = write_safetensors(sharded, w, shards=shards)
        with open(index) as f:
            weight_map = json.load(f)["weight_map"]
        files = sorted(set(weight_map.values()))
        assert len(files) == shards and set(weight_map) == set(w)
        assert not os.path.exists(os.path.join(sharded, "model.safetensors"))
        # layers are spread over the files, so a loader that read one file would miss some
        assert len({weight_map[n] for n in w if ".layers." in n}) > 1
        back = read_safetensors_folder(sharded)
        assert set(back) == set(w) and all(torch.equal(back[k], w[k]) for k in w)
        many = Transformer.from_folder(sharded, torch.float32, "cpu")
        for a, b in zip(one.spec.blocks, many.spec.blocks):
            assert torch.equal(a.mixer.w_qkv, b.mixer.w_qkv) and torch.equal(a.ffn.w_down, b.ffn.w_down)
        assert torch.equal(one.spec.head.weight, many.spec.head.weight)
    # a tensor missing from every shard is reported like any missing tensor
    del w["model.layers.2.mlp.down_proj.weight"]
    write_safetensors(sharded, w, shards=3)
    with pytest.raises(WeightsError, match="model.layers.2.mlp.down_proj.weight"):
        Transformer.from_folder(sharded, torch.float32, "cpu")
    os.remove(os.path.join(sharded, files[1]))
    with pytest.raises(WeightsError, match=files[1]):
        Transformer.from_folder(sharded, torch.float32, "cpu")


def test_missing_files(tmp_path):
    with pytest.raises(kvforge_amd.ConfigError):
        Transformer.from_folder(str(tmp_path), torch.float32, "cpu")
    registry.config_from_dict(preset_dict("tiny-a")).save(str(tmp_path))
    with pytest.raises(WeightsError, match="model.safetensors"):
        Transformer.from_folder(str(tmp_path), torch.float32, "cpu")


def test_engine_refuses_the_cpu(tmp_path):
    from kvforge_amd.engine.runner import ModelRunner
    m = Transformer.from_folder(make(tmp_path), torch.float32, "cpu")
    with pytest.raises(RuntimeError, match="GPU"):
        ModelRunner(m, 16, 8, 4, 64, 64)
