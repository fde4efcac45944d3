"""A position encoding that lives in the attention scores and not in q and k: every head has a
slope, and a key's score falls with its distance from the query.  The encoding is a part defined
here (it has no tensors; it only knows the slopes), a toy architecture hands its slopes to the
built-in attention part as constants, and the model is stepped in portions with pages that are
used again, decoded through captured steps and generated from, against the same model written
out over whole sequences.  Nothing in the framework's files knows of it, and it is nobody's
model."""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any

import pytest
import torch

import kvforge_amd
from kvforge_amd import registry
from kvforge_amd.config.model import ModelConfig
from kvforge_amd.engine.batch import StepEntry
from kvforge_amd.engine.runner import ModelRunner
from kvforge_amd.models.transformer import Transformer
from kvforge_amd.parts import (LMHead, ModelSpec, PagedAttention, Positions, PreNormBlock, RMSNorm, SwiGLU,
                               TokenEmbedding)
from tests.plain import llama as plain

pytestmark = pytest.mark.gpu
DEV = "cuda"


class ToyDistanceSlopes(Positions):
    """Head ``h`` of ``n`` gets the slope ``steepest * ratio**h``: the first heads look at their
    neighbourhood, the last ones far back."""

    replayable = True

    def __init__(self, steepest: float, ratio: float) -> None:
        self.prefix, self.steepest, self.ratio = "", steepest, ratio

    def slopes(self, num_heads: int) -> list[float]:
        return [self.steepest * self.ratio ** h for h in range(num_heads)]


@dataclass
class SlopesConfig(ModelConfig):
    hidden_size: int = 0
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    inter: int = 0
    layers: int = 0
    window: int = 0
    steepest: float = 0.0
    ratio: float = 0.0

    _KEYS = ("vocab_size", "max_position_embeddings", "hidden_size", "num_heads", "num_kv_heads", "head_dim",
             "inter", "layers", "window", "steepest", "ratio")

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "SlopesConfig":
        return cls(architecture=d["architectures"][0], **{k: d[k] for k in cls._KEYS})

    def to_dict(self) -> dict[str, Any]:
        return {"architectures": [self.architecture], **{k: getattr(self, k) for k in self._KEYS}}


def build_slopes(cfg: SlopesConfig) -> ModelSpec:
    h = cfg.hidden_size
    pos = registry.part_class(registry.POSITIONS, "toy_distance_slopes", "position encoding")(cfg.steepest, cfg.ratio)
    blocks = []
    for i in range(cfg.layers):
        # the odd layers look through a window as well
        att = PagedAttention(f"l.{i}.att", h, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim, None,
                             window=cfg.window if i % 2 else None, score_slopes=pos.slopes(cfg.num_heads))
        blocks.append(PreNormBlock(RMSNorm(f"l.{i}.n1", h, 1e-5), att, RMSNorm(f"l.{i}.n2", h, 1e-5),
                                   SwiGLU(f"l.{i}.ff", h, cfg.inter)))
    return ModelSpec(config=cfg, embedding=TokenEmbedding("embed", cfg.vocab_size, h), blocks=blocks,
                     final_norm=RMSNorm("norm", h, 1e-5), head=LMHead("head", cfg.vocab_size, h),
                     positions=[pos])


SLOPES = {"architectures": ["ToySlopesForCausalLM"], "vocab_size": 83, "max_position_embeddings": 160,
          "hidden_size": 48, "num_heads": 6, "num_kv_heads": 2, "head_dim": 16, "inter": 56, "layers": 3,
          "window": 21, "steepest": 0.5, "ratio": 0.5}


def slopes_plain(w, ids, with_bias=True):
    """Logits ``[T, vocab]`` of the model over one whole sequence."""
    wf = {k: v.float() for k, v in w.items()}
    c = SLOPES
    T, H, KV, d = len(ids), c["num_heads"], c["num_kv_heads"], c["head_dim"]
    slopes = [c["steepest"] * c["ratio"] ** hd for hd in range(H)]
    dist = (torch.arange(T)[None, :] - torch.arange(T)[:, None]).float()          # key - query
    h = wf["embed.weight"][torch.tensor(ids)]
    for i in range(c["layers"]):
        a = plain.rms_norm(h, wf[f"l.{i}.n1.weight"], 1e-5)
        q = (a @ wf[f"l.{i}.att.q_proj.weight"].T).view(T, H, d)
        k = (a @ wf[f"l.{i}.att.k_proj.weight"].T).view(T, KV, d)
        v = (a @ wf[f"l.{i}.att.v_proj.weight"].T).view(T, KV, d)
        seen = dist <= 0
        if i % 2:
            seen = seen & (dist > -c["window"])
        heads = []
        for hd in range(H):
            sc = (q[:, hd] @ k[:, hd // (H // KV)].T) / math.sqrt(d)
            if with_bias:
                sc = sc + slopes[hd] * dist
            heads.append(torch.softmax(sc.masked_fill(~seen, float("-inf")), -1) @ v[:, hd // (H // KV)])
        h = h + torch.cat(heads, -1) @ wf[f"l.{i}.att.o_proj.weight"].T
        m = plain.rms_norm(h, wf[f"l.{i}.n2.weight"], 1e-5)
        h = h + plain.swiglu(m, wf[f"l.{i}.ff.gate_proj.weight"], wf[f"l.{i}.ff.up_proj.weight"],
                             wf[f"l.{i}.ff.down_proj.weight"])
    return plain.rms_norm(h, wf["norm.weight"], 1e-5) @ wf["head.weight"].T


@pytest.fixture(scope="module")
def slopes_folder(tmp_path_factory):
    from tests.replay_util import liven
    kvforge_amd.register_positions("toy_distance_slopes", ToyDistanceSlopes)
    kvforge_amd.register_architecture("ToySlopesForCausalLM", SlopesConfig, build_slopes)
    folder = str(tmp_path_factory.mktemp("toy_slopes"))
    kvforge_amd.write_random_model(folder, SLOPES, seed=31)
    liven(folder)           # without it what attention adds is lost beside the embedding
    return folder


def test_the_bias_decides_the_logits(slopes_folder):
    w = plain.read_weights(slopes_folder)
    ids = torch.randint(0, 83, (60,), generator=torch.Generator().manual_seed(1)).tolist()
    a, b = slopes_plain(w, ids), slopes_plain(w, ids, with_bias=False)
    assert float((a - b).abs().max()) > 0.3               # five times the widest tolerance below
    assert (a.argmax(-1) != b.argmax(-1)).float().mean() > 0.2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_slopes_model_in_portions_with_pages_used_again(slopes_folder, dtype):
    w = plain.read_weights(slopes_folder)
    model = Transformer.from_folder(slopes_folder, dtype, DEV)
    assert len(model.cache_groups) == 2                  # whole-context layers and window layers
    bs = 8
    runner = ModelRunner(model, bs, 26, max_num_seqs=3, max_num_batched_tokens=128, max_model_len=160)
    g = torch.Generator().manual_seed(5)
    seqs = {r: torch.randint(0, 83, (n,), generator=g).tolist() for r, n in (("a", 131), ("b", 40), ("c", 57))}
    want = {r: slopes_plain(w, ids) for r, ids in seqs.items()}
    got = {r: [] for r in seqs}
    # 26 pages of 8 tokens: a (131 -> 17) and b (40 -> 5) fit, c (57 -> 8) gets b's pages
    plan = [[("a", 0, 30), ("b", 0, 40)], [("a", 30, 32)], [("a", 32, 129), ("c", 0, 3)],
            [("a", 129, 130), ("c", 3, 56)], [("a", 130, 131), ("c", 56, 57)]]
    for portions in plan:
        entries = []
        for rid, lo, hi in portions:
            if not runner.cache.has_request(rid):
                runner.cache.allocate(rid, 0)
            runner.cache.append_slots(rid, hi, lo)
            entries.append(StepEntry(rid, seqs[rid][lo:hi], lo, "all"))
        logits = runner.step(entries).cpu()
        off = 0
        for rid, lo, hi in portions:
            got[rid].append(logits[off:off + hi - lo])
            off += hi - lo
            runner.cache.mark_computed(rid, hi)
            runner.cache.release_behind(rid, hi)
            if hi == len(seqs[rid]):
                runner.cache.free(rid)
    t = dict(atol=2e-4, rtol=1e-4) if dtype == torch.float32 else dict(atol=6e-2, rtol=5e-2)
    for rid in seqs:
        torch.testing.assert_close(torch.cat(got[rid]), want[rid], **t)
    assert runner.cache.num_free_blocks == 26


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_slopes_model_generates_through_captured_steps(slopes_folder, dtype):
    w = plain.read_weights(slopes_folder)
    engine = kvforge_amd.InferenceEngine.from_folder(
        slopes_folder, kvforge_amd.EngineConfig(
            dtype=dtype, cache=kvforge_amd.CacheConfig(block_size=8, num_blocks=64),
            scheduler=kvforge_amd.SchedulerConfig(max_num_seqs=3, max_num_batched_tokens=16, max_model_len=160)))
    assert engine.runner.use_graphs
    g = torch.Generator().manual_seed(9)
    prompts = [torch.randint(0, 83, (n,), generator=g).tolist() for n in (37, 5, 18)]
    outs = engine.generate(prompts, kvforge_amd.SamplingParams(max_tokens=24, temperature=0.0))
    assert engine.runner.num_graph_replays > 0
    margin = 2e-4 if dtype == "float32" else 6e-2
    for p, o in zip(prompts, outs):
        logits = slopes_plain(w, p + o.output_token_ids)
        for i, tok in enumerate(o.output_token_ids):
            row = logits[len(p) - 1 + i]
            assert float(row.max() - row[tok]) <= margin
    assert engine.cache.num_free_blocks == engine.cache.num_blocks
