"""An embedding that is not a plain table, defined here: every row is multiplied by a constant
on its way into the residual stream.  The engine asks the parts what they can do and knows no
class by name: the embedding either names a bfloat16 table that holds exactly what it gives
(``Embedding.pick_table``; then captured greedy steps end in the head's own pick, which gathers
the next step's rows from that table) or says nothing (then those steps store logits, sample and
embed in kernels of their own).  The tokens are the same either way and are the plain
computation's.  Nothing in the framework's files knows of it, and it is nobody's model."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import pytest
import torch

import kvforge_amd
from kvforge_amd.config.model import LlamaConfig
from kvforge_amd.kernels import ops
from kvforge_amd.models.llama import build_llama
from kvforge_amd.parts import Embedding, ModelSpec, WeightSpec
from tests.plain import llama as plain

pytestmark = pytest.mark.gpu
SCALE = 32.0      # a power of two: the scaled table is exact in bfloat16


class ToyScaledEmbedding(Embedding):
    replayable = True

    def __init__(self, prefix: str, vocab: int, hidden: int, scale: float, offers_table: bool) -> None:
        self.prefix, self.vocab, self.hidden = prefix, vocab, hidden
        self.scale, self.offers_table = scale, offers_table
        self.table = self.scaled = None

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {self._name("weight"): WeightSpec((self.vocab, self.hidden))}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        self.table = tensors[self._name("weight")]
        self.scaled = (self.table.float() * self.scale).to(self.table.dtype)

    def kernel_modules(self, dtype: torch.dtype) -> set[str]:
        return {"elementwise"}

    def forward(self, ids: torch.Tensor, out: torch.Tensor) -> None:
        ops.embed(ids, self.table, out)
        out.mul_(self.scale)

    def pick_table(self):
        ok = self.offers_table and self.scaled is not None and self.scaled.dtype == torch.bfloat16
        return self.scaled if ok else None


@dataclass
class ScaledConfig(LlamaConfig):
    embedding_scale: float = 1.0
    embedding_offers_table: bool = False

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "ScaledConfig":
        base = LlamaConfig.from_dict(d)
        return cls(**base.__dict__, embedding_scale=float(d["embedding_scale"]),
                   embedding_offers_table=bool(d["embedding_offers_table"]))

    def to_dict(self) -> dict[str, Any]:
        return dict(super().to_dict(), embedding_scale=self.embedding_scale,
                    embedding_offers_table=self.embedding_offers_table)


def build_scaled(cfg: ScaledConfig) -> ModelSpec:
    spec = build_llama(cfg)
    spec.embedding = ToyScaledEmbedding("model.embed_tokens", cfg.vocab_size, cfg.hidden_size,
                                        cfg.embedding_scale, cfg.embedding_offers_table)
    return spec


def config(offers_table: bool) -> dict[str, Any]:
    # an untied head: the head's matrix is not the (unscaled) embedding table
    return dict(kvforge_amd.preset_dict("tiny-b"), architectures=["ToyScaledForCausalLM"],
                embedding_scale=SCALE, embedding_offers_table=offers_table)


def plain_logits(w, cfg, ids):
    """The plain model with the embedding table scaled: the only place the table is used, the
    head being untied."""
    assert not cfg["tie_word_embeddings"]
    scaled = dict(w)
    scaled["model.embed_tokens.weight"] = w["model.embed_tokens.weight"].float() * SCALE
    return plain.forward(scaled, cfg, ids)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from tests.replay_util import liven
    kvforge_amd.register_architecture("ToyScaledForCausalLM", ScaledConfig, build_scaled)
    out = {}
    for offers in (False, True):
        folder = str(tmp_path_factory.mktemp(f"toy_scaled_{int(offers)}"))
        kvforge_amd.write_random_model(folder, config(offers), seed=17)
        liven(folder)
        out[offers] = folder
    return out


def test_the_scale_decides_the_tokens(folders):
    w, cfg = plain.read_weights(folders[True]), plain.read_config(folders[True])
    ids = torch.randint(0, 384, (40,), generator=torch.Generator().manual_seed(2)).tolist()
    a, b = plain_logits(w, cfg, ids), plain.forward(w, cfg, ids)
    assert (a.argmax(-1) != b.argmax(-1)).float().mean() > 0.5
    assert float((a - b).abs().max()) > 0.3                   # ten times the widest margin below


def test_the_greedy_tail_follows_what_the_embedding_declares(folders):
    """Same weights, same tokens; the captured greedy steps end in the head's pick only for the
    embedding that names its table, and both are the plain model's choices."""
    g = torch.Generator().manual_seed(9)
    prompts = [torch.randint(0, 384, (n,), generator=g).tolist() for n in (23, 5, 41)]
    params = kvforge_amd.SamplingParams(max_tokens=20, temperature=0.0)
    tokens, tails = {}, {}
    for offers, folder in folders.items():
        engine = kvforge_amd.InferenceEngine.from_folder(folder, kvforge_amd.EngineConfig(
            dtype="bfloat16", cache=kvforge_amd.CacheConfig(block_size=8, num_blocks=64),
            scheduler=kvforge_amd.SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=32)))
        assert engine.runner.use_graphs and engine.model.can_pick(3) == offers
        tokens[offers] = [o.output_token_ids for o in engine.generate(prompts, params)]
        assert engine.runner.num_graph_replays > 0
        tails[offers] = engine.runner.num_greedy_tails
    assert tails[True] > 0 and tails[False] == 0
    w, cfg = plain.read_weights(folders[True]), plain.read_config(folders[True])
    for offers in (True, False):
        for p, out in zip(prompts, tokens[offers]):
            logits = plain_logits(w, cfg, p + out)
            for i, tok in enumerate(out):
                row = logits[len(p) - 1 + i]
                assert float(row.max() - row[tok]) <= 3e-2, (offers, i, tok)
    # where the plain model's choice is clear of bf16 rounding the two paths agree token for token
    for p, a, b in zip(prompts, tokens[True], tokens[False]):
        logits = plain_logits(w, cfg, p + a)
        for i, (x, y) in enumerate(zip(a, b)):
            top = torch.topk(logits[len(p) - 1 + i], 2).values
            if float(top[0] - top[1]) < 6e-2:
                break
            assert x == y, (i, x, y)


def test_an_embedding_that_offers_no_table_in_float32(folders):
    engine = kvforge_amd.InferenceEngine.from_folder(folders[False], kvforge_amd.EngineConfig(
        dtype="float32", cache=kvforge_amd.CacheConfig(block_size=8, num_blocks=64),
        scheduler=kvforge_amd.SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=32)))
    prompt = list(range(3, 30))
    out = engine.generate([prompt], kvforge_amd.SamplingParams(max_tokens=12, temperature=0.0))[0].output_token_ids
    w, cfg = plain.read_weights(folders[False]), plain.read_config(folders[False])
    logits = plain_logits(w, cfg, prompt + out)
    for i, tok in enumerate(out):
        row = logits[len(prompt) - 1 + i]
        assert float(row.max() - row[tok]) <= 1e-4
