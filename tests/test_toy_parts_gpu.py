"""Parts of other kinds than the built-in ones, defined here with torch ops and never a model of
anyone's: a feed-forward that routes each token to some of its experts, a norm with a mean and
a bias, learned absolute positions, and a block that runs mixer and feed-forward side by side.
A toy architecture picks them layer by layer from lists in its config.json through the
registries; it is built, loaded, stepped in portions and generated from without a change to the
framework's files, and compared with the same model written out over whole sequences."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

import pytest
import torch

import kvforge_amd
from kvforge_amd import registry
from kvforge_amd.config.model import ModelConfig
from kvforge_amd.engine.batch import StepEntry
from kvforge_amd.engine.runner import ModelRunner
from kvforge_amd.models.transformer import Transformer
from kvforge_amd.parts import (Block, FeedForward, LMHead, ModelSpec, Norm, PagedAttention,
                               Positions, TokenEmbedding, WeightSpec)
from tests.plain import llama as plain

pytestmark = pytest.mark.gpu
DEV = "cuda"


# ============================================================================ the toy parts
class ToyRoutedFeedForward(FeedForward):
    """``experts`` small ReLU feed-forwards; a token goes to the ``top_k`` with the largest
    router logits and their outputs are mixed with the softmax of those logits (fp32)."""

    replayable = True  # device work only, no look at the step's host fields

    def __init__(self, prefix: str, hidden: int, inter: int, experts: int, top_k: int) -> None:
        self.prefix, self.hidden, self.inter, self.experts, self.top_k = prefix, hidden, inter, experts, top_k

    def weight_specs(self):
        specs = {self._name("router.weight"): WeightSpec((self.experts, self.hidden), std=0.5)}
        for e in range(self.experts):
            specs[self._name(f"experts.{e}.up.weight")] = WeightSpec((self.inter, self.hidden), std=0.2)
            specs[self._name(f"experts.{e}.down.weight")] = WeightSpec((self.hidden, self.inter), std=0.2)
        return specs

    def load(self, tensors):
        self.router = tensors[self._name("router.weight")].float()
        self.up = torch.stack([tensors[self._name(f"experts.{e}.up.weight")] for e in range(self.experts)]).float()
        self.down = torch.stack([tensors[self._name(f"experts.{e}.down.weight")] for e in range(self.experts)]).float()

    def forward(self, x, step, residual):
        xf = x.float()
        logits = xf @ self.router.T
        top, idx = logits.topk(self.top_k, dim=-1)
        mix = torch.zeros_like(logits).scatter_(1, idx, torch.softmax(top, dim=-1))
        every = torch.relu(torch.einsum("nh,eih->eni", xf, self.up))
        residual += torch.einsum("eni,ehi,ne->nh", every, self.down, mix)


class ToyLayerNorm(Norm):
    """``(x - mean) * rsqrt(var + eps) * weight + bias``."""

    replayable = True

    def __init__(self, prefix: str, width: int, eps: float) -> None:
        self.prefix, self.width, self.eps = prefix, width, eps

    def weight_specs(self):
        return {self._name("weight"): WeightSpec((self.width,), init="norm", std=0.1),
                self._name("bias"): WeightSpec((self.width,), std=0.1)}

    def load(self, tensors):
        self.weight, self.bias = tensors[self._name("weight")].float(), tensors[self._name("bias")].float()

    def forward(self, x, out, rows=None, add=None):
        if add is not None:
            x += add
        y = x if rows is None else x.index_select(0, rows.long())
        out.copy_(torch.nn.functional.layer_norm(y, (self.width,), self.weight, self.bias, self.eps))


class ToyLearnedPositions(Positions):
    """One learned row per position, added to the embedding output."""

    replayable = True

    def __init__(self, prefix: str, max_positions: int, hidden: int) -> None:
        self.prefix, self.max_positions, self.hidden = prefix, max_positions, hidden

    def weight_specs(self):
        return {self._name("weight"): WeightSpec((self.max_positions, self.hidden), std=0.3)}

    def load(self, tensors):
        self.table = tensors[self._name("weight")].float()

    def on_embedding(self, residual, step):
        residual += self.table.index_select(0, step.positions.long())


class ToyParallelBlock(Block):
    """``h += mixer(norm(h)) + ffn(norm(h))``: one norm, both parts read the same activations."""

    def __init__(self, norm, mixer, ffn) -> None:
        self.norm, self.mixer, self.ffn = norm, mixer, ffn

    def parts(self):
        return [self.norm, self.mixer, self.ffn]

    def forward(self, residual, step, layer):
        x = step.ws.buf("toy_parallel_x", tuple(residual.shape), step.act_dtype)
        self.norm.forward(residual, x, add=step.take_owed(residual))
        self.mixer.forward(x, step, layer, residual)
        step.settle()  # the feed-forward here is a part that expects an up-to-date stream
        self.ffn.forward(x, step, residual)


@dataclass
class ToyMixConfig(ModelConfig):
    hidden_size: int = 0
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    inter: int = 0
    experts: int = 0
    experts_per_token: int = 0
    eps: float = 1e-5
    blocks: list[str] = field(default_factory=list)
    norms: list[str] = field(default_factory=list)
    feed_forwards: list[str] = field(default_factory=list)
    positions: str = ""

    _KEYS = ("vocab_size", "max_position_embeddings", "hidden_size", "num_heads", "num_kv_heads", "head_dim",
             "inter", "experts", "experts_per_token", "eps", "blocks", "norms", "feed_forwards", "positions")

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "ToyMixConfig":
        return cls(architecture=d["architectures"][0], **{k: d[k] for k in cls._KEYS})

    def to_dict(self) -> dict[str, Any]:
        return {"architectures": [self.architecture], **{k: getattr(self, k) for k in self._KEYS}}


def build_toy_mix(cfg: ToyMixConfig) -> ModelSpec:
    """Every layer's block, norm and feed-forward are looked up by the names the configuration
    gives for that layer."""
    h = cfg.hidden_size

    def norm(kind, name):
        return registry.part_class(registry.NORMS, kind, "norm")(name, h, cfg.eps)

    def ffn(kind, name):
        cls = registry.part_class(registry.FEED_FORWARDS, kind, "feed-forward")
        if kind == "toy_routed":
            return cls(name, h, cfg.inter, cfg.experts, cfg.experts_per_token)
        return cls(name, h, cfg.inter)

    blocks = []
    for i, (b, n, f) in enumerate(zip(cfg.blocks, cfg.norms, cfg.feed_forwards)):
        att = PagedAttention(f"l.{i}.att", h, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim, None)
        cls = registry.part_class(registry.BLOCKS, b, "block")
        if b == "toy_parallel":
            blocks.append(cls(norm(n, f"l.{i}.n"), att, ffn(f, f"l.{i}.ff")))
        else:
            blocks.append(cls(norm(n, f"l.{i}.n1"), att, norm(n, f"l.{i}.n2"), ffn(f, f"l.{i}.ff")))
    pos = registry.part_class(registry.POSITIONS, cfg.positions, "position encoding")(
        "pos", cfg.max_position_embeddings, h)
    return ModelSpec(config=cfg, embedding=TokenEmbedding("embed", cfg.vocab_size, h), blocks=blocks,
                     final_norm=norm(cfg.norms[-1], "norm"), head=LMHead("head", cfg.vocab_size, h),
                     positions=[pos])


MIX = {"architectures": ["ToyMixForCausalLM"], "vocab_size": 77, "max_position_embeddings": 96,
       "hidden_size": 40, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16, "inter": 24,
       "experts": 3, "experts_per_token": 2, "eps": 1e-4,
       "blocks": ["pre_norm", "toy_parallel", "pre_norm"],
       "norms": ["toy_layernorm", "rmsnorm", "toy_layernorm"],
       "feed_forwards": ["toy_routed", "swiglu", "toy_routed"],
       "positions": "toy_learned"}


# ============================================================================ the same model, plainly
def mix_plain(w, ids, margins=None):
    """Logits ``[T, vocab]``.  ``margins`` (a list) receives for every routed layer the gap
    between each token's last chosen and first rejected router logit."""
    wf = {k: v.float() for k, v in w.items()}
    T, cfg = len(ids), {"num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16}
    ones, zeros = torch.ones(T, 16), torch.zeros(T, 16)   # a rotation by nothing

    def norm(kind, h, name):
        if kind == "rmsnorm":
            return plain.rms_norm(h, wf[name + ".weight"], 1e-4)
        mu, var = h.mean(-1, keepdim=True), h.var(-1, unbiased=False, keepdim=True)
        return (h - mu) / torch.sqrt(var + 1e-4) * wf[name + ".weight"] + wf[name + ".bias"]

    def ffn(kind, x, name):
        if kind == "swiglu":
            return plain.swiglu(x, wf[name + ".gate_proj.weight"], wf[name + ".up_proj.weight"],
                                wf[name + ".down_proj.weight"])
        logits = x @ wf[name + ".router.weight"].T
        if margins is not None:
            ranked = logits.sort(-1, descending=True).values
            margins.append(ranked[:, 1] - ranked[:, 2])
        out = torch.zeros_like(x)
        for t in range(T):
            top = sorted(range(3), key=lambda e: -float(logits[t, e]))[:2]
            share = torch.softmax(logits[t, top], dim=0)
            for s, e in zip(share, top):
                mid = torch.relu(wf[f"{name}.experts.{e}.up.weight"] @ x[t])
                out[t] += s * (wf[f"{name}.experts.{e}.down.weight"] @ mid)
        return out

    def att(x, i):
        return plain.attention_block(x, wf, f"l.{i}.att.", cfg, ones, zeros, None)

    h = wf["embed.weight"][torch.tensor(ids)] + wf["pos.weight"][:T]
    for i, (b, n, f) in enumerate(zip(MIX["blocks"], MIX["norms"], MIX["feed_forwards"])):
        if b == "toy_parallel":
            x = norm(n, h, f"l.{i}.n")
            h = h + att(x, i) + ffn(f, x, f"l.{i}.ff")
        else:
            h = h + att(norm(n, h, f"l.{i}.n1"), i)
            h = h + ffn(f, norm(n, h, f"l.{i}.n2"), f"l.{i}.ff")
    return norm(MIX["norms"][-1], h, "norm") @ wf["head.weight"].T


def clearly_routed_tokens(w, n, gen, margin=0.3):
    """``n`` random token ids such that in the plain model every router's choice at every token
    is clear by ``margin``.  Two experts whose logits are closer than rounding may be chosen
    either way, and from that token on the sequence would be another one; a token's routing
    depends only on the tokens before it, so they are drawn one after the other."""
    ids: list[int] = []
    while len(ids) < n:
        for _ in range(200):
            tok, margins = int(torch.randint(0, 77, (1,), generator=gen)), []
            mix_plain(w, ids + [tok], margins)
            if min(float(m[-1]) for m in margins) >= margin:
                ids.append(tok)
                break
        else:
            raise AssertionError("no clearly routed token found: choose other weights")
    return ids


@pytest.fixture(scope="module")
def mix_folder(tmp_path_factory):
    kvforge_amd.register_feed_forward("toy_routed", ToyRoutedFeedForward)
    kvforge_amd.register_norm("toy_layernorm", ToyLayerNorm)
    kvforge_amd.register_positions("toy_learned", ToyLearnedPositions)
    kvforge_amd.register_block("toy_parallel", ToyParallelBlock)
    kvforge_amd.register_architecture("ToyMixForCausalLM", ToyMixConfig, build_toy_mix)
    folder = str(tmp_path_factory.mktemp("toy_mix"))
    kvforge_amd.write_random_model(folder, MIX, seed=11)
    return folder


def test_routing_spreads_over_experts(mix_folder):
    """The random router must not send everything to one pair, or the comparison below would
    not see a wrong choice."""
    w = {k: v.float() for k, v in plain.read_weights(mix_folder).items()}
    x = torch.randn(64, 40, generator=torch.Generator().manual_seed(0))
    first = (x @ w["l.0.ff.router.weight"].T).argmax(-1)
    assert len(set(first.tolist())) == 3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_parts_step_in_portions(mix_folder, dtype):
    w = plain.read_weights(mix_folder)
    model = Transformer.from_folder(mix_folder, dtype, DEV)
    kinds = [type(b).__name__ for b in model.spec.blocks]
    assert kinds == ["PreNormBlock", "ToyParallelBlock", "PreNormBlock"]
    assert type(model.spec.blocks[0].ffn) is ToyRoutedFeedForward
    assert type(model.spec.blocks[1].norm).__name__ == "RMSNorm"
    runner = ModelRunner(model, 4, 24, max_num_seqs=3, max_num_batched_tokens=64, max_model_len=96)
    assert runner.use_graphs
    g = torch.Generator().manual_seed(6)
    seqs = {r: clearly_routed_tokens(w, n, g) for r, n in (("a", 37), ("b", 20), ("c", 18))}
    want = {r: mix_plain(w, ids) for r, ids in seqs.items()}
    got = {r: [] for r in seqs}
    plan = [[("a", 0, 21), ("b", 0, 2)], [("a", 21, 23), ("b", 2, 19)], [("a", 23, 24), ("b", 19, 20)],
            [("a", 24, 37), ("c", 0, 17)], [("c", 17, 18)]]
    for portions in plan:
        entries = []
        for rid, a, b in portions:
            if not runner.cache.has_request(rid):
                runner.cache.allocate(rid, 0)
            runner.cache.append_slots(rid, b, a)
            entries.append(StepEntry(rid, seqs[rid][a:b], a, "all"))
        logits = runner.step(entries).cpu()
        off = 0
        for rid, a, b in portions:
            got[rid].append(logits[off:off + b - a])
            off += b - a
            if b == len(seqs[rid]):
                runner.cache.free(rid)
    t = dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32 else dict(atol=4e-2, rtol=4e-2)
    for rid in seqs:
        torch.testing.assert_close(torch.cat(got[rid]), want[rid], **t)
    assert runner.cache.num_free_blocks == 24


def test_toy_parts_generate_through_the_engine(mix_folder):
    """Greedy generation, decode steps replayed from graphs in runs: every produced token is the
    plain model's best (within rounding) at its place."""
    w = plain.read_weights(mix_folder)
    engine = kvforge_amd.InferenceEngine.from_folder(
        mix_folder, kvforge_amd.EngineConfig(
            dtype="float32", cache=kvforge_amd.CacheConfig(block_size=4, num_blocks=64),
            scheduler=kvforge_amd.SchedulerConfig(max_num_seqs=3, max_num_batched_tokens=8)))
    prompts = [[5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15], [70, 3], [44, 45, 46, 47, 48]]
    outs = engine.generate(prompts, kvforge_amd.SamplingParams(max_tokens=11, temperature=0.0))
    assert engine.runner.num_graph_replays > 0
    for p, o in zip(prompts, outs):
        assert len(o.output_token_ids) == 11
        margins = []
        logits = mix_plain(w, p + o.output_token_ids, margins)
        assert float(torch.stack(margins).min()) > 1e-4   # else a router's choice is a toss-up in fp32
        for i, tok in enumerate(o.output_token_ids):
            row = logits[len(p) - 1 + i]
            assert float(row.max() - row[tok]) <= 1e-4
