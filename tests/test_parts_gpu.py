"""Each part alone on the GPU against the plain function of the same name, at sizes of its own;
then a toy mixer with state of its own and a toy architecture (a block named twice, a call that
reads another call's cache), both defined here, registered, built, loaded and stepped without a
change to the framework's files."""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any

import pytest
import torch

import kvforge_amd
from kvforge_amd import registry
from kvforge_amd.cache import CacheGroup, CacheManager
from kvforge_amd.parts import attention_pages
from kvforge_amd.config.model import ModelConfig
from kvforge_amd.engine.batch import MetaBuffers, Step, StepEntry, Workspace, fill_step
from kvforge_amd.engine.runner import ModelRunner
from kvforge_amd.models.transformer import Transformer
from kvforge_amd.parts import (LayerCall, LayerState, LMHead, Mixer, ModelSpec, PagedAttention,
                               PreNormBlock, RMSNorm, RotaryPositions, StateSpec, SwiGLU,
                               TokenEmbedding, WeightSpec)
from tests.plain import llama as plain

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(atol=3e-5, rtol=3e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def make_step(entries, cache, dtype, n_groups=1, max_tokens=256):
    meta = MetaBuffers(max_tokens, 8, [32] * n_groups, DEV)
    step = Step()
    step.ws, step.act_dtype, step.device = Workspace(DEV), dtype, DEV
    fill_step(step, meta, entries, cache.block_table, lambda r: -1, cache.block_size)
    return step


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(dtype):
    part = RMSNorm("n", 100, 1e-4)
    assert part.weight_specs() == {"n.weight": WeightSpec((100,), init="norm", std=0.1)}
    w = 1 + rand(100, seed=1, scale=0.1)
    part.load({"n.weight": w.to(dtype).to(DEV)})
    x = rand(6, 100, seed=2, scale=4.0)
    out = torch.empty(6, 100, dtype=dtype, device=DEV)
    part.forward(x.to(DEV), out)
    torch.testing.assert_close(out.float().cpu(), plain.rms_norm(x, w.to(dtype), 1e-4), **tol(dtype))


def test_rotary_part_tables_are_the_plain_angles():
    cfg = registry.config_from_dict(kvforge_amd.preset_dict("tiny-b"))
    part = RotaryPositions(32, 500000.0, cfg.rope_scaling)
    part.prepare(300, DEV)
    inv = plain.inv_freq_for(kvforge_amd.preset_dict("tiny-b"))
    cos, sin = plain.rope_cos_sin(torch.arange(300), inv)
    assert torch.equal(part.cos.cpu(), cos[:, :16]) and torch.equal(part.sin.cpu(), sin[:, :16])
    plain_unscaled = plain.rope_inv_freq(32, 500000.0)
    assert not torch.equal(part.inv_freq, plain_unscaled)
    torch.testing.assert_close(RotaryPositions(32, 500000.0, None).inv_freq, plain_unscaled)


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_part(dtype):
    part = SwiGLU("m", 48, 112)
    w = {"m.gate_proj.weight": rand(112, 48, seed=3, scale=0.2).to(dtype),
         "m.up_proj.weight": rand(112, 48, seed=4, scale=0.2).to(dtype),
         "m.down_proj.weight": rand(48, 112, seed=5, scale=0.2).to(dtype)}
    assert {k: v.shape for k, v in part.weight_specs().items()} == {k: tuple(v.shape) for k, v in w.items()}
    part.load({k: v.to(DEV) for k, v in w.items()})
    part.seal()
    x = rand(9, 48, seed=6).to(dtype)
    res = rand(9, 48, seed=7)
    step = Step()
    step.ws, step.act_dtype = Workspace(DEV), dtype
    residual = res.clone().to(DEV)
    part.forward(x.to(DEV), step, residual)
    step.settle()
    want = res + plain.swiglu(x.float(), *(w[f"m.{n}_proj.weight"] for n in ("gate", "up", "down")))
    torch.testing.assert_close(residual.cpu(), want, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_head_parts(dtype):
    table = rand(37, 48, seed=8).to(dtype)
    emb = TokenEmbedding("e", 37, 48)
    emb.load({"e.weight": table.to(DEV)})
    ids = torch.tensor([3, 36, 0, 3], dtype=torch.int32, device=DEV)
    out = torch.empty(4, 48, device=DEV)
    emb.forward(ids, out)
    assert torch.equal(out.cpu(), table.float()[[3, 36, 0, 3]])
    tied = LMHead("lm_head", 37, 48, tied_to="e.weight")
    assert list(tied.weight_specs()) == ["e.weight"]
    tied.load({"e.weight": table.to(DEV)})
    x = rand(5, 48, seed=9).to(dtype)
    logits = torch.empty(5, 37, device=DEV)
    tied.forward(x.to(DEV), logits)
    torch.testing.assert_close(logits.cpu(), x.float() @ table.float().T, **tol(dtype))
    assert list(LMHead("lm_head", 37, 48).weight_specs()) == ["lm_head.weight"]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bs", [4, 8])
@pytest.mark.parametrize("H,KV,d,window", [(6, 2, 16, None), (3, 1, 48, 7), (4, 4, 32, None)])
@pytest.mark.parametrize("small_chip", [False, True])
def test_attention_part_over_portions(dtype, H, KV, d, window, bs, small_chip, monkeypatch):
    """The attention part alone: a sequence fed in three portions (the last a single token) beside
    a second whole sequence gives the plain whole-sequence attention block; q and k projections
    are scaled so the scores are peaked.  ``small_chip``: the part is told of a chip without any
    compute unit, which any rows fill, so it takes its items of two row tiles per wave
    where the kernel has them."""
    from kvforge_amd.kernels import ops as kernel_ops
    if small_chip:
        monkeypatch.setattr(kernel_ops, "_compute_units", {i: 0 for i in range(torch.cuda.device_count())})
    hidden = 40
    rot = RotaryPositions(d, 1000.0)
    rot.prepare(64, DEV)
    part = PagedAttention("a", hidden, H, KV, d, rot, window=window)
    w = {"a.q_proj.weight": rand(H * d, hidden, seed=10, scale=0.25).to(dtype),
         "a.k_proj.weight": rand(KV * d, hidden, seed=11, scale=0.25).to(dtype),
         "a.v_proj.weight": rand(KV * d, hidden, seed=12, scale=0.15).to(dtype),
         "a.o_proj.weight": rand(hidden, H * d, seed=13, scale=0.1).to(dtype)}
    part.load({k: v.to(DEV) for k, v in w.items()})
    part.seal()
    cache = CacheManager(bs, [CacheGroup((0,), attention_pages(KV, d), window)], 24)
    ls = LayerState(group=0, owns_cache=True,
                    pages={"k": torch.zeros(24, KV, bs, d, dtype=dtype, device=DEV),
                           "v": torch.zeros(24, KV, d, bs, dtype=dtype, device=DEV)})
    xs = {"s": rand(21, hidden, seed=14).to(dtype), "t": rand(9, hidden, seed=15).to(dtype)}
    cfg = {"num_attention_heads": H, "num_key_value_heads": KV, "head_dim": d}
    want = {}
    for rid, x in xs.items():
        cos, sin = plain.rope_cos_sin(torch.arange(x.shape[0]), plain.rope_inv_freq(d, 1000.0))
        want[rid] = plain.attention_block(x.float(), {k: v.float() for k, v in w.items()}, "a.",
                                          cfg, cos, sin, window)
    cache.allocate("junk", 5)                      # the pages of "s" and "t" are not contiguous
    cache.allocate("s", 0)
    cache.allocate("t", 0)
    got = {"s": [], "t": []}
    for portions in ([("s", 0, 12)], [("s", 12, 20), ("t", 0, 9)], [("s", 20, 21)]):
        entries = []
        for rid, a, b in portions:
            cache.append_slots(rid, b, a)
            entries.append(StepEntry(rid, [0] * (b - a), a, "none"))
        step = make_step(entries, cache, dtype)
        x = torch.cat([xs[rid][a:b] for rid, a, b in portions]).to(DEV)
        residual = torch.zeros(x.shape[0], hidden, device=DEV)
        part.forward(x, step, ls, residual)
        step.settle()  # with many rows the last product is left owed to the stream
        made = [v for k, v in step.scratch.items() if k[0] == "attention.prefill_work"]
        if made and dtype == torch.bfloat16 and bs % 8 == 0:
            assert made[0][1] == (128 if small_chip else 64)
        off = 0
        for rid, a, b in portions:
            got[rid].append(residual[off:off + b - a].cpu())
            off += b - a
            cache.release_behind(rid, b)
    for rid in xs:
        torch.testing.assert_close(torch.cat(got[rid]), want[rid], **tol(dtype))


@pytest.mark.parametrize("d,runs,rows_per_item", [
    (64, [(2048, 0)], 64),            # 512 workgroups of two tiles would leave half the chip's places empty
    (64, [(4096, 0)], 128),           # 1,024 of them fill it
    (64, [(2048, 2048)], 128),        # all items walk long: two a compute unit are enough
    (64, [(2048, 1024)], 64),         # the run starts less than its own length into its sequence
    (64, [(1024, 0)] * 4, 128),       # several runs count together
    (128, [(2048, 0)], 64),
    (128, [(4096, 0)], 128),
])
def test_attention_plans_rows_per_item_by_what_fills_the_chip(d, runs, rows_per_item, monkeypatch):
    """32 heads over 8 kv heads on a chip of 256 compute units: the planner's choice between one
    and two row tiles per wave, and its order (longest walk first)."""
    from types import SimpleNamespace
    from kvforge_amd.kernels import ops as kernel_ops
    monkeypatch.setattr(kernel_ops, "_compute_units", {i: 256 for i in range(torch.cuda.device_count())})
    part = PagedAttention("a", 2048, 32, 8, d, RotaryPositions(d, 1000.0))
    step = SimpleNamespace(q_lens=[n for n, _ in runs], start_pos=[s for _, s in runs],
                           prefill_seqs=list(range(len(runs))), scratch={}, device=torch.device(DEV),
                           upload_ints=lambda v: torch.tensor(v, dtype=torch.int32))
    rows, per_item = part._prefill_work(step, torch.bfloat16, 16)
    assert per_item == rows_per_item
    rows = rows.tolist()
    assert len(rows) == sum(-(-n * 4 // per_item) for n, _ in runs) and all(r[2] == -1 for r in rows)
    ends = [runs[b][1] + min(runs[b][0], -(-(i + 1) * per_item // 4)) for b, i, _ in rows]
    assert ends == sorted(ends, reverse=True)
    assert sorted((b, i) for b, i, _ in rows) == [(b, i) for b, (n, _) in enumerate(runs)
                                                  for i in range(-(-n * 4 // per_item))]


class ToyQKNormAttention(PagedAttention):
    """Attention with a bias on the q projection and an RMS norm per head of q and of k before
    the rotation, added from here through ``after_projection``: the framework's files know of
    neither.  The norm's weights are constants of the part (no tensors), one per element."""

    replayable = True

    def __init__(self, *args, q_bias=None, **kw):
        super().__init__(*args, **kw)
        self.q_bias = q_bias                           # [H * d], checkpoint order
        g = torch.Generator().manual_seed(99)
        self.qk_weight = 1 + 0.2 * torch.randn(self.d, generator=g)      # checkpoint order

    def after_projection(self, qkv, step):
        H, KV, d = self.H, self.KV, self.d
        perm = self.pair_permutation().to(qkv.device)   # the part's layout: perm[new] = old
        w = self.qk_weight.to(qkv.device)[perm]
        q = qkv[:, :H * d].float().view(-1, H, d)
        if self.q_bias is not None:
            q = q + self.q_bias.to(qkv.device).view(H, d)[:, perm]
        k = qkv[:, H * d:(H + KV) * d].float().view(-1, KV, d)
        for t, lo in ((q, 0), (k, H * d)):
            normed = t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + 1e-6) * w
            qkv[:, lo:lo + normed.shape[1] * d] = normed.reshape(normed.shape[0], -1).to(qkv.dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_variant_of_attention_changes_q_and_k_before_the_rotation(dtype):
    """``PagedAttention.after_projection``: a subclass defined here adds a bias to q and norms
    every head of q and k; fed in portions and token by token it gives what the same
    computation gives over the whole sequence, and without the hook's work the result is
    another one."""
    H, KV, d, hidden, bs = 4, 2, 32, 40, 8
    rot = RotaryPositions(d, 1000.0)
    rot.prepare(64, DEV)
    bias = rand(H * d, seed=31, scale=0.5)
    part = ToyQKNormAttention("a", hidden, H, KV, d, rot, q_bias=bias)
    assert not part.absorb_norm(RMSNorm("n", hidden, 1e-5))
    w = {"a.q_proj.weight": rand(H * d, hidden, seed=10, scale=0.25).to(dtype),
         "a.k_proj.weight": rand(KV * d, hidden, seed=11, scale=0.25).to(dtype),
         "a.v_proj.weight": rand(KV * d, hidden, seed=12, scale=0.15).to(dtype),
         "a.o_proj.weight": rand(hidden, H * d, seed=13, scale=0.1).to(dtype)}
    part.load({k: v.to(DEV) for k, v in w.items()})
    part.seal()
    x = rand(25, hidden, seed=14).to(dtype)
    wf = {k: v.float() for k, v in w.items()}
    T = x.shape[0]
    cos, sin = plain.rope_cos_sin(torch.arange(T), plain.rope_inv_freq(d, 1000.0))

    def whole(with_hook):
        q = (x.float() @ wf["a.q_proj.weight"].T).view(T, H, d)
        k = (x.float() @ wf["a.k_proj.weight"].T).view(T, KV, d)
        v = (x.float() @ wf["a.v_proj.weight"].T).view(T, KV, d)
        if with_hook:
            q = q + bias.view(H, d)
            q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + 1e-6) * part.qk_weight
            k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + 1e-6) * part.qk_weight
        q, k = plain.apply_rope(q, cos, sin), plain.apply_rope(k, cos, sin)
        att = plain.causal_attention(q, k, v, 1 / math.sqrt(d))
        return att.reshape(T, H * d) @ wf["a.o_proj.weight"].T

    want = whole(True)
    assert float((want - whole(False)).abs().max()) > 0.05
    cache = CacheManager(bs, [CacheGroup((0,), attention_pages(KV, d), None)], 8)
    ls = LayerState(group=0, owns_cache=True,
                    pages={"k": torch.zeros(8, KV, bs, d, dtype=dtype, device=DEV),
                           "v": torch.zeros(8, KV, d, bs, dtype=dtype, device=DEV)})
    cache.allocate("s", 0)
    got = []
    for a, b in ((0, 11), (11, 22), (22, 23), (23, 24), (24, 25)):
        cache.append_slots("s", b, a)
        step = make_step([StepEntry("s", [0] * (b - a), a, "none")], cache, dtype)
        residual = torch.zeros(b - a, hidden, device=DEV)
        part.forward(x[a:b].to(DEV), step, ls, residual)
        step.settle()
        got.append(residual.cpu())
    torch.testing.assert_close(torch.cat(got), want, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [7, 23])  # few rows: sums in the product kernels; many: owed to the stream
def test_pre_norm_block(dtype, n):
    hidden, H, KV, d, inter = 32, 2, 1, 16, 48
    rot = RotaryPositions(d, 100.0)
    rot.prepare(32, DEV)
    block = PreNormBlock(RMSNorm("b.n1", hidden, 1e-5), PagedAttention("b.att", hidden, H, KV, d, rot),
                         RMSNorm("b.n2", hidden, 1e-5), SwiGLU("b.ff", hidden, inter))
    g = torch.Generator().manual_seed(20)
    w = {}
    for name, spec in block.weight_specs().items():
        t = torch.randn(spec.shape, generator=g) * (0.1 if spec.init == "norm" else 0.15)
        w[name] = (t + 1 if spec.init == "norm" else t).to(dtype)
    block.load({k: v.to(DEV) for k, v in w.items()})
    block.seal()
    x = rand(n, hidden, seed=21)
    cache = CacheManager(4, [CacheGroup((0,), attention_pages(KV, d), None)], 8)
    cache.allocate("r", n)
    ls = LayerState(group=0, owns_cache=True,
                    pages={"k": torch.zeros(8, KV, 4, d, dtype=dtype, device=DEV),
                           "v": torch.zeros(8, KV, d, 4, dtype=dtype, device=DEV)})
    step = make_step([StepEntry("r", [0] * n, 0, "none")], cache, dtype)
    residual = x.clone().to(DEV)
    block.forward(residual, step, ls)
    step.settle()
    wf = {k: v.float() for k, v in w.items()}
    cfg = {"num_attention_heads": H, "num_key_value_heads": KV, "head_dim": d}
    cos, sin = plain.rope_cos_sin(torch.arange(n), plain.rope_inv_freq(d, 100.0))
    h = x + plain.attention_block(plain.rms_norm(x, wf["b.n1.weight"], 1e-5), wf, "b.att.", cfg,
                                  cos, sin, None)
    h = h + plain.swiglu(plain.rms_norm(h, wf["b.n2.weight"], 1e-5), wf["b.ff.gate_proj.weight"],
                         wf["b.ff.up_proj.weight"], wf["b.ff.down_proj.weight"])
    torch.testing.assert_close(residual.cpu(), h, **tol(dtype))


# ====================================================================== toy parts, defined here
class ToyDecayMixer(Mixer):
    """A recurrence with per-request state of fixed size, written with torch ops:
    ``s_t = sigmoid(decay) * s_{t-1} + x_t``,  ``y_t = s_t @ proj^T``.  The state lives in the
    request's slot between steps and is cleared where a request starts."""

    def __init__(self, prefix: str, hidden: int) -> None:
        self.prefix, self.hidden = prefix, hidden
        self.state_spec = StateSpec((hidden,), torch.float32)

    def weight_specs(self):
        return {self._name("decay"): WeightSpec((self.hidden,), init="norm", std=0.5),
                self._name("proj.weight"): WeightSpec((self.hidden, self.hidden), std=0.2)}

    def load(self, tensors):
        self.decay = tensors[self._name("decay")].float()
        self.proj = tensors[self._name("proj.weight")].float()

    def forward(self, x, step, layer, residual):
        gate = torch.sigmoid(self.decay)
        off = 0
        for b, n in enumerate(step.q_lens):
            slot = step.host_slot_ids[b]
            s = layer.state[slot].clone() if step.start_pos[b] > 0 else torch.zeros_like(gate)
            for t in range(n):
                s = gate * s + x[off + t].float()
                residual[off + t] += s @ self.proj.T
            layer.state[slot] = s
            off += n


@dataclass
class ToyConfig(ModelConfig):
    hidden_size: int = 0
    num_heads: int = 0
    head_dim: int = 0
    inter: int = 0
    eps: float = 1e-5

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "ToyConfig":
        return cls(architecture=d["architectures"][0], vocab_size=d["vocab_size"],
                   max_position_embeddings=d["max_position_embeddings"], hidden_size=d["hidden_size"],
                   num_heads=d["num_heads"], head_dim=d["head_dim"], inter=d["inter"], eps=d["eps"])

    def to_dict(self) -> dict[str, Any]:
        return {"architectures": [self.architecture], "vocab_size": self.vocab_size,
                "max_position_embeddings": self.max_position_embeddings,
                "hidden_size": self.hidden_size, "num_heads": self.num_heads,
                "head_dim": self.head_dim, "inter": self.inter, "eps": self.eps}


def build_toy(cfg: ToyConfig) -> ModelSpec:
    """Blocks: 0 attention, 1 toy recurrence, 2 attention without a cache of its own.
    Run order: 0, 1, 2 reading call 0's cache, then block 1 a second time."""
    h = cfg.hidden_size
    rot = RotaryPositions(cfg.head_dim, 100.0)
    mixer_cls = registry.MIXERS["toy_decay"]

    def block(i, mixer):
        return PreNormBlock(RMSNorm(f"layers.{i}.n1", h, cfg.eps), mixer,
                            RMSNorm(f"layers.{i}.n2", h, cfg.eps), SwiGLU(f"layers.{i}.ff", h, cfg.inter))
    blocks = [block(0, PagedAttention("layers.0.att", h, cfg.num_heads, 1, cfg.head_dim, rot)),
              block(1, mixer_cls("layers.1.mix", h)),
              block(2, PagedAttention("layers.2.att", h, cfg.num_heads, 1, cfg.head_dim, rot))]
    return ModelSpec(config=cfg, embedding=TokenEmbedding("embed", cfg.vocab_size, h), blocks=blocks,
                     final_norm=RMSNorm("norm", h, cfg.eps),
                     head=LMHead("head", cfg.vocab_size, h, tied_to="embed.weight"), positions=[rot],
                     schedule=[LayerCall(0), LayerCall(1), LayerCall(2, cache_of=0), LayerCall(1)])


TOY = {"architectures": ["ToyForCausalLM"], "vocab_size": 90, "max_position_embeddings": 128,
       "hidden_size": 48, "num_heads": 3, "head_dim": 16, "inter": 64, "eps": 1e-5}


def toy_plain(w, ids):
    """The toy model over one whole sequence, straight from its definition."""
    wf = {k: v.float() for k, v in w.items()}
    T = len(ids)
    h = wf["embed.weight"][torch.tensor(ids)]
    cos, sin = plain.rope_cos_sin(torch.arange(T), plain.rope_inv_freq(16, 100.0))
    cfg = {"num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 16}

    def ffn(h, i):
        m = plain.rms_norm(h, wf[f"layers.{i}.n2.weight"], 1e-5)
        return h + plain.swiglu(m, wf[f"layers.{i}.ff.gate_proj.weight"],
                                wf[f"layers.{i}.ff.up_proj.weight"], wf[f"layers.{i}.ff.down_proj.weight"])

    def recurrence(h):
        a = plain.rms_norm(h, wf["layers.1.n1.weight"], 1e-5)
        gate, s, ys = torch.sigmoid(wf["layers.1.mix.decay"]), torch.zeros(48), []
        for t in range(T):
            s = gate * s + a[t]
            ys.append(s @ wf["layers.1.mix.proj.weight"].T)
        return ffn(h + torch.stack(ys), 1)

    a0 = plain.rms_norm(h, wf["layers.0.n1.weight"], 1e-5)
    h = ffn(h + plain.attention_block(a0, wf, "layers.0.att.", cfg, cos, sin, None), 0)
    h = recurrence(h)
    # block 2 attends with its own query over the keys and values that call 0 cached
    a2 = plain.rms_norm(h, wf["layers.2.n1.weight"], 1e-5)
    q = plain.apply_rope((a2 @ wf["layers.2.att.q_proj.weight"].T).view(T, 3, 16), cos, sin)
    k = plain.apply_rope((a0 @ wf["layers.0.att.k_proj.weight"].T).view(T, 1, 16), cos, sin)
    v = (a0 @ wf["layers.0.att.v_proj.weight"].T).view(T, 1, 16)
    att = plain.causal_attention(q, k, v, 0.25).reshape(T, 48) @ wf["layers.2.att.o_proj.weight"].T
    h = ffn(h + att, 2)
    h = recurrence(h)
    return plain.rms_norm(h, wf["norm.weight"], 1e-5) @ wf["embed.weight"].T


@pytest.fixture(scope="module")
def toy_folder(tmp_path_factory):
    kvforge_amd.register_mixer("toy_decay", ToyDecayMixer)
    kvforge_amd.register_architecture("ToyForCausalLM", ToyConfig, build_toy)
    folder = str(tmp_path_factory.mktemp("toy"))
    kvforge_amd.write_random_model(folder, TOY, seed=4)
    return folder


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_architecture_registers_builds_and_steps(toy_folder, dtype):
    w = plain.read_weights(toy_folder)
    model = Transformer.from_folder(toy_folder, dtype, DEV)
    assert isinstance(model.config, ToyConfig)
    # one cache group with one owner (call 0); calls 1 and 3 each hold a state of their own
    assert [g.layers for g in model.cache_groups] == [(0,)]
    assert sorted(model.state_specs) == [1, 3]
    runner = ModelRunner(model, 4, 40, max_num_seqs=4, max_num_batched_tokens=64, max_model_len=128)
    g = torch.Generator().manual_seed(5)
    seqs = {r: torch.randint(0, 90, (n,), generator=g).tolist() for r, n in (("a", 23), ("b", 14), ("c", 9))}
    want = {r: toy_plain(w, ids) for r, ids in seqs.items()}
    got = {r: [] for r in seqs}
    plan = [[("a", 0, 7), ("b", 0, 14)], [("a", 7, 9)], [("a", 9, 22), ("c", 0, 1)],
            [("a", 22, 23), ("c", 1, 9)]]
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
                runner.cache.free(rid)          # "b"'s slot and pages go to "c"
    t = dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=3e-2)
    for rid in seqs:
        torch.testing.assert_close(torch.cat(got[rid]), want[rid], **t)
    assert runner.cache.slots.num_free == 4 and runner.cache.num_free_blocks == 40


def test_toy_architecture_generates_through_the_engine(toy_folder):
    w = plain.read_weights(toy_folder)
    engine = kvforge_amd.InferenceEngine.from_folder(
        toy_folder, kvforge_amd.EngineConfig(
            cache=kvforge_amd.CacheConfig(block_size=4, num_blocks=64),
            scheduler=kvforge_amd.SchedulerConfig(max_num_seqs=3, max_num_batched_tokens=8)))
    prompts = [[5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15], [80, 3], [44, 45, 46, 47, 48]]
    outs = engine.generate(prompts, kvforge_amd.SamplingParams(max_tokens=6, temperature=0.0))
    for p, o in zip(prompts, outs):
        logits = toy_plain(w, p + o.output_token_ids)
        for i, tok in enumerate(o.output_token_ids):
            row = logits[len(p) - 1 + i]
            assert float(row.max() - row[tok]) <= 1e-4
    assert engine.cache.slots.num_free == 3


def test_run_order_is_checked():
    cfg = ToyConfig.from_dict(TOY)
    spec = build_toy(cfg)
    spec.schedule = [LayerCall(0), LayerCall(2, cache_of=1)]
    with pytest.raises(ValueError, match="owns none"):
        Transformer(spec, torch.float32, DEV)
    spec.schedule = [LayerCall(5)]
    with pytest.raises(ValueError, match="outside"):
        Transformer(spec, torch.float32, DEV)


def test_ints_sent_along_with_a_step_arrive_in_stream_order():
    """``Step.upload_ints`` on the device: several lists in one step land behind each other in
    the step's own memory, a list too long for it goes the slow way, and the next step may
    overwrite them only behind this step's work in stream order."""
    cache = CacheManager(4, [CacheGroup((0,))], 16)
    cache.allocate("r", 12)
    step = make_step([StepEntry("r", [0] * 12, 0, "none")], cache, torch.float32)
    a = step.upload_ints(list(range(10)))
    b = step.upload_ints([(7, 8, -1), (9, 10, 11)])
    big = step.upload_ints(list(range(5000)))
    torch.cuda.synchronize()
    assert a.tolist() == list(range(10)) and b.tolist() == [7, 8, -1, 9, 10, 11]
    assert big.tolist() == list(range(5000)) and a.is_cuda and a.dtype == torch.int32
    assert a.data_ptr() != b.data_ptr() and b.data_ptr() % 16 == 0
    kept = a.clone()                     # queued before the next step's fill
    again = make_step([StepEntry("r", [0] * 12, 0, "none")], cache, torch.float32)
    c = again.upload_ints([5] * 10)
    torch.cuda.synchronize()
    assert kept.tolist() == list(range(10)) and c.tolist() == [5] * 10
