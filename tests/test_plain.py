"""Pins the plain implementation by what fixes it beside the reference's text: library routines
it must reduce to, hand-derived vectors, and invariants chosen so that a plausible mistake
(a wrong sign or pairing, eps outside the root, a norm in the wrong place) fails."""

from __future__ import annotations

import math

import pytest
import torch
import torch.nn.functional as F

from tests.plain import llama as plain
from tests.plain import sampling as plain_sampling


def rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


# ------------------------------------------------------------------ RMS norm
def test_rms_norm_is_the_library_routine():
    x, w = rand(7, 96) * 3, 1 + 0.1 * rand(96, seed=1)
    for eps in (1e-5, 1e-6, 0.3):  # a large eps tells "inside the root" from "outside"
        torch.testing.assert_close(plain.rms_norm(x, w, eps), F.rms_norm(x, (96,), w, eps))


def test_rms_norm_unit_rms_and_scale_invariance():
    x = rand(5, 64, seed=2)
    y = plain.rms_norm(x, torch.ones(64), 1e-12)
    torch.testing.assert_close(y.pow(2).mean(-1), torch.ones(5))
    torch.testing.assert_close(plain.rms_norm(x * 7.5, torch.ones(64), 1e-12), y)


def test_rms_norm_eps_sits_inside_the_root():
    x = torch.full((1, 4), 2.0)
    want = 2.0 / math.sqrt(4.0 + 0.5)
    assert plain.rms_norm(x, torch.ones(4), 0.5)[0, 0].item() == pytest.approx(want)


# ------------------------------------------------------------------ rotary
def test_rope_hand_vectors():
    # src/tokenvault/model.py:53-61 with d = 2: x = (1, 0) at angle a becomes (cos a, sin a)
    inv = torch.tensor([1.0])
    cos, sin = plain.rope_cos_sin(torch.tensor([1]), inv)
    out = plain.apply_rope(torch.tensor([[[1.0, 0.0]]]), cos, sin)
    torch.testing.assert_close(out, torch.tensor([[[math.cos(1.0), math.sin(1.0)]]]))
    out = plain.apply_rope(torch.tensor([[[0.0, 1.0]]]), cos, sin)
    torch.testing.assert_close(out, torch.tensor([[[-math.sin(1.0), math.cos(1.0)]]]))
    # d = 4 pairs element 0 with 2 and 1 with 3 (half split), not 0 with 1
    inv = plain.rope_inv_freq(4, 100.0)
    torch.testing.assert_close(inv, torch.tensor([1.0, 0.1]))
    cos, sin = plain.rope_cos_sin(torch.tensor([3]), inv)
    out = plain.apply_rope(torch.tensor([[[1.0, 0.0, 0.0, 0.0]]]), cos, sin)
    torch.testing.assert_close(out, torch.tensor([[[math.cos(3.0), 0.0, math.sin(3.0), 0.0]]]))
    out = plain.apply_rope(torch.tensor([[[0.0, 1.0, 0.0, 0.0]]]), cos, sin)
    torch.testing.assert_close(out, torch.tensor([[[0.0, math.cos(0.3), 0.0, math.sin(0.3)]]]))


def test_rope_position_zero_is_identity_and_pairs_keep_their_norm():
    inv = plain.rope_inv_freq(32, 10000.0)
    x = rand(6, 3, 32, seed=3)
    cos, sin = plain.rope_cos_sin(torch.zeros(6, dtype=torch.long), inv)
    torch.testing.assert_close(plain.apply_rope(x, cos, sin), x)
    cos, sin = plain.rope_cos_sin(torch.arange(6) * 17, inv)
    y = plain.apply_rope(x, cos, sin)
    pair = lambda t: t[..., :16] ** 2 + t[..., 16:] ** 2
    torch.testing.assert_close(pair(y), pair(x), atol=1e-5, rtol=1e-5)


def test_rope_scores_depend_on_distance_only():
    inv = plain.rope_inv_freq(16, 10000.0)
    q, k = rand(1, 1, 16, seed=4), rand(1, 1, 16, seed=5)

    def score(m, n):
        cq, sq = plain.rope_cos_sin(torch.tensor([m]), inv)
        ck, sk = plain.rope_cos_sin(torch.tensor([n]), inv)
        return (plain.apply_rope(q, cq, sq) * plain.apply_rope(k, ck, sk)).sum().item()

    assert score(9, 4) == pytest.approx(score(25, 20), abs=1e-5)
    assert score(9, 4) != pytest.approx(score(4, 9), abs=1e-3)  # direction matters


def test_llama3_scaling_invariants():
    base = plain.rope_inv_freq(32, 500000.0)
    # factor 1 is the identity
    torch.testing.assert_close(plain.llama3_scale_inv_freq(base, 1.0, 1.0, 4.0, 64), base)
    out = plain.llama3_scale_inv_freq(base, 4.0, 1.0, 4.0, 64)
    wavelen = 2 * math.pi / base
    assert out[0] == base[0]                                   # highest frequency untouched
    hi, lo = wavelen < 16, wavelen > 64
    assert hi.any() and lo.any() and (~hi & ~lo).any()         # all three branches
    torch.testing.assert_close(out[hi], base[hi])
    torch.testing.assert_close(out[lo], base[lo] / 4.0)
    assert (out[1:] <= out[:-1]).all()                         # still ordered
    mid = ~hi & ~lo
    assert ((out[mid] < base[mid]) & (out[mid] > base[mid] / 4.0)).all()
    # continuous at both thresholds
    f_low = torch.tensor([2 * math.pi / 64.0])
    f_high = torch.tensor([2 * math.pi / 16.0])
    assert plain.llama3_scale_inv_freq(f_low, 4.0, 1.0, 4.0, 64)[0].item() == pytest.approx(
        f_low.item() / 4.0, rel=1e-6)
    assert plain.llama3_scale_inv_freq(f_high, 4.0, 1.0, 4.0, 64)[0].item() == pytest.approx(
        f_high.item(), rel=1e-6)


def test_llama3_scaling_mid_band_value_worked_by_hand():
    """Tiny B's one frequency between the thresholds (theta 5e5, head size 32, factor 4, low 1,
    high 4, original length 64, so wavelengths between 16 and 64 are blended), by the rule
    "between them (1 - s) f / factor + s f with s = (orig / wavelength - low) / (high - low)":

        j = 2:  f = 500000^(-4/32) = 0.193922745,  wavelength = 2 pi / f = 32.4004557
        orig / wavelength = 1.97528086,  s = (1.97528086 - 1) / 3 = 0.325093619
        out = f (0.25 (1 - s) + s) = 0.193922745 * 0.493820214 = 0.0957629714

    A blend that is linear in the wavelength instead (s = (64 - 32.4) / 48) gives 0.1442 and
    passes every bound, order and continuity check above.  The plain model and the engine's
    tables must both give the worked value; neighbours j = 1 (wavelength 14.27, kept) and j = 3
    (73.58, divided by 4) pin the two thresholds' sides.

    Parity unpinned: the reference has no frequency scaling and nothing it ships holds a vector
    of scaled frequencies, so the worked value follows from the rule as written above and from
    no output of the reference."""
    from kvforge_amd.config.model import RopeScaling
    from kvforge_amd.parts.positions import scaled_inv_freq
    base = plain.rope_inv_freq(32, 500000.0)
    out = plain.llama3_scale_inv_freq(base, 4.0, 1.0, 4.0, 64)
    eng = scaled_inv_freq(32, 500000.0, RopeScaling("llama3", 4.0, 1.0, 4.0, 64))
    for got in (out, eng):
        assert got[2].item() == pytest.approx(0.0957629714, rel=2e-6)
        assert got[1].item() == pytest.approx(500000.0 ** (-2 / 32), rel=1e-6)
        assert got[3].item() == pytest.approx(500000.0 ** (-6 / 32) / 4.0, rel=1e-6)
    torch.testing.assert_close(eng, out, rtol=1e-6, atol=0)


# ------------------------------------------------------------------ attention
@pytest.mark.parametrize("H,KV,d", [(4, 2, 16), (3, 1, 32), (4, 4, 8)])
def test_attention_is_the_library_routine(H, KV, d):
    T = 13
    q, k, v = rand(T, H, d, seed=6), rand(T, KV, d, seed=7), rand(T, KV, d, seed=8)
    got = plain.causal_attention(q, k, v, 1 / math.sqrt(d))
    g = H // KV
    want = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.transpose(0, 1).repeat_interleave(g, 0)[None],
        v.transpose(0, 1).repeat_interleave(g, 0)[None], is_causal=True)[0].transpose(0, 1)
    torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)


def test_attention_special_cases():
    d = 8
    q, k, v = rand(1, 2, d, seed=9), rand(1, 1, d, seed=10), rand(1, 1, d, seed=11)
    out = plain.causal_attention(q, k, v, 0.3)           # one key: the output is its value
    torch.testing.assert_close(out, v.expand(1, 2, d))
    # query offset: the last query of a longer context equals the full computation's last row
    q, k, v = rand(9, 2, d, seed=12), rand(9, 1, d, seed=13), rand(9, 1, d, seed=14)
    full = plain.causal_attention(q, k, v, 0.3)
    torch.testing.assert_close(plain.causal_attention(q[5:], k, v, 0.3, q_offset=5), full[5:])
    # a window as long as the sequence is no window; a window of one sees only itself
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.3, window=9), full)
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.3, window=1), v.expand(9, 2, d))
    # zero scale gives the running mean of the values
    mean = v.cumsum(0) / torch.arange(1, 10)[:, None, None]
    torch.testing.assert_close(plain.causal_attention(q, k, v, 0.0), mean.expand(9, 2, d))


# ------------------------------------------------------------------ feed-forward
def test_swiglu():
    x = rand(5, 12, seed=15)
    g, u, dn = rand(20, 12, seed=16), rand(20, 12, seed=17), rand(12, 20, seed=18)
    want = F.linear(F.silu(F.linear(x, g)) * F.linear(x, u), dn)
    torch.testing.assert_close(plain.swiglu(x, g, u, dn), want)
    assert plain.swiglu(x, torch.zeros_like(g), u, dn).abs().max() == 0  # silu(0) = 0


# ------------------------------------------------------------------ whole model
def tiny_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    h, H, KV, d, I, V = (cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"],
                         cfg["head_dim"], cfg["intermediate_size"], cfg["vocab_size"])
    w = {"model.embed_tokens.weight": torch.randn(V, h, generator=g) * 0.5,
         "model.norm.weight": 1 + 0.1 * torch.randn(h, generator=g)}
    if not cfg["tie_word_embeddings"]:
        w["lm_head.weight"] = torch.randn(V, h, generator=g) * 0.5
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w[p + "input_layernorm.weight"] = 1 + 0.1 * torch.randn(h, generator=g)
        w[p + "post_attention_layernorm.weight"] = 1 + 0.1 * torch.randn(h, generator=g)
        w[p + "self_attn.q_proj.weight"] = torch.randn(H * d, h, generator=g) * 0.2
        w[p + "self_attn.k_proj.weight"] = torch.randn(KV * d, h, generator=g) * 0.2
        w[p + "self_attn.v_proj.weight"] = torch.randn(KV * d, h, generator=g) * 0.2
        w[p + "self_attn.o_proj.weight"] = torch.randn(h, H * d, generator=g) * 0.2
        w[p + "mlp.gate_proj.weight"] = torch.randn(I, h, generator=g) * 0.2
        w[p + "mlp.up_proj.weight"] = torch.randn(I, h, generator=g) * 0.2
        w[p + "mlp.down_proj.weight"] = torch.randn(h, I, generator=g) * 0.2
    return w


CFG = {"hidden_size": 24, "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 8,
       "intermediate_size": 40, "vocab_size": 50, "num_hidden_layers": 2, "rms_norm_eps": 1e-5,
       "rope_theta": 100.0, "tie_word_embeddings": True}


def test_model_is_causal_and_shift_invariant():
    w = tiny_weights(CFG)
    ids = [3, 14, 15, 9, 26, 5, 35, 8]
    full = plain.forward(w, CFG, ids)
    torch.testing.assert_close(plain.forward(w, CFG, ids[:5]), full[:5], atol=1e-5, rtol=1e-5)
    # only distances count under rotary positions
    torch.testing.assert_close(plain.forward(w, CFG, ids, first_position=11), full,
                               atol=2e-4, rtol=2e-4)


def test_model_tied_and_untied_head():
    w = tiny_weights(CFG)
    ids = [1, 2, 3]
    logits = plain.forward(w, CFG, ids)
    cfg2 = dict(CFG, tie_word_embeddings=False)
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    torch.testing.assert_close(plain.forward(w2, cfg2, ids), logits)
    w2["lm_head.weight"] = w2["lm_head.weight"] * 2
    torch.testing.assert_close(plain.forward(w2, cfg2, ids), logits * 2)


def test_model_one_layer_by_hand():
    """One layer, one head, identity-like pieces: the residual order of
    src/tokenvault/model.py:185-188 (norm before each sub-layer, sums outside)."""
    cfg = dict(CFG, num_hidden_layers=1, num_attention_heads=1, head_dim=24)
    w = tiny_weights(cfg, seed=3)
    ids = [7]
    # with one token attention returns v: h1 = h0 + Wo Wv norm(h0)
    h0 = w["model.embed_tokens.weight"][7]
    a = plain.rms_norm(h0[None], w["model.layers.0.input_layernorm.weight"], 1e-5)
    h1 = h0 + (a @ w["model.layers.0.self_attn.v_proj.weight"].T) @ w["model.layers.0.self_attn.o_proj.weight"].T
    m = plain.rms_norm(h1, w["model.layers.0.post_attention_layernorm.weight"], 1e-5)
    h2 = h1 + plain.swiglu(m, w["model.layers.0.mlp.gate_proj.weight"],
                           w["model.layers.0.mlp.up_proj.weight"],
                           w["model.layers.0.mlp.down_proj.weight"])
    want = plain.rms_norm(h2, w["model.norm.weight"], 1e-5) @ w["model.embed_tokens.weight"].T
    torch.testing.assert_close(plain.forward(w, cfg, ids), want, atol=1e-5, rtol=1e-5)


def test_sliding_layers_change_only_long_range():
    cfg = dict(CFG, layer_types=["sliding_attention", "full_attention"], sliding_window=4)
    w = tiny_weights(CFG)
    ids = list(range(10, 22))
    a, b = plain.forward(w, cfg, ids), plain.forward(w, CFG, ids)
    torch.testing.assert_close(a[:4], b[:4])           # inside the window nothing changes
    assert (a[6:] - b[6:]).abs().max() > 1e-4


# ------------------------------------------------------------------ sampling
def test_sampling_reference_vectors():
    # tests/test_continuous_batching.py:160-169 of the reference
    logits = torch.tensor([4.0, 3.0, 2.0, 1.0, 0.0])
    p = plain_sampling.processed_probs(logits, 1.0, top_k=2)
    assert (p[2:] == 0).all() and p[:2].sum().item() == pytest.approx(1.0)
    p = plain_sampling.processed_probs(logits, 1.0, top_p=0.5)
    assert p[0].item() == pytest.approx(1.0)
    assert plain_sampling.processed_probs(logits, 0.0).tolist() == [1.0, 0.0, 0.0, 0.0, 0.0]
    p = plain_sampling.processed_probs(logits, 0.7)
    torch.testing.assert_close(p, torch.softmax(logits.double() / 0.7, -1), atol=1e-6, rtol=1e-6)


def test_draw_and_uniform():
    p = torch.tensor([0.1, 0.2, 0.3, 0.4], dtype=torch.float64)
    assert [plain_sampling.draw(p, u) for u in (0.0, 0.09, 0.11, 0.29, 0.31, 0.61, 0.999)] == \
        [0, 0, 1, 1, 2, 3, 3]
    us = [plain_sampling.uniform(1, 2, i) for i in range(2000)]
    assert all(0 <= u < 1 for u in us) and abs(sum(us) / 2000 - 0.5) < 0.03
    assert plain_sampling.uniform(1, 2, 3) == plain_sampling.uniform(1, 2, 3)
    assert plain_sampling.uniform(1, 2, 3) != plain_sampling.uniform(1, 3, 3)


def test_attention_in_query_blocks_gives_the_same_logits():
    """``forward(query_block=...)`` never holds all scores at once (for sequences of tens of
    thousands of tokens); it is the same computation, also with a window and with ``last``."""
    cfg = dict(CFG, layer_types=["sliding_attention", "full_attention"], sliding_window=5)
    w = tiny_weights(CFG)
    ids = [(7 * i + 3) % 50 for i in range(37)]
    for c in (CFG, cfg):
        # in float64, where two orders of summation differ by nothing that could hide a mistake
        f64 = dict(dtype=torch.float64)
        full = plain.forward(w, c, ids, **f64)
        for block in (1, 8, 37, 64):
            torch.testing.assert_close(plain.forward(w, c, ids, query_block=block, **f64), full, atol=1e-7, rtol=1e-7)
        torch.testing.assert_close(plain.forward(w, c, ids, query_block=8, last=5, **f64), full[-5:],
                                   atol=1e-7, rtol=1e-7)
