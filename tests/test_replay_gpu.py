"""Trace replay through ``bin/trace_run`` (a fresh process, as a user runs it) against the plain
model: every request whole; most of it in one step and the last 32 tokens one by one; in
portions of changing size down to two tokens; and mixed, up to four live requests, portions of
some beside decoded tokens of others, with so few pages that they are used again.  In 32-bit and
in bfloat16, on three tiny configurations that differ in every size and option."""

from __future__ import annotations

import pytest

import kvforge_amd
from tests import replay_util as ru

pytestmark = pytest.mark.gpu

CONFIGS = {
    "tiny-a": (lambda: kvforge_amd.preset_dict("tiny-a"), 0, [37, 64, 81, 100, 53, 90]),
    "tiny-b": (lambda: kvforge_amd.preset_dict("tiny-b"), 1, [33, 70, 129, 96, 45, 160]),
    "tiny-c": (lambda: dict(ru.TINY_C), 2, [40, 97, 66, 130, 49, 111]),
}
TOL = {"float32": (2e-5, 1e-4), "bfloat16": (1.5e-2, 1.5e-2)}


def build_all_modes(prompts, seed):
    tb = ru.TraceBuilder()
    names = {}
    for rid, toks in prompts.items():
        for mode, fn in (("w", ru.whole), ("d", ru.decode_tail), ("p", ru.portions)):
            name = f"{rid}#{mode}"
            names[name] = toks
            fn(tb, name, toks)
    mixed_prompts = {f"{rid}#m": toks for rid, toks in prompts.items()}
    names.update(mixed_prompts)
    ru.mixed(tb, mixed_prompts, seed)
    return tb, names


# with the weights as drawn (flat attention) the two given configurations are enough
# a float32 engine meets weights stored in 32-bit, which bfloat16 cannot hold; once it is given
# weights stored in bfloat16 (widening at load is a path too)
# (one configuration is enough for the widening load)
@pytest.mark.parametrize("name,sharp,dtype,store", [
    (n, s, dtype, store) for n in CONFIGS for s in (0.0, 6.0) if s or n != "tiny-c"
    for dtype, store in (("float32", "float32"), ("bfloat16", "bfloat16"), ("float32", "bfloat16"))
    if store == dtype or (n, s) == ("tiny-b", 6.0)])
def test_replay_all_modes(tmp_path, name, dtype, store, sharp):
    make, seed, lengths = CONFIGS[name]
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, make(), seed=seed, dtype=store)
    if sharp:
        ru.sharpen(folder, sharp)
    cfg = make()
    prompts = ru.random_prompts(cfg["vocab_size"], lengths, seed)
    tb, names = build_all_modes(prompts, seed)
    # the pool holds exactly the peak of live tokens (each request rounded up to 64): the six
    # requests of the mixed phase need more pages in total than there are, so pages are reused
    assert sum(ru.round64(len(t)) for t in prompts.values()) > tb.peak
    out = str(tmp_path / "out")
    ru.run_trace(folder, dtype, tb, out)
    atol, rtol = TOL[dtype]
    ru.compare(folder, tb, out, names, atol, rtol)


ODD = {  # sizes off every beaten path: head sizes in steps of 16 up to 256, odd numbers of heads and
    # groups, widths that are multiples of 8 only, prime vocabularies, pages of 8, 24 and 32 tokens
    "d112": (dict(head_dim=112, num_key_value_heads=5, num_attention_heads=5, hidden_size=104,
                  intermediate_size=600, vocab_size=4099, num_hidden_layers=2, tie_word_embeddings=False,
                  layer_types=["sliding_attention", "full_attention"], sliding_window=33), 32),
    "d144": (dict(head_dim=144, num_key_value_heads=3, num_attention_heads=27, hidden_size=520,
                  intermediate_size=100, vocab_size=5003, num_hidden_layers=3, tie_word_embeddings=False,
                  layer_types=["full_attention", "sliding_attention", "full_attention"], sliding_window=24,
                  rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                                "high_freq_factor": 4.0, "original_max_position_embeddings": 64}), 8),
    "d256": (dict(head_dim=256, num_key_value_heads=3, num_attention_heads=12, hidden_size=72,
                  intermediate_size=24, vocab_size=9001, num_hidden_layers=1, tie_word_embeddings=True,
                  layer_types=["full_attention"]), 16),
    "d16": (dict(head_dim=16, num_key_value_heads=7, num_attention_heads=49, hidden_size=520,
                 intermediate_size=600, vocab_size=8999, num_hidden_layers=1, tie_word_embeddings=True,
                 layer_types=["sliding_attention"], sliding_window=64, rms_norm_eps=3e-4), 24),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", sorted(ODD))
def test_replay_sizes_that_no_kernel_was_tuned_for(tmp_path, dtype, which):
    """All four ways of cutting the requests, against the plain model, on shapes that the
    configuration allows and nothing was built around: each kernel takes them or a slower one
    does, never a wrong result."""
    change, block_size = ODD[which]
    cfg = dict(ru.TINY_C, max_position_embeddings=512, **change)
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, cfg, seed=len(which), dtype=dtype)
    ru.sharpen(folder, 4.0)
    prompts = ru.random_prompts(cfg["vocab_size"], [37, 64, 81, 100], 3)
    tb, names = build_all_modes(prompts, 3)
    out = str(tmp_path / "out")
    ru.run_trace(folder, dtype, tb, out, user_args=["--block-size", str(block_size)])
    atol, rtol = TOL[dtype]
    ru.compare(folder, tb, out, names, atol, rtol,
               measured_rounding="bfloat16" if dtype == "bfloat16" else False)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["WIDE", "WIDE_B", "WIDE_C"])
def test_replay_layers_wide_enough_for_the_serving_kernels(tmp_path, dtype, which):
    """The tiny configurations are below the sizes at which the bf16 engine changes kernels.
    This one is not: its down projection is cut in two halves of K for up to 16 rows, and the
    half that stays owed travels to the next layer's fused q/k/v projection and to the final
    norm; attention runs on the matrix cores at head size 64.  All four ways of cutting the
    requests, against the plain model."""
    import torch
    from kvforge_amd.kernels import ops
    bf = torch.bfloat16
    cfg = dict(getattr(ru, which))
    few = torch.empty(3, cfg["intermediate_size"], dtype=bf)
    deep = torch.empty(cfg["hidden_size"], cfg["intermediate_size"], dtype=bf)
    assert ops.k_halves_pay(few, deep) and not ops.is_library_product(few, deep)
    if which == "WIDE_C":     # the output projection as well
        heads = cfg["num_attention_heads"] * cfg["head_dim"]
        assert ops.k_halves_pay(torch.empty(3, heads, dtype=bf), torch.empty(cfg["hidden_size"], heads, dtype=bf))
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, cfg, seed=4, dtype=dtype)
    prompts = ru.random_prompts(cfg["vocab_size"], [41, 75, 52, 66], 9)
    tb, names = build_all_modes(prompts, 9)
    out = str(tmp_path / "out")
    ru.run_trace(folder, dtype, tb, out)
    ru.compare(folder, tb, out, names, *TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_tiny_b_at_its_own_pages_of_eight_tokens(tmp_path, dtype):
    """Tiny B as its configuration has it: pages of 8 tokens (``--block-size 8``), all four ways
    of cutting the requests, with a pool so small that pages are used again."""
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, kvforge_amd.preset_dict("tiny-b"), seed=1, dtype=dtype)
    ru.sharpen(folder, 6.0)
    prompts = ru.random_prompts(384, [1, 9, 40, 70, 129, 57], 1)
    tb, names = build_all_modes(prompts, 1)
    out = str(tmp_path / "out")
    ru.run_trace(folder, dtype, tb, out, user_args=["--block-size", "8", "--max-live", "4"])
    ru.compare(folder, tb, out, names, *TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_an_id_that_ends_and_comes_back_with_other_tokens(tmp_path, dtype):
    """What preemption does to the cache, seen from the step function: request "x" is fed and
    decodes beside "y", ends (its pages go back to the pool), "y" and a newcomer grow into those
    pages, and "x" comes back under the same id from position 0, first with its old tokens and
    more (recomputation), later once again with entirely different tokens, each time
    landing in pages that others have written since.  The engine keeps, per row of the block
    tables on the device, who the row belongs to; an id that returns must not be taken for its
    former self.  Every logit is compared with the plain model."""
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, dict(ru.TINY_C), seed=6, dtype=dtype)
    ru.sharpen(folder, 6.0)
    p = ru.random_prompts(200, [90, 120, 70, 80], 21)
    first, y, z, other = p["p0"], p["p1"], p["p2"], p["p3"]
    every = lambda n: list(range(n))
    tb = ru.TraceBuilder()
    tb.step([("x", first[:40], every(40), "x1"), ("y", y[:33], every(33))])
    for i in range(6):
        tb.step([("x", [first[40 + i]], [0], "x1"), ("y", [y[33 + i]], [0])])
    tb.step([("y", y[39:60], every(21))], end=["x"])                       # x loses its pages
    tb.step([("y", y[60:100], every(40)), ("z", z[:50], every(50))])       # others grow into them
    # x again: what it held before and ten tokens more, from position 0, as a recomputation does
    tb.step([("y", [y[100]], [0]), ("x", first[:56], every(56), "x1"), ("z", [z[50]], [0])])
    for i in range(8):
        tb.step([("y", [y[101 + i]], [0]), ("x", [first[56 + i]], [0], "x1"), ("z", [z[51 + i]], [0])])
    tb.step([("z", z[59:], every(11))], end=["x", "z"])
    # A third life with other tokens, in the batch row x sat in last (the second), which no step
    # has used in between, and with as many pages as it had there: only the allocation's serial
    # number tells the engine that the row's table on the device is not this request's.
    tb.step([("y", y[109:], every(11)), ("x", other[:64], every(64), "x2")])
    tb.step([("x", other[64:], every(16), "x2")], end=["x", "y"])
    names = {"x1": first, "x2": other, "y": y, "z": z}
    out = str(tmp_path / "out")
    # room for three live requests at most: x's pages must be among those that y and z take
    ru.run_trace(folder, dtype, tb, out, max_tokens=tb.peak)
    ru.compare(folder, tb, out, names, *TOL[dtype])


SERVED = {
    # two layers of the Llama 3.2 1B shape with its whole vocabulary (8,016 groups of 16 columns
    # in the head), tied
    "1b": lambda: dict(kvforge_amd.preset_dict("llama-1b"), num_hidden_layers=2,
                       max_position_embeddings=2048),
    # two layers of the Llama 3.1 8B layer shape: width 4096, head size 128, 14336 wide
    # feed-forward, untied head over a vocabulary that ends inside a group of 16 columns
    "8b": lambda: dict(kvforge_amd.preset_dict("llama-8b"), num_hidden_layers=2, vocab_size=32003,
                       max_position_embeddings=2048),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", list(SERVED))
def test_replay_at_the_served_width(tmp_path, shape, dtype):
    """The bf16 engine changes kernels by size: the norm folded into the projection up to 16
    rows, the weight-streaming kernel up to 32 (64 where its epilogue replaces a kernel), the
    library's product beyond, two column groups per wave for wide weights, the down projection
    in two halves of K.  Here the layers have the widths that are served, and steps of exactly
    16, 17, 32, 33, 64 and 65 tokens stand on both sides of every threshold; all four ways of
    cutting requests, against the plain model (some places of each step, the vocabulary being
    large)."""
    cfg = SERVED[shape]()
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, cfg, seed=12, dtype=dtype)
    # At these widths q.k already spreads over a few units (its spread grows with the width);
    # 1.5 makes the scores' spread about 2 (1B shape) and 4 (8B shape): peaked enough for one
    # wrong key to show, without multiplying the rounding of q and k into the logits.
    ru.sharpen(folder, 1.5)
    prompts = ru.random_prompts(cfg["vocab_size"], [240, 80, 100, 60], 13)
    a, b, c, d = (prompts[f"p{i}"] for i in range(4))
    tb = ru.TraceBuilder()
    names = {}
    # whole
    names["a#w"], names["b#w"] = a, b
    tb.step([("a#w", a, [0, 15, 16, 100, 239])], end=["a#w"])
    tb.step([("b#w", b, [0, 40, 79])], end=["b#w"])
    # most in one step, the last 32 one by one
    names["c#d"] = c
    ru.decode_tail(tb, "c#d", c)
    tb.steps[-33]["entries"][0]["want"] = [0, 33, 67]
    tb.expect[-33] = [("c#d", 0), ("c#d", 33), ("c#d", 67)]
    # portions on both sides of every threshold, then single tokens
    names["a#p"] = a
    pos = 0
    for n in (16, 17, 32, 33, 64, 65):
        tb.step([("a#p", a[pos:pos + n], [0, n // 2, n - 1])])
        pos += n
    for i in range(pos, len(a)):
        tb.step([("a#p", [a[i]], [0])], end=["a#p"] if i == len(a) - 1 else [])
    # mixed, pages used again
    mixed_prompts = {"b#m": b, "c#m": c, "d#m": d, "a#m": a[:120]}
    names.update(mixed_prompts)
    ru.mixed(tb, mixed_prompts, 5, max_want=3)
    out = str(tmp_path / "out")
    ru.run_trace(folder, dtype, tb, out)
    ru.compare(folder, tb, out, names, *TOL[dtype], measured_rounding=True if dtype == "float32" else dtype)


def test_replay_first_tokens_and_one_token_requests(tmp_path):
    """The first tokens of a sequence: a request of one token, of two, a first step of one token
    followed by a portion, and position 0 decoded alone."""
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, kvforge_amd.preset_dict("tiny-b"), seed=1, dtype="float32")
    ru.sharpen(folder, 6.0)
    prompts = ru.random_prompts(384, [1, 2, 20, 17], 5)
    tb = ru.TraceBuilder()
    tb.step([("p0", prompts["p0"], [0])], end=["p0"])
    tb.step([("p1", prompts["p1"], [0, 1])], end=["p1"])
    tb.step([("p2", prompts["p2"][:1], [0]), ("p3", prompts["p3"][:2], [0, 1])])
    tb.step([("p2", prompts["p2"][1:9], list(range(8))), ("p3", prompts["p3"][2:3], [0])])
    tb.step([("p2", prompts["p2"][9:], list(range(11))), ("p3", prompts["p3"][3:], list(range(14)))],
            end=["p2", "p3"])
    for dtype in ("float32", "bfloat16"):
        out = str(tmp_path / dtype)
        stored = ru.stored_as(folder, dtype)
        ru.run_trace(stored, dtype, tb, out)
        ru.compare(stored, tb, out, prompts, *TOL[dtype])


def test_replay_decoding_with_split_key_range(tmp_path):
    """One request decoded past 1,200 tokens: few sequences over a long context make the decode
    kernel cut the key range into several runs that are merged afterwards."""
    cfg = dict(ru.TINY_C, max_position_embeddings=2048)
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, cfg, seed=5, dtype="float32")
    ru.sharpen(folder, 6.0)
    prompts = ru.random_prompts(200, [1240], 11)
    tb = ru.TraceBuilder()
    tb.step([("p0", prompts["p0"][:700], [699])])
    tb.step([("p0", prompts["p0"][700:1200], [499])])
    for i in range(40):
        tb.step([("p0", [prompts["p0"][1200 + i]], [0])], end=["p0"] if i == 39 else [])
    for dtype in ("float32", "bfloat16"):
        out = str(tmp_path / dtype)
        stored = ru.stored_as(folder, dtype)
        ru.run_trace(stored, dtype, tb, out)
        ru.compare(stored, tb, out, prompts, *TOL[dtype])


def test_replay_long_decoding(tmp_path):
    """Two requests decoded token by token for 300 steps past a short prompt, across many
    pages."""
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, ru.TINY_C, seed=3, dtype="float32")
    ru.sharpen(folder, 6.0)
    prompts = ru.random_prompts(200, [330, 318], 7)
    tb = ru.TraceBuilder()
    tb.step([("p0", prompts["p0"][:30], [29]), ("p1", prompts["p1"][:18], [17])])
    for i in range(300):
        tb.step([("p0", [prompts["p0"][30 + i]], [0]), ("p1", [prompts["p1"][18 + i]], [0])],
                end=["p0", "p1"] if i == 299 else [])
    for dtype in ("float32", "bfloat16"):
        out = str(tmp_path / dtype)
        stored = ru.stored_as(folder, dtype)
        ru.run_trace(stored, dtype, tb, out)
        ru.compare(stored, tb, out, prompts, *TOL[dtype])


LONG = {  # small layers around attention heads of the size long contexts are served with
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 200,
    "hidden_size": 64, "num_hidden_layers": 2, "num_attention_heads": 2, "num_key_value_heads": 1,
    "head_dim": 128, "intermediate_size": 96, "max_position_embeddings": 40960,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
    "rms_norm_eps": 1e-5, "hidden_act": "silu", "tie_word_embeddings": False,
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_a_prompt_of_32k_tokens_in_portions_then_token_by_token(tmp_path, dtype):
    """A prompt of 32,768 tokens is fed in sixteen portions of 2,048 and then goes on for 16
    tokens one by one, a short request beside it for the second half (so the single-token steps
    hold a context of 32k beside one of a few dozen): page numbers past 2,000 per request, query
    runs at the end of tens of thousands of keys, the key range of one token in many cuts.
    Attention is peaked (q and k scaled), so that keys far back carry weight.  All logits of
    the last portion and of the single tokens, and some of every other portion, against the
    plain model computed a block of queries at a time; the tolerance is measured as for the
    served widths, since a softmax over 32k terms rounds differently in any two orders."""
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, dict(LONG), seed=15, dtype=dtype)
    ru.sharpen(folder, 6.0)
    prompts = ru.random_prompts(200, [32768 + 16, 56], 17)
    big, small = prompts["p0"], prompts["p1"]
    tb = ru.TraceBuilder()
    for i in range(16):
        lo = i * 2048
        want = list(range(2048)) if i == 15 else [0, 1000, 2047]
        entries = [("p0", big[lo:lo + 2048], want)]
        if i == 8:
            entries.append(("p1", small[:40], [0, 39]))
        tb.step(entries)
    for i in range(16):
        tb.step([("p1", [small[40 + i]], [0]), ("p0", [big[32768 + i]], [0])],
                end=["p0", "p1"] if i == 15 else [])
    out = str(tmp_path / "out")
    ru.run_trace(folder, dtype, tb, out)
    ru.compare(folder, tb, out, prompts, *TOL[dtype], measured_rounding=True if dtype == "float32" else dtype,
               query_block=512)
