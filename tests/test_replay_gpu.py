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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("sharp", [0.0, 6.0])
def test_replay_all_modes(tmp_path, name, dtype, sharp):
    make, seed, lengths = CONFIGS[name]
    if sharp == 0.0 and name == "tiny-c":
        pytest.skip("the flat-weights run covers the two given configurations")
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, make(), seed=seed)
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["WIDE", "WIDE_B"])
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
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, cfg, seed=4)
    prompts = ru.random_prompts(cfg["vocab_size"], [41, 75, 52, 66], 9)
    tb, names = build_all_modes(prompts, 9)
    out = str(tmp_path / "out")
    ru.run_trace(folder, dtype, tb, out)
    ru.compare(folder, tb, out, names, *TOL[dtype])


def test_replay_first_tokens_and_one_token_requests(tmp_path):
    """The first tokens of a sequence: a request of one token, of two, a first step of one token
    followed by a portion, and position 0 decoded alone."""
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, kvforge_amd.preset_dict("tiny-b"), seed=1)
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
        ru.run_trace(folder, dtype, tb, out)
        ru.compare(folder, tb, out, prompts, *TOL[dtype])


def test_replay_decoding_with_split_key_range(tmp_path):
    """One request decoded past 1,200 tokens: few sequences over a long context make the decode
    kernel cut the key range into several runs that are merged afterwards."""
    cfg = dict(ru.TINY_C, max_position_embeddings=2048)
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, cfg, seed=5)
    ru.sharpen(folder, 6.0)
    prompts = ru.random_prompts(200, [1240], 11)
    tb = ru.TraceBuilder()
    tb.step([("p0", prompts["p0"][:700], [699])])
    tb.step([("p0", prompts["p0"][700:1200], [499])])
    for i in range(40):
        tb.step([("p0", [prompts["p0"][1200 + i]], [0])], end=["p0"] if i == 39 else [])
    for dtype in ("float32", "bfloat16"):
        out = str(tmp_path / dtype)
        ru.run_trace(folder, dtype, tb, out)
        ru.compare(folder, tb, out, prompts, *TOL[dtype])


def test_replay_long_decoding(tmp_path):
    """Two requests decoded token by token for 300 steps past a short prompt, across many
    pages."""
    folder = str(tmp_path / "model")
    kvforge_amd.write_random_model(folder, ru.TINY_C, seed=3)
    ru.sharpen(folder, 6.0)
    prompts = ru.random_prompts(200, [330, 318], 7)
    tb = ru.TraceBuilder()
    tb.step([("p0", prompts["p0"][:30], [29]), ("p1", prompts["p1"][:18], [17])])
    for i in range(300):
        tb.step([("p0", [prompts["p0"][30 + i]], [0]), ("p1", [prompts["p1"][18 + i]], [0])],
                end=["p0", "p1"] if i == 299 else [])
    for dtype in ("float32", "bfloat16"):
        out = str(tmp_path / dtype)
        ru.run_trace(folder, dtype, tb, out)
        ru.compare(folder, tb, out, prompts, *TOL[dtype])
