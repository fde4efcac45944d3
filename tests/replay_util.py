"""Builds replay traces (the JSON steps ``bin/trace_run`` reads) and checks its output files
against the plain model.  Four families, as a user of the engine would cut the same requests:
whole; most in one step then the last 32 one by one; portions of changing size down to two
tokens; and mixed, up to four live requests with so few pages that they are used again."""

from __future__ import annotations

import json
import os
import random
import subprocess
import sys

import numpy as np
import torch

from tests.plain import llama as plain

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

TINY_C = {  # differs from tiny-a and tiny-b in every size; two kinds of attention layer
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 200,
    "hidden_size": 80, "num_hidden_layers": 4, "num_attention_heads": 6, "num_key_value_heads": 2,
    "head_dim": 48, "intermediate_size": 112, "max_position_embeddings": 512,
    "rope_theta": 1000.0, "rope_scaling": None, "rms_norm_eps": 1e-4, "hidden_act": "silu",
    "tie_word_embeddings": False, "sliding_window": 24,
    "layer_types": ["full_attention", "sliding_attention", "sliding_attention", "full_attention"],
}


WIDE = {  # layers wide enough for the kernels that serving a real model takes: head size 64 on
    # the matrix cores, a down projection deep and narrow enough to be cut in two halves of K (one
    # of them stays owed to the stream until the next layer's projections), gate/up wide enough
    # for two groups of columns per wave, a vocabulary that ends inside a group of 16 columns
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 1000,
    "hidden_size": 256, "num_hidden_layers": 3, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 64, "intermediate_size": 4096, "max_position_embeddings": 512,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 128},
    "rms_norm_eps": 1e-5, "hidden_act": "silu", "tie_word_embeddings": True,
}


# the same with head size 128, one kv head, a width that is not heads x head size, untied head
WIDE_B = dict(WIDE, vocab_size=777, hidden_size=192, num_hidden_layers=2, num_attention_heads=2,
              num_key_value_heads=1, head_dim=128, intermediate_size=4608, rms_norm_eps=1e-6,
              tie_word_embeddings=False)


def sharpen(folder: str, factor: float) -> None:
    """Scale every q and k projection so that attention is peaked: with N(0, 0.02) weights the
    scores are nearly flat and one misplaced key would hide among hundreds."""
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    for k in list(w):
        if k.endswith("q_proj.weight") or k.endswith("k_proj.weight"):
            w[k] = (w[k].float() * factor).to(w[k].dtype)
    save_file(w, path, metadata={"format": "pt"})


def round64(n: int) -> int:
    return -(-n // 64) * 64


class TraceBuilder:
    def __init__(self) -> None:
        self.steps: list[dict] = []
        self.expect: list[list[tuple[str, int]]] = []   # per step: (request, position) per row
        self.held: dict[str, int] = {}
        self.peak = 0

    def step(self, entries: list[tuple[str, list[int], list[int]]], end: list[str] = ()) -> None:
        rec = {"step": len(self.steps), "entries": [], "end": list(end)}
        rows = []
        for rid, toks, want in entries:
            start = self.held.get(rid, 0)
            rec["entries"].append({"id": rid, "tokens": toks, "want": want})
            rows += [(rid, start + i) for i in want]
            self.held[rid] = start + len(toks)
        self.peak = max(self.peak, sum(round64(v) for v in self.held.values()))
        for rid in end:
            self.held.pop(rid, None)
        self.steps.append(rec)
        self.expect.append(rows)


def whole(tb: TraceBuilder, rid: str, toks: list[int]) -> None:
    tb.step([(rid, toks, list(range(len(toks))))], end=[rid])


def decode_tail(tb: TraceBuilder, rid: str, toks: list[int], tail: int = 32) -> None:
    head = len(toks) - tail
    tb.step([(rid, toks[:head], list(range(head)))])
    for i in range(head, len(toks)):
        tb.step([(rid, [toks[i]], [0])], end=[rid] if i == len(toks) - 1 else [])


def portions(tb: TraceBuilder, rid: str, toks: list[int], sizes=(7, 2, 5, 3, 2, 11, 2, 16, 4, 2, 9)) -> None:
    p, k = 0, 0
    while p < len(toks):
        n = sizes[k % len(sizes)]
        k += 1
        if len(toks) - p - n == 1:      # never leave a single token for a "portion"
            n += 1
        n = min(n, len(toks) - p)
        last = p + n == len(toks)
        tb.step([(rid, toks[p:p + n], list(range(n)))], end=[rid] if last else [])
        p += n


def mixed(tb: TraceBuilder, prompts: dict[str, list[int]], seed: int, live_max: int = 4,
          decode_tail_len: int = 12) -> None:
    """Up to ``live_max`` requests live: portions of some beside single tokens of others; a
    request is sometimes left out of a step; new ones join as others end."""
    rng = random.Random(seed)
    waiting = list(prompts)
    live: dict[str, int] = {}
    while waiting or live:
        while waiting and len(live) < live_max and (not live or rng.random() < 0.6):
            live[waiting.pop(0)] = 0
        entries, ending = [], []
        for rid in list(live):
            if len(live) > 1 and rng.random() < 0.2:
                continue                                     # left out of this step
            toks, p = prompts[rid], live[rid]
            if p >= len(toks) - decode_tail_len:
                n = 1
            else:
                n = min(rng.randint(2, 13), len(toks) - decode_tail_len - p)
                if n == 1:
                    n = 2 if p + 2 <= len(toks) else 1
            want = list(range(n)) if rng.random() < 0.7 else ([n - 1] if rng.random() < 0.7 else [])
            entries.append((rid, toks[p:p + n], want))
            live[rid] = p + n
            if live[rid] == len(toks):
                ending.append(rid)
        if entries:
            tb.step(entries, end=ending)
            for rid in ending:
                del live[rid]


def run_trace(folder: str, dtype: str, tb: TraceBuilder, out_dir: str, max_tokens: int | None = None,
              env: dict | None = None, user_args: list[str] | None = None) -> None:
    os.makedirs(out_dir, exist_ok=True)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens or tb.peak)]
    text = "\n".join(json.dumps(s) for s in tb.steps) + "\n"
    p = subprocess.run(cmd, input=text, text=True, capture_output=True, timeout=600, env=env)
    assert p.returncode == 0, f"trace_run failed ({p.returncode}):\n{p.stderr[-4000:]}"
    done = [ln for ln in p.stdout.splitlines() if ln.startswith("done ")]
    assert done == [f"done {i}" for i in range(len(tb.steps))], p.stdout[-2000:]


def compare(folder: str, tb: TraceBuilder, out_dir: str, prompts: dict[str, list[int]], atol: float,
            rtol: float) -> float:
    """Every row trace_run wrote against the plain model's logits at that request's position.
    Reports the first wrong place by step, request and position."""
    w = {k: v for k, v in __import__("kvforge_amd").read_safetensors_folder(folder).items()}
    cfg = plain.read_config(folder)
    V = cfg["vocab_size"]
    want = {rid: plain.forward(w, cfg, toks) for rid, toks in prompts.items()}
    worst = 0.0
    for sid, rows in enumerate(tb.expect):
        path = os.path.join(out_dir, f"{sid}.f32")
        if not rows:
            assert not os.path.exists(path), f"step {sid} wanted nothing but wrote a file"
            continue
        got = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(-1, V).copy())
        assert got.shape[0] == len(rows), f"step {sid}: {got.shape[0]} rows, {len(rows)} wanted"
        for r, (rid, pos) in enumerate(rows):
            ref = want[rid.split("#")[0] if rid not in want else rid][pos]
            err = (got[r] - ref).abs()
            bound = atol + rtol * ref.abs()
            worst = max(worst, float(err.max()))
            if not bool((err <= bound).all()):
                j = int((err - bound).argmax())
                raise AssertionError(
                    f"step {sid}, request {rid}, position {pos}: logit {j} is {got[r, j]:.6f}, "
                    f"plain model gives {ref[j]:.6f} (|diff| {err[j]:.3e} > {bound[j]:.3e}); "
                    f"page offset {pos % 16}, page {pos // 16}")
    return worst


def random_prompts(vocab: int, lengths: list[int], seed: int) -> dict[str, list[int]]:
    g = torch.Generator().manual_seed(seed)
    return {f"p{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}
