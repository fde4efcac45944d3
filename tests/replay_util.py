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


# more heads than the width divides into: the output projection is as deep (32 heads x 128 = 4096)
# and as narrow as the down projection, so both are cut in two halves of K and the half that
# the one leaves owed is still owed when the other writes its own
WIDE_C = dict(WIDE, vocab_size=500, hidden_size=256, num_hidden_layers=2, num_attention_heads=32,
              num_key_value_heads=4, head_dim=128, intermediate_size=4096)


_STORED: dict[tuple[str, str], str] = {}


def stored_as(folder: str, dtype: str) -> str:
    """The folder's model with its floating tensors stored as ``dtype`` ("float32" or
    "bfloat16"): the folder itself if it stores them so, else a copy beside it, made once by
    conversion.  A float32 engine is to be given weights that bfloat16 cannot hold, a bfloat16
    engine weights stored in bfloat16 (one stored in 32-bit would stay 32-bit there)."""
    import shutil
    from safetensors.torch import save_file
    want = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    key = (os.path.abspath(folder), dtype)
    if key not in _STORED:
        w = plain.read_weights(folder)
        if all(t.dtype == want for t in w.values() if t.is_floating_point()):
            _STORED[key] = folder
        else:
            twin = f"{folder.rstrip(os.sep)}.{dtype}"
            os.makedirs(twin, exist_ok=True)
            for name in os.listdir(folder):
                if not name.endswith(".safetensors") and not name.endswith(".index.json"):
                    shutil.copy(os.path.join(folder, name), os.path.join(twin, name))
            save_file({k: (t.to(want) if t.is_floating_point() else t).contiguous() for k, t in w.items()},
                      os.path.join(twin, "model.safetensors"), metadata={"format": "pt"})
            _STORED[key] = twin
    return _STORED[key]


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


def liven(folder: str, qk: float = 6.0, out: float = 8.0) -> None:
    """Make a random model's next token depend on its context.  With N(0, 0.02) weights (and
    tied embeddings above all) what the layers add to the residual stream is small beside the
    last token's own embedding, so greedy decoding repeats the last token whatever the cache
    holds, and a test of generated tokens could not see a broken cache.  Peaked attention
    (q and k times ``qk``) and layer outputs that outweigh the embedding (v, o and down
    projections times ``out``) change that; ``context_matters`` checks it."""
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    w = load_file(path)
    for k in list(w):
        name = k.rsplit(".", 2)[-2]
        if name in ("q_proj", "k_proj"):
            w[k] = (w[k].float() * qk).to(w[k].dtype)
        elif name in ("v_proj", "o_proj", "down_proj"):
            w[k] = (w[k].float() * out).to(w[k].dtype)
    save_file(w, path, metadata={"format": "pt"})


def context_matters(folder: str, prompts: list[list[int]], n: int = 6) -> bool:
    """Whether the plain model's greedy continuation of every prompt differs from the
    continuation of the prompt's last token alone."""
    w = plain.read_weights(folder)
    cfg = plain.read_config(folder)
    return all(plain.greedy(w, cfg, p, n) != plain.greedy(w, cfg, p[-1:], n) for p in prompts if len(p) > 1)


def round64(n: int) -> int:
    return -(-n // 64) * 64


class TraceBuilder:
    def __init__(self) -> None:
        self.steps: list[dict] = []
        self.expect: list[list[tuple[str, int]]] = []   # per step: (request, position) per row
        self.held: dict[str, int] = {}
        self.peak = 0

    def step(self, entries: list[tuple], end: list[str] = ()) -> None:
        """``entries``: (id, tokens, wanted places) or (id, tokens, wanted places, key), where
        ``key`` names the sequence the rows are compared with when an id is used a second time
        for other tokens."""
        rec = {"step": len(self.steps), "entries": [], "end": list(end)}
        rows = []
        for rid, toks, want, *key in entries:
            start = self.held.get(rid, 0)
            rec["entries"].append({"id": rid, "tokens": toks, "want": want})
            rows += [(key[0] if key else rid, start + i) for i in want]
            self.held[rid] = start + len(toks)
        self.peak = max(self.peak, sum(round64(v) for v in self.held.values()))
        for rid in end:
            self.held.pop(rid, None)
        self.steps.append(rec)
        self.expect.append(rows)


def whole(tb: TraceBuilder, rid: str, toks: list[int]) -> None:
    tb.step([(rid, toks, list(range(len(toks))))], end=[rid])


def decode_tail(tb: TraceBuilder, rid: str, toks: list[int], tail: int = 32) -> None:
    head = max(1, len(toks) - tail)        # short requests: the first token, then one by one
    tb.step([(rid, toks[:head], list(range(head)))], end=[rid] if head == len(toks) else [])
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
          decode_tail_len: int = 12, max_want: int | None = None) -> None:
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
            if max_want is not None and len(want) > max_want:
                want = sorted(rng.sample(want[:-1], max_want - 1)) + [want[-1]]
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
           "--out", out_dir, "--max-tokens", str(max_tokens or tb.peak), *(user_args or [])]
    text = "\n".join(json.dumps(s) for s in tb.steps) + "\n"
    p = subprocess.run(cmd, input=text, text=True, capture_output=True, timeout=600, env=env)
    assert p.returncode == 0, f"trace_run failed ({p.returncode}):\n{p.stderr[-4000:]}"
    done = [ln for ln in p.stdout.splitlines() if ln.startswith("done ")]
    assert done == [f"done {i}" for i in range(len(tb.steps))], p.stdout[-2000:]


def compare(folder: str, tb: TraceBuilder, out_dir: str, prompts: dict[str, list[int]], atol: float,
            rtol: float, measured_rounding: "bool | str" = False, query_block: int | None = None) -> float:
    """Every row trace_run wrote against the plain model's logits at that request's position.
    Reports the first wrong place by step, request and position.

    ``measured_rounding`` (for 32-bit runs of wide layers): sums over thousands of terms round
    differently in any two 32-bit implementations, and at widths of 2,048 and more that alone
    exceeds the tolerance the tiny models are held to.  The rows are then compared with the
    plain model computed in float64, and the absolute tolerance is no smaller than five times
    what the plain model's own 32-bit run differs from that by, measured per request (its
    library sums a long dot product in blocks, the engine's 32-bit kernel one term after the
    other, which rounds a few times more; a wrong index or a lost term shows at 1e-3 and up).

    ``measured_rounding="bfloat16"`` (for bfloat16 runs of wide layers, where peaked attention
    multiplies what rounding q and k to 8 bits does, and the largest of millions of errors is
    compared): the plain model is also run with the least rounding a bfloat16 engine can do
    (``plain.forward(dtype=bfloat16, residual_in_fp32=True)``: only the tensors between
    operations are rounded), and a row's absolute tolerance is no smaller than three times the
    largest difference that run shows from the 32-bit one in the same row.  A wrong key or page
    moves a row by about the logits' spread, many times that.

    ``query_block``: the plain model attends so many queries at a time (for sequences whose
    scores would not fit in memory all at once)."""
    w = {k: v for k, v in plain.read_weights(folder).items()}
    cfg = plain.read_config(folder)
    V = cfg["vocab_size"]
    by_tokens: dict[tuple, torch.Tensor] = {}
    want = {}
    for rid, toks in prompts.items():
        key = tuple(toks)
        if key not in by_tokens:
            ref = plain.forward(w, cfg, toks, query_block=query_block)
            floor = 0.0
            if measured_rounding == "bfloat16":
                least = plain.forward(w, cfg, toks, dtype=torch.bfloat16, residual_in_fp32=True,
                                      query_block=query_block)
                floor = 3.0 * (least - ref).abs().max(dim=1).values          # per row
            elif measured_rounding:
                exact = plain.forward(w, cfg, toks, dtype=torch.float64, query_block=query_block)
                floor = 5.0 * float((ref.double() - exact).abs().max())
                ref = exact.float()
            by_tokens[key] = (ref, floor)
        want[rid] = by_tokens[key]
    worst = 0.0
    for sid, rows in enumerate(tb.expect):
        path = os.path.join(out_dir, f"{sid}.f32")
        if not rows:
            assert not os.path.exists(path), f"step {sid} wanted nothing but wrote a file"
            continue
        got = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(-1, V).copy())
        assert got.shape[0] == len(rows), f"step {sid}: {got.shape[0]} rows, {len(rows)} wanted"
        for r, (rid, pos) in enumerate(rows):
            ref, floor = want[rid.split("#")[0] if rid not in want else rid]
            if torch.is_tensor(floor):
                floor = float(floor[pos])
            ref = ref[pos]
            err = (got[r] - ref).abs()
            bound = max(atol, floor) + rtol * ref.abs()
            worst = max(worst, float(err.max()))
            if not bool((err <= bound).all()):
                j = int((err - bound).argmax())
                raise AssertionError(
                    f"step {sid}, request {rid}, position {pos}: logit {j} is {got[r, j]:.6f}, "
                    f"plain model gives {ref[j]:.6f} (|diff| {err[j]:.3e} > {bound[j]:.3e}); "
                    f"offset {pos % 16} in a page of 16, {pos % 8} in a page of 8")
    return worst


def random_prompts(vocab: int, lengths: list[int], seed: int) -> dict[str, list[int]]:
    g = torch.Generator().manual_seed(seed)
    return {f"p{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}
