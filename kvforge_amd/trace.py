"""Trace replay: feeds given token ids through a model step by step and writes logits.

It samples nothing and owns no forward pass, cache or loader: it builds the same
``Transformer``, ``ModelRunner`` (step function, cache manager, pages) and kernels that
generation uses.  Steps arrive on standard input, one JSON object a line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step with wanted places the logits ``[wanted, vocab]`` are written as little-endian
float32 to ``<out>/<step>.f32``; after every step ``done <step>`` is printed and flushed.
"""

from __future__ import annotations

import argparse
import json
import os
import sys



def pool_pages(max_tokens: int, block_size: int) -> int:
    """Pages for ``max_tokens`` tokens of live requests, each request's count rounded up to a
    multiple of 64 by the caller: a unit of 64 tokens takes ``ceil(64 / block_size)`` pages (a
    request's pages are its own, so a page size that does not divide 64 rounds every unit up);
    pages larger than 64 tokens round the total up to their own size."""
    if block_size >= 64:
        return max(1, -(-max_tokens // block_size))
    units = max(1, -(-max_tokens // 64))
    return units * -(-64 // block_size)


def _say(msg: str) -> None:
    print(f"[trace_run] {msg}", file=sys.stderr, flush=True)


def main(argv: list[str] | None = None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--out", required=True, help="folder the logits files are written to")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--max-live", type=int, default=16, help="most requests live at a time")
    args = ap.parse_args(argv)
    if args.block_size < 1 or args.max_live < 1 or args.max_tokens < 1:
        ap.error("--block-size, --max-live and --max-tokens must be positive")

    _say("loading torch ...")
    import numpy as np
    import torch

    from kvforge_amd.config.engine import parse_dtype
    from kvforge_amd.engine.batch import StepEntry
    from kvforge_amd.engine.runner import ModelRunner
    from kvforge_amd.models.transformer import Transformer

    if not torch.cuda.is_available():
        _say("error: no GPU is visible; the engine has no CPU path")
        return 2
    os.makedirs(args.out, exist_ok=True)
    dtype = parse_dtype(args.dtype)
    _say(f"loading model from {args.model} as {args.dtype}")
    model = Transformer.from_folder(args.model, dtype, "cuda")
    block_size = args.block_size
    num_blocks = pool_pages(args.max_tokens, block_size)
    capacity = num_blocks * block_size
    runner = ModelRunner(model, block_size, num_blocks, max_num_seqs=args.max_live,
                         max_num_batched_tokens=capacity, max_model_len=capacity)
    _say(f"ready: {num_blocks} pages of {block_size} tokens per cache group")
    held: dict[str, int] = {}
    cache = runner.cache
    while True:
        line = sys.stdin.readline()
        if not line:
            break
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        sid = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            rid, toks = str(e["id"]), [int(t) for t in e["tokens"]]
            if not toks:
                raise ValueError(f"step {sid}: request {rid} brings no tokens")
            start = held.get(rid, 0)
            if rid not in held:
                cache.allocate(rid, 0)
            cache.append_slots(rid, start + len(toks), start)
            entries.append(StepEntry(rid, toks, start, list(e.get("want", []))))
        if entries:
            logits = runner.step(entries)
            for e in entries:
                held[e.request_id] = e.start_pos + len(e.token_ids)
                cache.release_behind(e.request_id, held[e.request_id])
            if logits.shape[0] > 0:
                arr = logits.detach().to("cpu", torch.float32).numpy().astype("<f4", copy=False)
                tmp = os.path.join(args.out, f".{sid}.f32.tmp")
                np.ascontiguousarray(arr).tofile(tmp)
                os.replace(tmp, os.path.join(args.out, f"{sid}.f32"))
            else:
                torch.cuda.synchronize()
        for rid in rec.get("end", []):
            rid = str(rid)
            cache.free(rid)
            held.pop(rid, None)
        print(f"done {sid}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
