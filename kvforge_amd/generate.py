"""Command line: generate from a model folder or a random-weight preset.

    python -m kvforge_amd.generate --preset tiny-a --prompt-ids 5,17,3 --max-tokens 16 --temperature 0
    python -m kvforge_amd.generate --model DIR --prompt "hello" --dtype bfloat16

Engine options carry the names of the reference's launcher (scripts/serve.py:43-60: --preset,
--device, --dtype, --block-size, --num-blocks, --kv-cache-gb, --max-num-seqs,
--max-num-batched-tokens, --max-model-len) and of its benchmark (benchmarks/run_bench.py:327-353:
--seed); ``--model`` stands where the reference has ``--hf-model``.
"""

from __future__ import annotations

import argparse
import json
import sys


def parse_args(argv: list[str] | None = None) -> argparse.Namespace:
    from kvforge_amd.config.presets import PRESETS

    p = argparse.ArgumentParser(prog="kvforge_amd.generate", description=__doc__,
                                formatter_class=argparse.RawDescriptionHelpFormatter)
    src = p.add_mutually_exclusive_group()
    src.add_argument("--preset", choices=sorted(PRESETS), default=None,
                     help="random weights of a named shape")
    src.add_argument("--model", "--hf-model", dest="model", default=None,
                     help="folder with config.json and model.safetensors")
    what = p.add_mutually_exclusive_group()
    what.add_argument("--prompt-ids", action="append", default=None,
                      help="comma-separated token ids; repeat for several prompts")
    what.add_argument("--prompt-file", default=None, help="one prompt of token ids per line")
    what.add_argument("--prompt", action="append", default=None,
                      help="text, tokenised by the model folder's tokenizer.json if it has one, "
                           "else byte by byte (needs vocab_size >= 258)")
    p.add_argument("--max-tokens", type=int, default=64)
    p.add_argument("--temperature", type=float, default=0.0)
    p.add_argument("--top-k", type=int, default=0)
    p.add_argument("--top-p", type=float, default=1.0)
    p.add_argument("--ignore-eos", action="store_true")
    p.add_argument("--stop-token-ids", default="", help="comma-separated token ids")
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--device", default="cuda")
    p.add_argument("--dtype", choices=["float32", "bfloat16"], default="float32")
    p.add_argument("--block-size", type=int, default=16)
    p.add_argument("--num-blocks", type=int, default=None)
    p.add_argument("--kv-cache-gb", type=float, default=0.25)
    p.add_argument("--max-num-seqs", type=int, default=32)
    p.add_argument("--max-num-batched-tokens", type=int, default=2048)
    p.add_argument("--max-model-len", type=int, default=2048)
    p.add_argument("--no-graphs", action="store_true", help="do not replay decode steps from HIP graphs")
    p.add_argument("--decode-run-steps", type=int, default=8,
                   help="decode steps the device takes between two looks of the host")
    p.add_argument("--no-decode-run-ahead", action="store_true",
                   help="do not queue the next run of decode steps before the current one is read")
    p.add_argument("--json", action="store_true", help="print one JSON object instead of text")
    return p.parse_args(argv)


def _ids(text: str) -> list[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def main(argv: list[str] | None = None) -> int:
    args = parse_args(argv)
    from kvforge_amd.config.engine import CacheConfig, EngineConfig, SchedulerConfig
    from kvforge_amd.engine.engine import InferenceEngine
    from kvforge_amd.sampling.params import SamplingParams
    from kvforge_amd.tokenizer import tokenizer_for

    tokenizer = tokenizer_for(args.model) if args.prompt else None
    if args.prompt:
        prompts: list = list(args.prompt)
    elif args.prompt_file:
        with open(args.prompt_file) as f:
            prompts = [_ids(line) for line in f if line.strip()]
    else:
        prompts = [_ids(t) for t in (args.prompt_ids or ["1,2,3"])]
    config = EngineConfig(
        cache=CacheConfig(block_size=args.block_size, num_blocks=args.num_blocks,
                          kv_cache_memory_gb=None if args.num_blocks else args.kv_cache_gb),
        scheduler=SchedulerConfig(max_num_seqs=args.max_num_seqs,
                                  max_num_batched_tokens=args.max_num_batched_tokens,
                                  max_model_len=args.max_model_len),
        device=args.device, dtype=args.dtype, seed=args.seed, use_graphs=not args.no_graphs,
        decode_run_steps=args.decode_run_steps, decode_run_ahead=not args.no_decode_run_ahead)
    if args.model:
        engine = InferenceEngine.from_folder(args.model, config, tokenizer)
        name = args.model
    else:
        preset = args.preset or "tiny-a"
        engine = InferenceEngine.from_config(preset, config, tokenizer)
        name = f"{preset}-random(seed={args.seed})"
    params = SamplingParams(max_tokens=args.max_tokens, temperature=args.temperature,
                            top_k=args.top_k, top_p=args.top_p, ignore_eos=args.ignore_eos,
                            stop_token_ids=_ids(args.stop_token_ids))
    outs = engine.generate(prompts, params)
    stats = engine.stats()
    if args.json:
        print(json.dumps({"model": name, "outputs": [
            {"request_id": o.request_id, "prompt_token_ids": o.prompt_token_ids,
             "output_token_ids": o.output_token_ids, "finish_reason": o.finish_reason.value,
             "text": o.text} for o in outs], "stats": stats}))
        return 0
    kv = stats["kv_cache"]
    print(f"kvforge_amd: model={name} blocks={kv['num_blocks']}x{kv['block_size']} "
          f"kv={kv['bytes_total'] / 2**20:.1f} MiB dtype={args.dtype}")
    for o in outs:
        print(f"{o.request_id} [{o.finish_reason.value}] prompt={len(o.prompt_token_ids)} tokens -> "
              f"{o.output_token_ids}")
        if o.text is not None:
            print(f"  text: {o.text!r}")
    m = stats["metrics"]
    print(f"steps={int(m['num_steps'])} output_tokens_per_s={m['output_tokens_per_s']:.1f} "
          f"ttft_p50_ms={m['ttft_p50_ms']:.2f} tpot_p50_ms={m['tpot_p50_ms']:.2f} "
          f"preemptions={stats['scheduler']['num_preemptions']}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
