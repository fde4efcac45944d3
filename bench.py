"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--prompt-len 512]
                    [--dtype bfloat16] [--layers L] [--no-points] [--phase all|decode|prefill]
                    [--preset llama-1b|llama-3b|llama-8b] [--context-len 8192]
    python bench.py --phase mixed --preset llama-3b --batch 32 --steps 256
    python bench.py --phase burst --preset small [--dtype float32]

Default run: the layer sizes of Llama 3.2 1B (16 layers, hidden 2048, 32 heads, 8 kv heads, head
size 64, SwiGLU 8192, vocabulary 128256, llama3 rope scaling, tied embeddings), random weights
N(0, 0.02), batch 8, 512-token uniform-random prompts, greedy, context cap 8192, pages of 16
tokens.  A step is one decode step of the whole engine (scheduler, batch building, forward,
sampling, bookkeeping).  One JSON line is printed; besides the decode figure it carries a
2,048-token prefill, the decode step's share of the HBM roofline, and decode at batch 1 and 64.
``points`` also holds (unless ``--no-points``) the same model over contexts of 4,096 and 8,192
tokens (decode at batch 8 and 64, one prompt of 8,192 tokens), the same model in true 32-bit (decode at batch 1
and 8, prefill of 2,048 tokens, with their shares of the fp32 bounds), the mixed workload at the
Llama 3.2 3B shape (32 requests, prompts of 128 to 4,096 tokens, chunked prefill under a
2,048-token budget beside decode steps, 256 new tokens each) and long-context decoding at the
Llama 3.1 8B shape, all 32 layers (batch 16 at 32,768-token prompts, 128 new tokens; before it
decode at batch 1 and 8 over 512-token prompts); the 32-bit, 3B and 8B models draw their random
weights on the device.
Peaks are the published MI355X ones: HBM 8 TB/s; dense MFMA 2.5 PFLOP/s for bf16, 157.3 TFLOP/s
for fp32.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK = {"bfloat16": 2.5e15, "float32": 157.3e12}
CONTEXT_CAP = 8192
BLOCK_SIZE = 16
PREFILL_TOKENS = 2048
MODEL_NAMES = {"llama-1b": "Llama 3.2 1B", "llama-3b": "Llama 3.2 3B", "llama-8b": "Llama 3.1 8B"}
# The model of the reference's own serving benchmark (benchmarks/BENCHMARK_REPORT.md:28-29,
# src/tokenvault/model_loader.py:24-27): 26.1M parameters.
SMALL = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "vocab_size": 8192,
         "hidden_size": 512, "num_hidden_layers": 6, "num_attention_heads": 8, "num_key_value_heads": 4,
         "head_dim": 64, "intermediate_size": 1408, "max_position_embeddings": 2048,
         "rope_theta": 10000.0, "rope_scaling": None, "rms_norm_eps": 1e-6, "hidden_act": "silu",
         "tie_word_embeddings": False}


def build_engine(model, dtype, max_num_seqs, num_tokens_cached, use_graphs=True, run_steps=None,
                 context_cap=CONTEXT_CAP):
    """``model``: a model folder, or a config.json dictionary whose random weights are drawn on
    the device."""
    import kvforge_amd
    from kvforge_amd import CacheConfig, EngineConfig, InferenceEngine, SchedulerConfig

    num_blocks = -(-num_tokens_cached // BLOCK_SIZE) + max_num_seqs + 8
    cfg = EngineConfig(
        cache=CacheConfig(block_size=BLOCK_SIZE, num_blocks=num_blocks, watermark=0.0),
        scheduler=SchedulerConfig(max_num_seqs=max_num_seqs, max_num_batched_tokens=PREFILL_TOKENS,
                                  max_model_len=context_cap),
        dtype=dtype, use_graphs=use_graphs)
    if run_steps is not None:
        cfg.decode_run_steps = run_steps
    if isinstance(model, dict):
        return InferenceEngine.from_config(model, cfg, on_device=True)
    return InferenceEngine.from_folder(model, cfg)


def random_prompts(vocab, n, length, seed):
    import torch
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(1, vocab, (length,), generator=g).tolist() for _ in range(n)]


def early_tokens(batch, prompt_len):
    """Most tokens a request decodes before the last prompt of the batch has been read."""
    return -(-batch * prompt_len // PREFILL_TOKENS) + 1


def decode_run(engine, vocab, batch, prompt_len, steps, warmup, seed=0):
    """Prefill ``batch`` prompts, run ``warmup`` decode steps untimed, then time ``steps``."""
    import torch
    from kvforge_amd import SamplingParams

    # requests admitted first decode while the later prompts are still being read: leave them
    # room for that, so that every request lives through the timed steps
    params = SamplingParams(max_tokens=steps + warmup + early_tokens(batch, prompt_len) + 8,
                            temperature=0.0, ignore_eos=True)
    for p in random_prompts(vocab, batch, prompt_len, seed):
        engine.add_request(p, params)
    while any(not r.decoding for r in engine.scheduler.requests.values()) or engine.scheduler.num_waiting:
        engine.step()
    sched = engine.scheduler
    run_limit, run_ahead = sched.run_limit, sched.run_ahead

    def decode_steps(n):
        """Exactly ``n`` decode steps of the whole batch (the engine may take several between two
        looks of the host; the last run is cut to fit, and no run is queued ahead that these
        ``n`` steps would not read); returns the tokens produced."""
        produced, start = 0, engine.runner.num_forward_passes
        while engine.runner.num_forward_passes - start < n:
            left = n - (engine.runner.num_forward_passes - start)
            sched.run_limit = min(run_limit, left)
            sched.run_ahead = run_ahead and left >= 2 * run_limit
            produced += sum(len(o.new_token_ids) for o in engine.step())
        sched.run_limit, sched.run_ahead = run_limit, run_ahead
        assert engine.runner.num_forward_passes - start == n
        return produced

    decode_steps(warmup)
    assert len(engine.scheduler.running) == batch
    ctx_start = [r.num_tokens for r in engine.scheduler.running]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    produced = decode_steps(steps)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ctx_end = [r.num_tokens for r in engine.scheduler.running]
    assert len(ctx_end) == batch and produced == batch * steps, (len(ctx_end), produced)
    for rid in list(engine.scheduler.requests):
        engine.abort_request(rid)
    mean_ctx = (sum(ctx_start) + sum(ctx_end)) / 2.0 / max(1, batch)
    return {"tokens": produced, "seconds": dt, "tok_s": produced / dt, "ms_per_step": dt / steps * 1e3,
            "mean_ctx": mean_ctx}


def prefill_run(engine, vocab, tokens, repeats=3, seed=1):
    import torch
    from kvforge_amd import SamplingParams

    best = None
    params = SamplingParams(max_tokens=1, temperature=0.0, ignore_eos=True)
    for i in range(repeats + 1):
        prompt = random_prompts(vocab, 1, tokens, seed + i)[0]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.generate([prompt], params)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if i > 0:                      # the first run warms buffers and kernels
            best = dt if best is None else min(best, dt)
    return best


def mixed_run(engine, vocab, requests, new_tokens, seed=0):
    """``requests`` prompts of 128 to 4,096 tokens (uniform), all there at once: chunked prefill
    under the token budget mixed with the decode steps of those already running, ``new_tokens``
    each.  Returns prompt tokens, generated tokens and seconds."""
    import random
    import torch
    from kvforge_amd import SamplingParams

    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    lens = [rng.randint(128, 4096) for _ in range(requests)]
    prompts = [torch.randint(1, vocab, (n,), generator=g).tolist() for n in lens]
    params = SamplingParams(max_tokens=new_tokens, temperature=0.0, ignore_eos=True)
    engine.generate(prompts[:2], SamplingParams(max_tokens=24, temperature=0.0, ignore_eos=True))  # warm-up
    engine.metrics.reset()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    outs = engine.generate(prompts, params)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    mixed_run.last = {"lens": lens, "steps": engine.metrics.num_steps,
                      "step_tokens": list(engine.metrics.batched_tokens)}
    return sum(lens), sum(len(o.output_token_ids) for o in outs), dt


def burst_run(folder, vocab, dtype, use_graphs, seed=0):
    """The workload of the reference's serving benchmark (benchmarks/BENCHMARK_REPORT.md:30-36):
    48 requests, all there at once, prompts of 16 to 128 tokens and 8 to 128 new tokens (uniform),
    greedy, eos ignored; at most 16 sequences and 1,024 tokens in a step, 1,024 pages of 16
    tokens, chunked prefill, first come first served."""
    import random
    import torch
    from kvforge_amd import CacheConfig, EngineConfig, InferenceEngine, SamplingParams, SchedulerConfig

    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    lens = [rng.randint(16, 128) for _ in range(48)]
    news = [rng.randint(8, 128) for _ in range(48)]
    prompts = [torch.randint(1, vocab, (n,), generator=g).tolist() for n in lens]
    params = [SamplingParams(max_tokens=n, temperature=0.0, ignore_eos=True) for n in news]
    cfg = EngineConfig(cache=CacheConfig(block_size=16, num_blocks=1024),
                       scheduler=SchedulerConfig(max_num_seqs=16, max_num_batched_tokens=1024),
                       dtype=dtype, use_graphs=use_graphs)
    best = None
    engine = InferenceEngine.from_folder(folder, cfg)
    for _ in range(3):                               # the first pass compiles, captures and warms
        engine.metrics.reset()
        passes = engine.runner.num_forward_passes
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        outs = engine.generate(prompts, params)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        generated = sum(len(o.output_token_ids) for o in outs)
        assert generated == sum(news)
        summary = engine.metrics.summary()
        if best is None or dt < best[0]:
            best = (dt, generated, summary, engine.runner.num_forward_passes - passes)
    return sum(lens), best


def decode_bytes(engine, nums, elem, batch, mean_ctx):
    """What a decode step has to read: every weight it uses once, and the cache of the live
    requests."""
    return engine.model.weight_bytes + batch * mean_ctx * nums["kv_values_per_token"] * elem


def prefill_flops(nums, n):
    """Linear layers over ``n`` tokens, the head for one row, causal attention."""
    return (2.0 * n * nums["linear_params"] + 2.0 * nums["head_params"]
            + 2.0 * n * n * nums["attn_hd"] * nums["layers"])


def fp32_points(cfg, vocab, nums, steps=48, warmup=8):
    """The 1B shape in true 32-bit, weights drawn and held in 32-bit on the device: decode at
    batch 1 and 8, prefill of 2,048 tokens."""
    import torch
    out = {}
    for b in (8, 1):
        need = b * (512 + steps + warmup + early_tokens(b, 512) + 32)
        engine = build_engine(cfg, "float32", b, max(need, PREFILL_TOKENS + 64))
        r = decode_run(engine, vocab, b, 512, steps, warmup)
        out[f"fp32_decode_b{b}"] = round(r["tok_s"], 1)
        out[f"fp32_decode_b{b}_ms"] = round(r["ms_per_step"], 4)
        out[f"fp32_decode_b{b}_hbm_frac"] = round(
            decode_bytes(engine, nums, 4, b, r["mean_ctx"]) / (r["seconds"] / steps) / 1e9 / HBM_PEAK_GBS, 4)
        if b == 8:
            s = prefill_run(engine, vocab, PREFILL_TOKENS, repeats=2)
            out["fp32_prefill_tok_s"] = round(PREFILL_TOKENS / s, 1)
            out["fp32_prefill_ms"] = round(s * 1e3, 3)
            out["fp32_prefill_frac"] = round(prefill_flops(nums, PREFILL_TOKENS) / s / MFMA_PEAK["float32"], 4)
        del engine
        torch.cuda.empty_cache()
    return out


def longer_1b_points(folder, vocab, nums, steps=32, warmup=4):
    """The 1B shape in bf16 further out: decode at batch 8 and 64 over contexts of 4,096 and
    8,192 tokens (their share of the HBM roofline), and one prompt of 8,192 tokens read in
    portions of 2,048 (its share of the matrix-core peak)."""
    import torch
    out = {}
    for ctx in (4096, 8192):
        for b in (8, 64):
            prompt = ctx - steps - warmup - 8
            need = b * (prompt + steps + warmup + early_tokens(b, prompt) + 32)
            engine = build_engine(folder, "bfloat16", b, need, context_cap=ctx + 1024)
            r = decode_run(engine, vocab, b, prompt, steps, warmup)
            key = f"decode_b{b}_ctx{ctx}"
            out[key] = round(r["tok_s"], 1)
            out[key + "_ms"] = round(r["ms_per_step"], 4)
            out[key + "_hbm_frac"] = round(
                decode_bytes(engine, nums, 2, b, r["mean_ctx"]) / (r["seconds"] / steps) / 1e9 / HBM_PEAK_GBS, 4)
            if ctx == 8192 and b == 8:
                s = prefill_run(engine, vocab, 8192, repeats=2)
                out["prefill_8192_tok_s"] = round(8192 / s, 1)
                out["prefill_8192_ms"] = round(s * 1e3, 3)
                out["prefill_8192_frac"] = round(prefill_flops(nums, 8192) / s / MFMA_PEAK["bfloat16"], 4)
            del engine
            torch.cuda.empty_cache()
    return out


def mixed_3b_points(requests=32, new_tokens=256):
    """The mixed workload at the Llama 3.2 3B shape, bf16: 32 requests with prompts of 128 to 4,096
    tokens, chunked prefill under a 2,048-token budget, 256 decoded tokens each."""
    import torch
    import kvforge_amd
    cfg = kvforge_amd.preset_dict("llama-3b")
    nums = model_numbers(cfg, cfg["num_hidden_layers"])
    engine = build_engine(cfg, "bfloat16", requests, requests * (4096 + new_tokens + 64))
    prompt_tokens, generated, dt = mixed_run(engine, cfg["vocab_size"], requests, new_tokens)
    info = mixed_run.last
    flops = 2.0 * nums["linear_params"] * (prompt_tokens + generated)
    cache_read = 0.0
    per_token = nums["kv_values_per_token"] * 2
    for n in info["lens"]:
        flops += 2.0 * n * n * nums["attn_hd"] * nums["layers"]                      # the prompt, causal
        flops += 4.0 * new_tokens * (n + new_tokens / 2) * nums["attn_hd"] * nums["layers"]
        cache_read += new_tokens * (n + new_tokens / 2) * per_token                  # decode steps
    read = info["steps"] * engine.model.weight_bytes + cache_read
    out = {"mixed_3b_tok_s": round((prompt_tokens + generated) / dt, 1),
           "mixed_3b_gen_tok_s": round(generated / dt, 1), "mixed_3b_s": round(dt, 4),
           "mixed_3b_steps": info["steps"], "mixed_3b_ms_per_step": round(dt / info["steps"] * 1e3, 4),
           "mixed_3b_mfma_frac": round(flops / dt / MFMA_PEAK["bfloat16"], 4),
           "mixed_3b_hbm_frac": round(read / dt / 1e9 / HBM_PEAK_GBS, 4)}
    del engine
    torch.cuda.empty_cache()
    return out


def long_8b_points(batch=16, prompt_len=32768, new_tokens=128, warmup=8):
    """Long-context decode at the Llama 3.1 8B shape, all 32 layers, bf16: batch 16 at prompts of
    32,768 tokens, 128 new tokens each; before it decode at batch 1 and 8 over short prompts."""
    import torch
    import kvforge_amd
    cfg = kvforge_amd.preset_dict("llama-8b")
    nums = model_numbers(cfg, cfg["num_hidden_layers"])
    steps = new_tokens - 1
    need = batch * (prompt_len + steps + warmup + early_tokens(batch, prompt_len) + 32)
    engine = build_engine(cfg, "bfloat16", batch, need, context_cap=prompt_len + 1024)
    short = {}
    for b in (1, 8):        # the same model over short contexts: 512-token prompts, batch 1 and 8
        r = decode_run(engine, cfg["vocab_size"], b, 512, 48, 8)
        short[f"decode_8b_b{b}"] = round(r["tok_s"], 1)
        short[f"decode_8b_b{b}_ms"] = round(r["ms_per_step"], 4)
        short[f"decode_8b_b{b}_hbm_frac"] = round(
            decode_bytes(engine, nums, 2, b, r["mean_ctx"]) / (r["seconds"] / 48) / 1e9 / HBM_PEAK_GBS, 4)
    t0 = time.perf_counter()
    r = decode_run(engine, cfg["vocab_size"], batch, prompt_len, steps, warmup)
    total = time.perf_counter() - t0
    read = decode_bytes(engine, nums, 2, batch, r["mean_ctx"])
    out = {"long_8b_tok_s": round(r["tok_s"], 1), "long_8b_ms_per_step": round(r["ms_per_step"], 4),
           "long_8b_hbm_frac": round(read / (r["seconds"] / steps) / 1e9 / HBM_PEAK_GBS, 4),
           "long_8b_layers": cfg["num_hidden_layers"], "long_8b_batch": batch,
           "long_8b_context": int(r["mean_ctx"]), "long_8b_steps": steps,
           "long_8b_prefill_tok_s": round(batch * prompt_len / max(total - r["seconds"], 1e-9), 1),
           **short}
    del engine
    torch.cuda.empty_cache()
    return out


def products_run(cfg, rows, repeats=6):
    """The four matrix products of one layer alone, ``rows`` rows of bf16 activations each over
    ``repeats`` copies of its weight in turn (so that no copy is found in a cache), through the
    same entry points the parts use: microseconds per product.  For profiles and counters of a
    single kernel."""
    import torch
    from kvforge_amd.kernels import ops
    h, H, KV, d, I = (cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"],
                      cfg["head_dim"], cfg["intermediate_size"])
    dev, bf = "cuda", torch.bfloat16
    ops.library_ready(dev)
    out = {}
    for name, (n, k) in {"qkv": ((H + 2 * KV) * d, h), "o": (h, H * d), "gate_up": (2 * I, h), "down": (h, I)}.items():
        ws = [ops.streamed((torch.randn(n, k, device=dev) * 0.02).to(bf)) for _ in range(repeats)]
        a = (torch.randn(rows, k, device=dev)).to(bf)
        stream = torch.zeros(rows, n, device=dev)
        plain = torch.empty(rows, n, device=dev, dtype=bf)
        gated = torch.empty(rows, n // 2, device=dev, dtype=bf)

        def launch(w):
            if name in ("o", "down"):
                ops.gemm(a, w, stream, accumulate=True)
            elif name == "gate_up" and ops.bf16_kernel_takes(a, w, False, True):
                ops.gemm_fused(a, w, gated, silu_pairs=True)
            else:
                ops.gemm(a, w, plain)
        for w in ws:
            launch(w)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for w in ws:
            launch(w)
        e1.record()
        torch.cuda.synchronize()
        out[f"{name}_us"] = round(e0.elapsed_time(e1) * 1e3 / repeats, 2)
        del ws
    return out


def model_numbers(cfg, layers_run):
    h, H, KV, d, I, V = (cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"],
                         cfg["head_dim"], cfg["intermediate_size"], cfg["vocab_size"])
    per_layer = h * d * (2 * H + 2 * KV) + 3 * h * I
    return {"linear_params": layers_run * per_layer, "head_params": V * h,
            "kv_values_per_token": 2 * layers_run * KV * d, "attn_hd": H * d, "layers": layers_run}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=255)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--preset", choices=["llama-1b", "llama-3b", "llama-8b", "small"], default="llama-1b",
                    help="layer sizes of the model (random weights); the default is the headline run")
    ap.add_argument("--context-len", type=int, default=CONTEXT_CAP,
                    help="longest request the engine admits (prompt and new tokens)")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the model has")
    ap.add_argument("--no-points", action="store_true",
                    help="skip decode at batch 1 and 64, the 32-bit run and the 3B and 8B workloads")
    ap.add_argument("--only-points", default=None,
                    help="comma-separated subset of longer_1b,fp32,mixed_3b,long_8b to run besides the main line")
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--decode-run-steps", type=int, default=None,
                    help="decode steps the device takes between two looks of the host (engine default: 8)")
    ap.add_argument("--phase", choices=["all", "decode", "prefill", "mixed", "burst", "products"], default="all",
                    help="for profiles: only the decode steps at --batch, or only the prefill; "
                         "mixed: --batch requests with prompts of 128 to 4,096 tokens, chunked "
                         "prefill beside decode steps, --steps new tokens each; burst: the "
                         "workload of the reference's own serving benchmark (48 short requests "
                         "at once, 16 sequences a step), for --preset small or any other; "
                         "products: the four matrix products of a layer alone at --batch rows "
                         "(launch to launch, so short ones show the host's time)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2

    import torch
    import kvforge_amd

    if args.preset == "small" and args.phase != "burst":
        print("--preset small goes with --phase burst")
        return 2
    cfg = dict(SMALL) if args.preset == "small" else kvforge_amd.preset_dict(args.preset)
    full_layers = cfg["num_hidden_layers"]
    layers_run = args.layers or full_layers
    cfg["num_hidden_layers"] = layers_run
    elem = 2 if args.dtype == "bfloat16" else 4
    nums = model_numbers(cfg, layers_run)
    vocab = cfg["vocab_size"]

    if args.phase == "products":
        print(json.dumps({"phase": "products", "model": args.preset, "rows": args.batch, "dtype": "bfloat16",
                          **products_run(cfg, args.batch)}))
        return 0
    with tempfile.TemporaryDirectory(prefix="kvforge_bench_") as folder:
        kvforge_amd.write_random_model(folder, cfg, seed=0, dtype=args.dtype)
        if args.phase == "burst":
            prompt_tokens, (dt, generated, summary, passes) = burst_run(folder, vocab, args.dtype,
                                                                        not args.no_graphs)
            print(json.dumps({
                "phase": "burst", "model": args.preset, "dtype": args.dtype, "requests": 48,
                "prompt_tokens": prompt_tokens, "generated_tokens": generated, "seconds": round(dt, 4),
                "output_tok_s": round(generated / dt, 1), "forward_passes": passes,
                "ttft_p50_ms": round(summary["ttft_p50_ms"], 2), "ttft_p99_ms": round(summary["ttft_p99_ms"], 2),
                "tpot_p50_ms": round(summary["tpot_p50_ms"], 3),
                "reference_published": "84.6 output tok/s, TTFT p50 9,340 ms, TPOT p50 157.6 ms: "
                                       "small preset, fp32, one laptop CPU thread "
                                       "(benchmarks/BENCHMARK_REPORT.md:80)"}))
            return 0
        if args.phase == "mixed":
            engine = build_engine(folder, args.dtype, args.batch, args.batch * (4096 + args.steps + 64),
                                  use_graphs=not args.no_graphs, run_steps=args.decode_run_steps,
                                  context_cap=args.context_len)
            prompt_tokens, generated, dt = mixed_run(engine, vocab, args.batch, args.steps)
            print(json.dumps({"phase": "mixed", "model": args.preset, "requests": args.batch,
                              "dtype": args.dtype, "prompt_tokens": prompt_tokens,
                              "generated_tokens": generated, "seconds": round(dt, 4),
                              "total_tok_s": round((prompt_tokens + generated) / dt, 1),
                              "generated_tok_s": round(generated / dt, 1)}))
            return 0
        results = {}
        points = args.phase == "all" and not args.no_points
        batches = [args.batch] + ([b for b in (1, 64) if b != args.batch] if points else [])
        prefill_s = None
        for b in batches:
            need = b * (args.prompt_len + args.steps + args.warmup + early_tokens(b, args.prompt_len) + 32)
            engine = build_engine(folder, args.dtype, max(b, 1), max(need, PREFILL_TOKENS + 64),
                                  use_graphs=not args.no_graphs, run_steps=args.decode_run_steps,
                                  context_cap=args.context_len)
            if args.phase != "prefill":
                results[b] = decode_run(engine, vocab, b, args.prompt_len, args.steps, args.warmup)
            if b == args.batch:
                if args.phase != "decode":
                    prefill_s = prefill_run(engine, vocab, PREFILL_TOKENS)
                weight_bytes = engine.model.weight_bytes
            del engine
            torch.cuda.empty_cache()
        more = {}
        if points and args.preset == "llama-1b" and layers_run == full_layers:
            chosen = set((args.only_points or "longer_1b,fp32,mixed_3b,long_8b").split(","))
            for name, fn in (("longer_1b", lambda: longer_1b_points(folder, vocab, nums)),
                             ("fp32", lambda: fp32_points(cfg, vocab, nums)),
                             ("mixed_3b", mixed_3b_points), ("long_8b", long_8b_points)):
                if name not in chosen:
                    continue
                try:
                    more.update(fn())
                except Exception as e:   # the main line is printed whatever happens to an extra
                    print(f"bench: {name} failed: {type(e).__name__}: {e}", file=sys.stderr)
                    more[f"{name}_failed"] = 1
                    torch.cuda.empty_cache()

    if args.phase != "all":  # a partial run for a profile: say what was timed and stop
        part = ({"prefill_ms": round(prefill_s * 1e3, 3)} if args.phase == "prefill" else
                {"ms_per_step": round(results[args.batch]["ms_per_step"], 4)})
        print(json.dumps({"phase": args.phase, "batch": args.batch, "dtype": args.dtype, **part}))
        return 0
    main_run = results[args.batch]
    run_steps_used = args.decode_run_steps or kvforge_amd.EngineConfig().decode_run_steps
    step_s = main_run["seconds"] / args.steps
    kv_bytes = args.batch * main_run["mean_ctx"] * nums["kv_values_per_token"] * elem
    achieved = (weight_bytes + kv_bytes) / step_s / 1e9
    n = PREFILL_TOKENS
    line = {
        "metric": "decode tok/s (%s shape, batch %d)" % (MODEL_NAMES[args.preset], args.batch),
        "value": round(main_run["tok_s"], 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(main_run["ms_per_step"], 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: random weights N(0, 0.02), uniform-random token ids",
        "config": {
            "model": MODEL_NAMES[args.preset].lower().replace(" ", "-") + "-shape", "layers": full_layers, "layers_run": layers_run,
            "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
            "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
            "intermediate": cfg["intermediate_size"], "vocab": vocab,
            "tied_embeddings": cfg["tie_word_embeddings"],
            "rope": "theta %.0e, llama3 factor %g" % (cfg["rope_theta"], cfg["rope_scaling"]["factor"]), "rms_norm_eps": cfg["rms_norm_eps"],
            "global_batch": args.batch, "seq_len": args.prompt_len, "new_tokens": args.steps + 1,
            "context_len": args.context_len, "block_size": BLOCK_SIZE, "parallelism": "single-gpu",
            "sampling": "greedy", "decode_run_steps": run_steps_used,
        },
        "prefill": {"value": round(n / prefill_s, 1), "tokens": n, "ms": round(prefill_s * 1e3, 3),
                    "frac": round(prefill_flops(nums, n) / prefill_s / MFMA_PEAK[args.dtype], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": {**{f"decode_b{b}": round(r["tok_s"], 1) for b, r in results.items() if b != args.batch},
                   **more},
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
