"""Decode and prefill throughput of the engine at Qwen3-4B size on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--preset qwen3-8b]
    python bench.py --mixed [--preset qwen3-8b] [--requests 160]

A step is one decode step of the engine: plan, run the batch through the model from
the cache, sample, read the tokens back. Random weights (seeded), prompts of uniform
random token ids, every request prefilled through the engine to a context of
``--context`` tokens before timing. Prints one JSON line.
"""

import argparse
import json
import random
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

# Published MI355X peaks used for the roofline fractions.
HBM_GBPS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

DEFAULT_PRESET = "qwen3-4b"        # socrates_amd/config/presets/qwen3-4b.json, the headline configuration
MIXED_PRESET = "qwen3-8b"          # the serving workload's: prompt portions beside decoding rows


def preset_dict(name):
    import json

    from socrates_amd.config import preset_path
    return json.loads(preset_path(name).read_text())


def build_engine(cfg_dict, dtype, max_batch, max_len, seed, compile_, chunk=2048, block_size=16):
    import torch

    from socrates_amd.cache import CacheManager, blocks_for
    from socrates_amd.config import config_class_for
    from socrates_amd.engine import Engine, ModelRunner
    from socrates_amd.kernels import HipKernels
    from socrates_amd.parts import DecoderModel, cache_needs, expected_tensors
    from socrates_amd.weights import random_tensors

    config = config_class_for(cfg_dict["architectures"][0]).from_dict(cfg_dict)
    plan = config.plan()
    ops = HipKernels(dtype, "cuda:0")
    weights = random_tensors(expected_tensors(plan), seed, dtype=dtype, device="cuda:0")
    model = DecoderModel(plan, weights, ops)
    del weights
    cache = CacheManager(cache_needs(plan), max_rows=max_batch, max_len=max_len, block_size=block_size,
                         num_blocks=max_batch * blocks_for(max_len, block_size), dtype=dtype, device="cuda:0")
    runner = ModelRunner(model, cache)
    engine = Engine(runner, max_batch=max_batch, max_len=max_len, max_new_tokens=max_len,
                    chunk=chunk, compile=compile_)
    return config, engine


def mixed_workload(args, dtype):
    """The serving workload: requests with prompts of uniform length in [128, 4096] arrive all
    at once; up to ``--decode-rows`` of them decode while the next prompt is run in portions
    of up to 2,048 tokens beside them (the step's token budget is the portion plus the rows).
    Every step is timed on the host around the engine's whole step (plan, run, sample, read
    back) and sorted by what it ran. Prints one JSON line; ``value`` is all tokens (prompt
    and generated) per second over the whole run."""
    import torch

    from socrates_amd.sampling import SamplingParams
    cfg = preset_dict(args.preset)
    full_layers = cfg["num_hidden_layers"]
    layers = args.layers or full_layers
    cfg["num_hidden_layers"] = layers
    rows, portion = args.decode_rows, args.prefill_tokens
    config, engine = build_engine(cfg, dtype, rows + 1, args.max_len, seed=0, compile_=not args.no_graphs,
                                  block_size=args.block_size,
                                  chunk=portion + rows)
    engine.runner.ops.fuse_norms = not args.no_fused_norms
    if args.dtype == "bf16" and not args.no_tune:
        engine.tune([portion + rows, rows])
    rng = random.Random(7)
    params = SamplingParams(max_new_tokens=args.new_tokens, eos_token_ids=())
    reqs = [engine.submit([rng.randrange(config.vocab_size) for _ in range(rng.randint(128, 4096))], sampling=params)
            for _ in range(args.requests)]
    kinds = {"mixed": [0, 0.0, 0, 0], "prompt_only": [0, 0.0, 0, 0], "decode_only": [0, 0.0, 0, 0]}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while not engine.scheduler.idle:
        a = time.perf_counter()
        n = engine.step()
        b = time.perf_counter()
        if n == 0:
            if engine.scheduler.idle:           # the last requests were retired by this call
                break
            raise RuntimeError("requests are waiting but nothing can be scheduled")
        lens = engine.last_portions
        n_decode = sum(1 for t in lens if t == 1)
        kind = "decode_only" if n_decode == len(lens) else ("mixed" if n_decode else "prompt_only")
        k = kinds[kind]
        k[0] += 1
        k[1] += b - a
        k[2] += n
        k[3] += n_decode
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    new = sum(len(r.output) for r in reqs)
    prompt = sum(len(r.ids) for r in reqs)
    sized = {"qwen3-4b": "Qwen3-4B-sized", "qwen3-8b": "Qwen3-8B-sized", "qwen3-32b": "Qwen3-32B-sized"}.get(
        args.preset, args.preset)
    summary = {kind: {"steps": k[0], "ms_per_step": round(k[1] / k[0] * 1e3, 3), "tokens_per_step": round(k[2] / k[0], 1),
                      "decode_rows_per_step": round(k[3] / k[0], 1), "tok_s": round(k[2] / k[1], 1)}
               for kind, k in kinds.items() if k[0]}
    out = {
        "metric": f"tokens/s through mixed steps: portions of up to {portion} prompt tokens beside up to {rows} "
                  f"decoding rows ({sized}, {args.dtype})",
        "value": round((prompt + new) / dt, 1), "unit": "tok/s", "n_gpus": 1,
        "steps": sum(k[0] for k in kinds.values()), "warmup": 0,
        "ms_per_step": round(dt / sum(k[0] for k in kinds.values()) * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: seeded random weights, uniform random token ids, prompt lengths uniform in [128, 4096]",
        "config": {"model": sized, "global_batch": rows, "seq_len": args.max_len, "parallelism": "single GPU",
                   "layers": layers, "layers_full": full_layers, "hidden_size": config.hidden_size,
                   "num_attention_heads": config.num_attention_heads,
                   "num_key_value_heads": config.num_key_value_heads, "head_dim": config.head_dim,
                   "intermediate_size": config.intermediate_size, "vocab_size": config.vocab_size,
                   "requests": args.requests, "new_tokens_per_request": args.new_tokens,
                   "portion_tokens": portion, "block_size": args.block_size, "hip_graphs": not args.no_graphs},
        "new_tok_s": round(new / dt, 1), "prompt_tokens": prompt, "new_tokens": new, "seconds": round(dt, 3),
        "preemptions": engine.scheduler.n_preemptions,
    }
    out.update(summary)
    print(json.dumps(out))
    return 0


def decode_rate(engine, batch, context, steps, warmup, vocab, seed):
    """Prefill ``batch`` prompts of ``context`` - 1 tokens through the engine, then time
    ``steps`` decode steps. Returns (tokens per second, ms per step)."""
    import torch
    rng = random.Random(seed)
    from socrates_amd.sampling import SamplingParams
    # requests whose prompt is done decode beside the portions of the others, and take their
    # share of a step's token budget: room for the tokens they generate meanwhile
    portions = -(-context // max(1, engine.scheduler.token_budget - batch))
    params = SamplingParams(max_new_tokens=batch * portions + warmup + steps + 8, eos_token_ids=())
    reqs = [engine.submit([rng.randrange(vocab) for _ in range(context - 1)], sampling=params)
            for _ in range(batch)]
    while any(not r.output for r in reqs):          # prefill, a portion per step
        engine.step()
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        n = engine.step()
        assert n == batch, f"a timed step ran {n} tokens, expected {batch}"
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    for r in reqs:
        r.cancelled = True
    engine.scheduler.retire_finished()
    return batch * steps / dt, dt / steps * 1e3


def prefill_rate(engine, tokens, vocab, seed, repeats=3):
    """Time one step that runs a whole prompt of ``tokens`` tokens and samples its first token."""
    import torch
    from socrates_amd.sampling import SamplingParams
    rng = random.Random(seed)
    best = None
    for _ in range(repeats + 1):
        req = engine.submit([rng.randrange(vocab) for _ in range(tokens)],
                            sampling=SamplingParams(max_new_tokens=1, eos_token_ids=()))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        n = engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert n == tokens and req.done
        engine.scheduler.retire_finished()
        best = dt if best is None else min(best, dt)      # the first repeat warms up
    return best


def release(engine):
    """Give an engine's memory back (weights, cache, captured steps) before the next is built."""
    import gc

    import torch
    engine.runner._graphs = None
    engine.runner.model = engine.runner.cache = None
    engine.cache = engine.sampler = engine.scheduler = None
    del engine
    gc.collect()
    torch.cuda.empty_cache()


def other_sizes(args, dtype, item):
    """Decode at batch 8 at longer contexts, and decode and a 2,048-token prefill at the larger
    models' layer sizes: flat entries for ``points``, each rate with the fraction of its
    roofline (decode: bytes read over 8 TB/s; prefill: flops over the dtype's peak)."""
    import torch
    out = {}

    def decode_point(name, config, engine, batch, context):
        tok_s, ms = decode_rate(engine, batch, context, 16, 4, config.vocab_size, seed=11)
        step_bytes = (config.param_counts()["read_per_step"] * item
                      + batch * context * config.kv_bytes_per_token(item))
        out[name] = round(tok_s, 1)
        out[name + "_ms"] = round(ms, 4)
        out[name + "_hbm_frac"] = round(step_bytes / (ms * 1e-3) / 1e9 / HBM_GBPS, 4)

    # the headline model behind longer contexts
    cfg = preset_dict(DEFAULT_PRESET)
    config, engine = build_engine(cfg, dtype, 8, 32768 + 512, seed=0, compile_=not args.no_graphs,
                                  block_size=args.block_size)
    for context in (8192, 32768):
        decode_point(f"decode_b8_ctx{context}", config, engine, 8, context)
    release(engine)
    # the larger models: all layers of each, the contexts that BASELINE.json gives them
    for tag, preset, context in (("8b", "qwen3-8b", 2048), ("32b", "qwen3-32b", 8192)):
        cfg = preset_dict(preset)
        config, engine = build_engine(cfg, dtype, 8, context + 512, seed=0, compile_=not args.no_graphs,
                                      block_size=args.block_size)
        if args.dtype == "bf16" and not args.no_tune:
            engine.tune([args.prefill_tokens])
        decode_point(f"decode_b8_{tag}_ctx{context}", config, engine, 8, context)
        pre_s = prefill_rate(engine, args.prefill_tokens, config.vocab_size, seed=12, repeats=2)
        out[f"prefill_{tag}_ms"] = round(pre_s * 1e3, 3)
        out[f"prefill_{tag}_frac"] = round(config.prefill_flops(args.prefill_tokens) / pre_s / PEAK_FLOPS[args.dtype], 4)
        out[f"layers_{tag}"] = config.num_hidden_layers
        release(engine)
        torch.cuda.synchronize()
    return out


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048)
    ap.add_argument("--max-len", type=int, default=4096)
    ap.add_argument("--preset", default=None, help="a configuration of socrates_amd/config/presets "
                    f"(default {DEFAULT_PRESET}; with --mixed {MIXED_PRESET})")
    ap.add_argument("--mixed", action="store_true",
                    help="the serving workload: prompt portions beside decoding rows (see mixed_workload)")
    ap.add_argument("--requests", type=int, default=160, help="--mixed: requests in the run")
    ap.add_argument("--new-tokens", type=int, default=128, help="--mixed: tokens generated per request")
    ap.add_argument("--decode-rows", type=int, default=64, help="--mixed: requests that decode side by side")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has")
    ap.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per page of the cache (the reference's 16)")
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64")
    ap.add_argument("--no-sizes", action="store_true",
                    help="skip the points at longer contexts and at the larger models' layer sizes")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--no-tune", action="store_true", help="library products with the library's default choice")
    ap.add_argument("--split-waves", type=int, default=None, help="key splits of the decode attention: waves aimed at")
    ap.add_argument("--split-keys", type=int, default=None, help="key splits of the decode attention: fewest keys of a split")
    ap.add_argument("--addnorm-splits", type=int, default=None,
                    help="workgroups that share one tile's K in the projections with a residual epilogue")
    ap.add_argument("--no-fused-norms", action="store_true",
                    help="decode steps with the residual sums and norms in kernels of their own")
    ap.add_argument("--sweep-rows", type=int, default=None,
                    help="rows of a decode step from which its products take the sweep form (0: never)")
    ap.add_argument("--set", action="append", default=[], metavar="NAME=VALUE",
                    help="set an attribute of the kernel set (a switch or a threshold of HipKernels), e.g. stream_rows=0")
    args = ap.parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine is "
              "single-GPU by design)")
        return 2

    import torch
    dtype = {"bf16": torch.bfloat16, "fp32": torch.float32}[args.dtype]
    item = 2 if args.dtype == "bf16" else 4
    if args.mixed:
        args.preset = args.preset or MIXED_PRESET
        args.max_len = max(args.max_len, 8192)
        return mixed_workload(args, dtype)
    args.preset = args.preset or DEFAULT_PRESET
    cfg = preset_dict(args.preset)
    full_layers = cfg["num_hidden_layers"]
    args.layers = args.layers or full_layers
    cfg["num_hidden_layers"] = args.layers
    sized = {"qwen3-4b": "Qwen3-4B-sized", "qwen3-8b": "Qwen3-8B-sized", "qwen3-32b": "Qwen3-32B-sized"}.get(
        args.preset, args.preset)
    biggest = max(args.batch, 1 if args.no_points else 64)
    if args.prefill_tokens + 1 > args.max_len:
        ap.error(f"--prefill-tokens {args.prefill_tokens} needs --max-len of at least {args.prefill_tokens + 1}")
    # the timed prefill is one step: the scheduler's portion holds the whole prompt
    config, engine = build_engine(cfg, dtype, biggest, args.max_len, seed=0, compile_=not args.no_graphs,
                                  chunk=max(2048, args.prefill_tokens), block_size=args.block_size)
    V = config.vocab_size
    engine.runner.ops.fuse_norms = not args.no_fused_norms
    for item_ in args.set:
        name, _, value = item_.partition("=")
        if not hasattr(engine.runner.ops, name):
            ap.error(f"--set {name}: the kernel set has no such attribute")
        setattr(engine.runner.ops, name, json.loads(value))
    if args.sweep_rows is not None:
        engine.runner.ops.sweep_rows = args.sweep_rows
    if args.split_waves:
        engine.runner.ops.split_target_waves = args.split_waves
    if args.split_keys:
        engine.runner.ops.split_min_keys = args.split_keys
    if args.addnorm_splits is not None:
        engine.runner.ops.addnorm_splits = args.addnorm_splits
    if args.dtype == "bf16" and not args.no_tune:
        # the library's products (more than 16 rows): its fastest solution for the prompt's shapes
        # and, up to 16 rows, the faster of the library and this package's own kernel for the timed batch
        engine.tune([args.prefill_tokens] + ([] if args.no_points else [64]) + [args.batch])

    tok_s, ms = decode_rate(engine, args.batch, args.context, args.steps, args.warmup, V, seed=1)
    # bytes one decode step has to read: every weight once, and the cache of the live requests
    step_bytes = (config.param_counts()["read_per_step"] * item
                  + args.batch * args.context * config.kv_bytes_per_token(item))
    achieved = step_bytes / (ms * 1e-3) / 1e9

    pre_s = prefill_rate(engine, args.prefill_tokens, V, seed=2)
    pre_flops = config.prefill_flops(args.prefill_tokens)
    points = {}
    if not args.no_points:
        for b in (1, 64):
            points[f"decode_b{b}"] = round(decode_rate(engine, b, args.context, max(8, args.steps // 2),
                                                       4, V, seed=3 + b)[0], 1)
    if not args.no_points and not args.no_sizes and args.preset == DEFAULT_PRESET and args.layers == full_layers:
        release(engine)
        points.update(other_sizes(args, dtype, item))
    out = {
        "metric": f"decode tok/s @ batch {args.batch}, context {args.context} ({sized}, {args.dtype})",
        "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: seeded random weights, uniform random token ids",
        "config": {"model": sized, "global_batch": args.batch, "seq_len": args.context,
                   "parallelism": "single GPU", "layers": args.layers, "layers_full": full_layers,
                   "hidden_size": config.hidden_size, "num_attention_heads": config.num_attention_heads,
                   "num_key_value_heads": config.num_key_value_heads, "head_dim": config.head_dim,
                   "intermediate_size": config.intermediate_size, "vocab_size": V,
                   "tie_word_embeddings": config.tie_word_embeddings, "max_len": args.max_len,
                   "block_size": args.block_size, "hip_graphs": not args.no_graphs,
                   "library_products_tuned": args.dtype == "bf16" and not args.no_tune},
        "prefill": {"value": round(args.prefill_tokens / pre_s, 1), "tokens": args.prefill_tokens,
                    "ms": round(pre_s * 1e3, 3),
                    "frac": round(pre_flops / pre_s / PEAK_FLOPS[args.dtype], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 4)},
        "points": points,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
