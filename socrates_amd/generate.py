"""Command line: generate from a model folder.

    python -m socrates_amd.generate --model DIR --prompt-ids 5,17,3 --max-new-tokens 16

The reference's command line is ``python -m model.inference_paged`` with no arguments
and environment variables for the knobs (model/inference_paged.py:240-255,
model/inference_cont.py:21-30): it submits a list of prompts, runs the engine, prints
each result and a line ``wall | total tok | tok/s``. The same happens here; every knob
is an option named after the reference's ``Engine`` argument, and the reference's
environment variables give the defaults where they exist (MODEL_ID for --model, DEVICE,
KV_BLOCK for --block-size, COMPILE).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

from .engine import KV_BLOCK, MAX_BATCH, MAX_LEN, MAX_NEW_TOKENS, PREFILL_CHUNK, Engine
from .sampling import SamplingParams


def _ids(text: str):
    return [int(t) for t in text.replace(",", " ").split()]


def parse_args(argv=None):
    ap = argparse.ArgumentParser(prog="python -m socrates_amd.generate", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", default=os.getenv("MODEL_ID"),
                    help="model folder: config.json + model.safetensors (env MODEL_ID)")
    ap.add_argument("--random-weights", metavar="CONFIG_JSON",
                    help="write a random model for this config.json into --model first (seeded by --seed)")
    ap.add_argument("--preset", help="like --random-weights with a configuration that comes with the package: "
                                     "tiny-a, tiny-b, qwen3-4b, qwen3-8b, qwen3-32b")
    ap.add_argument("--device", default=os.getenv("DEVICE", "cuda:0"))
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--compile", type=int, default=int(os.getenv("COMPILE", "1") not in ("0", "false", "False")),
                    help="1: replay decode steps from captured HIP graphs (env COMPILE)")
    ap.add_argument("--max-batch", type=int, default=MAX_BATCH)
    ap.add_argument("--max-len", type=int, default=MAX_LEN)
    ap.add_argument("--max-new-tokens", type=int, default=MAX_NEW_TOKENS)
    ap.add_argument("--block-size", type=int, default=int(os.getenv("KV_BLOCK", str(KV_BLOCK))))
    ap.add_argument("--num-blocks", type=int, default=None)
    ap.add_argument("--chunk", type=int, default=PREFILL_CHUNK, help="token budget of one step")
    ap.add_argument("--temperature", type=float, default=0.0, help="0: greedy")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--eos", type=_ids, default=None, help="stop token ids (default: the model's)")
    ap.add_argument("--prompt-ids", type=_ids, action="append", default=[],
                    help="a prompt as token ids, e.g. 5,17,3 (repeatable)")
    ap.add_argument("--prompt-file", help="JSON lines, each a list of token ids")
    ap.add_argument("--prompt", action="append", default=[], help="a text prompt (needs --tokenizer)")
    ap.add_argument("--tokenizer", help="folder of a Hugging Face tokenizer, for text prompts")
    args = ap.parse_args(argv)
    if not args.model:
        ap.error("--model (or MODEL_ID) is required")
    return args


def main(argv=None) -> int:
    args = parse_args(argv)
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.dtype]
    if args.random_weights and args.preset:
        print("--random-weights and --preset both name a configuration; give one", file=sys.stderr)
        return 2
    if args.preset:
        from .config import preset_path
        args.random_weights = str(preset_path(args.preset))
    if args.random_weights:
        from .config import config_class_for
        from .weights import write_random_model
        raw = json.loads(open(args.random_weights).read())
        config = config_class_for(raw["architectures"][0]).from_dict(raw)
        write_random_model(args.model, config, args.seed)
    tok = None
    if args.tokenizer:
        from transformers import AutoTokenizer      # tokenizer only; no model code is used
        tok = AutoTokenizer.from_pretrained(args.tokenizer)
    prompts = list(args.prompt_ids)
    if args.prompt_file:
        prompts += [json.loads(line) for line in open(args.prompt_file) if line.strip()]
    if args.prompt and tok is None:
        print("text prompts need --tokenizer", file=sys.stderr)
        return 2
    prompts += args.prompt
    if not prompts:
        print("no prompts given (--prompt-ids, --prompt-file or --prompt)", file=sys.stderr)
        return 2
    engine = Engine(args.model, tok=tok, device=args.device, dtype=dtype, compile=bool(args.compile),
                    max_batch=args.max_batch, max_len=args.max_len, max_new_tokens=args.max_new_tokens,
                    block_size=args.block_size, num_blocks=args.num_blocks, chunk=args.chunk)
    reqs = [engine.submit(p, sampling=SamplingParams(
        temperature=args.temperature, seed=args.seed + i,
        eos_token_ids=None if args.eos is None else tuple(args.eos))) for i, p in enumerate(prompts)]
    pools = ", ".join(f"{g.allocator.num_blocks} pages of {g.block_size} tokens" for g in engine.cache.groups)
    print(f"{len(reqs)} requests, {engine.max_batch} rows, {pools or 'no paged cache'}\n")
    t0 = time.perf_counter()
    engine.run()
    wall = time.perf_counter() - t0
    for r in reqs:
        shown = tok.decode(r.output) if tok is not None else " ".join(map(str, r.output))
        asked = r.prompt if isinstance(r.prompt, str) else " ".join(map(str, r.ids))
        print(f"> {asked}\n{shown}\n")
    total = sum(len(r.output) for r in reqs)
    print(f"{wall:.2f} s wall | {total} tok | {total / wall:.2f} tok/s")
    return 0


if __name__ == "__main__":
    sys.exit(main())
