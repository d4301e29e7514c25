"""Command line in the manner of computerex/dlgo's examples/simple_chat/main.go:19-40:
`--ctx` (runtime context length), `--max-tokens`, `--temp` (0 = greedy) and the model
path as the positional argument, each checked the same way (> 0, > 0, >= 0).  Prompts
are token ids, since tokenizers are not part of this library.

    python -m dlgo_amd [--ctx N] [--max-tokens N] [--temp T] [--prompt-ids 1,2,3 ...] MODEL_DIR
    python -m dlgo_amd --random-config CONFIG_JSON [--weight-seed S] [...]        (weights drawn for the seed, nothing read or written)
"""
from __future__ import annotations

import argparse
import json
import sys
from typing import List


def _ids(text: str) -> List[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="dlgo_amd", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("model", nargs="?", help="folder with config.json and model.safetensors")
    ap.add_argument("--ctx", type=int, default=8192, help="runtime context length (tokens)")
    ap.add_argument("--max-tokens", type=int, default=256, help="max tokens per response")
    ap.add_argument("--temp", type=float, default=0.7, help="sampling temperature (0 = greedy)")
    ap.add_argument("--top-k", type=int, default=None)
    ap.add_argument("--top-p", type=float, default=None)
    ap.add_argument("--min-p", type=float, default=None)
    ap.add_argument("--repetition-penalty", type=float, default=None)
    ap.add_argument("--greedy", action="store_true", help="argmax decoding (same as --temp 0)")
    ap.add_argument("--seed", type=int, default=-1, help="sampling seed (< 0: from the clock)")
    ap.add_argument("--ignore-eos", action="store_true", help="do not stop at stop tokens")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--prompt-ids", action="append", default=[], help="a prompt as token ids, e.g. 1,15,27 (repeatable)")
    ap.add_argument("--prompts-file", help="a file with one prompt of token ids per line")
    ap.add_argument("--random-config", metavar="CONFIG_JSON",
                    help="instead of MODEL_DIR: run the model this config.json describes with weights drawn for --weight-seed")
    ap.add_argument("--write-random", metavar="CONFIG_JSON",
                    help="write a model folder with random weights for this config.json into MODEL_DIR, then exit")
    ap.add_argument("--weight-seed", type=int, default=0, help="seed of --random-config and --write-random")
    ap.add_argument("--weight-std", type=float, default=None,
                    help="standard deviation of the drawn matrices (default: the configuration's initializer_range)")
    ap.add_argument("--info", action="store_true", help="print the model's description and exit")
    args = ap.parse_args(argv)
    if (args.model is None) == (args.random_config is None):
        ap.error("a model folder or --random-config CONFIG_JSON is required (one of them)")
    if args.write_random and args.model is None:
        ap.error("--write-random writes into MODEL_DIR")
    if args.ctx <= 0:
        print("Error: --ctx must be > 0", file=sys.stderr)
        return 1
    if args.max_tokens <= 0:
        print("Error: --max-tokens must be > 0", file=sys.stderr)
        return 1
    if args.temp < 0:
        print("Error: --temp must be >= 0", file=sys.stderr)
        return 1

    if args.write_random:
        from . import models  # noqa: F401
        from .config import load_config
        from .weights import write_random_model
        try:
            write_random_model(load_config(args.write_random), args.weight_seed, args.model, std=args.weight_std)
        except Exception as e:
            print(f"Error writing model: {e}" + (" (--weight-std)" if "initializer_range" in str(e) else ""), file=sys.stderr)
            return 1
        print(f"wrote {args.model}")
        return 0

    try:
        prompts = [_ids(p) for p in args.prompt_ids]
        if args.prompts_file:
            with open(args.prompts_file) as f:
                prompts += [_ids(line) for line in f if line.strip()]
    except (OSError, ValueError) as e:
        print(f"Error reading prompts (token ids separated by commas or spaces): {e}", file=sys.stderr)
        return 1
    from . import (with_greedy, with_ignore_eos, with_max_tokens, with_min_p, with_repetition_penalty, with_seed,
                   with_temperature, with_top_k, with_top_p)
    from .api import load_llm
    try:
        batch = max(1, min(64, len(prompts) or 1))
        if args.random_config:
            llm = load_llm(args.random_config, args.ctx, args.dtype, max_batch=batch, random_seed=args.weight_seed,
                           random_std=args.weight_std)
        else:
            llm = load_llm(args.model, args.ctx, args.dtype, max_batch=batch)
    except Exception as e:
        print(f"Error loading model: {e}", file=sys.stderr)
        return 1
    print(f"Model: {llm.model_info()}")
    if args.info or not prompts:
        return 0
    opts = [with_max_tokens(args.max_tokens), with_temperature(0.0 if args.greedy else args.temp), with_seed(args.seed)]
    for value, opt in ((args.top_k, with_top_k), (args.top_p, with_top_p), (args.min_p, with_min_p),
                       (args.repetition_penalty, with_repetition_penalty)):
        if value is not None:
            opts.append(opt(value))
    if args.greedy:
        opts.append(with_greedy())
    if args.ignore_eos:
        opts.append(with_ignore_eos())
    try:
        results = llm.generate(prompts, *opts)
    except Exception as e:
        print(f"Error generating: {e}", file=sys.stderr)
        return 1
    for i, r in enumerate(results):
        print(json.dumps({"request": i, "tokens": r.tokens, "finish_reason": r.finish_reason}))
    print(f"[{results[0]}]")
    return 0


if __name__ == "__main__":
    sys.exit(main())
