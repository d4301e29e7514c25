#!/usr/bin/env python3
"""Decode and prefill throughput of the Llama 3.2 1B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--dtype bf16|fp32]

A step is one decode step of the whole batch as the library's own generation loop
runs it (dlgo_amd.engine.generate): greedy choice of the next tokens on the device,
the step function on those tokens, the ids' return to the host.  The loop times
every step itself (Stats.step_ms, as computerex/dlgo's loop does,
models/llm/generate.go:227-229,275-282): after W warm-up steps the next K steps
are the timed ones, taken as five regions; the figures are the median region's.
Random weights, seeded uniform-random token ids, no stop tokens.  Prints ONE JSON
line.  --breakdown adds "kernels": the time of every launch of one decode step,
by kind, made one by one between events (gpu_timing_main.go:73-119), and
"prefill_kernels": the same for one prompt step.

Peaks used for the fractions (MI355X, published): HBM 8 TB/s; dense MFMA bf16
2.5 PFLOP/s, fp32 157.3 TFLOP/s.
"""
import argparse
import json
import statistics
import sys
import time

# The benchmark's model: Llama 3.2 1B as config.json states it.
LLAMA_1B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "vocab_size": 128256, "hidden_size": 2048, "num_hidden_layers": 16, "intermediate_size": 8192,
    "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 64,
    "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
    "max_position_embeddings": 131072, "tie_word_embeddings": True, "initializer_range": 0.02,
    "hidden_act": "silu", "torch_dtype": "bfloat16", "bos_token_id": 128000, "eos_token_id": 128001,
}
# Other shapes of the family, for measurements beside the default: the same keys with other sizes.
SHAPES = {
    "llama-3.2-1b": LLAMA_1B,
    "llama-3.2-3b": dict(LLAMA_1B, hidden_size=3072, num_hidden_layers=28, num_attention_heads=24, head_dim=128),
    "llama-3.1-8b": dict(LLAMA_1B, hidden_size=4096, num_hidden_layers=32, intermediate_size=14336, head_dim=128,
                         tie_word_embeddings=False, rope_scaling=dict(LLAMA_1B["rope_scaling"], factor=8.0)),
}
CONTEXT = 4096
PROMPT = 2048
REGIONS = 5        # timed regions of a decode measurement; the median one is reported
HBM_PEAK = 8.0e12
FLOP_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}


def weight_bytes(cfg, elem):
    """Bytes a decode step must read of the weights: every matrix once (the tied table serves as the head)."""
    d, f = cfg.hidden_size, cfg.intermediate_size
    per_layer = (cfg.q_dim + 2 * cfg.kv_dim) * d + d * cfg.q_dim + 3 * d * f
    head = cfg.vocab_size * d       # the output head; the embedding table gives only the step's rows
    norms = (2 * cfg.num_hidden_layers + 1) * d * 4
    return (cfg.num_hidden_layers * per_layer + head) * elem + norms


def kv_bytes_per_token(cfg, elem):
    return cfg.num_hidden_layers * 2 * cfg.kv_dim * elem


def prefill_flops(cfg, t):
    d, f = cfg.hidden_size, cfg.intermediate_size
    per_layer = (cfg.q_dim + 2 * cfg.kv_dim) * d + d * cfg.q_dim + 3 * d * f
    linear = 2.0 * t * per_layer * cfg.num_hidden_layers
    attn = cfg.num_hidden_layers * cfg.num_attention_heads * 2.0 * 2.0 * cfg.head_dim * t * (t + 1) / 2.0   # QK^T and PV, causal
    head = 2.0 * cfg.vocab_size * d
    return linear + attn + head


def ragged(args, cfg, full_layers, elem) -> int:
    """Unequal prompts through the generation loop (the larger shapes' workloads): one batch, greedy, no stop tokens."""
    import numpy as np
    import torch

    from dlgo_amd.engine import Engine
    from dlgo_amd.engine.generate import generate
    from dlgo_amd.sampling import Sampler, SamplerConfig
    from dlgo_amd.sampling.options import GenerateConfig
    n, lo, hi, new, ctx = (int(v) for v in args.ragged.split(":"))
    rng = np.random.default_rng(0)
    lens = rng.integers(lo, hi + 1, size=n)
    prompts = [rng.integers(0, cfg.vocab_size, size=int(k)).tolist() for k in lens]
    held = sum((int(k) + new + 63) // 64 * 64 for k in lens)
    eng = Engine.from_random(cfg, seed=0, dtype=args.dtype, max_tokens=held, max_ctx=ctx, max_slots=n, graph_max_batch=n)
    sampler = Sampler(eng.vocab, eng.device, max_rows=n)
    conf = GenerateConfig(max_tokens=new, sampler=SamplerConfig(temperature=0.0), seed=1, ignore_eos=True)
    runs = []
    for _ in range(5):      # the first records the decode step; the second is still some 8% slower than the ones after it
        _, st = generate(eng, sampler, prompts, [conf] * n, max_batch=n, sync=torch.cuda.synchronize)
        runs.append(st)
    st = sorted(runs, key=lambda r: r.generate_ms)[2]
    steps = st.steps
    mean_ctx = float(lens.mean()) + (new + 1) / 2.0
    step_bytes = weight_bytes(cfg, elem) + n * mean_ctx * kv_bytes_per_token(cfg, elem)
    achieved = step_bytes / (st.generate_ms / 1e3 / steps)
    flops = sum(prefill_flops(cfg, int(k)) for k in lens)
    line = {
        "metric": f"decode tok/s, {n} requests with prompts of {lo}..{hi} tokens ({args.shape} shape, context {ctx})",
        "value": round(st.tokens_per_sec, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": 1,
        "ms_per_step": round(st.generate_ms / steps, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: random weights N(0, 0.02), uniform random token ids and prompt lengths",
        "config": {"model": args.shape + "-shape", "layers": cfg.num_hidden_layers, "layers_of_model": full_layers,
                   "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                   "tied_embeddings": cfg.tie_word_embeddings, "global_batch": n, "seq_len": ctx,
                   "prompt_tokens": int(lens.sum()), "new_tokens": new, "parallelism": "single-gpu",
                   "kv_cache_dtype": args.dtype, "sampling": "greedy, through the generation loop"},
        "prefill": {"value": round(st.prompt_tokens / st.prefill_ms * 1e3, 1), "tokens": int(st.prompt_tokens),
                    "ms": round(st.prefill_ms, 3), "frac": round(flops / (st.prefill_ms / 1e3) / FLOP_PEAK[args.dtype], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4)},
    }
    print(json.dumps(line))
    return 0


def breakdown(eng, sampler, cfg, batch, rng, steps=8):
    """One decode step of `batch` sequences, launch by launch: the same launches a recorded step replays, made one by
    one with an event before and after each.  So that the device does not wait for the host between them, every step
    is queued behind a fill of several gigabytes that keeps the device busy meanwhile (and leaves the caches cold, as
    the weights of the layers before leave them in a real step); "event_pair" is what two events with nothing between
    them measure, which is taken off every bracket.  Returns {kind of launch: [microseconds a step, launches a step]},
    their sum, the launches of a step and the events' share."""
    import torch

    from dlgo_amd.engine import Entry
    from dlgo_amd.kernels import ops
    from dlgo_amd.sampling import SamplerConfig
    prompts = [rng.integers(0, cfg.vocab_size, size=PROMPT).tolist() for _ in range(batch)]
    slots = eng.open(batch)
    greedy = [SamplerConfig(temperature=0.0)] * batch
    logits = eng.step([Entry(s, p, [PROMPT - 1]) for s, p in zip(slots, prompts)])
    for _ in range(2):
        logits = eng.decode(slots, sampler.choose_device(logits, greedy, [0.0] * batch), replay=False)
    ballast = torch.empty(6 << 30, dtype=torch.uint8, device=eng.device)
    torch.cuda.synchronize()
    pairs = []
    with ops.Timings() as t:
        for _ in range(steps):
            ballast.fill_(1)
            logits = eng.decode(slots, sampler.choose_device(logits, greedy, [0.0] * batch), replay=False)
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            b.record()
            pairs.append((a, b))
            torch.cuda.synchronize()
    us, n = t.microseconds(), t.launches()
    eng.close(slots)
    del ballast
    pair = sum(a.elapsed_time(b) for a, b in pairs) * 1000.0 / len(pairs)
    # per kind: microseconds a step with the events' own share taken off, and the launches a step
    out = {k: [round(max(0.0, v / steps - n[k] / steps * pair), 1), n[k] // steps] for k, v in sorted(us.items(), key=lambda kv: -kv[1])}
    out["sum"] = round(sum(v[0] for v in out.values()), 1)
    out["launches"] = sum(n.values()) // steps
    out["event_pair"] = round(pair, 2)
    return out


def prefill_breakdown(eng, cfg, rng, tokens):
    """One prompt step of `tokens` rows, launch by launch between events, as `breakdown` does for a decode step.  The
    prompt is one token shorter than the benchmark's, a shape the engine has not seen, so the step is made of its
    launches and not replayed from a recording; its kernels are long enough that the device does not wait for the host
    between them.  Returns {kind of launch: [microseconds, launches]}, their sum, the launches and the events' share."""
    import torch

    from dlgo_amd.engine import Entry
    from dlgo_amd.kernels import ops
    prompt = rng.integers(0, cfg.vocab_size, size=tokens).tolist()
    slots = eng.open(1)
    torch.cuda.synchronize()
    with ops.Timings() as t:
        eng.step([Entry(slots[0], prompt, [tokens - 1])])
        pairs = []
        for _ in range(8):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            b.record()
            pairs.append((a, b))
        torch.cuda.synchronize()
    us, n = t.microseconds(), t.launches()
    eng.close(slots)
    pair = sum(a.elapsed_time(b) for a, b in pairs) * 1000.0 / len(pairs)
    out = {k: [round(max(0.0, v - n[k] * pair), 1), n[k]] for k, v in sorted(us.items(), key=lambda kv: -kv[1])}
    out["sum"] = round(sum(v[0] for v in out.values()), 1)
    out["launches"] = sum(n.values())
    out["event_pair"] = round(pair, 2)
    out["tokens"] = tokens
    return out


def main() -> int:
    global PROMPT, CONTEXT
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the model has (0 = all)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--points", default="1,64", help="other batch sizes to report, comma separated ('' = none)")
    ap.add_argument("--point-steps", type=int, default=64)
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--breakdown", action="store_true",
                    help="add \"kernels\": microseconds of one decode step of --batch by kind of launch, each launch timed between events, "
                         "and \"prefill_kernels\": the same for one prompt step")
    ap.add_argument("--ragged", default="", metavar="N:LO:HI:NEW:CTX",
                    help="instead of the default run: N requests with prompts of LO..HI tokens (uniform, seeded), NEW "
                         "generated tokens each, context CTX, through the generation loop")
    ap.add_argument("--shape", default="llama-3.2-1b", choices=sorted(SHAPES), help="layer sizes (default: the benchmark's)")
    ap.add_argument("--prompt-len", type=int, default=PROMPT, help="tokens of each prompt (default: the benchmark's 2,048)")
    ap.add_argument("--context", type=int, default=CONTEXT, help="context length (default: the benchmark's 4,096)")
    args = ap.parse_args()
    PROMPT, CONTEXT = args.prompt_len, args.context
    if args.gpus != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import numpy as np
    import torch

    from dlgo_amd import models  # noqa: F401
    from dlgo_amd.config import config_from_dict
    from dlgo_amd.engine import Engine
    from dlgo_amd.engine.generate import generate
    from dlgo_amd.sampling import Sampler, SamplerConfig
    from dlgo_amd.sampling.options import GenerateConfig

    raw = dict(SHAPES[args.shape])
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    cfg = config_from_dict(raw)
    elem = 2 if args.dtype == "bf16" else 4
    if args.ragged:
        return ragged(args, cfg, full_layers, elem)
    batches = [args.batch] + [int(b) for b in args.points.split(",") if b.strip()]
    most = max(batches)
    per_seq = PROMPT + args.warmup + max(args.steps, args.point_steps) + 64
    if per_seq > CONTEXT:
        print(f"bench.py: {PROMPT} prompt tokens, warmup and timed steps need {per_seq} tokens, the context is {CONTEXT}")
        return 2
    eng = Engine.from_random(cfg, seed=0, dtype=args.dtype, max_tokens=most * ((per_seq + 63) // 64 * 64), max_ctx=CONTEXT,
                             max_step_tokens=8192, graph_max_batch=max(most, 8))
    sampler = Sampler(eng.vocab, eng.device, max_rows=most)
    rng = np.random.default_rng(0)

    def conf(new_tokens):
        return GenerateConfig(max_tokens=new_tokens, sampler=SamplerConfig(temperature=0.0), seed=1, ignore_eos=True)

    def decode(batch, steps, warmup):
        """`warmup` + `steps` decode steps of `batch` sequences through the generation loop; the loop's own times of the
        last `steps` of them.  A short run first, so that the step of this batch size is recorded before the run that
        counts (the loop runs a size as it is twice, then records it)."""
        prompts = [rng.integers(0, cfg.vocab_size, size=PROMPT).tolist() for _ in range(batch)]
        generate(eng, sampler, prompts, [conf(4)] * batch, max_batch=batch, sync=torch.cuda.synchronize)
        # the first token comes from the prompt step; every further one is a decode step
        _, st = generate(eng, sampler, prompts, [conf(warmup + steps + 1)] * batch, max_batch=batch, sync=torch.cuda.synchronize)
        times = st.step_ms[1:]                       # [0] is the prompt step
        assert len(times) == warmup + steps + 1, (len(times), warmup, steps)
        timed = times[warmup:warmup + steps]         # the last entry is the loop's final turn, which runs no step
        n_regions = REGIONS if steps >= REGIONS else 1
        sizes = [steps // n_regions + (1 if r < steps % n_regions else 0) for r in range(n_regions)]
        per_step, o = [], 0
        for size in sizes:
            per_step.append(sum(timed[o:o + size]) / size / 1000.0)
            o += size
        mean_ctx = PROMPT + warmup + (steps + 1) / 2.0       # keys a step reads per sequence, averaged over the timed steps
        return statistics.median(per_step), mean_ctx, per_step

    # the other batch sizes first: the headline figure is then taken on a device that has been working for a while
    points = {}
    for b in batches[1:]:
        p_step, _, _ = decode(b, args.point_steps, min(args.warmup, 8))
        points[f"decode_b{b}"] = round(b / p_step, 1)
    step_s, mean_ctx, regions = decode(args.batch, args.steps, args.warmup)
    ms_step = step_s * 1000.0
    value = args.batch / step_s
    step_bytes = weight_bytes(cfg, elem) + args.batch * mean_ctx * kv_bytes_per_token(cfg, elem)
    achieved = step_bytes / step_s

    prefill = None
    if not args.no_prefill:
        times = []
        for i in range(6):       # the loop's own time of the prompt step (it waits for the device before and after)
            prompt = rng.integers(0, cfg.vocab_size, size=PROMPT).tolist()
            _, st = generate(eng, sampler, [prompt], [conf(1)], max_batch=1, sync=torch.cuda.synchronize)
            times.append(st.prefill_ms / 1000.0)
        pt = statistics.median(times[1:])
        prefill = {"value": round(PROMPT / pt, 1), "tokens": PROMPT, "ms": round(pt * 1000.0, 3),
                   "frac": round(prefill_flops(cfg, PROMPT) / pt / FLOP_PEAK[args.dtype], 4)}

    kernels = prefill_kernels = None
    if args.breakdown:
        kernels = breakdown(eng, sampler, cfg, args.batch, rng)
        if not args.no_prefill and PROMPT > 1:
            try:
                prefill_kernels = prefill_breakdown(eng, cfg, rng, PROMPT - 1)
            except Exception as e:      # the line's other figures are measured by now: say what went wrong beside them
                prefill_kernels = {"error": f"{type(e).__name__}: {e}"}

    line = {
        "metric": f"decode tok/s @ batch {args.batch} ({args.shape} shape, {PROMPT}-token prompts, context {CONTEXT})",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: random weights N(0, 0.02), uniform random token ids",
        "config": {"model": args.shape + "-shape", "layers": cfg.num_hidden_layers, "layers_of_model": full_layers,
                   "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                   "tied_embeddings": cfg.tie_word_embeddings, "global_batch": args.batch, "seq_len": CONTEXT,
                   "prompt_len": PROMPT, "parallelism": "single-gpu", "kv_cache_dtype": args.dtype,
                   "sampling": "greedy, through the generation loop"},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4)},
        "points": points,
        "regions_ms_per_step": [round(r * 1000.0, 4) for r in regions],
    }
    if prefill is not None:
        line["prefill"] = prefill
    if kernels is not None:
        line["kernels"] = kernels
    if prefill_kernels is not None:
        line["prefill_kernels"] = prefill_kernels
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
