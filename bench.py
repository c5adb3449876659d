#!/usr/bin/env python3
"""Serving benchmark on one MI355X: decoded tokens a second of a Llama-3.2-1B-shaped model with
random weights at batch 8 and a context of 4,096 tokens, plus the prefill of 2,048 tokens and
decoding at batch 1 and 64.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C]

A step is one decode step inside the generation loop (``Generator.stream``, the loop that serves
requests): the step function over the cache as a captured graph, arg-max sampling on the device,
the sampled tokens fed back, the loop's own bookkeeping.  The prompts go through the loop's prompt
steps, sized so that the timed steps end at the context length.  Beside the published peaks the
line gives what this GPU reaches in kernels of this library that only read memory or only issue
matrix instructions (``peak_measured``).  One JSON line is printed; everything else goes to
standard error.

The reference's own tool reports prompt and decoding speed of one sequence
(src/libllm/benchmark_main.cc:52-86); it publishes no numbers, so ``vs_baseline`` is null.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_BYTES_PER_S = 8.0e12
DENSE_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

# Llama-3.2-1B sizes
FULL = {
    "model_type": "llama", "num_hidden_layers": 16, "hidden_size": 2048, "num_attention_heads": 32,
    "num_key_value_heads": 8, "head_dim": 64, "intermediate_size": 8192, "vocab_size": 128256,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
    "rms_norm_eps": 1e-5, "tie_word_embeddings": True, "max_position_embeddings": 131072,
    "hidden_act": "silu", "bos_token_id": 128000, "eos_token_id": 128001,
}


# the other Llama shapes the reference family covers, for measurements beside the default
SHAPES = {
    "1b": {},
    "3b": {"num_hidden_layers": 28, "hidden_size": 3072, "num_attention_heads": 24, "head_dim": 128},
    "8b": {"num_hidden_layers": 32, "hidden_size": 4096, "num_attention_heads": 32, "head_dim": 128,
           "intermediate_size": 14336, "tie_word_embeddings": False,
           "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                            "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}},
}
NAMES = {"1b": "Llama-3.2-1B shape", "3b": "Llama-3.2-3B shape", "8b": "Llama-3.1-8B shape"}


def log(msg):
    print("[bench] " + msg, file=sys.stderr, flush=True)


def weight_bytes(cfg, itemsize):
    """Bytes of every weight a decode step reads once (the tied table serves as output matrix)."""
    h, i = cfg.hidden_size, cfg.intermediate_size
    q, kv = cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
    per_layer = (q + 2 * kv) * h + h * q + 3 * h * i
    head = cfg.vocab_size * h
    norms = (2 * cfg.num_hidden_layers + 1) * h * 4
    return (cfg.num_hidden_layers * per_layer + head) * itemsize + norms


def kv_bytes_per_token(cfg, itemsize):
    return 2 * cfg.num_hidden_layers * cfg.num_key_value_heads * cfg.head_dim * itemsize


def prefill_flops(cfg, t):
    h, i = cfg.hidden_size, cfg.intermediate_size
    q, kv = cfg.num_attention_heads * cfg.head_dim, cfg.num_key_value_heads * cfg.head_dim
    linear = 2.0 * t * cfg.num_hidden_layers * ((q + 2 * kv) * h + h * q + 3 * h * i)
    attention = cfg.num_hidden_layers * 4.0 * q * (t * (t + 1) / 2.0)
    head = 2.0 * cfg.vocab_size * h                       # logits of the last position only
    return linear + attention + head


def time_decode(gen, params, torch, batch, context, steps, warmup, vocab):
    """Seconds that ``steps`` decode steps of ``batch`` sequences take inside the generation loop
    (``Generator.stream``: the loop that serves requests, with its bookkeeping, the next step
    queued while the host reads the last one's tokens), the last of them at ``context`` tokens.
    The prompts are random tokens and go through the loop's own prompt steps; ``warmup`` decode
    steps run before the clock starts.  The clock is read after a device-wide wait on both sides."""
    start = context - steps - warmup - 1
    if start < 1:
        raise SystemExit("context %d is too short for %d steps" % (context, steps + warmup))
    g = torch.Generator().manual_seed(batch)
    prompts = [torch.randint(0, vocab, (start,), generator=g).tolist() for _ in range(batch)]
    stream = gen.stream(prompts, params, max_new_tokens=warmup + steps + 4, stop_tokens=())
    seen, t0, dt = 0, None, None
    # When the tokens of decode step s have come, step s + 1 is queued already: the wait at the
    # first mark ends with step warmup + 1, the wait at the second with step warmup + steps + 1.
    first_mark, second_mark = (warmup + 1) * batch, (warmup + steps + 1) * batch
    for _ in stream:
        seen += 1
        if seen == first_mark:
            torch.cuda.synchronize()
            t0 = time.perf_counter()
        elif seen == second_mark:
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            break
    stream.close()                                         # ends the requests, gives their slots back
    return dt


def time_prefill(engine, torch, tokens, vocab, reps):
    """Seconds of one prompt step of ``tokens`` tokens with the last row's logits wanted: the best
    of ``reps`` runs after the first (the second run of a shape captures its graph, the later ones
    replay it; the first replays still run slower than the ones after)."""
    from libllm_amd.engine import StepEntry
    g = torch.Generator().manual_seed(99)
    prompt = torch.randint(0, vocab, (tokens,), generator=g).tolist()
    best = None
    for r in range(reps + 1):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([StepEntry("prefill", prompt, [tokens - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        engine.end(["prefill"])
        if r > 0:                                           # the first run warms up
            best = dt if best is None else min(best, dt)
    return best


def run_workload(args, torch):
    """The two generation workloads beside the headline: 16 prompts of unequal lengths (uniform in
    [64, 2048]) with 256 tokens each, or 64 prompts of 1,024 tokens with 512 tokens each, through
    the generation loop (greedy, no stop token)."""
    import numpy as np

    from libllm_amd.cache import PAGE
    from libllm_amd.config import config_from_dict
    from libllm_amd.engine import Generator
    from libllm_amd.runtime import random_engine
    from libllm_amd.sampling import Sampler, SamplingParams
    d = dict(FULL)
    d.update(SHAPES[args.shape])
    d["eos_token_id"] = None
    cfg = config_from_dict(d)
    rng = np.random.default_rng(0)
    if args.workload == "batch64":
        prompts = [rng.integers(0, cfg.vocab_size, size=1024).tolist() for _ in range(64)]
        new = 512
    else:
        prompts = [rng.integers(0, cfg.vocab_size, size=int(n)).tolist()
                   for n in rng.integers(64, 2049, size=16)]
        new = 256
    need = sum((len(p) + new + PAGE) // PAGE * PAGE for p in prompts) + 4096
    engine = random_engine(cfg, seed=0, dtype=args.dtype, max_tokens=need)
    gen = Generator(engine, Sampler(engine.ops, cfg.vocab_size), (), cfg.max_position_embeddings,
                    engine.cache.n_pages, PAGE, max_batch=64)
    result = None
    for rep in range(3):                                   # the first run warms up; a shape's second coming captures its graph
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        first = []

        def on_token(i, tok):
            if not first:
                torch.cuda.synchronize()
                first.append(time.perf_counter() - t0)
        out = gen.generate(prompts, SamplingParams(temperature=0.0), max_new_tokens=new, on_token=on_token)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        n_prompt, n_out = sum(len(p) for p in prompts), sum(len(o) for o in out)
        result = {
            "metric": "generated tok/s, %s workload (%s)" % (args.workload, NAMES[args.shape]),
            "value": round((n_out - len(prompts)) / (dt - first[0]), 1), "unit": "tokens/s", "n_gpus": 1,
            "steps": new - 1, "warmup": 0, "ms_per_step": round((dt - first[0]) / (new - 1) * 1e3, 3),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
            "data": "synthetic: uniform random token ids, random weights N(0, 0.02)",
            "config": {"model": NAMES[args.shape], "layers": cfg.num_hidden_layers, "prompts": len(prompts),
                       "prompt_tokens": n_prompt, "new_tokens_each": new, "sampling": "greedy"},
            "prefill": {"value": round(n_prompt / first[0], 1), "tokens": n_prompt, "ms": round(first[0] * 1e3, 2)},
        }
        log("run %d: first tokens after %.1f ms, then %.2f ms a step" % (rep, first[0] * 1e3, result["ms_per_step"]))
    print(json.dumps(result), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--shape", default="1b", choices=sorted(SHAPES), help="layer sizes (default: the 1B shape)")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (0: all)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--prefill", type=int, default=2048)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip decoding at batch 1 and 64")
    ap.add_argument("--sampling", default="greedy", choices=["greedy", "default"],
                    help="greedy, or the command line's default (temperature 1, top-k 50, top-p 0.8)")
    ap.add_argument("--workload", choices=["unequal16", "batch64"],
                    help="run a generation workload through the generation loop instead")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this library does not run on several (--gpus %d)" % args.gpus)
        return 2

    import torch

    if args.workload:
        return run_workload(args, torch)

    from libllm_amd.cache import PAGE
    from libllm_amd.config import config_from_dict
    from libllm_amd.engine import Generator
    from libllm_amd.runtime import random_engine
    from libllm_amd.sampling import Sampler, SamplingParams

    d = dict(FULL)
    d.update(SHAPES[args.shape])
    layers_full = d["num_hidden_layers"]
    if args.layers:
        d["num_hidden_layers"] = args.layers
    args.layers = d["num_hidden_layers"]
    cfg = config_from_dict(d)
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    itemsize = 2 if short == "bf16" else 4
    biggest = max(args.batch, 1 if args.no_points else 64)
    max_tokens = biggest * (args.context + 64) + 4096
    log("building %d layers of %d with random weights, cache for %d tokens" %
        (args.layers, layers_full, max_tokens))
    engine = random_engine(cfg, seed=0, dtype=args.dtype, max_tokens=max_tokens)
    gen = Generator(engine, Sampler(engine.ops, cfg.vocab_size), (), cfg.max_position_embeddings,
                    engine.cache.n_pages, PAGE, max_batch=biggest)
    params = SamplingParams(temperature=0.0) if args.sampling == "greedy" else SamplingParams()
    vocab = cfg.vocab_size
    peaks = engine.ops.measured_peaks()
    log("measured on this GPU: read %.0f GB/s, copy %.0f GB/s, bf16 matrix cores %.0f TFLOP/s, fp32 %.1f TFLOP/s"
        % (peaks["read_GBs"], peaks["copy_GBs"], peaks["bf16_TFs"], peaks["fp32_TFs"]))

    pre_s = time_prefill(engine, torch, args.prefill, vocab, reps=10)
    pf = prefill_flops(cfg, args.prefill)
    log("prefill of %d tokens: %.2f ms" % (args.prefill, pre_s * 1e3))

    dt = time_decode(gen, params, torch, args.batch, args.context, args.steps, args.warmup, vocab)
    ms = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    log("decode at batch %d: %.3f ms a step, %.0f tokens/s" % (args.batch, ms, value))
    mean_ctx = args.context - args.steps / 2.0
    step_bytes = weight_bytes(cfg, itemsize) + args.batch * mean_ctx * kv_bytes_per_token(cfg, itemsize)
    achieved = step_bytes / (dt / args.steps) / 1e9

    flops_measured = (peaks["bf16_TFs"] if short == "bf16" else peaks["fp32_TFs"]) * 1e12
    points = {}
    if not args.no_points:
        for b in (1, 64):
            dtb = time_decode(gen, params, torch, b, args.context, args.steps, args.warmup, vocab)
            points["decode_b%d" % b] = round(b * args.steps / dtb, 1)
            log("decode at batch %d: %.3f ms a step, %.0f tokens/s" % (b, dtb / args.steps * 1e3, b * args.steps / dtb))

    out = {
        "metric": "decode tok/s at batch %d, context %d (%s)" % (args.batch, args.context, NAMES[args.shape]),
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": short,
        "data": "synthetic: uniform random token ids, random weights N(0, 0.02)",
        "config": {
            "model": NAMES[args.shape], "layers": args.layers, "layers_full": layers_full,
            "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads,
            "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
            "tied_head": cfg.tie_word_embeddings,
            "rope": "theta 5e5, llama3 factor %g" % cfg.rope_scaling["factor"], "global_batch": args.batch, "seq_len": args.context,
            "prefill_tokens": args.prefill, "sampling": "greedy" if args.sampling == "greedy" else "temperature 1, top-k 50, top-p 0.8", "parallelism": "single GPU",
        },
        "prefill": {"value": round(args.prefill / pre_s, 1), "tokens": args.prefill,
                    "ms": round(pre_s * 1e3, 3), "frac": round(pf / pre_s / DENSE_FLOPS[short], 4),
                    "peak_measured": round(flops_measured / 1e12, 1), "unit_measured": "TFLOP/s",
                    "frac_measured": round(pf / pre_s / flops_measured, 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_BYTES_PER_S / 1e9,
                     "unit": "GB/s", "frac": round(achieved / (HBM_BYTES_PER_S / 1e9), 4),
                     "peak_measured": round(peaks["read_GBs"], 1),
                     "frac_measured": round(achieved / peaks["read_GBs"], 4)},
        "points": points,
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
