#!/usr/bin/env python3
"""Serving benchmark on one MI355X: decoded tokens a second of a Llama-3.2-1B-shaped model with
random weights at batch 8 and a context of 4,096 tokens, plus the prefill of 2,048 tokens and
decoding at batch 1, 64 and 256.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C]
    python bench.py --sweep            # decode at batch 1..256 x context 4,096..131,072, as a table
    python bench.py --unequal          # decode steps of batches whose contexts differ widely

A step is one decode step inside the generation loop (``Generator.stream``, the loop that serves
requests): the step function over the cache as a captured graph, arg-max sampling on the device,
the sampled tokens fed back, the loop's own bookkeeping.  The prompts go through the loop's prompt
steps, sized so that the timed steps end at the context length.  Beside the published peaks the
line gives what this GPU reaches in kernels of this library that only read memory or only issue
matrix instructions (``peak_measured``).  The default run then builds the 3B and the 8B shape and
runs their generation workloads (16 unequal prompts with 256 tokens each; 64 prompts of 1,024
tokens with 512 tokens each), whose figures go into ``points``.  One JSON line is printed;
everything else goes to standard error.

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
    # further sizes of the same architecture (layer sizes and vocabulary only; the position encoding
    # stays the default's, which does not change a step's time): every head with keys of its own,
    # a feed-forward that is no multiple of 256, and the widest layers of the family, of which
    # ``--layers`` runs as many as fit beside their tiled copies
    "7b": {"num_hidden_layers": 32, "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 32,
           "head_dim": 128, "intermediate_size": 11008, "vocab_size": 32000, "tie_word_embeddings": False},
    "13b": {"num_hidden_layers": 40, "hidden_size": 5120, "num_attention_heads": 40, "num_key_value_heads": 40,
            "head_dim": 128, "intermediate_size": 13824, "vocab_size": 32000, "tie_word_embeddings": False},
    "70b": {"num_hidden_layers": 80, "hidden_size": 8192, "num_attention_heads": 64, "num_key_value_heads": 8,
            "head_dim": 128, "intermediate_size": 28672, "tie_word_embeddings": False},
}
NAMES = {"1b": "Llama-3.2-1B shape", "3b": "Llama-3.2-3B shape", "8b": "Llama-3.1-8B shape",
         "7b": "Llama-2-7B sizes", "13b": "Llama-2-13B sizes", "70b": "Llama-3.1-70B sizes"}


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
    """Seconds of one prompt step of ``tokens`` tokens with the last row's logits wanted, ``reps``
    runs after the first two (the second run of a shape captures its graph, the later ones replay
    it): (median, minimum)."""
    from libllm_amd.engine import StepEntry
    g = torch.Generator().manual_seed(99)
    prompt = torch.randint(0, vocab, (tokens,), generator=g).tolist()
    times = []
    for r in range(reps + 2):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([StepEntry("prefill", prompt, [tokens - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        engine.end(["prefill"])
        if r > 1:                                           # the first run warms up, the second captures
            times.append(dt)
    times.sort()
    return times[len(times) // 2], times[0]


def workload_prompts(workload, vocab):
    """(prompts, new tokens each) of a generation workload: 16 prompts of unequal lengths
    (uniform in [64, 2048]) with 256 tokens each, or 64 prompts of 1,024 tokens with 512 each."""
    import numpy as np
    rng = np.random.default_rng(0)
    if workload == "batch64":
        return [rng.integers(0, vocab, size=1024).tolist() for _ in range(64)], 512
    return [rng.integers(0, vocab, size=int(n)).tolist() for n in rng.integers(64, 2049, size=16)], 256


def time_workload(shape, workload, dtype, torch, reps=3):
    """A generation workload through the generation loop (greedy, no stop token) on an engine of
    its own: what the last of ``reps`` runs took (the first warms up; a shape's second coming
    captures its graph).  Returns a record of plain numbers."""
    from libllm_amd.cache import PAGE
    from libllm_amd.config import config_from_dict
    from libllm_amd.engine import Generator
    from libllm_amd.runtime import random_engine
    from libllm_amd.sampling import Sampler, SamplingParams
    d = dict(FULL)
    d.update(SHAPES[shape])
    d["eos_token_id"] = None
    cfg = config_from_dict(d)
    prompts, new = workload_prompts(workload, cfg.vocab_size)
    need = sum((len(p) + new + PAGE) // PAGE * PAGE for p in prompts) + 4096
    engine = random_engine(cfg, seed=0, dtype=dtype, max_tokens=need)
    gen = Generator(engine, Sampler(engine.ops, cfg.vocab_size), (), cfg.max_position_embeddings,
                    engine.cache.n_pages, PAGE, max_batch=64)
    itemsize = 2 if dtype == "bfloat16" else 4
    rec = None
    for rep in range(reps):
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
        step_s = (dt - first[0]) / (new - 1)
        # bytes of a decode step in the middle of the run: every weight once, and the cache the live requests hold
        held = n_prompt + len(prompts) * new / 2.0
        step_bytes = weight_bytes(cfg, itemsize) + held * kv_bytes_per_token(cfg, itemsize)
        rec = {"cfg": cfg, "prompts": len(prompts), "prompt_tokens": n_prompt, "new": new,
               "tok_s": (n_out - len(prompts)) / (dt - first[0]), "ms_per_step": step_s * 1e3,
               "prefill_ms": first[0] * 1e3, "prefill_tok_s": n_prompt / first[0],
               "prefill_frac": sum(prefill_flops(cfg, len(p)) for p in prompts) / first[0] / DENSE_FLOPS["bf16" if itemsize == 2 else "fp32"],
               "hbm_frac": step_bytes / step_s / HBM_BYTES_PER_S}
        log("%s %s run %d: first tokens after %.1f ms, then %.2f ms a step" % (shape, workload, rep, rec["prefill_ms"], rec["ms_per_step"]))
    del gen, engine
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    return rec


def run_workload(args, torch):
    """One of the two generation workloads beside the headline, as a line of its own."""
    rec = time_workload(args.shape, args.workload, args.dtype, torch)
    cfg = rec["cfg"]
    result = {
        "metric": "generated tok/s, %s workload (%s)" % (args.workload, NAMES[args.shape]),
        "value": round(rec["tok_s"], 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": rec["new"] - 1, "warmup": 0, "ms_per_step": round(rec["ms_per_step"], 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: uniform random token ids, random weights N(0, 0.02)",
        "config": {"model": NAMES[args.shape], "layers": cfg.num_hidden_layers, "prompts": rec["prompts"],
                   "prompt_tokens": rec["prompt_tokens"], "new_tokens_each": rec["new"], "sampling": "greedy"},
        "prefill": {"value": round(rec["prefill_tok_s"], 1), "tokens": rec["prompt_tokens"], "ms": round(rec["prefill_ms"], 2),
                    "frac": round(rec["prefill_frac"], 4)},
        "roofline": {"bound": "hbm", "achieved": round(rec["hbm_frac"] * HBM_BYTES_PER_S / 1e9, 1),
                     "peak": HBM_BYTES_PER_S / 1e9, "unit": "GB/s", "frac": round(rec["hbm_frac"], 4)},
    }
    print(json.dumps(result), flush=True)
    return 0


SWEEP_BATCHES = (1, 8, 16, 32, 64, 128, 256)
SWEEP_CONTEXTS = (4096, 16384, 32768, 131072)


def run_sweep(args, torch):
    """Decode steps at batch 1 to 256 and contexts of 4,096 to 131,072 tokens (where the cache fits
    the device), each with its bytes / time against 8 TB/s.  The cache is not filled by prompts
    (at 131,072 tokens a batch that alone would take minutes): the requests are given their pages
    and lengths in the cache's books, the pages hold random values, and the step function decodes
    from there, arg-max on the device and the tokens fed back without the host reading them, as
    the generation loop queues them."""
    from libllm_amd.config import config_from_dict
    from libllm_amd.engine import StepEntry
    from libllm_amd.runtime import random_engine
    d = dict(FULL)
    d.update(SHAPES[args.shape])
    cfg = config_from_dict(d)
    itemsize = 2 if args.dtype == "bfloat16" else 4
    free, _ = torch.cuda.mem_get_info()
    per_token = kv_bytes_per_token(cfg, itemsize)
    room = int((free - 2.2 * weight_bytes(cfg, itemsize) - (8 << 30)) / per_token)
    cells = [(b, c) for c in SWEEP_CONTEXTS for b in SWEEP_BATCHES if b * (c + 64) <= room]
    max_tokens = max(b * (c + 64) for b, c in cells)
    log("cache for %d tokens (%.0f GB); %d cells" % (max_tokens, max_tokens * per_token / 1e9, len(cells)))
    engine = random_engine(cfg, seed=0, dtype=args.dtype, max_tokens=max_tokens, max_slots=max(SWEEP_BATCHES))
    for g in engine.cache.groups:
        for plane in g.planes.values():
            plane.normal_()
    steps, warmup = args.steps, args.warmup
    points, table = {}, {}
    for b, c in cells:
        ids = [("sweep", b, c, i) for i in range(b)]
        for r in ids:                                       # the books only: pages and lengths, no prompt step
            slot = engine.cache.admit(r)
            engine.cache.reserve(slot, c - steps - warmup - 1)
            engine.cache.commit(slot, c - steps - warmup - 1)
        engine.cache.flush()
        tokens = torch.zeros((b,), dtype=torch.int32, device=engine.device)
        entries = [StepEntry(r, [0], [0]) for r in ids]
        for k in range(warmup + steps):
            if k == warmup:
                torch.cuda.synchronize()
                t0 = time.perf_counter()
            tokens = engine.ops.argmax(engine.step(entries, tokens_device=tokens))
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        engine.end(ids)
        step_bytes = weight_bytes(cfg, itemsize) + b * (c - steps / 2.0) * per_token
        frac = step_bytes / dt / HBM_BYTES_PER_S
        points["b%d_c%d" % (b, c)] = round(b / dt, 1)
        points["b%d_c%d_hbm_frac" % (b, c)] = round(frac, 4)
        table[(b, c)] = (dt * 1e3, frac)
        log("batch %3d, context %6d: %.3f ms a step, %.0f tok/s, %.2f of 8 TB/s" % (b, c, dt * 1e3, b / dt, frac))
    log("ms a step (fraction of 8 TB/s), %s, %s:" % (NAMES[args.shape], args.dtype))
    log("%8s" % "batch" + "".join("%18d" % c for c in SWEEP_CONTEXTS))
    for b in SWEEP_BATCHES:
        log("%8d" % b + "".join(("%11.3f (%.2f)" % table[(b, c)]) if (b, c) in table else "%18s" % "-" for c in SWEEP_CONTEXTS))
    best = max(points[k] for k in points if not k.endswith("_frac"))
    print(json.dumps({
        "metric": "decode tok/s over batch x context (%s)" % NAMES[args.shape], "value": best, "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": None, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if itemsize == 2 else "fp32",
        "data": "synthetic: random cache contents, random weights N(0, 0.02)",
        "config": {"model": NAMES[args.shape], "layers": cfg.num_hidden_layers, "sampling": "greedy"},
        "points": points}), flush=True)
    return 0


UNEQUAL_CASES = (
    ("8x16384", [16384] * 8), ("1x131072", [131072]), ("1x131072_7x128", [131072] + [128] * 7),
    ("64x4096", [4096] * 64), ("1x131072_63x2048", [131072] + [2048] * 63), ("8x32768_56x256", [32768] * 8 + [256] * 56),
    ("64x64to8128", [64 + 128 * i for i in range(64)]),
)


def time_contexts(engine, torch, name, ctxs, steps, warmup):
    """Seconds a decode step of sequences that end at ``ctxs`` tokens takes: the cache's books are
    filled without prompt steps (pages and lengths only), then the step function decodes, arg-max
    on the device and the tokens fed back without the host reading them."""
    from libllm_amd.engine import StepEntry
    ids = [("contexts", name, i) for i in range(len(ctxs))]
    for r, c in zip(ids, ctxs):
        slot = engine.cache.admit(r)
        engine.cache.reserve(slot, c - steps - warmup - 1)
        engine.cache.commit(slot, c - steps - warmup - 1)
    engine.cache.flush()
    tokens = torch.zeros((len(ids),), dtype=torch.int32, device=engine.device)
    entries = [StepEntry(r, [0], [0]) for r in ids]
    for k in range(warmup + steps):
        if k == warmup:
            torch.cuda.synchronize()
            t0 = time.perf_counter()
        tokens = engine.ops.argmax(engine.step(entries, tokens_device=tokens))
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    engine.end(ids)
    return dt


def run_unequal(args, torch):
    """Decode steps of batches whose sequences hold very different numbers of tokens, beside
    batches of like lengths with about as many bytes, each with its bytes / time against 8 TB/s
    (the cache's books are filled as in the sweep).  Decode attention sizes its grid by the
    longest sequence of a step unless the lengths differ widely; then it deals the pages out by
    length."""
    from libllm_amd.config import config_from_dict
    from libllm_amd.engine import StepEntry
    from libllm_amd.runtime import random_engine
    d = dict(FULL)
    d.update(SHAPES[args.shape])
    cfg = config_from_dict(d)
    itemsize = 2 if args.dtype == "bfloat16" else 4
    per_token = kv_bytes_per_token(cfg, itemsize)
    max_tokens = max(sum(c + 64 for c in ctxs) for _, ctxs in UNEQUAL_CASES)
    engine = random_engine(cfg, seed=0, dtype=args.dtype, max_tokens=max_tokens, max_slots=64)
    for g in engine.cache.groups:
        for plane in g.planes.values():
            plane.normal_()
    steps, warmup = min(args.steps, 32), min(args.warmup, 8)        # (the shortest sequences end at 128 tokens)
    points = {}
    for name, ctxs in UNEQUAL_CASES:
        dt = time_contexts(engine, torch, name, ctxs, steps, warmup)
        frac = (weight_bytes(cfg, itemsize) + (sum(ctxs) - len(ctxs) * steps / 2.0) * per_token) / dt / HBM_BYTES_PER_S
        points[name + "_ms"] = round(dt * 1e3, 3)
        points[name + "_hbm_frac"] = round(frac, 4)
        log("%-20s %.3f ms a step, %.2f of 8 TB/s" % (name, dt * 1e3, frac))
    print(json.dumps({
        "metric": "decode ms a step over batches of unequal contexts (%s)" % NAMES[args.shape],
        "value": points["1x131072_63x2048_ms"], "unit": "ms", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": points["1x131072_63x2048_ms"], "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if itemsize == 2 else "fp32", "data": "synthetic: random cache contents, random weights N(0, 0.02)",
        "config": {"model": NAMES[args.shape], "layers": cfg.num_hidden_layers, "sampling": "greedy"},
        "points": points}), flush=True)
    return 0


def run_requests(args, torch):
    """Many requests of mixed lengths through the generation loop, more than a batch holds: prompt
    lengths log-normal (median about 240 tokens, clipped to [4, 6000]) with four long ones of
    12,000 to 50,000, greedy, at most 256 new tokens, and stop tokens drawn so that a reply ends
    after about 200 tokens on average (random weights give a near-uniform next token).  The loop
    forms batch after batch, shorter replies end earlier, slots and pages are used again.  The
    second of two runs counts (the first captures the graphs of the shapes that come up)."""
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
    n, new = args.requests, 256
    lens = np.clip(np.exp(rng.normal(5.5, 1.2, size=n)).astype(int), 4, 6000)
    lens[rng.integers(0, n, size=4)] = [30000, 50000, 12000, 20000]
    prompts = [rng.integers(0, cfg.vocab_size, size=int(l)).tolist() for l in lens]
    stop = tuple(int(t) for t in rng.integers(0, cfg.vocab_size, size=cfg.vocab_size // 200))
    engine = random_engine(cfg, seed=0, dtype=args.dtype, max_tokens=2_000_000, max_slots=args.max_batch)
    gen = Generator(engine, Sampler(engine.ops, cfg.vocab_size), stop, cfg.max_position_embeddings,
                    engine.cache.n_pages, PAGE, max_batch=args.max_batch)
    log("%d requests, %d prompt tokens (median %d, longest %d), batches of at most %d"
        % (n, lens.sum(), np.median(lens), lens.max(), args.max_batch))
    for rep in range(2):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = gen.generate(prompts, SamplingParams(temperature=0.0), max_new_tokens=new)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        n_out = sum(len(o) for o in out)
        log("run %d: %.2f s, %d new tokens, %.0f generated tok/s, %.0f tok/s with the prompts' tokens"
            % (rep, dt, n_out, n_out / dt, (n_out + lens.sum()) / dt))
    print(json.dumps({
        "metric": "generated tok/s over %d requests of mixed lengths (%s)" % (n, NAMES[args.shape]),
        "value": round(n_out / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": None, "warmup": None,
        "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: uniform random token ids, random weights N(0, 0.02)",
        "config": {"model": NAMES[args.shape], "layers": cfg.num_hidden_layers, "requests": n, "max_batch": args.max_batch,
                   "prompt_tokens": int(lens.sum()), "new_tokens": n_out, "max_new_tokens": new, "sampling": "greedy"},
        "points": {"seconds": round(dt, 3), "tok_s_with_prompts": round((n_out + lens.sum()) / dt, 1)}}), flush=True)
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
    ap.add_argument("--no-points", action="store_true", help="skip decoding at batch 1, 64 and 256")
    ap.add_argument("--sampling", default="greedy", choices=["greedy", "default"],
                    help="greedy, or the command line's default (temperature 1, top-k 50, top-p 0.8)")
    ap.add_argument("--workload", choices=["unequal16", "batch64"],
                    help="run a generation workload through the generation loop instead")
    ap.add_argument("--sweep", action="store_true",
                    help="decode steps at batch 1 to 256 and contexts of 4,096 to 131,072 tokens, as a table")
    ap.add_argument("--unequal", action="store_true",
                    help="decode steps of batches whose sequences hold very different numbers of tokens")
    ap.add_argument("--requests", type=int, default=0,
                    help="run so many requests of mixed lengths through the generation loop instead")
    ap.add_argument("--max-batch", type=int, default=256, help="the largest batch of --requests")
    ap.add_argument("--no-workloads", action="store_true",
                    help="skip the generation workloads of the 3B and 8B shapes")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this library does not run on several (--gpus %d)" % args.gpus)
        return 2

    import torch

    if args.workload:
        return run_workload(args, torch)
    if args.sweep:
        return run_sweep(args, torch)
    if args.unequal:
        return run_unequal(args, torch)
    if args.requests:
        return run_requests(args, torch)

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
    # decoding is also measured at batch 1 and 64, and at 256 (the largest captured graph) where
    # the cache for that is small beside the device's memory
    point_batches = () if args.no_points else ((1, 64, 256) if args.shape == "1b" else (1, 64))
    biggest = max((args.batch,) + point_batches)
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

    pre_s, pre_min = time_prefill(engine, torch, args.prefill, vocab, reps=11)
    pf = prefill_flops(cfg, args.prefill)
    log("prefill of %d tokens: %.2f ms (the median of 11 runs; the fastest %.2f)" % (args.prefill, pre_s * 1e3, pre_min * 1e3))

    dt = time_decode(gen, params, torch, args.batch, args.context, args.steps, args.warmup, vocab)
    ms = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    log("decode at batch %d: %.3f ms a step, %.0f tokens/s" % (args.batch, ms, value))
    mean_ctx = args.context - args.steps / 2.0
    step_bytes = weight_bytes(cfg, itemsize) + args.batch * mean_ctx * kv_bytes_per_token(cfg, itemsize)
    achieved = step_bytes / (dt / args.steps) / 1e9

    flops_measured = (peaks["bf16_TFs"] if short == "bf16" else peaks["fp32_TFs"]) * 1e12
    points = {}
    if point_batches:
        for b in point_batches:
            dtb = time_decode(gen, params, torch, b, args.context, args.steps, args.warmup, vocab)
            points["decode_b%d" % b] = round(b * args.steps / dtb, 1)
            bytes_b = weight_bytes(cfg, itemsize) + b * mean_ctx * kv_bytes_per_token(cfg, itemsize)
            points["decode_b%d_hbm_frac" % b] = round(bytes_b / (dtb / args.steps) / HBM_BYTES_PER_S, 4)
            log("decode at batch %d: %.3f ms a step, %.0f tokens/s" % (b, dtb / args.steps * 1e3, b * args.steps / dtb))
    if 256 in point_batches:
        # one sequence of 131,072 tokens among 63 of 2,048 (the cache for batch 256 holds them): decode
        # attention deals such a step's pages out by length
        ctxs = [131072] + [2048] * 63
        dtu = time_contexts(engine, torch, "unequal64", ctxs, 32, 8)
        points["decode_1x131072_63x2048_ms_per_step"] = round(dtu * 1e3, 3)
        points["decode_1x131072_63x2048_hbm_frac"] = round(
            (weight_bytes(cfg, itemsize) + (sum(ctxs) - 64 * 16) * kv_bytes_per_token(cfg, itemsize)) / dtu / HBM_BYTES_PER_S, 4)
        log("decode of 1 x 131,072 + 63 x 2,048 tokens: %.3f ms a step" % (dtu * 1e3))
    if not (args.no_points or args.no_workloads) and args.shape == "1b" and args.layers == layers_full:
        # the family's other two shapes with the workloads named for them, each on an engine of its own
        del gen, engine
        import gc
        gc.collect()
        torch.cuda.empty_cache()
        for shape, workload, reps in (("3b", "unequal16", 3), ("8b", "batch64", 2)):
            rec = time_workload(shape, workload, args.dtype, torch, reps=reps)
            name = "%s_%s" % (shape, workload)
            points["decode_" + name] = round(rec["tok_s"], 1)
            points["decode_%s_ms_per_step" % name] = round(rec["ms_per_step"], 3)
            points["decode_%s_hbm_frac" % name] = round(rec["hbm_frac"], 4)
            points["prefill_" + name] = round(rec["prefill_tok_s"], 1)
            points["prefill_%s_ms" % name] = round(rec["prefill_ms"], 2)
            points["prefill_%s_frac" % name] = round(rec["prefill_frac"], 4)

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
                    "statistic": "median of 11 runs", "ms_min": round(pre_min * 1e3, 3),
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
