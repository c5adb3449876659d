"""The engine against the plain implementation, through the trace replay that drives the
framework's own step function and cache: each request alone and whole; with its last 32 tokens one
by one; in batches of unequal lengths whose shorter requests end earlier, one batch after another
so that slots and pages are used again; long decoding; the first tokens of a sequence.  In 32-bit
and in bfloat16, for tiny configurations that differ in every size and option."""
import io
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import traces
from helpers import assert_clear_argmax_agrees, assert_logits_close, bounds
from plain import files, llama
from tiny import TINY_A, TINY_B, TINY_C, make_model

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C}
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    base = tmp_path_factory.mktemp("models")
    out = {}
    for name, cfg in CONFIGS.items():
        path = make_model(base, cfg, seed=17 + len(name), name=name)
        cfg_json, weights = files.read_model_dir(path)
        out[name] = (path, llama.PlainConfig(cfg_json), weights)
    return out


def make_requests(cfg, lengths, seed):
    rng = np.random.default_rng(seed)
    return {"r%d" % i: rng.integers(0, cfg.vocab, size=min(n, cfg.max_pos)).tolist()
            for i, n in enumerate(lengths)}


_oracle_cache = {}


def oracle(name, cfg, weights, toks, rounded=False):
    """The plain implementation's logits at every position; ``rounded``: with stored tensors
    rounded to bfloat16 (the model of bfloat16's cost that the bounds are sized by)."""
    key = (name, tuple(toks), rounded)
    if key not in _oracle_cache:
        _oracle_cache[key] = llama.logits_all(cfg, weights, toks, store=llama.to_bfloat16 if rounded else llama.exact)
    return _oracle_cache[key]


def run_replay(path, dtype, steps, out_dir, max_tokens=None, use_graphs=True):
    from libllm_amd.engine.trace import replay
    from libllm_amd.runtime import load_engine
    need = traces.max_tokens_needed(steps)
    engine = load_engine(path, dtype=dtype, max_tokens=max_tokens or need, use_graphs=use_graphs)
    log = io.StringIO()
    replay(engine, traces.lines(steps), str(out_dir), log=log)
    assert log.getvalue().split() == [w for s in steps for w in ("done", str(s["step"]))]
    engine.cache.check()
    assert engine.cache.slots.n_free == engine.cache.slots.n_slots          # everything given back
    assert all(g.pool.n_free == g.pool.n_pages for g in engine.cache.groups)
    return engine


WORST = {}


def check(name, cfg, weights, requests, got, dtype):
    """Every position of every request against the plain implementation: both metrics within
    their bounds (helpers.bounds), and the arg-max wherever the oracle's margin is clear."""
    worst = WORST.get(dtype, (0.0, 0.0))
    for rid, toks in requests.items():
        ref = oracle(name, cfg, weights, toks)
        rounded = oracle(name, cfg, weights, toks, rounded=True) if dtype == "bfloat16" else None
        assert sorted(got[rid]) == list(range(len(toks))), "positions of %s" % rid
        out = np.stack([got[rid][p] for p in range(len(toks))])
        what = "%s %s %s" % (name, dtype, rid)
        err, row = assert_logits_close(out, ref, dtype, what, rounded)
        tol, row_tol = bounds(dtype, ref, rounded)
        assert_clear_argmax_agrees(out, ref, row_tol, what)
        worst = (max(worst[0], err / tol), max(worst[1], row / row_tol))
    WORST[dtype] = worst
    print("largest fraction of a bound used so far (%s): max metric %.2f, row metric %.2f" % ((dtype,) + worst))
    return worst


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_tail_and_batches_agree_with_plain(models, tmp_path, name, dtype):
    path, cfg, weights = models[name]
    lengths = [70, 33, 100, 5, 64, 129, 1, 65]
    requests = make_requests(cfg, lengths, seed=3)
    ids = list(requests)
    groups = [{r: requests[r] for r in ids[0:3]}, {r: requests[r] for r in ids[3:6]},
              {r: requests[r] for r in ids[6:8]}]
    decode = {"r0": 20, "r1": 32, "r2": 3, "r3": 4, "r4": 1, "r5": 40, "r6": 0, "r7": 64}
    results = {}
    for mode, steps in (("whole", traces.whole(requests)), ("tail", traces.tail_one_by_one(requests)),
                        ("batches", traces.batches(groups, decode))):
        out_dir = tmp_path / mode
        run_replay(path, dtype, steps, out_dir)            # the cache is exactly as large as needed
        got = traces.collect(steps, str(out_dir), cfg.vocab)
        check(name, cfg, weights, requests, got, dtype)
        results[mode] = got
    # the three ways of cutting agree with each other, beyond rounding
    for rid, toks in requests.items():
        a = np.stack([results["whole"][rid][p] for p in range(len(toks))])
        for mode in ("tail", "batches"):
            b = np.stack([results[mode][rid][p] for p in range(len(toks))])
            assert_logits_close(b, a, dtype, "%s against whole, %s" % (mode, rid))


@pytest.mark.parametrize("dtype", DTYPES)
def test_slots_and_pages_are_reused(models, tmp_path, dtype):
    """Six batches through a cache that holds one batch: every page and slot is used again,
    with stale keys of earlier requests still in it."""
    name = "B"
    path, cfg, weights = models[name]
    requests = make_requests(cfg, [90, 40, 120, 66, 10, 128, 77, 30, 64, 100, 3, 50], seed=8)
    ids = list(requests)
    groups = [{r: requests[r] for r in ids[i:i + 2]} for i in range(0, len(ids), 2)]
    steps = traces.batches(groups)
    run_replay(path, dtype, steps, tmp_path, max_tokens=traces.max_tokens_needed(steps))
    check(name, cfg, weights, requests, traces.collect(steps, str(tmp_path), cfg.vocab), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("use_graphs", [True, False])
def test_long_decoding(models, tmp_path, dtype, use_graphs):
    """A short prompt, then 200 tokens one by one across three page borders, three requests
    of different lengths together."""
    name = "A" if use_graphs else "C"
    path, cfg, weights = models[name]
    base = 120 if name == "A" else 260
    requests = make_requests(cfg, [base, base - 57, base - 101], seed=5)
    decode = {r: len(t) - 3 for r, t in requests.items()}
    steps = traces.batches([requests], decode)
    run_replay(path, dtype, steps, tmp_path, use_graphs=use_graphs)
    check(name, cfg, weights, requests, traces.collect(steps, str(tmp_path), cfg.vocab), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_first_tokens(models, tmp_path, dtype):
    name = "B"
    path, cfg, weights = models[name]
    requests = make_requests(cfg, [1, 2, 3, 4], seed=6)
    for mode, steps in (("whole", traces.whole(requests)), ("tail", traces.tail_one_by_one(requests)),
                        ("batch", traces.batches([requests], {r: len(t) - 1 for r, t in requests.items()}))):
        out_dir = tmp_path / mode
        run_replay(path, dtype, steps, out_dir)
        check(name, cfg, weights, requests, traces.collect(steps, str(out_dir), cfg.vocab), dtype)


def _is_matrix(name, arr):
    return arr.ndim == 2


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,stored", [("A", "float32"), ("B", "float32"), ("C", "float16")])
def test_files_of_other_float_types(tmp_path, name, stored, dtype):
    """Model files that store float32 (full significands, jittered norm scales) or float16.  The
    32-bit engine must keep every bit of them: a path that rounded a weight, a norm scale or a bias
    to bfloat16 between the file and a kernel would be a thousand times beyond the 32-bit bound.
    The bfloat16 engine must turn every matrix into bfloat16 at load, as the reference casts every
    float tensor to its device's type (src/libllm/var_builder.cc:113-125), keep the vectors in
    32-bit, and run the matrix-core products: it is compared with the plain implementation on
    matrices rounded the same way."""
    from libllm_amd.hip.ops import PreparedWeight
    path = make_model(tmp_path, CONFIGS[name], seed=23, name=name + stored, stored=stored)
    cfg_json, weights = files.read_model_dir(path)
    cfg = llama.PlainConfig(cfg_json)
    assert any(np.any(w != llama.to_bfloat16(w)) for w in weights.values())     # the file needs more than bfloat16
    if dtype == "bfloat16":
        weights = {n: llama.to_bfloat16(w) if _is_matrix(n, w) else w for n, w in weights.items()}
    requests = make_requests(cfg, [70, 9, 100, 33, 1], seed=31)
    steps = traces.batches([requests], {r: min(8, len(t) - 1) for r, t in requests.items()})
    engine = run_replay(path, dtype, steps, tmp_path / dtype)
    tag = name + stored + dtype
    check(tag, cfg, weights, requests, traces.collect(steps, str(tmp_path / dtype), cfg.vocab), dtype)
    for block in engine.model.blocks:
        for lin in (block.mixer.qkv, block.mixer.out, block.feed_forward.gate_up, block.feed_forward.down):
            if dtype == "bfloat16":
                assert isinstance(lin.prepared, PreparedWeight) and lin.weight.dtype == torch.bfloat16
            else:
                assert lin.weight.dtype == torch.float32
        assert all(n.weight.dtype == torch.float32 for n in block.norms)


def test_matrices_kept_in_32_bit_on_request(tmp_path):
    """``keep_float32``: in bfloat16 mode the matrices of a float32 file stay float32 and their
    products run in true 32-bit; activations and the cache are bfloat16 all the same."""
    from libllm_amd.engine.trace import replay
    from libllm_amd.runtime import load_engine
    path = make_model(tmp_path, CONFIGS["A"], seed=24, name="kept", stored="float32")
    cfg_json, weights = files.read_model_dir(path)
    cfg = llama.PlainConfig(cfg_json)
    requests = make_requests(cfg, [40, 7, 66], seed=32)
    steps = traces.batches([requests], {r: 4 for r in requests})
    engine = load_engine(path, dtype="bfloat16", max_tokens=traces.max_tokens_needed(steps), keep_float32=True)
    assert engine.model.blocks[0].mixer.qkv.weight.dtype == torch.float32
    replay(engine, traces.lines(steps), str(tmp_path / "out"), log=io.StringIO())
    check("kept", cfg, weights, requests, traces.collect(steps, str(tmp_path / "out"), cfg.vocab), "bfloat16")


@pytest.fixture(scope="module")
def long_models(tmp_path_factory):
    """The tiny configurations with position limits beyond a thousand, so that one request of a
    batch can be long while the others are short."""
    base = tmp_path_factory.mktemp("long_models")
    out = {}
    for name, limit in (("A", 1536), ("B", 2304), ("C", 1100)):
        cfg = dict(CONFIGS[name], max_position_embeddings=limit)
        path = make_model(base, cfg, seed=5 + len(out), name=name)
        cfg_json, weights = files.read_model_dir(path)
        out[name] = (path, llama.PlainConfig(cfg_json), weights)
    return out


EDGE_LENGTHS = [1, 2, 15, 16, 17, 31, 33, 63, 64, 65, 127, 128, 129, 191, 192, 193, 255, 256, 257]


def random_trace(rng, cfg):
    """One to three batches after one another.  A batch has up to 33 requests that start together,
    lengths drawn around page and tile borders, sometimes one of about a thousand tokens among
    them.  Half the time the prompts come in chunks of unequal sizes, a chunk for every request
    that still has prompt left; then one token a step, the shorter requests ending earlier."""
    steps, requests = [], {}
    for _ in range(int(rng.integers(1, 4))):
        group = {}
        long_one = rng.random() < 0.4
        for i in range(int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 13, 16, 17, 25, 33]))):
            if long_one and i == 0:
                n = int(rng.integers(900, cfg.max_pos))
            elif rng.random() < 0.5:
                n = int(rng.choice(EDGE_LENGTHS)) + 64 * int(rng.integers(0, 2))
            else:
                n = int(rng.integers(1, 300))
            group["q%d" % (len(requests) + len(group))] = rng.integers(0, cfg.vocab, size=min(n, cfg.max_pos)).tolist()
        requests.update(group)
        sub = traces.batches([group], {r: int(rng.integers(0, min(len(t), 40))) for r, t in group.items()})
        if rng.random() < 0.5:
            left = {e["id"]: list(e["tokens"]) for e in sub[0]["entries"]}
            chunks = []
            while any(left.values()):
                entries = []
                for r in left:
                    if left[r]:
                        k = int(rng.choice([1, 3, 16, 63, 64, 65, 100, 400]))
                        entries.append({"id": r, "tokens": left[r][:k], "want": list(range(len(left[r][:k])))})
                        left[r] = left[r][k:]
                chunks.append({"entries": entries, "end": []})
            for r in sub[0]["end"]:                          # a request that is all prompt ends with its last chunk
                [c for c in chunks if any(e["id"] == r for e in c["entries"])][-1]["end"].append(r)
            sub = chunks + sub[1:]
        for s in sub:
            s["step"] = len(steps)
            steps.append(s)
    return steps, requests


@pytest.mark.parametrize("case", range(66))
def test_random_traces(long_models, tmp_path, case):
    """Drawn batches, cuts and cache sizes (see random_trace) in both dtypes, with and without
    captured graphs (every fourth group of six without), every position of every request against
    the plain implementation."""
    name, dtype, use_graphs = "ABC"[case % 3], DTYPES[(case // 3) % 2], (case // 6) % 4 != 3
    path, cfg, weights = long_models[name]
    rng = np.random.default_rng(1000 + case)
    steps, requests = random_trace(rng, cfg)
    spare = int(rng.choice([0, 0, 64, 640]))
    run_replay(path, dtype, steps, tmp_path, max_tokens=traces.max_tokens_needed(steps) + spare, use_graphs=use_graphs)
    check("long" + name, cfg, weights, requests, traces.collect(steps, str(tmp_path), cfg.vocab), dtype)


def drawn_config(rng):
    """A tiny configuration with every size and option drawn: 1 to 5 kv heads with 1 to 8 query
    heads each, head sizes of 16 to 128, widths and feed-forwards in multiples of 8, any
    vocabulary, the three rotary scalings, biases, tied or untied output, either eps."""
    n_kv = int(rng.choice([1, 2, 3, 4, 5]))
    scaling = [None, {"rope_type": "linear", "factor": float(rng.choice([2.0, 4.0]))},
               {"rope_type": "llama3", "factor": float(rng.choice([8.0, 32.0])), "low_freq_factor": 1.0,
                "high_freq_factor": 4.0,
                "original_max_position_embeddings": int(rng.choice([32, 64, 128]))}][int(rng.integers(0, 3))]
    return {"model_type": "llama", "num_hidden_layers": int(rng.integers(1, 4)),
            "hidden_size": 8 * int(rng.integers(4, 48)), "num_attention_heads": n_kv * int(rng.choice([1, 2, 3, 4, 8])),
            "num_key_value_heads": n_kv, "head_dim": int(rng.choice([16, 32, 48, 64, 80, 96, 112, 128])),
            "intermediate_size": 8 * int(rng.integers(6, 90)), "vocab_size": int(rng.integers(64, 3000)),
            "rope_theta": float(rng.choice([10000.0, 500000.0])), "rope_scaling": scaling,
            "rms_norm_eps": float(rng.choice([1e-5, 1e-6])), "tie_word_embeddings": bool(rng.integers(0, 2)),
            "max_position_embeddings": 256, "attention_bias": bool(rng.integers(0, 2)), "hidden_act": "silu",
            "eos_token_id": 2}


@pytest.mark.parametrize("seed", range(12))
def test_drawn_configurations(tmp_path, seed):
    """Configurations drawn at random (see drawn_config) with requests of drawn lengths: whole,
    with the last tokens one by one, and in two batches, in both dtypes, every position against
    the plain implementation."""
    rng = np.random.default_rng(7000 + seed)
    name = "drawn%d" % seed
    path = make_model(tmp_path, drawn_config(rng), seed=seed, name=name)
    cfg_json, weights = files.read_model_dir(path)
    cfg = llama.PlainConfig(cfg_json)
    requests = make_requests(cfg, [int(n) for n in rng.integers(1, 150, size=int(rng.integers(3, 8)))], seed=seed)
    ids = list(requests)
    half = max(1, len(ids) // 2)
    groups = [{r: requests[r] for r in ids[:half]}, {r: requests[r] for r in ids[half:]}]
    for dtype in DTYPES:
        for mode, steps in (("whole", traces.whole(requests)), ("tail", traces.tail_one_by_one(requests)),
                            ("batches", traces.batches(groups))):
            out_dir = tmp_path / (dtype + mode)
            run_replay(path, dtype, steps, out_dir)
            check(name, cfg, weights, requests, traces.collect(steps, str(out_dir), cfg.vocab), dtype)


@pytest.mark.parametrize("case", range(6))
def test_batches_of_more_than_128_requests(long_models, tmp_path, case):
    """160 to 250 short requests start together and decode a few tokens each, the shorter ones
    ending earlier: the decode graphs of 160 to 256 rows and those below as the batch thins out
    (the last two cases without graphs), every position against the plain implementation."""
    name, dtype, use_graphs = "ABC"[case % 3], DTYPES[case % 2], case < 4
    path, cfg, weights = long_models[name]
    rng = np.random.default_rng(5000 + case)
    n = [250, 170, 200, 161, 250, 160][case]
    group = {"q%d" % i: rng.integers(0, cfg.vocab, size=int(rng.integers(1, 40))).tolist() for i in range(n)}
    tails = {r: int(rng.integers(1, 12)) if len(t) > 12 else int(rng.integers(0, len(t))) for r, t in group.items()}
    steps = traces.batches([group], tails)
    for i, s in enumerate(steps):
        s["step"] = i
    engine = run_replay(path, dtype, steps, tmp_path, max_tokens=traces.max_tokens_needed(steps), use_graphs=use_graphs)
    assert (max(k[0] for k in engine._graphs) > 128) if use_graphs else not engine._graphs
    check("long" + name, cfg, weights, group, traces.collect(steps, str(tmp_path), cfg.vocab), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("use_graphs", [True, False])
def test_a_long_request_among_short_ones(long_models, tmp_path, monkeypatch, dtype, use_graphs):
    """One request of two thousand tokens decodes beside nine of a few dozen: such a step is run
    with its decode attention dealt out by length (a graph of its own kind), and when the long
    request has ended the others go on in the uniform kind; every position against the plain
    implementation."""
    from libllm_amd.engine import Engine
    monkeypatch.setattr(Engine, "UNEQUAL_MIN", 512)          # (the tiny configurations stop far below 4,096 tokens)
    path, cfg, weights = long_models["B"]
    rng = np.random.default_rng(77)
    group = {"long": rng.integers(0, cfg.vocab, size=2050).tolist()}
    group.update({"s%d" % i: rng.integers(0, cfg.vocab, size=int(n)).tolist() for i, n in enumerate(rng.integers(20, 70, size=9))})
    tails = {r: 18 for r in group}
    tails["long"] = 6                                           # it ends first; the short ones decode on
    steps = traces.batches([group], tails)
    for i, s in enumerate(steps):
        s["step"] = i
    engine = run_replay(path, dtype, steps, tmp_path, max_tokens=traces.max_tokens_needed(steps), use_graphs=use_graphs)
    if use_graphs:
        assert {k[2] for k in engine._graphs} == {True, False}      # graphs of both kinds were made
    check("long" + "B", cfg, weights, group, traces.collect(steps, str(tmp_path), cfg.vocab), dtype)


BENCH_SHAPES = {
    "1b": dict(hidden_size=2048, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
               intermediate_size=8192, tie_word_embeddings=True, factor=32.0),
    # the shape of the reference's own model test (src/libllm/llama_test.cc:44-45): groups of three heads
    "3b": dict(hidden_size=3072, num_attention_heads=24, num_key_value_heads=8, head_dim=128,
               intermediate_size=8192, tie_word_embeddings=True, factor=32.0),
    "8b": dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
               intermediate_size=14336, tie_word_embeddings=False, factor=8.0),
}


@pytest.mark.parametrize("shape", list(BENCH_SHAPES))
def test_layers_of_the_measured_shapes(tmp_path, shape):
    """Two layers of the sizes that the measurements run (a smaller vocabulary, no power of two)
    against the plain implementation.  The launcher picks the form of a product and of attention
    by the sizes and by the rows of a step, so the tiny configurations do not reach every form:
    batches of 1, 8, 20, 48 and 64 decode through each form of the skinny product and, from 33
    rows on, the product for 33 to 128 rows, as do batches of 96 and 128 and a prompt of 100
    tokens; a batch of 200, a prompt of 230 tokens and two of 75 (a step of some 160 rows) go through
    the same product in two slabs of rows; the three prompts of 670 tokens (a step of some 2,030 rows) go through the library's
    products and, for the gate and up weights of the 1B and 3B shapes, the product for many rows
    (test_the_gate_and_up_product_of_a_long_prompt_is_ours sees that it runs)."""
    sh = dict(BENCH_SHAPES[shape])
    cfg_dict = {"model_type": "llama", "num_hidden_layers": 2, "vocab_size": 8009, "rope_theta": 500000.0,
                "rope_scaling": {"rope_type": "llama3", "factor": sh.pop("factor"), "low_freq_factor": 1.0,
                                 "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
                "rms_norm_eps": 1e-5, "max_position_embeddings": 4096, "hidden_act": "silu",
                "eos_token_id": 2, **sh}
    path = make_model(tmp_path, cfg_dict, seed=3, std=0.02, norm_std=0.1, name=shape)
    cfg_json, weights = files.read_model_dir(path)
    cfg = llama.PlainConfig(cfg_json)
    rng = np.random.default_rng(1)
    for batch, prompt, decode, dtypes in ((1, 40, 5, DTYPES), (8, 30, 5, DTYPES), (20, 20, 3, DTYPES),
                                          (48, 10, 3, ["bfloat16"]), (64, 8, 3, DTYPES), (3, 670, 2, ["bfloat16"]),
                                          (96, 6, 3, ["bfloat16"]), (1, 100, 2, ["bfloat16"]), (128, 1, 2, ["bfloat16"]),
                                          (200, 1, 2, ["bfloat16"]), (1, 230, 2, ["bfloat16"]), (2, 75, 2, ["bfloat16"])):
        group = {"s%d_%d" % (batch, i): rng.integers(0, cfg.vocab, size=prompt + int(rng.integers(0, 9)) + decode).tolist()
                 for i in range(batch)}
        steps = traces.batches([group], {r: decode for r in group})
        checked = dict(list(group.items())[:3] + list(group.items())[-1:])
        for dtype in dtypes:
            out_dir = tmp_path / ("%s_%d_%s" % (shape, batch, dtype))
            run_replay(path, dtype, steps, out_dir, max_tokens=traces.max_tokens_needed(steps) + 64)
            check(shape, cfg, weights, checked, traces.collect(steps, str(out_dir), cfg.vocab), dtype)


def test_the_gate_and_up_product_of_a_long_prompt_is_ours():
    """A step of 2,030 rows at the 1B shape's widths: every layer's gate and up product with its
    SwiGLU is the kernel for many rows, also in the captured prompt graph that the second such step
    makes; a step of 600 rows, whose tiles would fill half a round of the device, is the library's."""
    from libllm_amd.config import config_from_dict
    from libllm_amd.engine import StepEntry
    from libllm_amd.runtime import random_engine
    sh = dict(BENCH_SHAPES["1b"])
    cfg_dict = {"model_type": "llama", "num_hidden_layers": 2, "vocab_size": 8009, "rope_theta": 500000.0,
                "rope_scaling": {"rope_type": "llama3", "factor": sh.pop("factor"), "low_freq_factor": 1.0,
                                 "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
                "rms_norm_eps": 1e-5, "max_position_embeddings": 4096, "hidden_act": "silu",
                "eos_token_id": 2, **sh}
    engine = random_engine(config_from_dict(cfg_dict), seed=5, dtype="bfloat16", max_tokens=8192)
    calls = []
    real = engine.ops._wide
    engine.ops._wide = lambda *a: (calls.append(a[0].shape[0]), real(*a))[1]
    rng = np.random.default_rng(9)
    outs = []
    toks = rng.integers(0, 8009, size=2030).tolist()
    for rep in range(3):                                   # the second coming of the shape captures a graph
        outs.append(engine.step([StepEntry(("long", rep), toks, [2029])]).clone())
        engine.end([("long", rep)])
    assert calls and all(m >= 2030 for m in calls) and len(calls) >= 2 * 2, calls
    assert torch.equal(outs[1], outs[2])                   # the same prompt from the graph, twice
    # (that the graph's values are right is test_library_products_inside_prompt_graphs' matter, bit
    # for bit at rows that fill a graph, and test_gemm_wide_swiglu's; the first step here has 2,030
    # rows where the graph has 2,048, so the library may pick other kernels for it)
    calls.clear()
    engine.step([StepEntry("short", rng.integers(0, 8009, size=600).tolist(), [599])])
    assert not calls


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_prompt_of_thousands_of_rows(tmp_path, dtype):
    """A prompt of 3,700 tokens in one step (beyond the captured prompt graphs; in bfloat16 the
    form of prompt attention in which a wave takes two tiles of rows), then a second request in a
    batch with its last tokens one by one across a page border, every position against the plain
    implementation."""
    cfg_dict = dict(TINY_A, max_position_embeddings=4096)
    path = make_model(tmp_path, cfg_dict, seed=41, name="long")
    cfg_json, weights = files.read_model_dir(path)
    cfg = llama.PlainConfig(cfg_json)
    requests = make_requests(cfg, [3700, 3650], seed=42)
    steps = traces.whole({"r0": requests["r0"]}) + traces.batches([{"r1": requests["r1"]}], {"r1": 20})
    for i, s in enumerate(steps):
        s["step"] = i
    out_dir = tmp_path / dtype
    run_replay(path, dtype, steps, out_dir)
    check("long", cfg, weights, requests, traces.collect(steps, str(out_dir), cfg.vocab), dtype)


def test_a_request_of_nine_thousand_tokens(tmp_path):
    """One request of 9,300 tokens, whole and with its last 32 tokens one by one, in both dtypes,
    every position against the plain implementation (src/libllm/llama_test.cc:194-224 walks a
    prompt whole and token by token): a prompt step of thousands of rows beyond the captured
    graphs, and decode steps over 146 pages, where a wave of decode attention walks several."""
    cfg_dict = dict(TINY_A, max_position_embeddings=16384)
    path = make_model(tmp_path, cfg_dict, seed=43, name="long9k")
    cfg_json, weights = files.read_model_dir(path)
    cfg = llama.PlainConfig(cfg_json)
    requests = make_requests(cfg, [9300], seed=44)
    for dtype in DTYPES:
        for mode, steps in (("whole", traces.whole(requests)), ("tail", traces.tail_one_by_one(requests))):
            out_dir = tmp_path / (dtype + mode)
            run_replay(path, dtype, steps, out_dir)
            check("long9k", cfg, weights, requests, traces.collect(steps, str(out_dir), cfg.vocab), dtype)


def test_the_1b_shape_whole_in_32_bit_and_bfloat16():
    """All 16 layers of the measured 1B shape with its vocabulary of 128,256, random weights drawn
    on the device, in true 32-bit and in bfloat16: an unequal batch of three prompts (247 rows: the
    library's products in bfloat16), then four tokens each, the logits at the wanted places
    against the plain implementation run on the same weights."""
    import bench
    from libllm_amd.config import config_from_dict
    from libllm_amd.engine import StepEntry
    from libllm_amd.runtime import random_engine
    from libllm_amd.weights import random_tensors
    config = config_from_dict(dict(bench.FULL, max_position_embeddings=4096))
    cfg = llama.PlainConfig(config.to_dict())
    rng = np.random.default_rng(77)
    toks = {i: rng.integers(0, cfg.vocab, size=n + 4).tolist() for i, n in enumerate((200, 40, 7))}
    weights, ref, rounded = None, {}, {}
    for dtype in DTYPES:
        engine = random_engine(config, seed=3, dtype=dtype, max_tokens=1024)
        if weights is None:
            # the random-weights mode draws every tensor from (seed, name): the same draw here
            declared = engine.model.declared()
            weights = {name: random_tensors({name: declared[name]}, 3, std=0.02, dtype=torch.bfloat16,
                                            device="cuda")[name].double().cpu().numpy() for name in declared}
            for i, t in toks.items():
                rows = list(range(len(t) - 5, len(t)))
                ref[i] = llama.lm_head(cfg, weights, llama.hidden_states(cfg, weights, t)[rows])
                rounded[i] = llama.lm_head(cfg, weights, llama.hidden_states(cfg, weights, t, store=llama.to_bfloat16)[rows])
        got = {i: [] for i in toks}
        out = engine.step([StepEntry(i, t[:-4], [len(t) - 5]) for i, t in toks.items()])
        for j, i in enumerate(toks):
            got[i].append(out[j].double().cpu().numpy())
        for k in range(4):
            out = engine.step([StepEntry(i, [t[len(t) - 4 + k]], [0]) for i, t in toks.items()])
            for j, i in enumerate(toks):
                got[i].append(out[j].double().cpu().numpy())
        for i in toks:
            assert_logits_close(np.stack(got[i]), ref[i], dtype, "1b %s request %d" % (dtype, i),
                                rounded[i] if dtype == "bfloat16" else None)
        del engine


ODD = {
    "width 100, feed-forward 150, vocabulary 101": dict(hidden_size=100, num_attention_heads=5, num_key_value_heads=5,
                                                        intermediate_size=150, vocab_size=101),
    "odd width 65, vocabulary 3": dict(hidden_size=65, intermediate_size=91, vocab_size=3),
    "head size 80": dict(hidden_size=160, num_attention_heads=2, num_key_value_heads=1, head_dim=80),
    "head size 112": dict(hidden_size=112, num_attention_heads=2, num_key_value_heads=2, head_dim=112),
    "head size 256": dict(hidden_size=256, num_attention_heads=2, num_key_value_heads=1, head_dim=256),
    "head size 24": dict(hidden_size=96, num_attention_heads=4, num_key_value_heads=2, head_dim=24),
    "seven heads, seven kv heads": dict(hidden_size=112, num_attention_heads=7, num_key_value_heads=7),
    "a group of 20 heads": dict(hidden_size=80, num_attention_heads=20, num_key_value_heads=1),
    "a group of 40 heads": dict(hidden_size=80, num_attention_heads=40, num_key_value_heads=1, head_dim=32),
    "one layer, one head": dict(num_hidden_layers=1, hidden_size=16, num_attention_heads=1, num_key_value_heads=1,
                                intermediate_size=8, vocab_size=9),
    "feed-forward of one, vocabulary 70001": dict(intermediate_size=1, vocab_size=70001),
    "width 72, a multiple of 8 only": dict(hidden_size=72, num_attention_heads=3, num_key_value_heads=1, head_dim=32,
                                          intermediate_size=88, vocab_size=33),
    "width 66, a multiple of 2 only": dict(hidden_size=66, intermediate_size=90, vocab_size=77),
    "head size 96": dict(hidden_size=96, num_attention_heads=3, num_key_value_heads=3, head_dim=96),
    "head size 8": dict(hidden_size=32, num_attention_heads=4, num_key_value_heads=2, head_dim=8),
    "a group of 8 heads": dict(hidden_size=128, num_attention_heads=16, num_key_value_heads=2),
    # Widths that are multiples of 8 and not of 32 or 16: the skinny product's last step of K is
    # short, the SwiGLU epilogue is not taken, the library's products run at 65 rows and more.  At
    # the tests' spread of 0.08 a row of 2,056 columns gives products of spread 3.6: the softmax
    # is sharply peaked and bfloat16 costs six times what it costs the tiny configurations (the
    # plain implementation with stored tensors rounded to bfloat16 is 0.078 off in the row metric
    # and 0.32 in the max metric, where Tiny A is 0.012 and 0.05 off).  The bounds follow that, so in
    # bfloat16 this case decides nothing (a bound of 0.8 in the max metric would let a wrong tile
    # through): what holds here is the 32-bit run of the same case, bound 1e-4, and the kernel
    # tests of the short last step of K (test_gemm_skinny at K = 136, 264, 4,104 and 72).
    "width 2056, feed-forward 8200": dict(hidden_size=2056, num_attention_heads=8, num_key_value_heads=4, head_dim=64,
                                          intermediate_size=8200, vocab_size=500),
    # the same at a spread of 0.02 (products of spread 0.9): bfloat16 costs what it costs Tiny A,
    # and the bounds are as tight as there
    "width 2056, feed-forward 8200, spread 0.02": dict(hidden_size=2056, num_attention_heads=8, num_key_value_heads=4,
                                                       head_dim=64, intermediate_size=8200, vocab_size=500, spread=0.02),
}


@pytest.mark.parametrize("what", list(ODD))
def test_odd_sizes_end_to_end(tmp_path, what):
    """Sizes that a configuration may have and no released model has, through the whole engine in
    both dtypes: a batch of up to 18 unequal prompts, then six tokens each."""
    cfg_dict = dict(TINY_A, max_position_embeddings=512, **ODD[what])
    path = make_model(tmp_path, cfg_dict, seed=len(what), name="odd", std=cfg_dict.pop("spread", 0.08))
    cfg_json, weights = files.read_model_dir(path)
    cfg = llama.PlainConfig(cfg_json)
    lengths = [70, 9, 131, 20, 1, 64, 33, 200, 5, 17, 90, 40, 3, 66, 128, 12, 7, 100]
    requests = make_requests(cfg, lengths[:18 if len(what) % 2 else 5], seed=len(what))
    steps = traces.batches([requests], {r: min(6, len(t) - 1) for r, t in requests.items()})
    for dtype in DTYPES:
        out_dir = tmp_path / dtype
        run_replay(path, dtype, steps, out_dir)
        check(what, cfg, weights, requests, traces.collect(steps, str(out_dir), cfg.vocab), dtype)


def test_a_head_size_beyond_the_kernels_is_refused(tmp_path):
    from libllm_amd.errors import KernelError
    from libllm_amd.engine import StepEntry
    from libllm_amd.runtime import load_engine
    path = make_model(tmp_path, dict(TINY_A, hidden_size=272, num_attention_heads=1, num_key_value_heads=1,
                                     head_dim=272), seed=1, name="wide_head")
    with pytest.raises(KernelError, match="head_dim 272"):
        load_engine(path, dtype="bfloat16", max_tokens=64).step([StepEntry("a", [1, 2, 3], [2])])


def _decode_rows(engine, requests, n_last):
    from libllm_amd.engine import StepEntry
    engine.step([StepEntry(r, t[:-n_last], []) for r, t in requests.items()])
    rows = []
    for i in range(n_last, 0, -1):
        out = engine.step([StepEntry(r, [t[-i]], [0]) for r, t in requests.items()])
        rows.append(out.cpu().numpy().copy())
    return np.stack(rows)                                    # [steps, requests, vocab]


def test_padding_changes_nothing(models):
    """Five sequences decode through the graph captured for six rows, the sixth row being
    padding.  In 32-bit the same bits come out without graphs (no padding row at all); in
    bfloat16 the same bits come out when the sixth row is a real sequence."""
    from libllm_amd.runtime import load_engine
    path, cfg, weights = models["A"]
    five = make_requests(cfg, [9, 70, 31, 12, 44], seed=12)
    six = dict(five, extra=make_requests(cfg, [50], seed=13)["r0"])
    padded = load_engine(path, dtype="float32", max_tokens=1024, use_graphs=True)
    plain_path = load_engine(path, dtype="float32", max_tokens=1024, use_graphs=False)
    a, b = _decode_rows(padded, five, 4), _decode_rows(plain_path, five, 4)
    assert [k[0] for k in padded._graphs] == [6] and not plain_path._graphs
    assert np.array_equal(a, b)
    e5 = load_engine(path, dtype="bfloat16", max_tokens=1024, use_graphs=True)
    e6 = load_engine(path, dtype="bfloat16", max_tokens=1024, use_graphs=True)
    a, b = _decode_rows(e5, five, 4), _decode_rows(e6, six, 4)
    assert [k[0] for k in e5._graphs] == [6] and [k[0] for k in e6._graphs] == [6]
    assert np.array_equal(a, b[:, :5])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("use_graphs", [False, True])
def test_steps_seen_before_ask_the_device_for_no_memory(models, use_graphs, dtype):
    """Once steps of some shapes have run, steps of those shapes ask the device for no memory:
    what the operations allocate is cut from blocks that the process holds already (a captured
    graph's own pool; for steps queued kernel by kernel the pool that hands a step's blocks
    back as its tensors die, as the reference's stream-ordered pool does,
    src/flint/cuda/common.h:116-142).  Counted by the pool's requests to the device and by the
    bytes it holds."""
    import torch
    from libllm_amd.engine import StepEntry
    from libllm_amd.runtime import load_engine
    path, cfg, _ = models["A"]
    engine = load_engine(path, dtype=dtype, max_tokens=1024, use_graphs=use_graphs)
    lengths = [9, 70, 31]

    def batch(seed):
        requests = make_requests(cfg, lengths, seed=seed)
        engine.step([StepEntry(r, t, [len(t) - 1]) for r, t in requests.items()])
        for k in range(6):
            out = engine.step([StepEntry(r, [(seed + k) % cfg.vocab], [0]) for r in requests])
        engine.end(list(requests))
        return out.float().sum().item()                      # waits for the device

    for seed in range(3):                                    # a prompt's graph is captured when its shape comes again
        batch(seed)
    stats = torch.cuda.memory_stats()
    asked, held = stats["num_device_alloc"], stats["reserved_bytes.all.current"]
    for seed in range(3, 7):
        batch(seed)
    stats = torch.cuda.memory_stats()
    assert stats["num_device_alloc"] == asked and stats["reserved_bytes.all.current"] == held
    assert bool(engine._graphs) == use_graphs and bool(engine._prompt_graphs) == use_graphs


def test_a_captured_step_whose_replay_differs_is_not_used(models, monkeypatch):
    """A captured decode step is replayed twice before it serves and compared, bit for bit, with
    the same step queued kernel by kernel (work may be recorded that does not replay).  Here the
    comparison is made to fail: the engine warns, keeps no graph for that shape, and its steps
    give what an engine without graphs gives."""
    from libllm_amd.engine import step as step_mod
    from libllm_amd.runtime import load_engine
    path, cfg, _ = models["A"]
    requests = make_requests(cfg, [9, 70, 31], seed=5)
    plain_path = load_engine(path, dtype="bfloat16", max_tokens=1024, use_graphs=False)
    want = _decode_rows(plain_path, requests, 4)
    checked = load_engine(path, dtype="bfloat16", max_tokens=1024)
    assert np.array_equal(_decode_rows(checked, requests, 4), want) and checked._graphs and not checked._no_graph
    calls = []
    monkeypatch.setattr(step_mod._CapturedForward, "_same", staticmethod(lambda out, ref: bool(calls.append(1))))
    engine = load_engine(path, dtype="bfloat16", max_tokens=1024)
    with pytest.warns(UserWarning, match="run without a captured graph"):
        got = _decode_rows(engine, requests, 4)
    assert len(calls) == 1 and not engine._graphs
    assert engine._no_graph == {("decode", 3, 128, False)}  # (the position limit of this configuration is 128; lengths not far apart)
    assert np.array_equal(got, want)


def test_a_library_product_that_does_not_replay_is_not_captured(models, monkeypatch):
    """Before a product of the vendor library is recorded into a graph, its shape is tried alone:
    recorded, replayed over new rows and compared with the product queued directly.  Shapes that
    pass are remembered; here the trial is then made to fail, and the prompt step that holds such
    a product runs without a graph, with a warning, and gives the same logits."""
    from libllm_amd.engine import StepEntry
    from libllm_amd.hip.ops import HipOps
    from libllm_amd.runtime import load_engine
    path, cfg, _ = models["C"]
    prompt = make_requests(cfg, [150], seed=8)["r0"]

    def logits(engine):
        engine.PROMPT_SEEN = 1
        out = []
        for k in range(3):
            out.append(engine.step([StepEntry("p", prompt, [len(prompt) - 1])]).cpu().numpy().copy())
            engine.end(["p"])
        assert all(np.array_equal(o, out[0]) for o in out)
        return out[0]

    engine = load_engine(path, dtype="bfloat16", max_tokens=1024)
    monkeypatch.setattr(HipOps, "_replayable", {})
    want = logits(engine)
    assert list(engine._prompt_graphs) == [(176, 2)]
    tried = engine.ops._replayable
    assert tried and all(tried.values()) and all(key[0] == 176 for key in tried)
    monkeypatch.setattr(HipOps, "_replayable", {})
    monkeypatch.setattr(HipOps, "_product_replays", lambda self, x, w: False)
    other = load_engine(path, dtype="bfloat16", max_tokens=1024)
    with pytest.warns(UserWarning, match="does not replay from a captured graph"):
        got = logits(other)
    assert not other._prompt_graphs and other._no_graph == {("prompt", 176, 2)}
    assert np.array_equal(got, want)


@pytest.mark.parametrize("name", list(CONFIGS))
def test_norms_between_products_get_no_kernel(models, name):
    """Decoding up to 16 rows in bfloat16, the product that adds into the stream prepares the RMS
    norm after it and the next product applies the row's scale; the embedding prepares the first
    norm of a step in the same way, and where every row's logits are wanted the last product
    prepares the final norm: the norm kernel then does not run at all.  Logits against the plain
    implementation, and against an engine that runs every norm as a kernel."""
    from libllm_amd.runtime import load_engine
    path, cfg, weights = models[name]
    requests = make_requests(cfg, [9, 30, 17, 6], seed=45)
    folded = load_engine(path, dtype="bfloat16", max_tokens=1024, use_graphs=False)
    kernels = load_engine(path, dtype="bfloat16", max_tokens=1024, use_graphs=False)
    kernels.ops.fold_norms = False
    calls = {}
    for tag, e in (("folded", folded), ("kernels", kernels)):
        real = e.ops.add_rmsnorm
        def counted(*a, _real=real, _tag=tag, **k):
            calls[_tag] = calls.get(_tag, 0) + 1
            return _real(*a, **k)
        e.ops.add_rmsnorm = counted
    a, b = _decode_rows(folded, requests, 4), _decode_rows(kernels, requests, 4)
    n_layers = len(folded.model.spec.schedule)
    prompt = 2 * n_layers                                       # the prompt step: more than 16 rows, no logits wanted
    assert calls["kernels"] == prompt + 4 * (2 * n_layers + 1)
    assert calls.get("folded", 0) == prompt
    assert_logits_close(a, b.astype(np.float64), "bfloat16", "folded norms against norm kernels")
    for i, (rid, toks) in enumerate(requests.items()):
        ref, rounded = oracle(name, cfg, weights, toks), oracle(name, cfg, weights, toks, rounded=True)
        rows = slice(len(toks) - 4, len(toks))                  # step s fed token -(4 - s): logits at that position
        assert_logits_close(a[:, i], ref[rows], "bfloat16", rid, rounded[rows])


@pytest.mark.parametrize("dtype", DTYPES)
def test_batch_order_changes_nothing(models, dtype):
    """The same requests in the opposite order take other slots and other rows of every step.
    Prompts short enough for the kernels whose sums do not depend on the row (at most 64 rows a
    step): the same bits for every request, in 32-bit and in bfloat16.  And a request alone
    gives what it gives inside the batch."""
    from libllm_amd.runtime import load_engine
    path, cfg, weights = models["B"]
    requests = make_requests(cfg, [9, 30, 17], seed=44)              # 44 rows of prompt, then 4 tokens each
    swapped = dict(reversed(list(requests.items())))
    e1 = load_engine(path, dtype=dtype, max_tokens=1024)
    e2 = load_engine(path, dtype=dtype, max_tokens=1024)
    a, b = _decode_rows(e1, requests, 4), _decode_rows(e2, swapped, 4)
    assert np.array_equal(a, b[:, ::-1])
    e3 = load_engine(path, dtype=dtype, max_tokens=1024)
    alone = _decode_rows(e3, {"r1": requests["r1"]}, 4)
    if dtype == "float32":
        assert np.array_equal(alone[:, 0], a[:, 1])
    else:
        assert_logits_close(alone[:, 0], a[:, 1].astype(np.float64), dtype, "alone against in a batch")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_prompt_steps_through_graphs(models, name, dtype):
    """Steps that bring whole prompts replay captured graphs, padded to fixed numbers of rows and
    sequences (here from the first time a shape comes).  Unequal batches, prompts continued over
    several steps, one wanted row or none, then single tokens that read what the prompts cached:
    against the plain implementation, and in 32-bit the bits of an engine without graphs."""
    from libllm_amd.engine import StepEntry
    from libllm_amd.runtime import load_engine
    path, cfg, weights = models[name]
    limit = min(cfg.max_pos, 120)
    rng = np.random.default_rng(17)
    eng = load_engine(path, dtype=dtype, max_tokens=4096)
    eng.PROMPT_SEEN = 1
    ref = load_engine(path, dtype=dtype, max_tokens=4096, use_graphs=False)
    for rnd in range(3):                                   # the same shapes again: replays, and slots used again
        lengths = [int(x) for x in rng.integers(2, limit - 8, size=int(rng.integers(1, 5)))]
        toks = {i: rng.integers(3, cfg.vocab, size=n + 6).tolist() for i, n in enumerate(lengths)}
        cut = {i: int(rng.integers(1, n)) for i, n in enumerate(lengths)}
        steps = [[StepEntry(i, toks[i][:cut[i]], []) for i in toks],                        # nothing wanted
                 [StepEntry(i, toks[i][cut[i]:lengths[i]], [lengths[i] - cut[i] - 1]) for i in toks]]
        steps += [[StepEntry(i, [toks[i][lengths[i] + k]], [0]) for i in toks] for k in range(6)]
        for k, entries in enumerate(steps):
            a, b = eng.step(entries), ref.step(entries)
            if k == 0:
                assert a is None and b is None
                continue
            if dtype == "float32":
                assert torch_equal(a, b), "round %d step %d" % (rnd, k)
            for j, e in enumerate(entries):
                upto = (lengths[e.request] if k == 1 else lengths[e.request] + k - 1)
                want = oracle(name, cfg, weights, toks[e.request])[upto - 1]
                assert_logits_close(a[j].cpu().numpy()[None], want[None], dtype, "round %d step %d" % (rnd, k))
        eng.end(list(toks)); ref.end(list(toks))
    assert eng._prompt_graphs and not ref._prompt_graphs
    eng.cache.check()


def torch_equal(a, b):
    import torch
    return torch.equal(a, b)


def test_a_dropped_engine_goes_at_once_with_its_graphs(models):
    """An engine that has captured graphs of both kinds is freed the moment it is dropped, with
    the collector of cycles switched off: its graphs hold no reference back to it.  Otherwise it
    would wait for the collector, which may run while another graph is being captured; the capture
    is in global mode, and a graph, a pinned buffer or an event freed then ends the process.
    ``HipOps.capture`` also collects before a capture and keeps the collector off during it."""
    import gc
    import weakref
    import torch
    from libllm_amd.engine import StepEntry
    from libllm_amd.runtime import load_engine
    path, cfg, _ = models["B"]
    gc.collect()
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    gc.disable()
    try:
        engine = load_engine(path, dtype="bfloat16", max_tokens=1024)
        engine.PROMPT_SEEN = 1
        engine.step([StepEntry(i, [5 + i, 6, 7, 8][:2 + i], [1 + i]) for i in range(3)])
        for k in range(3):
            engine.step([StepEntry(i, [9 + k], [0]) for i in range(3)])
        assert engine._graphs and engine._prompt_graphs
        assert gc.isenabled() is False                      # captures leave the collector as they found it
        ref = weakref.ref(engine)
        graphs = [weakref.ref(g) for g in list(engine._graphs.values()) + list(engine._prompt_graphs.values())]
        del engine
        assert ref() is None and all(g() is None for g in graphs)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() <= before + (1 << 20)
    finally:
        gc.enable()


def test_prompt_graphs_are_bounded(models):
    """At most ``PROMPT_GRAPHS`` prompt graphs are kept, the one unused for longest goes first, and a
    shape that comes again after its graph went is captured again and gives the same logits."""
    import torch
    from libllm_amd.engine import StepEntry
    from libllm_amd.runtime import load_engine
    path, cfg, _ = models["A"]
    engine = load_engine(path, dtype="float32", max_tokens=2048)
    engine.PROMPT_SEEN, engine.PROMPT_GRAPHS = 1, 2
    ref = load_engine(path, dtype="float32", max_tokens=2048, use_graphs=False)
    rng = np.random.default_rng(6)
    seen = []
    for n in (5, 20, 40, 5, 70, 20):                    # rows 16, 32, 48, 16, 80, 32
        prompt = rng.integers(3, cfg.vocab, size=n).tolist()
        a, b = engine.step([StepEntry("p", prompt, [n - 1])]), ref.step([StepEntry("p", prompt, [n - 1])])
        assert torch.equal(a, b)
        engine.end(["p"]); ref.end(["p"])
        seen.append([k[0] for k in engine._prompt_graphs])
    assert seen == [[16], [16, 32], [32, 48], [48, 16], [16, 80], [80, 32]]


def test_decode_graphs_are_bounded(models):
    """At most ``DECODE_GRAPHS`` decode graphs are kept, the one unused for longest goes first, and
    a batch size that comes again after its graph went is captured again and gives the same
    logits."""
    import torch
    from libllm_amd.engine import StepEntry
    from libllm_amd.runtime import load_engine
    path, cfg, _ = models["A"]
    engine = load_engine(path, dtype="float32", max_tokens=2048)
    engine.DECODE_GRAPHS = 2
    ref = load_engine(path, dtype="float32", max_tokens=2048, use_graphs=False)
    seen = []
    for n in (1, 3, 5, 1, 8, 3):                         # graphs of 1, 3, 6, 1, 8 and 3 rows
        names = ["r%d" % i for i in range(n)]
        for e in (engine, ref):
            e.step([StepEntry(r, [7 + i, 9], []) for i, r in enumerate(names)])
        a = engine.step([StepEntry(r, [11 + i], [0]) for i, r in enumerate(names)]).clone()
        b = ref.step([StepEntry(r, [11 + i], [0]) for i, r in enumerate(names)])
        assert torch.equal(a, b)
        engine.end(names); ref.end(names)
        seen.append([k[0] for k in engine._graphs])
    assert seen == [[1], [1, 3], [3, 6], [6, 1], [1, 8], [8, 3]]


def test_captures_with_an_eager_collector(models):
    """The collector of cycles set to run at almost every allocation, engines built and dropped one
    after another, each capturing graphs of both kinds, some cyclic garbage that owns device
    memory lying about: captures collect first and keep the collector off while they last, so the
    steps give what an engine without graphs gives."""
    import gc
    import torch
    from libllm_amd.engine import StepEntry
    from libllm_amd.runtime import load_engine
    path, cfg, _ = models["A"]
    ref = load_engine(path, dtype="float32", max_tokens=1024, use_graphs=False)
    steps = [[StepEntry(i, [5 + i, 6, 7, 8, 9][:3 + i], [2 + i]) for i in range(3)]]
    steps += [[StepEntry(i, [11 + k], [0]) for i in range(3)] for k in range(4)]
    want = [ref.step(e).clone() for e in steps]
    ref.end([0, 1, 2])
    old = gc.get_threshold()
    gc.set_threshold(1, 1, 1)
    try:
        for rnd in range(3):
            junk = [torch.empty(1024, device="cuda")]
            junk.append(junk)                                  # a cycle that owns device memory
            del junk
            engine = load_engine(path, dtype="float32", max_tokens=1024)
            engine.PROMPT_SEEN = 1
            for e, w in zip(steps, want):
                assert torch.equal(engine.step(e), w)
            assert engine._graphs and engine._prompt_graphs
            assert gc.isenabled()
            del engine
    finally:
        gc.set_threshold(*old)


@pytest.mark.parametrize("rows", [176, 224, 512, 2048])
def test_library_products_inside_prompt_graphs(rows):
    """A prompt of real width fills its graph exactly, so that the graph and an engine without
    graphs run the same kernels, the library's for large products among them: six replays with
    other prompts, eager work and a synchronisation between them, each the bits of the eager step;
    then a token for each, which reads the keys and values the graphs wrote."""
    import torch
    from libllm_amd.config import config_from_dict
    from libllm_amd.engine import StepEntry
    from libllm_amd.runtime import random_engine
    cfg = config_from_dict({
        "model_type": "llama", "num_hidden_layers": 2, "hidden_size": 2048, "num_attention_heads": 32,
        "num_key_value_heads": 8, "head_dim": 64, "intermediate_size": 8192, "vocab_size": 4096,
        "rope_theta": 500000.0, "rms_norm_eps": 1e-5, "tie_word_embeddings": True,
        "max_position_embeddings": 4096, "hidden_act": "silu", "bos_token_id": 1, "eos_token_id": 2})
    engines = [random_engine(cfg, seed=5, dtype="bfloat16", max_tokens=8192, use_graphs=g) for g in (True, False)]
    engines[0].PROMPT_SEEN = 1
    rng = np.random.default_rng(8)
    scratch = torch.randn((512, 512), device="cuda")
    for k in range(6):
        prompt = rng.integers(3, 4096, size=rows).tolist()
        outs, nxt = [], []
        for e in engines:
            outs.append(e.step([StepEntry("p", prompt, [rows - 1])]).clone())
            scratch = (scratch @ scratch).clamp_(-1, 1)
            torch.cuda.synchronize()
            nxt.append(e.step([StepEntry("p", [7 + k], [0])]).clone())
            e.end(["p"])
        assert torch.equal(outs[0], outs[1]), "replay %d differs from the eager step" % k
        assert torch.equal(nxt[0], nxt[1]), "the token after replay %d differs" % k
    assert list(engines[0]._prompt_graphs) == [(rows, 2)] and not engines[1]._prompt_graphs


@pytest.mark.parametrize("n_prompts", [40, 96, 224])    # 224: a graph of exactly as many rows, so that the library chooses the same product for both engines
@pytest.mark.parametrize("widths", [(2048, 32, 64, 8192), (4096, 32, 128, 14336)])
def test_decode_graphs_of_many_rows(widths, n_prompts):
    """From 17 rows on the products that add into the stream are computed over slices of K, which
    the next norm kernel adds; from 33 rows on by the product for 33 to 128 rows where its
    slices fill the device, beyond 128 by the library's.  Layers of real width: a graph of 48, 96 or 224 rows replayed twelve times, an engine
    without graphs stepping beside it, other work and a synchronisation between the replays;
    every replay gives the bits of the eager step."""
    import torch
    from libllm_amd.config import config_from_dict
    from libllm_amd.engine import StepEntry
    from libllm_amd.runtime import random_engine
    hidden, heads, head_dim, inter = widths
    cfg = config_from_dict({
        "model_type": "llama", "num_hidden_layers": 2, "hidden_size": hidden, "num_attention_heads": heads,
        "num_key_value_heads": 8, "head_dim": head_dim, "intermediate_size": inter, "vocab_size": 4096,
        "rope_theta": 500000.0, "rms_norm_eps": 1e-5, "tie_word_embeddings": True,
        "max_position_embeddings": 4096, "hidden_act": "silu", "bos_token_id": 1, "eos_token_id": 2})
    rng = np.random.default_rng(3)
    prompts = {i: rng.integers(3, 4096, size=int(n)).tolist() for i, n in enumerate(rng.integers(3, 40, size=n_prompts))}
    engines = [random_engine(cfg, seed=5, dtype="bfloat16", max_tokens=16384, use_graphs=g) for g in (True, False)]
    ops = engines[0].ops
    assert ops.ACCUM_ROWS < 40 <= ops.SPLIT_ROWS < 96 <= ops.MID_ROWS and ops.mid_gemm
    for e in engines:
        e.step([StepEntry(r, t, []) for r, t in prompts.items()])
    scratch = torch.randn((512, 512), device="cuda")
    for k in range(12):
        toks = {r: int((7 * r + 13 * k) % 4096) for r in prompts}
        outs = []
        for e in engines:
            outs.append(e.step([StepEntry(r, [toks[r]], [0]) for r in prompts]).clone())
            scratch = (scratch @ scratch).clamp_(-1, 1)         # the program's own eager work
            torch.cuda.synchronize()
        assert torch.equal(outs[0], outs[1]), "replay %d differs from the eager step" % k
    assert [key[0] for key in engines[0]._graphs] == [{40: 48, 96: 96, 224: 224}[n_prompts]] and not engines[1]._graphs


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_run_program(models, tmp_path, dtype):
    """bin/trace_run as a user starts it: a child process fed through its standard input, one
    step after each ``done`` line."""
    name = "C"
    path, cfg, weights = models[name]
    requests = make_requests(cfg, [40, 7, 66], seed=21)
    steps = traces.batches([requests], {"r0": 5, "r1": 6, "r2": 2})
    out_dir = tmp_path / "out"
    proc = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", path,
                             "--dtype", dtype, "--out", str(out_dir), "--max-tokens",
                             str(traces.max_tokens_needed(steps))],
                            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    for s in steps:
        proc.stdin.write(json.dumps(s) + "\n")
        proc.stdin.flush()
        assert proc.stdout.readline().strip() == "done %d" % s["step"]
    proc.stdin.close()
    assert proc.wait(timeout=60) == 0
    check(name, cfg, weights, requests, traces.collect(steps, str(out_dir), cfg.vocab), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_run_program_with_random_weights(tmp_path, dtype):
    """``trace_run --random-weights CONFIG.json --seed S``: no weight file; the tensors are drawn on
    the device from (seed, name).  The plain implementation runs on the same draw."""
    from libllm_amd.config import config_from_dict
    from libllm_amd.engine import declared_weights
    from libllm_amd.weights import random_tensors
    cfg_path = tmp_path / "tiny_b.json"
    cfg_path.write_text(json.dumps(TINY_B))
    declared = declared_weights(config_from_dict(TINY_B).to_spec())
    weights = {k: v.double().cpu().numpy() for k, v in random_tensors(declared, 6, std=0.02, device="cuda").items()}
    cfg = llama.PlainConfig(TINY_B)
    requests = make_requests(cfg, [33, 70], seed=22)
    steps = traces.batches([requests], {"r0": 4, "r1": 3})
    out_dir = tmp_path / "out"
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--random-weights", str(cfg_path),
                          "--seed", "6", "--dtype", dtype, "--out", str(out_dir), "--max-tokens",
                          str(traces.max_tokens_needed(steps))], input="\n".join(traces.lines(steps)) + "\n",
                         capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stderr
    assert run.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    check("random B", cfg, weights, requests, traces.collect(steps, str(out_dir), cfg.vocab), dtype)
    both = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--dtype", dtype, "--out", str(out_dir),
                           "--max-tokens", "64"], input="", capture_output=True, text=True, timeout=60)
    assert both.returncode == 2 and "--random-weights" in both.stderr


def test_cache_full_is_an_error(models):
    from libllm_amd import CacheError
    from libllm_amd.engine import StepEntry
    from libllm_amd.runtime import load_engine
    path, cfg, _ = models["A"]
    engine = load_engine(path, dtype="float32", max_tokens=128)
    engine.step([StepEntry("a", [1] * 64, [])])
    engine.step([StepEntry("b", [1] * 64, [])])
    with pytest.raises(CacheError):
        engine.step([StepEntry("a", [1], [0])])               # a third page does not exist
    engine.end(["b"])
    assert engine.step([StepEntry("a", [1], [0])]).shape == (1, cfg.vocab)
    with pytest.raises(CacheError):
        engine.step([StepEntry("c", [1] * 100, [])])          # beyond what is free; nothing is admitted
    assert not engine.holds("c")
    engine.cache.check()
