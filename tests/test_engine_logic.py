"""The engine's own logic (packing, cache, schedule, generation) on the CPU, with a torch stand-in
for the kernels: the same traces as on the GPU, against the plain implementation."""
import io

import numpy as np
import pytest
import torch

import toy
import traces
from cpu_ops import CpuOps
from libllm_amd import CacheError, Model, RequestError
from libllm_amd.config import ScheduleEntry, config_from_dict
from libllm_amd.engine import DecoderModel, Engine, StepEntry
from libllm_amd.engine.trace import replay
from libllm_amd.runtime import load_engine
from libllm_amd.weights import random_tensors
from plain import files, llama, sampling
from tiny import TINY_A, TINY_B, TINY_C, make_model


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    base = tmp_path_factory.mktemp("models")
    out = {}
    for name, cfg in (("A", TINY_A), ("B", TINY_B), ("C", TINY_C)):
        path = make_model(base, cfg, seed=40 + len(out), name=name)
        cfg_json, weights = files.read_model_dir(path)
        out[name] = (path, llama.PlainConfig(cfg_json), weights)
    return out


def err(out, ref):
    return float(np.abs(np.asarray(out, dtype=np.float64) - ref).max() / np.abs(ref).mean())


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_traces_agree_with_plain(models, tmp_path, name):
    path, cfg, weights = models[name]
    rng = np.random.default_rng(1)
    requests = {"r%d" % i: rng.integers(0, cfg.vocab, size=n).tolist() for i, n in enumerate([70, 5, 1, 66, 33])}
    ids = list(requests)
    groups = [{r: requests[r] for r in ids[:3]}, {r: requests[r] for r in ids[3:]}]
    for mode, steps in (("whole", traces.whole(requests)), ("tail", traces.tail_one_by_one(requests, 6)),
                        ("batches", traces.batches(groups))):
        engine = load_engine(path, dtype="float32", max_tokens=traces.max_tokens_needed(steps), ops=CpuOps())
        out_dir = tmp_path / mode
        replay(engine, traces.lines(steps), str(out_dir), log=io.StringIO())
        engine.cache.check()
        assert engine.cache.slots.n_free == engine.cache.slots.n_slots
        got = traces.collect(steps, str(out_dir), cfg.vocab)
        for rid, toks in requests.items():
            ref = llama.logits_all(cfg, weights, toks)
            assert err(np.stack([got[rid][p] for p in range(len(toks))]), ref) < 1e-4


def test_step_refuses_bad_requests(models):
    path, cfg, _ = models["A"]
    engine = load_engine(path, dtype="float32", max_tokens=128, ops=CpuOps())
    for bad in ([], [StepEntry("a", [], [])], [StepEntry("a", [1], [1])], [StepEntry("a", [cfg.vocab], [])],
                [StepEntry("a", [-1], [])], [StepEntry("a", [1], []), StepEntry("a", [2], [])],
                [StepEntry("a", [1, 2.5], [])], [StepEntry("a", [[1, 2]], [])], [StepEntry("a", ["1"], [])]):
        with pytest.raises(RequestError):
            engine.step(bad)
    assert not engine.live_requests()
    with pytest.raises(CacheError):
        engine.step([StepEntry("a", [1] * 129, [])])           # beyond max_position_embeddings 128
    with pytest.raises(CacheError):
        engine.end(["nobody"])
    assert engine.step([StepEntry("a", [1, 2], [])]) is None and engine.length("a") == 2
    engine.end(["a"])
    engine.cache.check()


def test_generation_matches_plain(models):
    path, cfg, weights = models["B"]
    rng = np.random.default_rng(2)
    prompts = [rng.integers(10, cfg.vocab, size=n).tolist() for n in (1, 17, 40, 70)]
    model = Model(path, dtype="float32", max_tokens=512, ops=CpuOps(), max_batch=3)
    assert model.name == "llama"
    got = model.generate(prompts, max_new_tokens=5, temperature=0.0)
    assert got == [sampling.generate(cfg, weights, p, 5) for p in prompts]
    got = model.generate(prompts, max_new_tokens=5, temperature=0.8, top_k=50, top_p=0.8, seed=3)
    want = [sampling.generate(cfg, weights, p, 5, 0.8, 50, 0.8, seed=3, stream=i) for i, p in enumerate(prompts)]
    assert got == want
    assert model.generate(prompts[:1], max_new_tokens=5, temperature=0.8, seed=3) == want[:1]   # whatever the batch
    first = got[1][0]
    assert model.generate(prompts, 5, temperature=0.8, seed=3, stop_tokens=[first])[1] == []
    model.engine.cache.check()
    chunks = list(model.complete(prompts[1], temperature=0.0, max_new_tokens=3))
    assert [c.token_id for c in chunks if c.token_id is not None] == sampling.generate(cfg, weights, prompts[1], 3)


@pytest.mark.parametrize("seed", range(6))
def test_generation_of_drawn_requests_matches_plain(models, seed):
    """Requests, batch size, cache size, the bound on a prompt step's rows and stop tokens drawn at
    random: every reply is what the plain implementation gives for that prompt alone, and the
    cache's books are whole afterwards."""
    path, cfg, weights = models["ABC"[seed % 3]]
    rng = np.random.default_rng(100 + seed)
    n = int(rng.integers(1, 10))
    new = int(rng.integers(1, 7))
    prompts = [rng.integers(0, cfg.vocab, size=int(l)).tolist() for l in rng.integers(1, 90, size=n)]
    longest = max(len(p) for p in prompts) + new
    max_tokens = int(rng.integers(1, 4)) * (-(-longest // 64) * 64)              # room for one to three of the longest
    stop = rng.integers(0, cfg.vocab, size=cfg.vocab // 6).tolist()               # ends about every sixth token
    model = Model(path, dtype="float32", max_tokens=max_tokens, ops=CpuOps(), max_batch=int(rng.integers(1, 6)),
                  max_prompt_rows=int(rng.integers(16, 120)))
    for temperature in (0.0, 0.9):
        got = model.generate(prompts, max_new_tokens=new, temperature=temperature, top_k=40, top_p=0.9, seed=seed,
                             stop_tokens=stop)
        want = [sampling.generate(cfg, weights, p, new, temperature, 40, 0.9, seed=seed, stream=i, stop=stop)
                for i, p in enumerate(prompts)]
        assert got == want
        model.engine.cache.check()
        assert model.engine.cache.slots.n_free == model.engine.cache.slots.n_slots
        assert not model.engine.live_requests()


def test_completions_taken_in_turns_and_one_left_unfinished(models):
    """Two completions of one model whose chunks are taken in turns give what each gives alone
    (each holds a slot of the cache of its own), and one that is dropped half way gives its slot
    and pages back."""
    import gc
    path, cfg, weights = models["B"]
    model = Model(path, dtype="float32", max_tokens=1024, ops=CpuOps())
    prompts = ([21, 500, 13, 640, 15, 77], [100, 200, 300])
    alone = [sampling.generate(cfg, weights, p, 8) for p in prompts]
    assert all(len(a) > 2 for a in alone)
    turns = [iter(model.complete(p, temperature=0.0, max_new_tokens=8)) for p in prompts]
    got = [[], []]
    for _ in range(10):
        for it, out in zip(turns, got):
            out.extend(c.token_id for c in [next(it, None)] if c is not None and c.token_id is not None)
    assert got == alone
    dropped = iter(model.complete(prompts[0], temperature=0.0, max_new_tokens=8))
    next(dropped)
    assert model.engine.live_requests()
    del dropped
    gc.collect()
    model.engine.cache.check()
    assert not model.engine.live_requests() and model.engine.cache.slots.n_free == model.engine.cache.slots.n_slots


def test_generation_beside_an_unfinished_completion(models):
    """A completion that its caller has not finished holds a slot and pages of the cache: the
    generation loop cuts its batches to what is free when each starts (here one batch of four
    becomes two), and the completion goes on afterwards as if nothing had happened."""
    path, cfg, weights = models["B"]
    model = Model(path, dtype="float32", max_tokens=256, ops=CpuOps())
    rng = np.random.default_rng(0)
    prompts = [rng.integers(10, cfg.vocab, size=n).tolist() for n in (60, 50, 40, 30)]
    want = [sampling.generate(cfg, weights, p, 4) for p in prompts]
    assert model.generate(prompts, max_new_tokens=4, temperature=0.0) == want
    first = model._generator._serial
    long_prompt = [21, 500, 13, 640, 15, 77] * 10
    reply = sampling.generate(cfg, weights, long_prompt, 6)
    assert len(reply) == 6
    held = iter(model.complete(long_prompt, temperature=0.0, max_new_tokens=6))
    got = [next(held).token_id]
    assert model.generate(prompts, max_new_tokens=4, temperature=0.0) == want
    assert model._generator._serial - first > 2            # the completion's batch, and more than one for the four
    got += [c.token_id for c in held if c.token_id is not None]
    assert got == reply
    model.engine.cache.check()
    assert model.engine.cache.slots.n_free == model.engine.cache.slots.n_slots
    # nothing free at all is an error that says so
    from libllm_amd.engine import StepEntry
    for i in range(model.engine.cache.slots.n_slots):
        model.engine.step([StepEntry(("held", i), [1], [])])
    with pytest.raises(CacheError, match="other requests hold"):
        model.generate(prompts[:1], max_new_tokens=2, temperature=0.0)
    model.engine.end([("held", i) for i in range(model.engine.cache.slots.n_slots)])


def test_messages_become_the_architectures_chat_format(models, tmp_path):
    """The messages of a chat, block by block as the reference's model class appends them
    (src/libllm/llama.cc:406-442), where the tokenizer beside the model knows the control tokens;
    lines of text where there is no tokenizer file; the last message the user's or the
    assistant's."""
    import shutil
    from libllm_amd import ControlToken
    from libllm_amd.prompt import llama3_prompt, plain_prompt
    tokenizers = pytest.importorskip("tokenizers")
    path, cfg, _ = models["B"]
    chat = [{"role": "system", "content": "be brief"}, {"role": "user", "content": "hello there"},
            {"role": "assistant", "content": "hi"}, {"role": "user", "content": "hello hi"}]
    c = ControlToken
    head = lambda role: [c("<|start_header_id|>"), role, c("<|end_header_id|>")]          # noqa: E731
    assert llama3_prompt(chat) == (
        [c("<|begin_of_text|>")] + head("system") + ["\n\nbe brief", c("<|eot_id|>")]
        + head("user") + ["\n\nhello there", c("<|eot_id|>")] + head("assistant") + ["\n\nhi", c("<|eot_id|>")]
        + head("user") + ["\n\nhello hi", c("<|eot_id|>")] + head("assistant") + ["\n\n"])
    assert llama3_prompt(chat[:3])[-4:] == head("assistant") + ["\n\nhi"]                # left open: the reply continues it
    for bad in ([], chat[:1], [{"role": "user"}]):
        with pytest.raises(RequestError):
            llama3_prompt(bad)
    # no tokenizer file beside the model: bytes are the tokens, the messages lines of text
    plain = Model(path, dtype="float32", max_tokens=512, ops=CpuOps())
    assert plain.build_prompt(chat) == plain_prompt(chat) == (
        "system: be brief\nuser: hello there\nassistant: hi\nuser: hello hi\nassistant: ")
    # a tokenizer that knows the control tokens
    folder = tmp_path / "with_tokenizer"
    shutil.copytree(path, folder)
    words = ["<|begin_of_text|>", "<|start_header_id|>", "<|end_header_id|>", "<|eot_id|>", "[UNK]", "system", "user",
             "assistant", "be", "brief", "hello", "there", "hi"]
    tok = tokenizers.Tokenizer(tokenizers.models.WordLevel({w: i for i, w in enumerate(words)}, unk_token="[UNK]"))
    tok.pre_tokenizer = tokenizers.pre_tokenizers.Whitespace()
    tok.add_special_tokens(words[:4])
    tok.save(str(folder / "tokenizer.json"))
    model = Model(str(folder), dtype="float32", max_tokens=512, ops=CpuOps())
    blocks = model.build_prompt(chat)
    assert blocks == llama3_prompt(chat)
    bot, sh, eh, eot = 0, 1, 2, 3
    assert model._prepare_prompt(blocks) == [bot, sh, 5, eh, 8, 9, eot, sh, 6, eh, 10, 11, eot, sh, 7, eh, 12, eot,
                                             sh, 6, eh, 10, 12, eot, sh, 7, eh]
    assert model.chat_stop_ids() == [eot] and plain.chat_stop_ids() == []
    reply = [ch.token_id for ch in model.complete(blocks, top_k=1, max_new_tokens=3) if ch.token_id is not None]
    assert len(reply) <= 3
    # a tokenizer without them: lines of text again
    tok2 = tokenizers.Tokenizer(tokenizers.models.WordLevel({w: i for i, w in enumerate(words[4:])}, unk_token="[UNK]"))
    tok2.pre_tokenizer = tokenizers.pre_tokenizers.Whitespace()
    tok2.save(str(folder / "tokenizer.json"))
    assert Model(str(folder), dtype="float32", max_tokens=512, ops=CpuOps()).build_prompt(chat) == plain_prompt(chat)


def build(spec, seed, ops, max_tokens=512):
    model = DecoderModel(spec)
    tensors = random_tensors(model.declared(), seed, std=0.1, norm_std=0.2, dtype=torch.float32)
    model.bind(tensors, ops, torch.float32)
    return Engine(model, ops, torch.float32, max_tokens), {k: v.double().numpy() for k, v in tensors.items()}


def test_schedule_may_repeat_a_layer_or_share_a_cache_entry():
    cfg_t = config_from_dict(TINY_A)
    cfg = llama.PlainConfig(TINY_A)
    ids = np.random.default_rng(3).integers(0, cfg.vocab, size=20).tolist()
    # layer 0 twice: the same weights run twice, each run with keys of its own
    spec = cfg_t.to_spec()
    spec.schedule = [ScheduleEntry(0, 0), ScheduleEntry(0, 1), ScheduleEntry(1, 2)]
    engine, w = build(spec, 5, CpuOps())
    x = llama.embedding(w["model.embed_tokens.weight"], ids)
    for layer in (0, 0, 1):
        x = llama.decode_layer(cfg, w, layer, x, np.arange(len(ids)))
    ref = llama.lm_head(cfg, w, llama.rms_norm(x, w["model.norm.weight"], cfg.eps))
    whole = engine.step([StepEntry("a", ids, list(range(20)))]).double().numpy()
    assert err(whole, ref) < 1e-4
    parts = [engine.step([StepEntry("b", ids[:13], list(range(13)))])] + \
            [engine.step([StepEntry("b", [t], [0])]) for t in ids[13:]]
    assert err(torch.cat(parts).double().numpy(), ref) < 1e-4
    # layer 1 reads the keys and values that layer 0 wrote: it differs from its own-cache result
    spec = cfg_t.to_spec()
    spec.schedule = [ScheduleEntry(0, 0), ScheduleEntry(1, 0, writes=False)]
    shared, _ = build(spec, 5, CpuOps())
    assert shared.model.spec.n_cache_entries() == 1 and len(shared.cache.groups[0].entries) == 1
    a = shared.step([StepEntry("a", ids, list(range(20)))])
    b = torch.cat([shared.step([StepEntry("b", ids[:7], list(range(7)))])] +
                  [shared.step([StepEntry("b", [t], [0])]) for t in ids[7:]])
    assert err(b.double().numpy(), a.double().numpy()) < 1e-4       # consistent however it is cut
    own, _ = build(cfg_t.to_spec(), 5, CpuOps())
    assert err(own.step([StepEntry("a", ids, list(range(20)))]).double().numpy(), a.double().numpy()) > 1e-2


def test_layers_may_differ_and_groups_get_storage_of_their_own():
    spec = config_from_dict(TINY_A).to_spec()
    spec.layers[1].mixer.n_kv_heads = 4                              # another grouping in layer 1
    spec.layers[1].mixer.window = 70                                 # and a window
    spec.layers[1].feed_forward.intermediate = 96
    engine, _ = build(spec, 6, CpuOps(), max_tokens=256)
    kinds = [(g.need.kind, g.planes["k"].shape[2], g.need.window, g.entries) for g in engine.cache.groups]
    assert kinds == [("full", 2, 0, [0]), ("window", 4, 70, [1])]
    ids = np.random.default_rng(4).integers(0, 256, size=128).tolist()
    whole = engine.step([StepEntry("a", ids, list(range(128)))])
    engine.end(["a"])
    cut = torch.cat([engine.step([StepEntry("b", ids[:90], list(range(90)))])] +
                    [engine.step([StepEntry("b", [t], [0])]) for t in ids[90:]])
    assert err(cut.double().numpy(), whole.double().numpy()) < 1e-4
    win = engine.cache.groups[1]
    assert sorted(win.held[engine.cache.slot_of("b")]) == [0, 1] or sorted(win.held[engine.cache.slot_of("b")]) == [1]
    engine.end(["b"])
    engine.cache.check()


def test_toy_mixer_with_state_of_its_own():
    cfg_t = config_from_dict(TINY_A)
    cfg = llama.PlainConfig(TINY_A)
    engine, w = build(toy.toy_spec(cfg_t), 7, CpuOps())
    assert not engine.use_graphs and list(engine.cache.state) == [1] and engine.cache.state[1].shape[1:] == (64,)
    assert engine.cache.groups[0].entries == [0]                     # the toy keeps no keys or values
    rng = np.random.default_rng(5)
    reqs = {"a": rng.integers(0, 256, size=30).tolist(), "b": rng.integers(0, 256, size=11).tolist()}
    steps = traces.batches([reqs, {"c": reqs["b"]}], {"a": 12, "b": 4, "c": 10})
    got = {}
    for s in steps:
        out = engine.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        row = 0
        for e in s["entries"]:
            for _ in e["want"]:
                got.setdefault(e["id"], []).append(out[row].double().numpy())
                row += 1
        engine.end(s["end"])
    for rid, toks in (("a", reqs["a"]), ("b", reqs["b"]), ("c", reqs["b"])):   # c reuses a slot: clean state
        ref = toy.toy_oracle(cfg, w, w["model.layers.1.toy.mix.weight"], toks)
        assert err(np.stack(got[rid]), ref) < 1e-4


def test_toy_mixer_with_a_plane_of_its_own_and_toy_input_layer():
    """A mixer that keeps one latent row a token in the cache's pages (no keys and values), and an
    input layer with learned positions, both defined in tests/toy.py: batches of unequal prompts
    cut in two ways, slots and pages used again."""
    cfg_t = config_from_dict(dict(TINY_A, max_position_embeddings=256))
    cfg = llama.PlainConfig(cfg_t.to_dict())
    engine, w = build(toy.planes_spec(cfg_t), 9, CpuOps(), max_tokens=320)
    g_latent, g_kv = engine.cache.groups
    assert g_latent.entries == [0] and list(g_latent.planes) == ["z"] and g_latent.planes["z"].dtype == torch.float32
    assert g_latent.planes["z"].shape == (1, 6, 64, 8) and sorted(g_kv.planes) == ["k", "v"]
    assert "model.embed_positions.weight" in engine.model.declared()
    rng = np.random.default_rng(6)
    reqs = {"a": rng.integers(0, 256, size=150).tolist(), "b": rng.integers(0, 256, size=70).tolist()}
    steps = traces.batches([reqs, {"c": reqs["b"], "d": reqs["a"][:100]}], {"a": 12, "b": 8, "c": 3, "d": 40})
    got = {}
    for s in steps:
        out = engine.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        row = 0
        for e in s["entries"]:
            for _ in e["want"]:
                got.setdefault(e["id"], []).append(out[row].double().numpy())
                row += 1
        engine.end(s["end"])
        engine.cache.check()
    for rid, toks in (("a", reqs["a"]), ("b", reqs["b"]), ("c", reqs["b"]), ("d", reqs["a"][:100])):
        assert err(np.stack(got[rid]), toy.planes_oracle(cfg, w, toks)) < 1e-4
    assert all(g.pool.n_free == g.pool.n_pages for g in engine.cache.groups)


def test_toy_norm_and_toy_block_arrangement():
    """A norm of another kind and another arrangement of a block (one norm, mixer and
    feed-forward side by side), both defined in tests/toy.py and chosen in the model's record:
    whole prompts and cut ones agree with their restatement."""
    cfg_t = config_from_dict(TINY_A)
    cfg = llama.PlainConfig(TINY_A)
    engine, w = build(toy.arrangement_spec(cfg_t), 13, CpuOps())
    declared = engine.model.declared()
    assert "model.layers.1.ln_a.bias" in declared and "model.layers.0.post_attention_layernorm.weight" not in declared
    ids = np.random.default_rng(3).integers(0, 256, size=100).tolist()
    ref = toy.arrangement_oracle(cfg, w, ids)
    whole = engine.step([StepEntry("a", ids, list(range(100)))])
    engine.end(["a"])
    cut = torch.cat([engine.step([StepEntry("b", ids[:70], list(range(70)))])] +
                    [engine.step([StepEntry("b", [t], [0])]) for t in ids[70:]])
    engine.end(["b"])
    assert err(whole.double().numpy(), ref) < 1e-4 and err(cut.double().numpy(), ref) < 1e-4


def test_a_dropped_engine_goes_at_once(models):
    """Nothing an engine owns refers back to it, so dropping it frees it there and then, without
    the collector of cycles (which may run at any later time, for instance while a graph is being
    captured, when freeing device resources ends the process)."""
    import gc
    import weakref
    path, cfg, _ = models["A"]
    gc.collect()
    gc.disable()
    try:
        model = Model(path, dtype="float32", max_tokens=512, ops=CpuOps(), max_batch=3)
        model.generate([[5, 6, 7], [8, 9]], max_new_tokens=3, temperature=0.0)
        engine = weakref.ref(model.engine)
        cache = weakref.ref(model.engine.cache)
        del model
        assert engine() is None and cache() is None
    finally:
        gc.enable()
