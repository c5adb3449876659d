"""Each part of a layer alone on the GPU against the plain function it stands for, at sizes of its
own, and the parts that tests define themselves."""
import numpy as np
import pytest
import torch

import toy
import traces
from helpers import assert_logits_close, make_ctx, make_kv, rel_err
from libllm_amd.config import ScheduleEntry, config_from_dict
from libllm_amd.engine import DecoderModel, Engine, StepEntry
from libllm_amd.parts import Stream, build_block, build_feed_forward, build_mixer, build_norm
from libllm_amd.parts.attention import AttentionSpec
from libllm_amd.parts.mlp_swiglu import SwiGLUSpec
from libllm_amd.parts.norm_rms import RMSNormSpec
from libllm_amd.parts.rope import RotaryPosition, RotarySpec
from libllm_amd.weights import random_tensors
from plain import llama
from tiny import TINY_A, TINY_B

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]

# a layer of its own shape: 5 heads in 5 groups... no: 10 heads over 5 kv heads, head size 48, width 112
LAYER = {"hidden_size": 112, "num_attention_heads": 10, "num_key_value_heads": 5, "head_dim": 48,
         "intermediate_size": 264, "num_hidden_layers": 1, "vocab_size": 300, "rms_norm_eps": 3e-6,
         "rope_theta": 77777.0, "max_position_embeddings": 512, "tie_word_embeddings": False,
         "rope_scaling": {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0,
                          "high_freq_factor": 4.0, "original_max_position_embeddings": 128},
         "model_type": "llama"}


@pytest.fixture(scope="module")
def ops():
    from libllm_amd.hip import HipOps
    return HipOps()


def tol(dtype):
    return 1e-4 if dtype == torch.float32 else 0.06


def weights_for(part, prefix, seed, dtype):
    decl = {prefix + k: v for k, v in part.weights().items()}
    t = random_tensors(decl, seed, std=0.1, norm_std=0.3, dtype=torch.bfloat16)   # exactly representable
    dev = {}
    for k, v in t.items():
        vector = decl[k].role == "vector"
        dev[k[len(prefix):]] = v.to("cuda", torch.float32 if (vector or dtype == torch.float32) else dtype)
    return dev, {k: v.double().numpy() for k, v in t.items()}


def rows(m, width, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn((m, width), generator=g).to(torch.bfloat16).to(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_part(ops, dtype):
    norm = build_norm(RMSNormSpec(kind="rms", width=112, eps=3e-6))
    dev, host = weights_for(norm, "n.", 1, dtype)
    norm.bind(dev, ops, dtype)
    ctx = make_ctx(ops, dtype, [(0, 0, 9)])
    res = rows(9, 112, torch.float32, 2).cuda()
    delta = rows(9, 112, dtype, 3).cuda()
    stream = Stream(res.clone())
    stream.delta = delta
    out = norm.add_norm(ctx, stream)
    x = res.double().cpu().numpy() + delta.double().cpu().numpy()
    assert stream.delta is None and np.allclose(stream.res.cpu().numpy(), x, atol=1e-6)
    assert rel_err(out.double().cpu().numpy(), llama.rms_norm(x, host["n.weight"], 3e-6)) < tol(dtype)


def test_rotary_part_tables(ops):
    for cfg in (TINY_B, LAYER, TINY_A):
        spec = RotarySpec(kind="rotary", rot_dim=cfg["head_dim"], theta=cfg["rope_theta"],
                          max_position=cfg["max_position_embeddings"], scaling=cfg["rope_scaling"])
        part = RotaryPosition(spec)
        inv = llama.rope_inv_freq(cfg["head_dim"], cfg["rope_theta"], cfg["rope_scaling"])
        assert np.allclose(part.inv_freq().numpy(), inv, rtol=1e-12)
        cos, sin = part.tables("cuda")
        c, s = llama.rope_table(np.arange(cfg["max_position_embeddings"]), inv)
        half = cfg["head_dim"] // 2
        assert cos.dtype == torch.float32 and tuple(cos.shape) == (cfg["max_position_embeddings"], half)
        assert np.abs(cos.cpu().numpy() - c[:, :half]).max() < 1e-7 and np.abs(sin.cpu().numpy() - s[:, :half]).max() < 1e-7


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_part(ops, dtype):
    cfg = llama.PlainConfig(LAYER)
    spec = config_from_dict(LAYER).to_spec().layers[0].mixer
    assert isinstance(spec, AttentionSpec)
    mixer = build_mixer(spec)
    dev, host = weights_for(mixer, "model.layers.0.self_attn.", 4, dtype)
    mixer.bind(dev, ops, dtype)
    x = rows(150, 112, dtype, 5)
    ref = llama.attention_block(cfg, host, 0, x.double().numpy(), np.arange(150))
    # the whole sequence at once, then the same in two steps with a single token at the end
    for cuts in ([150], [100, 49, 1]):
        kv = make_kv("cuda", dtype, 2, 3, 5, 48, seed=len(cuts))
        got, start = [], 0
        for n in cuts:
            ctx = make_ctx(ops, dtype, [(1, start, n)])
            ctx._kv[0] = kv
            got.append(mixer.forward(ctx, x[start:start + n].cuda().contiguous(), ScheduleEntry(0, 0)))
            start += n
        assert rel_err(torch.cat(got).double().cpu().numpy(), ref) < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_feed_forward_part(ops, dtype):
    cfg = llama.PlainConfig(LAYER)
    ff = build_feed_forward(SwiGLUSpec(kind="swiglu", width=112, intermediate=264))
    dev, host = weights_for(ff, "model.layers.0.mlp.", 6, dtype)
    ff.bind(dev, ops, dtype)
    for m in (1, 70):                                              # few rows and many take different kernels
        x = rows(m, 112, dtype, 7)
        out = ff.forward(make_ctx(ops, dtype, [(0, 0, m)]), x.cuda())
        assert rel_err(out.double().cpu().numpy(), llama.mlp(cfg, host, 0, x.double().numpy())) < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_arrangement(ops, dtype):
    cfg = llama.PlainConfig(LAYER)
    ls = config_from_dict(LAYER).to_spec().layers[0]
    block = build_block(ls.block, build_mixer(ls.mixer), build_feed_forward(ls.feed_forward),
                        [build_norm(n) for n in ls.norms])
    host = {}
    for role, part in (("mixer", block.mixer), ("feed_forward", block.feed_forward),
                       ("norm0", block.norms[0]), ("norm1", block.norms[1])):
        dev, h = weights_for(part, ls.prefixes[role], 8 + len(host), dtype)
        part.bind(dev, ops, dtype)
        host.update(h)
    x = rows(75, 112, torch.float32, 9)
    kv = make_kv("cuda", dtype, 1, 2, 5, 48)
    ctx = make_ctx(ops, dtype, [(0, 0, 75)])
    ctx._kv[0] = kv
    stream = Stream(x.cuda().clone())
    block.forward(ctx, stream, ScheduleEntry(0, 0))
    out = stream.res.double().cpu().numpy() + stream.delta.double().cpu().numpy()   # the next norm adds it
    assert rel_err(out, llama.decode_layer(cfg, host, 0, x.double().numpy(), np.arange(75))) < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_head_without_layers(ops, dtype):
    spec = config_from_dict(dict(LAYER, tie_word_embeddings=True)).to_spec()
    spec.layers, spec.schedule = [], []
    model = DecoderModel(spec)
    t = random_tensors(model.declared(), 3, std=0.1, norm_std=0.3)
    model.bind({k: v.to("cuda", torch.float32 if (dtype == torch.float32 or v.dim() == 1) else dtype)
                for k, v in t.items()}, ops, dtype)
    engine = Engine(model, ops, dtype, max_tokens=64)
    ids = [3, 299, 0, 17]
    out = engine.step([StepEntry("a", ids, [0, 1, 2, 3])])
    e = t["model.embed_tokens.weight"].double().numpy()
    ref = llama.rms_norm(e[ids], t["model.norm.weight"].double().numpy(), 3e-6) @ e.T   # tied: the table again
    assert rel_err(out.double().cpu().numpy(), ref) < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_mixer_registers_builds_and_steps(ops, dtype):
    """A mixer with state of its own, defined in tests/toy.py, inside a Llama model on the GPU."""
    cfg_t = config_from_dict(TINY_A)
    cfg = llama.PlainConfig(TINY_A)
    model = DecoderModel(toy.toy_spec(cfg_t))
    t = random_tensors(model.declared(), 7, std=0.1, norm_std=0.2)
    model.bind({k: v.to("cuda", torch.float32 if (dtype == torch.float32 or v.dim() == 1) else dtype)
                for k, v in t.items()}, ops, dtype)
    engine = Engine(model, ops, dtype, max_tokens=512)
    engine.PROMPT_SEEN = 1                               # prompt steps through captured graphs from the first
    # the toy reads the step's sequences on the host: its layer runs from the host, the stretches
    # of the schedule before and after it are captured graphs all the same
    assert engine.use_graphs and [safe for safe, _ in model.stretches()] == [True, False, True]
    assert list(engine.cache.state) == [1]
    w = {k: v.double().numpy() for k, v in t.items()}
    rng = np.random.default_rng(5)
    reqs = {"a": rng.integers(0, 256, size=30).tolist(), "b": rng.integers(0, 256, size=11).tolist()}
    steps = traces.batches([reqs, {"c": reqs["b"]}], {"a": 12, "b": 4, "c": 10})
    got = {}
    for s in steps:
        out = engine.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        row = 0
        for e in s["entries"]:
            for _ in e["want"]:
                got.setdefault(e["id"], []).append(out[row].double().cpu().numpy())
                row += 1
        engine.end(s["end"])
    for rid, toks in (("a", reqs["a"]), ("b", reqs["b"]), ("c", reqs["b"])):
        ref = toy.toy_oracle(cfg, w, w["model.layers.1.toy.mix.weight"], toks)
        assert_logits_close(np.stack(got[rid]), ref, dtype, rid)
    # a prompt of which only the last row is wanted goes through a captured prompt step too
    d = rng.integers(0, 256, size=25).tolist()
    rows = [engine.step([StepEntry("d", d[:20], [19])]).double().cpu().numpy()]
    rows += [engine.step([StepEntry("d", [x], [0])]).double().cpu().numpy() for x in d[20:]]
    engine.end(["d"])
    ref = toy.toy_oracle(cfg, w, w["model.layers.1.toy.mix.weight"], d)
    assert_logits_close(np.concatenate(rows), ref[19:], dtype, "d")
    engine.cache.check()
    graphs = list(engine._graphs.values()) + list(engine._prompt_graphs.values())
    assert engine._graphs and engine._prompt_graphs
    assert all(g.forward.n_graphs == 2 and g.forward.n_host_pieces == 1 for g in graphs)


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_routed_feed_forward_and_position_encoding(ops, dtype):
    """A feed-forward with routing and a position encoding of another kind, both defined in
    tests/toy.py, chosen for one layer each: whole prompts and cut ones agree with the plain
    restatement (rows whose routing is a near tie aside, in bfloat16)."""
    cfg = llama.PlainConfig(TINY_A)
    model = DecoderModel(toy.toys_spec(config_from_dict(TINY_A)))
    assert "model.layers.1.moe.experts.w_in" in model.declared()
    t = random_tensors(model.declared(), 21, std=0.1, norm_std=0.2)
    model.bind({k: v.to("cuda", torch.float32 if (dtype == torch.float32 or v.dim() == 1) else dtype)
                for k, v in t.items()}, ops, dtype)
    engine = Engine(model, ops, dtype, max_tokens=512)
    # the routed part picks rows on the host's say: its layer runs from the host between two graphs
    assert engine.use_graphs and [(safe, units) for safe, units in model.stretches()] == [
        (True, [0, 1]), (False, [2]), (True, [3])]
    w = {k: v.double().numpy() for k, v in t.items()}
    ids = np.random.default_rng(8).integers(0, 256, size=100).tolist()
    ref, margin = toy.toys_oracle(cfg, w, ids)
    whole = engine.step([StepEntry("a", ids, list(range(100)))]).double().cpu().numpy()
    engine.end(["a"])
    cut = torch.cat([engine.step([StepEntry("b", ids[:70], list(range(70)))]).clone()] +
                    [engine.step([StepEntry("b", [x], [0])]).clone() for x in ids[70:]]).double().cpu().numpy()
    engine.end(["b"])
    clear = margin > (1e-6 if dtype == torch.float32 else 0.05)
    assert clear.sum() > 80
    # the routed layer is the last one: a near tie at one row does not touch the other rows
    assert_logits_close(whole[clear], ref[clear], dtype, "whole")
    assert_logits_close(cut[clear], ref[clear], dtype, "cut")
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_norm_and_toy_block_arrangement(ops, dtype):
    """A norm of another kind (mean taken out, a bias) and another arrangement of a block (one
    norm whose rows the mixer and the feed-forward both read, their results handed to the stream
    as two float32 matrices), both defined in tests/toy.py and chosen in the model's record.  The
    layer arranged in parallel is captured with its neighbours; the layer with the toy norm,
    which works through library calls, runs from the host between the graphs.  Whole prompts,
    cut ones, and batches of unequal lengths agree with the restatement."""
    cfg = llama.PlainConfig(TINY_A)
    model = DecoderModel(toy.arrangement_spec(config_from_dict(TINY_A)))
    t = random_tensors(model.declared(), 13, std=0.1, norm_std=0.2)
    model.bind({k: v.to("cuda", torch.float32 if (dtype == torch.float32 or v.dim() == 1) else dtype)
                for k, v in t.items()}, ops, dtype)
    engine = Engine(model, ops, dtype, max_tokens=512)
    engine.PROMPT_SEEN = 1
    assert engine.use_graphs and [(safe, units) for safe, units in model.stretches()] == [
        (True, [0, 1]), (False, [2]), (True, [3])]
    w = {k: v.double().numpy() for k, v in t.items()}
    ids = np.random.default_rng(3).integers(0, 256, size=100).tolist()
    ref = toy.arrangement_oracle(cfg, w, ids)
    whole = engine.step([StepEntry("a", ids, list(range(100)))]).double().cpu().numpy()
    engine.end(["a"])
    cut = torch.cat([engine.step([StepEntry("b", ids[:70], list(range(70)))]).clone()] +
                    [engine.step([StepEntry("b", [x], [0])]).clone() for x in ids[70:]]).double().cpu().numpy()
    engine.end(["b"])
    assert_logits_close(whole, ref, dtype, "whole")
    assert_logits_close(cut, ref, dtype, "cut")
    # two requests of unequal lengths in one batch, their last rows through a captured prompt step
    short = ids[:23]
    out = engine.step([StepEntry("c", ids[:60], [59]), StepEntry("d", short, [22])]).double().cpu().numpy()
    assert_logits_close(out[:1], ref[59:60], dtype, "c")
    assert_logits_close(out[1:], toy.arrangement_oracle(cfg, w, short)[22:], dtype, "d")
    nxt = engine.step([StepEntry("c", [ids[60]], [0]), StepEntry("d", [ids[23]], [0])]).double().cpu().numpy()
    assert_logits_close(nxt[:1], ref[60:61], dtype, "c next")
    engine.end(["c", "d"])
    engine.cache.check()
    assert engine._graphs and engine._prompt_graphs
    graphs = list(engine._graphs.values()) + list(engine._prompt_graphs.values())
    assert all(g.forward.n_graphs == 2 and g.forward.n_host_pieces == 1 for g in graphs)


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_mixer_with_a_plane_of_its_own_and_toy_input_layer(ops, dtype):
    """A mixer that keeps one latent row a token in the cache's pages, in a plane of its own
    width and element type instead of keys and values, and an input layer with learned positions:
    both defined in tests/toy.py, chosen in the model's record, and stepped on the GPU (the input
    layer inside the captured graphs, the mixer from the host between them) against their own
    restatement.  Batches of unequal prompts, one after another, so that pages are used again."""
    cfg_t = config_from_dict(dict(TINY_A, max_position_embeddings=256))
    cfg = llama.PlainConfig(cfg_t.to_dict())
    model = DecoderModel(toy.planes_spec(cfg_t))
    t = random_tensors(model.declared(), 9, std=0.1, norm_std=0.2)
    model.bind({k: v.to("cuda", torch.float32 if (dtype == torch.float32 or v.dim() == 1) else dtype)
                for k, v in t.items()}, ops, dtype)
    engine = Engine(model, ops, dtype, max_tokens=320)
    engine.PROMPT_SEEN = 1
    assert engine.use_graphs and [(safe, units) for safe, units in model.stretches()] == [
        (True, [0]), (False, [1]), (True, [2, 3])]
    g_latent, g_kv = engine.cache.groups
    assert list(g_latent.planes) == ["z"] and g_latent.planes["z"].shape == (1, 6, 64, 8)
    assert g_latent.planes["z"].dtype == torch.float32 and sorted(g_kv.planes) == ["k", "v"]
    w = {k: v.double().numpy() for k, v in t.items()}
    rng = np.random.default_rng(6)
    reqs = {"a": rng.integers(0, 256, size=150).tolist(), "b": rng.integers(0, 256, size=70).tolist()}
    steps = traces.batches([reqs, {"c": reqs["b"], "d": reqs["a"][:100]}], {"a": 12, "b": 8, "c": 3, "d": 40})
    got = {}
    for s in steps:
        out = engine.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        row = 0
        for e in s["entries"]:
            for _ in e["want"]:
                got.setdefault(e["id"], []).append(out[row].double().cpu().numpy())
                row += 1
        engine.end(s["end"])
        engine.cache.check()
    for rid, toks in (("a", reqs["a"]), ("b", reqs["b"]), ("c", reqs["b"]), ("d", reqs["a"][:100])):
        assert_logits_close(np.stack(got[rid]), toy.planes_oracle(cfg, w, toks), dtype, rid)
    # a prompt of which only the last row is wanted goes through a captured prompt step
    e = rng.integers(0, 256, size=90).tolist()
    rows = [engine.step([StepEntry("e", e[:80], [79])]).double().cpu().numpy()]
    rows += [engine.step([StepEntry("e", [x], [0])]).double().cpu().numpy() for x in e[80:]]
    engine.end(["e"])
    assert_logits_close(np.concatenate(rows), toy.planes_oracle(cfg, w, e)[79:], dtype, "e")
    assert engine._graphs and engine._prompt_graphs
    assert all(g.pool.n_free == g.pool.n_pages for g in engine.cache.groups)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("activation", ["gelu_tanh", "relu"])
def test_feed_forward_with_another_activation(ops, dtype, activation):
    """The gated feed-forward with another activation of the gate, chosen in the part's record:
    steps of 3, 20, 50, 100 and 200 rows go through each form of the gated product (few rows,
    33 to 128 rows, the library's with the gating kernel behind it)."""
    from test_gpu_kernels import gate_act
    spec = SwiGLUSpec(kind="swiglu", width=128, intermediate=384, activation=activation)
    ff = build_feed_forward(spec)
    dev, host = weights_for(ff, "ff.", 5, dtype)
    ff.bind(dev, ops, dtype)
    for m in (3, 20, 50, 100, 200):
        ctx = make_ctx(ops, dtype, [(0, 0, m)])
        x = rows(m, 128, dtype, m)
        out = ff.forward(ctx, x.cuda())
        xd = x.double().numpy()
        gate, up = xd @ host["ff.gate_proj.weight"].T, xd @ host["ff.up_proj.weight"].T
        ref = (up * gate_act(activation, torch.from_numpy(gate)).numpy()) @ host["ff.down_proj.weight"].T
        assert rel_err(out.double().cpu().numpy(), ref) < tol(dtype), (m, activation)
    with pytest.raises(Exception, match="not supported"):
        build_feed_forward(SwiGLUSpec(kind="swiglu", width=128, intermediate=384, activation="swish9"))


def test_attention_refuses_a_cache_entry_without_its_planes(ops):
    """The attention kernels check what they are handed: a cache entry with other planes, or with
    keys in another layout, is refused with an error that names what is there."""
    from libllm_amd.errors import KernelError
    from libllm_amd.parts import CacheNeed, CacheView, Plane, rows_plane
    from libllm_amd.parts import kv_pages
    ctx = make_ctx(ops, torch.bfloat16, [(0, 0, 3)])
    q = torch.zeros((3, 2 * 16 * 3), dtype=torch.bfloat16, device="cuda")
    table = torch.zeros((1, 1), dtype=torch.int32, device="cuda")
    latent = CacheNeed("full", (rows_plane("z", (8,), 64),))
    view = CacheView({"z": torch.zeros((2, 64, 8), device="cuda")}, table, 64, latent)
    with pytest.raises(KernelError, match='planes "k" and "v"; this one has: z'):
        ops.attention(q, 2, 2, 16, ctx, view, 0.25, 0)
    good = kv_pages.kv_need(2, 16, 0, 64)
    other = CacheNeed("full", (Plane("k", good.planes[0].page_shape, "rows"), good.planes[1]))
    planes = {p.name: torch.zeros((2,) + p.page_shape, dtype=torch.bfloat16, device="cuda") for p in good.planes}
    with pytest.raises(KernelError, match="laid out as 'rows'"):
        ops.attention(q, 2, 2, 16, ctx, CacheView(planes, table, 64, other), 0.25, 0)
    assert ops.attention(q, 2, 2, 16, ctx, CacheView(planes, table, 64, good), 0.25, 0).shape == (3, 32)


def _halves_from_neighbours(w, n_heads, hd, rot):
    """Rows of a q or k projection (or bias) reordered so that the dims an interleaved encoding
    rotates together, (2j, 2j+1), become the pair (j, j + rot/2) of the rotate-half form."""
    head = np.arange(hd)
    head[:rot // 2], head[rot // 2:rot] = np.arange(0, rot, 2), np.arange(1, rot, 2)
    order = (np.arange(n_heads)[:, None] * hd + head[None, :]).reshape(-1)
    return w[order]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("base", [TINY_A, dict(TINY_B, attention_bias=True)])
def test_interleaved_rotary_pairing(ops, dtype, base):
    """A position encoding that rotates neighbouring dims (2j, 2j+1) instead of the halves of a
    head: chosen in the model's record, no other change.  The plain implementation rotates halves;
    it is given the q and k projections with their rows reordered accordingly, which leaves every
    score unchanged.  Whole prompts, cut prompts and single tokens."""
    cfg = llama.PlainConfig(base)
    spec = config_from_dict(base).to_spec()
    for layer in spec.layers:
        layer.mixer.position.pairing = "interleaved"
    model = DecoderModel(spec)
    t = random_tensors(model.declared(), 31, std=0.1, norm_std=0.2)
    model.bind({k: v.to("cuda", torch.float32 if (dtype == torch.float32 or v.dim() == 1) else dtype)
                for k, v in t.items()}, ops, dtype)
    assert all(b.mixer.adjacent for b in model.blocks)
    engine = Engine(model, ops, dtype, max_tokens=512)
    w = {k: v.double().numpy() for k, v in t.items()}
    for name in list(w):
        for proj, heads in (("q_proj", cfg.n_heads), ("k_proj", cfg.n_kv)):
            if "." + proj + "." in name:
                w[name] = _halves_from_neighbours(w[name], heads, cfg.head_dim, cfg.head_dim)
    rng = np.random.default_rng(6)
    reqs = {"a": rng.integers(0, cfg.vocab, size=90).tolist(), "b": rng.integers(0, cfg.vocab, size=17).tolist()}
    steps = traces.batches([reqs], {"a": 20, "b": 5})
    got = {}
    for s in steps:
        out = engine.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        row = 0
        for e in s["entries"]:
            for _ in e["want"]:
                got.setdefault(e["id"], []).append(out[row].double().cpu().numpy())
                row += 1
        engine.end(s["end"])
    for rid, toks in reqs.items():
        assert_logits_close(np.stack(got[rid]), llama.logits_all(cfg, w, toks), dtype, rid)
    # and it is not the rotate-half form under another name: the unpermuted weights give other logits
    plain_half = llama.logits_all(cfg, {k: v.double().numpy() for k, v in t.items()}, reqs["a"])
    assert rel_err(np.stack(got["a"]), plain_half) > 0.5


@pytest.mark.parametrize("dtype", DTYPES)
def test_toy_output_layer(ops, dtype):
    """An output layer of another kind (capped logits), defined in tests/toy.py and chosen in the
    model's record; it runs inside captured graphs like the built-in one."""
    cfg = llama.PlainConfig(TINY_A)
    spec = config_from_dict(TINY_A).to_spec()
    spec.head = toy.CappedHeadSpec(spec.head.vocab, spec.head.width, spec.head.tensor, spec.head.tied,
                                   kind="capped", cap=2.0)
    model = DecoderModel(spec)
    t = random_tensors(model.declared(), 33, std=0.1, norm_std=0.2)
    model.bind({k: v.to("cuda", torch.float32 if (dtype == torch.float32 or v.dim() == 1) else dtype)
                for k, v in t.items()}, ops, dtype)
    engine = Engine(model, ops, dtype, max_tokens=256)
    assert engine.use_graphs
    w = {k: v.double().numpy() for k, v in t.items()}
    ids = np.random.default_rng(9).integers(0, 256, size=40).tolist()
    ref = 2.0 * np.tanh(llama.logits_all(cfg, w, ids) / 2.0)
    assert np.abs(ref).max() > 1.5                                   # the cap bites
    out = [engine.step([StepEntry("a", ids[:30], list(range(30)))]).double().cpu().numpy()]
    out += [engine.step([StepEntry("a", [x], [0])]).double().cpu().numpy() for x in ids[30:]]
    assert engine._graphs
    assert_logits_close(np.concatenate(out), ref, dtype, "capped")


@pytest.mark.parametrize("dtype", DTYPES)
def test_schedule_and_mixed_layers_on_the_gpu(ops, dtype):
    """A layer run twice, a run that reads another run's keys, and a layer with a window and
    another grouping: whole prompts and single tokens agree."""
    spec = config_from_dict(TINY_A).to_spec()
    spec.layers[1].mixer.n_kv_heads = 4
    spec.layers[1].mixer.window = 70
    spec.schedule = [ScheduleEntry(0, 0), ScheduleEntry(1, 1), ScheduleEntry(0, 2), ScheduleEntry(1, 1, writes=False)]
    model = DecoderModel(spec)
    t = random_tensors(model.declared(), 9, std=0.1, norm_std=0.2)
    model.bind({k: v.to("cuda", torch.float32 if (dtype == torch.float32 or v.dim() == 1) else dtype)
                for k, v in t.items()}, ops, dtype)
    engine = Engine(model, ops, dtype, max_tokens=256)
    assert [(g.need.kind, g.entries) for g in engine.cache.groups] == [("full", [0, 2]), ("window", [1])]
    ids = np.random.default_rng(4).integers(0, 256, size=128).tolist()
    whole = engine.step([StepEntry("a", ids, list(range(128)))]).double().cpu().numpy()
    engine.end(["a"])
    cut = torch.cat([engine.step([StepEntry("b", ids[:90], list(range(90)))]).clone()] +
                    [engine.step([StepEntry("b", [x], [0])]).clone() for x in ids[90:]]).double().cpu().numpy()
    assert_logits_close(cut, whole, dtype, "cut against whole")
    engine.end(["b"])
    engine.cache.check()
