"""Pins of the plain implementation: what fixes each formula beside the reference's text.  Vectors
that the reference's own tests hold, special cases that reduce to a library routine, and
invariants, each chosen so that a plausible mistake (a wrong sign or pairing, eps outside the
root, the wrong half gated, a mask aligned at the top) fails."""
import math

import numpy as np
import pytest
from scipy.special import softmax as scipy_softmax

from plain import llama, sampling
from tiny import LLAMA3_MIDDLE_BAND, TINY_A, TINY_B


def rng(seed=0):
    return np.random.default_rng(seed)


# ------------------------------------------------------------------------------- vectors of the reference
def test_softmax_reference_vectors():
    # src/flint/cpu/test.cc:146-155
    assert np.allclose(llama.softmax(np.array([0.1, 0.2, 0.3])), [0.3006, 0.3322, 0.3672], atol=1e-4)
    assert np.allclose(llama.softmax(np.array([0.1, 0.2, -np.inf])), [0.4750, 0.5250, 0.0], atol=1e-4)
    # src/flint/cuda/test.cc:230-238: extreme values stay finite
    out = llama.softmax(np.array([-999.0, -998.0, -997.0, -np.inf]))
    assert np.isfinite(out).all() and abs(out.sum() - 1) < 1e-12 and out[3] == 0


def test_embedding_reference_vector():
    # src/flint/cpu/test.cc:101-144
    wte = np.array([[0.1, 0.2], [0.3, 0.4], [0.2, 0.3], [0.4, 0.5], [0.7, 0.8]])
    out = llama.embedding(wte, [[0, 1, 2], [1, 3, 4]])
    assert np.array_equal(out, [[[0.1, 0.2], [0.3, 0.4], [0.2, 0.3]], [[0.3, 0.4], [0.4, 0.5], [0.7, 0.8]]])
    with pytest.raises(AssertionError):
        llama.embedding(wte, [5])


def test_sampling_reference_vectors():
    # src/flint/cuda/test.cc:376-392: top_k = 1 is arg-max
    p = np.log(np.array([[0.4, 0.3, 0.2, 0.1], [0.1, 0.2, 0.6, 0.1], [0.05, 0.05, 0.1, 0.8]]))
    assert [sampling.sample(row, 1.0, 1, 1.0, 0.99) for row in p] == [0, 2, 3]
    # src/flint/cuda/test.cc:405-415
    v = np.zeros((2, 2050))
    v[0, 2049], v[1, 1100] = 0.4, 0.7
    assert [sampling.sample(row, 1.0, 1, 1.0, 0.5) for row in v] == [2049, 1100]


# ------------------------------------------------------------------------------- norm, activation
def test_rms_norm_formula_and_eps_placement():
    x = np.array([[3.0, 4.0]])
    assert np.allclose(llama.rms_norm(x, np.ones(2), 0.0), x / math.sqrt(12.5))
    assert np.allclose(llama.rms_norm(x, np.array([2.0, 0.5]), 0.0), x * [2.0, 0.5] / math.sqrt(12.5))
    assert np.array_equal(llama.rms_norm(np.zeros((1, 4)), np.ones(4), 1e-5), np.zeros((1, 4)))
    # eps inside the root: for tiny x the result is x / sqrt(eps), not x / eps or x / rms
    tiny = np.full((1, 4), 1e-6)
    assert np.allclose(llama.rms_norm(tiny, np.ones(4), 1e-2), tiny / math.sqrt(1e-12 + 1e-2))
    big = rng(1).normal(size=(3, 10)) * 1e3
    assert np.allclose(llama.rms_norm(big, np.ones(10), 1e-5), llama.rms_norm(big * 7, np.ones(10), 1e-5), rtol=1e-6)
    assert np.allclose((llama.rms_norm(big, np.ones(10), 0.0) ** 2).mean(-1), 1.0)


def test_swiglu_gates_the_first_half():
    assert np.allclose(llama.swiglu(np.array([1.0, 2.0])), 1.0 / (1 + math.exp(-1.0)) * 2.0)
    assert not np.allclose(llama.swiglu(np.array([1.0, 2.0])), llama.swiglu(np.array([2.0, 1.0])))
    assert llama.swiglu(np.array([0.0, 5.0]))[0] == 0.0
    assert np.allclose(llama.swiglu(np.array([40.0, 3.0])), 120.0)
    x = rng(2).normal(size=(4, 12))
    g, u = x[:, :6], x[:, 6:]
    assert np.allclose(llama.swiglu(x), g * (1 / (1 + np.exp(-g))) * u)


def test_linear_is_x_wt():
    x, w = rng(3).normal(size=(5, 7)), rng(4).normal(size=(3, 7))
    assert np.allclose(llama.linear(x, w), np.einsum("mk,nk->mn", x, w))


# ------------------------------------------------------------------------------- rotary
def test_rope_position_zero_pairing_sign_and_norm():
    hd = 16
    inv = llama.rope_inv_freq(hd, 10000.0)
    x = rng(5).normal(size=(3, 2, hd))
    cos, sin = llama.rope_table([0, 0, 0], inv)
    assert np.allclose(llama.apply_rope(x, cos, sin), x)                    # position 0: identity
    cos, sin = llama.rope_table([5, 9, 77], inv)
    y = llama.apply_rope(x, cos, sin)
    pair = lambda v: v[..., :hd // 2] ** 2 + v[..., hd // 2:] ** 2        # noqa: E731
    assert np.allclose(pair(x), pair(y))                                    # each pair (j, j + hd/2) keeps its norm
    e0 = np.zeros((1, 1, hd))
    e0[0, 0, 0] = 1.0
    cos, sin = llama.rope_table([3], inv)
    out = llama.apply_rope(e0, cos, sin)[0, 0]
    assert abs(out[0] - math.cos(3.0)) < 1e-12 and abs(out[hd // 2] - math.sin(3.0)) < 1e-12
    assert np.count_nonzero(np.abs(out) > 1e-15) == 2                       # not the neighbour (interleaved) pairing
    assert np.allclose(llama.rotate_half(np.arange(1.0, 5.0)), [-3, -4, 1, 2])   # src/libllm/llama.cc:151-164


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_rope_scores_depend_on_distance_only(cfg):
    hd = cfg["head_dim"]
    inv = llama.rope_inv_freq(hd, cfg["rope_theta"], cfg["rope_scaling"])
    q, k = rng(6).normal(size=(1, 1, hd)), rng(7).normal(size=(1, 1, hd))

    def score(m, n):
        cq, sq = llama.rope_table([m], inv)
        ck, sk = llama.rope_table([n], inv)
        return float((llama.apply_rope(q, cq, sq) * llama.apply_rope(k, ck, sk)).sum())
    assert abs(score(17, 5) - score(112, 100)) < 1e-9
    assert abs(score(17, 5) - score(5, 17)) > 1e-3                          # the sign of the distance matters


def test_llama3_frequency_bands():
    cfg = TINY_B
    hd, sc = cfg["head_dim"], cfg["rope_scaling"]
    plain = llama.rope_inv_freq(hd, cfg["rope_theta"])
    scaled = llama.rope_inv_freq(hd, cfg["rope_theta"], sc)
    assert np.allclose(plain, cfg["rope_theta"] ** (-np.arange(0, hd, 2) / hd))
    wavelen = 2 * math.pi / plain
    orig = sc["original_max_position_embeddings"]
    short = wavelen < orig / sc["high_freq_factor"]
    long_ = wavelen > orig / sc["low_freq_factor"]
    assert short.any() and long_.any() and (~short & ~long_).any()          # all three bands occur
    assert np.array_equal(scaled[short], plain[short])
    assert np.allclose(scaled[long_], plain[long_] / sc["factor"])
    mid = ~short & ~long_
    assert ((scaled[mid] < plain[mid]) & (scaled[mid] > plain[mid] / sc["factor"])).all()
    assert (np.diff(scaled) < 0).all()                                       # still ordered
    # continuous at both edges of the middle band
    for edge, want in ((orig / sc["high_freq_factor"], 1.0), (orig / sc["low_freq_factor"], 1.0 / sc["factor"])):
        for nudge in (1 - 1e-9, 1 + 1e-9):
            freq = 2 * math.pi / (edge * nudge)
            assert abs(_scaled_single(freq, sc) / freq - want) < 1e-6
    one = dict(sc, factor=1.0)
    assert np.allclose(llama.rope_inv_freq(hd, cfg["rope_theta"], one), plain)


@pytest.mark.parametrize("params,want", LLAMA3_MIDDLE_BAND)
def test_llama3_middle_band_values(params, want):
    factor, low, high, orig, theta, hd = params
    sc = {"rope_type": "llama3", "factor": factor, "low_freq_factor": low, "high_freq_factor": high,
          "original_max_position_embeddings": orig}
    got = llama.rope_inv_freq(hd, theta, sc)
    for j, value in want.items():
        assert abs(got[j] / value - 1.0) < 1e-12, (j, got[j], value)


def _scaled_single(freq, sc):
    # a head of 4 dimensions has the frequencies [1, theta^-1/2]: choose theta so the second is freq
    return float(llama.rope_inv_freq(4, freq ** -2.0, sc)[1])


# ------------------------------------------------------------------------------- attention
def test_attention_reduces_to_library_softmax():
    q, k, v = rng(8).normal(size=(1, 6, 16)), rng(9).normal(size=(1, 6, 16)), rng(10).normal(size=(1, 6, 16))
    want = scipy_softmax(q[0] @ k[0].T / math.sqrt(16), axis=-1) @ v[0]
    assert np.allclose(llama.attention(q, k, v, causal=False)[0], want)


def test_attention_special_cases():
    v = rng(11).normal(size=(2, 1, 8))
    q, k = rng(12).normal(size=(2, 1, 8)), rng(13).normal(size=(2, 1, 8))
    assert np.allclose(llama.attention(q, k, v, True), v)                   # one query, one key: the value
    k, v = rng(14).normal(size=(1, 5, 8)), rng(15).normal(size=(1, 5, 8))
    out = llama.attention(np.zeros((1, 5, 8)), k, v, True)                   # equal scores: mean of the visible values
    for r in range(5):
        assert np.allclose(out[0, r], v[0, :r + 1].mean(0))


def test_attention_mask_is_aligned_bottom_right():
    k, v = rng(16).normal(size=(2, 10, 8)), rng(17).normal(size=(2, 10, 8))
    q = rng(18).normal(size=(4, 6, 8))                                       # 6 queries over 10 keys
    out = llama.attention(q, k, v, True)
    for r in range(6):
        visible = 10 - 6 + r + 1                                             # src/flint/operators.cc:119-124
        alone = llama.attention(q[:, r:r + 1], k[:, :visible], v[:, :visible], False)
        assert np.allclose(out[:, r:r + 1], alone)
    k2 = k.copy()
    k2[:, 7] += 5.0                                                          # a later key leaves earlier rows alone
    out2 = llama.attention(q, k2, v, True)
    assert np.allclose(out2[:, :3], out[:, :3]) and not np.allclose(out2[:, 3:], out[:, 3:])


def test_attention_in_blocks_of_rows_is_attention(monkeypatch):
    """Long sequences go a block of query rows at a time; the mask's rows are then made without
    the rows above them.  Both are the one-piece computation, term for term."""
    assert np.array_equal(llama.causal_mask_rows(10, 4), llama.causal_mask(10)[6:10])      # src/flint/cpu/tensor.cc:86-98
    assert np.array_equal(llama.causal_mask_rows(5, 5), llama.causal_mask(5))
    k, v = rng(30).normal(size=(2, 23, 8)), rng(31).normal(size=(2, 23, 8))
    q = rng(32).normal(size=(4, 19, 8))
    whole = llama.attention(q, k, v, True)
    monkeypatch.setattr(llama, "ROW_BLOCK", 5)
    assert np.allclose(llama.attention(q, k, v, True), whole, rtol=1e-13, atol=1e-15)


def test_grouped_heads_equal_repeated_kv_heads():
    q = rng(19).normal(size=(6, 4, 8))
    k, v = rng(20).normal(size=(2, 4, 8)), rng(21).normal(size=(2, 4, 8))
    rep = lambda x: np.repeat(x, 3, axis=0)                                  # noqa: E731  heads 0,1,2 -> kv 0
    assert np.allclose(llama.attention(q, k, v, True), llama.attention(q, rep(k), rep(v), True))
    assert np.array_equal(llama.expand_kv_heads(k, 6)[2], k[0]) and np.array_equal(llama.expand_kv_heads(k, 6)[3], k[1])


# ------------------------------------------------------------------------------- whole model
def random_weights(cfg, seed, std=0.1):
    r = rng(seed)
    h, hd, nh, nkv, inter = cfg.hidden, cfg.head_dim, cfg.n_heads, cfg.n_kv, cfg.inter
    w = {"model.embed_tokens.weight": r.normal(size=(cfg.vocab, h)) * std,
         "model.norm.weight": 1 + 0.2 * r.normal(size=h)}
    if not cfg.tied:
        w["lm_head.weight"] = r.normal(size=(cfg.vocab, h)) * std
    for i in range(cfg.n_layers):
        p = "model.layers.%d." % i
        w[p + "input_layernorm.weight"] = 1 + 0.2 * r.normal(size=h)
        w[p + "post_attention_layernorm.weight"] = 1 + 0.2 * r.normal(size=h)
        w[p + "self_attn.q_proj.weight"] = r.normal(size=(nh * hd, h)) * std
        w[p + "self_attn.k_proj.weight"] = r.normal(size=(nkv * hd, h)) * std
        w[p + "self_attn.v_proj.weight"] = r.normal(size=(nkv * hd, h)) * std
        w[p + "self_attn.o_proj.weight"] = r.normal(size=(h, nh * hd)) * std
        w[p + "mlp.gate_proj.weight"] = r.normal(size=(inter, h)) * std
        w[p + "mlp.up_proj.weight"] = r.normal(size=(inter, h)) * std
        w[p + "mlp.down_proj.weight"] = r.normal(size=(h, inter)) * std
    return w


@pytest.mark.parametrize("cfg_dict", [TINY_A, TINY_B])
def test_model_invariants(cfg_dict):
    cfg = llama.PlainConfig(cfg_dict)
    w = random_weights(cfg, 3)
    ids = rng(4).integers(0, cfg.vocab, size=12).tolist()
    logits = llama.logits_all(cfg, w, ids)
    assert logits.shape == (12, cfg.vocab)
    # only distances between positions count: a shift of all positions changes nothing
    assert np.allclose(llama.logits_all(cfg, w, ids, position_offset=37), logits, atol=1e-9)
    # causal: a later token leaves earlier logits alone
    ids2 = list(ids)
    ids2[8] = (ids2[8] + 1) % cfg.vocab
    logits2 = llama.logits_all(cfg, w, ids2)
    assert np.allclose(logits2[:8], logits[:8]) and not np.allclose(logits2[8:], logits[8:])
    # a prefix gives the same logits as the same positions of the whole
    assert np.allclose(llama.logits_all(cfg, w, ids[:5]), logits[:5])
    if cfg.tied:
        h = llama.hidden_states(cfg, w, ids)
        assert np.allclose(logits, h @ w["model.embed_tokens.weight"].T)


def test_block_is_identity_without_output_matrices():
    cfg = llama.PlainConfig(TINY_A)
    w = random_weights(cfg, 5)
    for i in range(cfg.n_layers):
        w["model.layers.%d.self_attn.o_proj.weight" % i][:] = 0
        w["model.layers.%d.mlp.down_proj.weight" % i][:] = 0
    x = rng(6).normal(size=(7, cfg.hidden))
    assert np.array_equal(llama.decode_layer(cfg, w, 0, x, np.arange(7)), x)


def test_fused_projection_equals_separate_ones():
    cfg = llama.PlainConfig(TINY_B)
    w = random_weights(cfg, 7)
    x = rng(8).normal(size=(3, cfg.hidden))
    p = "model.layers.1.self_attn."
    fused, _ = llama.fused_qkv(w, p)
    sep = np.concatenate([x @ w[p + n + "_proj.weight"].T for n in "qkv"], axis=-1)
    assert np.allclose(x @ fused.T, sep)


# ------------------------------------------------------------------------------- sampling
def test_uniform_is_a_function_of_its_keys():
    us = [sampling.uniform(1, s, c) for s in range(20) for c in range(20)]
    assert all(0.0 <= u < 1.0 for u in us) and len(set(us)) > 390
    assert sampling.uniform(1, 2, 3) == sampling.uniform(1, 2, 3) != sampling.uniform(2, 2, 3)
    assert abs(np.mean(us) - 0.5) < 0.05


def test_nucleus_and_top_k_order():
    logits = np.log(np.array([0.05, 0.4, 0.25, 0.2, 0.1]))
    labels, acc = sampling.candidates(logits, 1.0, 3, 1.0)
    assert labels == [1, 2, 3] and np.allclose(acc, [0.4, 0.65, 0.85])       # sorted, largest first
    labels, acc = sampling.candidates(logits, 1.0, 5, 0.6)
    assert labels == [1, 2]                                                   # shortest prefix reaching top_p
    assert sampling.sample(logits, 1.0, 5, 0.6, 0.0) == 1
    assert sampling.sample(logits, 1.0, 5, 0.6, 0.99) == 2                    # r = u * kept sum
    assert sampling.sample(logits, 0.0, 5, 0.6, 0.99) == 1                    # temperature 0: arg-max
    tie = np.array([1.0, 3.0, 3.0, 0.0])
    assert sampling.candidates(tie, 1.0, 2, 1.0)[0] == [1, 2] and sampling.sample(tie, 0.0, 0, 1.0, 0.3) == 1
    draws = [sampling.sample(logits, 1.0, 0, 1.0, (i + 0.5) / 2000) for i in range(2000)]
    assert np.abs(np.bincount(draws, minlength=5) / 2000 - np.exp(logits)).max() < 2e-3
    hot = [sampling.sample(logits, 0.25, 0, 1.0, (i + 0.5) / 2000) for i in range(2000)]
    assert np.mean(np.array(hot) == 1) > 0.75                                 # low temperature sharpens
