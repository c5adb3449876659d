"""Plain Llama decoder: whole sequences, no cache, one function per part, numpy float64.

Each function cites the reference file (relative to the reference tree) whose formula it
follows.  The rotary frequency table has no text in the reference (its exporter stores a table
computed by an external rotary module, tools/llama_exporter.py:54-62); the frequency formulas
here are the published Llama-3 ones and are pinned by the invariants in test_plain.py.
"""
import math

import numpy as np


# --------------------------------------------------------------------------- configuration

class PlainConfig:
    """config.json keys as the exporter maps them: tools/llama_exporter.py:90-100,
    src/libllm/llama.cc:53-75 (num_key_value_heads defaults to the number of heads)."""

    def __init__(self, d):
        self.hidden = int(d["hidden_size"])
        self.n_heads = int(d["num_attention_heads"])
        self.n_kv = int(d.get("num_key_value_heads") or self.n_heads)
        self.head_dim = int(d.get("head_dim") or self.hidden // self.n_heads)
        self.inter = int(d["intermediate_size"])
        self.n_layers = int(d["num_hidden_layers"])
        self.vocab = int(d["vocab_size"])
        self.eps = float(d["rms_norm_eps"])
        self.theta = float(d.get("rope_theta", 10000.0))
        self.scaling = d.get("rope_scaling")
        self.tied = bool(d.get("tie_word_embeddings", False))
        self.max_pos = int(d["max_position_embeddings"])
        self.qkv_bias = bool(d.get("attention_bias", False))
        eos = d.get("eos_token_id")
        self.stop = set() if eos is None else set(eos if isinstance(eos, list) else [eos])


# --------------------------------------------------------------------------- parts

def embedding(table, ids):
    """x[t] = table[ids[t]]  (src/libllm/layers.cc:43-47, src/flint/cpu/lookup.cc:44-53)."""
    ids = np.asarray(ids)
    assert ids.min() >= 0 and ids.max() < table.shape[0], "indices out of range"
    return table[ids]


def rms_norm(x, w, eps):
    """y = x * w / sqrt(mean(x^2) + eps), eps inside the root
    (src/flint/cpu/normalizations.cc:52-65, src/flint/cuda/rms_norm.cu:59-76)."""
    mean = np.mean(x * x, axis=-1, keepdims=True)
    return x * w / np.sqrt(mean + eps)


def linear(x, w, b=None):
    """y = x W^T (+ b), W stored [out, in]  (src/libllm/layers.cc:80-92)."""
    y = x @ w.T
    return y if b is None else y + b


def softmax(x):
    """Max-subtracted softmax over the last axis (src/flint/cpu/softmax.cc:40-60)."""
    m = np.max(x, axis=-1, keepdims=True)
    e = np.exp(x - m)
    return e / np.sum(e, axis=-1, keepdims=True)


def swiglu(x):
    """out = silu(first half) * second half  (src/flint/cpu/swiglu.cc:48-54,
    src/flint/cuda/swiglu.cu:44-49)."""
    n = x.shape[-1] // 2
    gate, up = x[..., :n], x[..., n:]
    return gate * (1.0 / (1.0 + np.exp(-gate))) * up


def rope_inv_freq(head_dim, theta, scaling=None):
    """inv_freq_i = theta^(-2i/head_dim), i < head_dim/2; with rope_type llama3 each frequency
    is kept, divided by `factor`, or blended, by its wavelength against the original window."""
    i = np.arange(0, head_dim, 2, dtype=np.float64)
    inv = 1.0 / (theta ** (i / head_dim))
    if not scaling:
        return inv
    kind = scaling.get("rope_type", scaling.get("type"))
    if kind in (None, "default"):
        return inv
    if kind == "linear":                       # positions divided by the factor
        return inv / float(scaling["factor"])
    if kind != "llama3":
        raise ValueError("unsupported rope scaling: %r" % (kind,))
    factor = float(scaling["factor"])
    low = float(scaling["low_freq_factor"])
    high = float(scaling["high_freq_factor"])
    orig = float(scaling["original_max_position_embeddings"])
    out = np.empty_like(inv)
    for j, f in enumerate(inv):
        wavelen = 2.0 * math.pi / f
        if wavelen < orig / high:
            out[j] = f
        elif wavelen > orig / low:
            out[j] = f / factor
        else:
            s = (orig / wavelen - low) / (high - low)
            out[j] = (1.0 - s) * f / factor + s * f
    return out


def rope_table(positions, inv_freq):
    """cos, sin of shape [T, head_dim]; each row holds the head_dim/2 angles twice, which is
    what the rotate-half application below needs (tools/llama_exporter.py:54-62)."""
    ang = np.asarray(positions, dtype=np.float64)[:, None] * inv_freq[None, :]
    ang = np.concatenate([ang, ang], axis=-1)
    return np.cos(ang), np.sin(ang)


def rotate_half(x):
    """[-x[hd/2:], x[:hd/2]]  (src/libllm/llama.cc:151-164)."""
    h = x.shape[-1] // 2
    return np.concatenate([-x[..., h:], x[..., :h]], axis=-1)


def apply_rope(x, cos, sin):
    """x [T, heads, hd]; cos, sin [T, hd] broadcast over heads: x*cos + rotate_half(x)*sin
    (src/libllm/llama.cc:166-176)."""
    return x * cos[:, None, :] + rotate_half(x) * sin[:, None, :]


def causal_mask(length):
    """mask[y][x] = -inf if x > y else 0  (src/flint/cpu/tensor.cc:86-98)."""
    m = np.zeros((length, length))
    m[np.triu_indices(length, k=1)] = -np.inf
    return m


def expand_kv_heads(x, n_heads):
    """[n_kv, L, hd] -> [n_heads, L, hd], each kv head repeated `group` times in place
    (src/flint/operators.cc:43-56)."""
    n_kv = x.shape[0]
    group = n_heads // n_kv
    return np.repeat(x, group, axis=0)


def attention(q, k, v, causal, store=None):
    """q [n_heads, Lq, hd], k, v [n_kv, Lk, hd] -> [n_heads, Lq, hd].
    Scores (q*s)(k*s)^T with s = sqrt(1/sqrt(hd)); the causal mask of size Lk is sliced to its
    last Lq rows (bottom-right aligned) and skipped for a single query
    (src/flint/operators.cc:100-127).  ``store`` (see attention_block) is applied to the
    probabilities, which are the left operand of the second product in the storage type; not to
    the scores, which the reference also stores between its operators but which an engine with
    one attention kernel keeps in 32-bit."""
    n_heads, lq, hd = q.shape
    n_kv, lk, _ = k.shape
    assert n_heads % n_kv == 0
    if n_heads != n_kv:
        k = expand_kv_heads(k, n_heads)
        v = expand_kv_heads(v, n_heads)
    s = math.sqrt(1.0 / math.sqrt(hd))
    if causal and lq > ROW_BLOCK:
        # Long sequences, a block of query rows at a time with the keys that the block's last row
        # sees: the keys left out are masked for every row of the block, so each row's softmax is
        # over the same terms as in one piece; only the memory for the scores is smaller.
        out = np.empty_like(q)
        for r0 in range(0, lq, ROW_BLOCK):
            r1 = min(lq, r0 + ROW_BLOCK)
            seen = lk - lq + r1
            out[:, r0:r1] = _attention_rows(q[:, r0:r1], k[:, :seen], v[:, :seen], s, True, store)
        return out
    return _attention_rows(q, k, v, s, causal, store)


ROW_BLOCK = 1024


def _attention_rows(q, k, v, s, causal, store):
    lq, lk = q.shape[1], k.shape[1]
    scores = (q * s) @ np.swapaxes(k * s, -1, -2)
    if causal and lq > 1:
        scores = scores + causal_mask_rows(lk, lq)[None]
    p = softmax(scores)
    return (p if store is None else store(p)) @ v


def causal_mask_rows(lk, lq):
    """The last ``lq`` rows of causal_mask(lk), made without the rows above them."""
    rows = np.arange(lk - lq, lk)[:, None]
    return np.where(np.arange(lk)[None, :] > rows, -np.inf, 0.0)


# --------------------------------------------------------------------------- blocks

def fused_qkv(weights, prefix):
    """q, k, v rows stacked in that order (tools/llama_exporter.py:64-70)."""
    w = np.concatenate([weights[prefix + n + "_proj.weight"] for n in "qkv"], axis=0)
    b = None
    if prefix + "q_proj.bias" in weights:
        b = np.concatenate([weights[prefix + n + "_proj.bias"] for n in "qkv"], axis=0)
    return w, b


def exact(x):
    """The default of ``store``: nothing is rounded."""
    return x


def attention_block(cfg, weights, layer, x, positions, store=exact):
    """x [T, H] normed input -> [T, H]  (src/libllm/llama.cc:178-225).  ``store`` is applied
    wherever the reference keeps a tensor in its device float type between two operators (its
    operators return tensors of that type, src/flint/functional.cc:205-207): the model of an
    engine that computes exactly and stores in reduced precision, used to size error bounds."""
    p = "model.layers.%d.self_attn." % layer
    t = x.shape[0]
    wqkv, bqkv = fused_qkv(weights, p)
    qkv = store(linear(x, wqkv, bqkv))
    qd, kd = cfg.n_heads * cfg.head_dim, cfg.n_kv * cfg.head_dim
    q = qkv[:, :qd].reshape(t, cfg.n_heads, cfg.head_dim)
    k = qkv[:, qd:qd + kd].reshape(t, cfg.n_kv, cfg.head_dim)
    v = qkv[:, qd + kd:qd + 2 * kd].reshape(t, cfg.n_kv, cfg.head_dim)
    cos, sin = rope_table(positions, rope_inv_freq(cfg.head_dim, cfg.theta, cfg.scaling))
    q = store(apply_rope(q, cos, sin))
    k = store(apply_rope(k, cos, sin))
    o = attention(q.transpose(1, 0, 2), k.transpose(1, 0, 2), v.transpose(1, 0, 2), True, store)
    o = store(o.transpose(1, 0, 2).reshape(t, qd))
    return store(linear(o, weights[p + "o_proj.weight"]))


def mlp(cfg, weights, layer, x, store=exact):
    """down(swiglu(gate_up(x))), gate rows first (src/libllm/llama.cc:92-98,
    tools/llama_exporter.py:73-78)."""
    p = "model.layers.%d.mlp." % layer
    wgu = np.concatenate([weights[p + "gate_proj.weight"], weights[p + "up_proj.weight"]], axis=0)
    h = store(swiglu(store(linear(x, wgu))))
    return store(linear(h, weights[p + "down_proj.weight"]))


def decode_layer(cfg, weights, layer, x, positions, store=exact):
    """Pre-norm residual block (src/libllm/llama.cc:251-267).  The running sum itself is not
    passed through ``store``: the bounds are for engines that keep it in 32-bit."""
    p = "model.layers.%d." % layer
    residual = x
    h = store(rms_norm(x, weights[p + "input_layernorm.weight"], cfg.eps))
    h = attention_block(cfg, weights, layer, h, positions, store)
    x = h + residual
    residual = x
    h = store(rms_norm(x, weights[p + "post_attention_layernorm.weight"], cfg.eps))
    h = mlp(cfg, weights, layer, h, store)
    return h + residual


def hidden_states(cfg, weights, ids, position_offset=0, store=exact):
    """Embedding, layers, final norm (src/libllm/llama.cc:294-303)."""
    x = embedding(weights["model.embed_tokens.weight"], ids)
    positions = np.arange(len(ids)) + position_offset
    for layer in range(cfg.n_layers):
        x = decode_layer(cfg, weights, layer, x, positions, store)
    return store(rms_norm(x, weights["model.norm.weight"], cfg.eps))


def lm_head(cfg, weights, h):
    """logits = h W_out^T (src/libllm/llama.cc:305-308); a tied model uses the embedding."""
    w = weights["model.embed_tokens.weight"] if cfg.tied else weights["lm_head.weight"]
    return linear(h, w)


def logits_all(cfg, weights, ids, position_offset=0, store=exact):
    """Logits at every position of one whole sequence: [T, V]
    (the forwardAll of src/libllm/llama_test.cc:92-97)."""
    return lm_head(cfg, weights, hidden_states(cfg, weights, ids, position_offset, store))


def to_bfloat16(x):
    """Rounds to the nearest value with 8 bits of significand, ties to even: what storing a
    float32 result as bfloat16 does (the upper 16 bits of the float32 pattern)."""
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    bits = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16
    return bits.astype(np.uint32).view(np.float32).astype(np.float64).reshape(np.shape(x))
