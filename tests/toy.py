"""A mixer defined outside the framework, with per-sequence state of its own: a running sum with
decay, h_t = decay * h_(t-1) + x_t, out_t = h_t W.  It is registered, built into a model, bound
and stepped without any change to the framework's files."""
from dataclasses import dataclass

import torch

from libllm_amd.parts import Mixer, StateNeed, WeightDecl, register_mixer
from libllm_amd.parts.base import PartSpec


@dataclass
class DecaySumSpec(PartSpec):
    width: int = 0
    decay: float = 0.5


@register_mixer("decay_sum")
class DecaySum(Mixer):
    graph_safe = False               # walks the step's sequences on the host

    def __init__(self, spec: DecaySumSpec):
        self.width, self.decay = spec.width, float(spec.decay)
        self.weight = None

    def weights(self):
        return {"mix.weight": WeightDecl((self.width, self.width))}

    def state_need(self):
        return StateNeed((self.width,), torch.float32)

    def bind(self, tensors, ops, dtype):
        self.weight = tensors["mix.weight"]

    def forward(self, ctx, x, entry):
        state = ctx.state(entry.cache)                       # [slots, width], zero for a new sequence
        out = torch.empty_like(x)
        row = 0
        for slot, n in zip(ctx.seq_slot_host, ctx.seq_lens):
            h = state[slot].clone()
            for _ in range(n):
                h = self.decay * h + x[row].float()
                out[row] = (h @ self.weight.float().t()).to(x.dtype)
                row += 1
            if entry.writes:
                state[slot] = h
        return out


def toy_spec(base_config, decay=0.5):
    """The Llama model as data, with the mixer of layer 1 replaced by the toy."""
    spec = base_config.to_spec()
    spec.layers[1].mixer = DecaySumSpec(kind="decay_sum", width=spec.width, decay=decay)
    spec.layers[1].prefixes["mixer"] = "model.layers.1.toy."
    return spec


def toy_oracle(cfg, weights, toy_weight, ids, decay=0.5):
    """The same model through the plain implementation: layer 1's attention output replaced."""
    import numpy as np

    from plain import llama
    x = llama.embedding(weights["model.embed_tokens.weight"], ids)
    positions = np.arange(len(ids))
    for layer in range(cfg.n_layers):
        p = "model.layers.%d." % layer
        if layer != 1:
            x = llama.decode_layer(cfg, weights, layer, x, positions)
            continue
        h = llama.rms_norm(x, weights[p + "input_layernorm.weight"], cfg.eps)
        acc, mixed = np.zeros(cfg.hidden), []
        for t in range(len(ids)):
            acc = decay * acc + h[t]
            mixed.append(acc @ toy_weight.T)
        x = x + np.stack(mixed)
        x = x + llama.mlp(cfg, weights, layer, llama.rms_norm(x, weights[p + "post_attention_layernorm.weight"], cfg.eps))
    return llama.lm_head(cfg, weights, llama.rms_norm(x, weights["model.norm.weight"], cfg.eps))


# ---------------------------------------------------------------------------------------------
# A feed-forward with routing and a position encoding of another kind, both defined here: they
# are registered, chosen per layer in a model record, bound and stepped like the built-in parts.
from libllm_amd.parts import FeedForward, register_feed_forward, register_position  # noqa: E402


@dataclass
class TopOneSpec(PartSpec):
    width: int = 0
    inner: int = 0
    n_experts: int = 2


@register_feed_forward("top1_experts")
class TopOneExperts(FeedForward):
    """Each row goes to the one expert whose router logit (in 32-bit) is largest:
    y = W_out[e] relu(W_in[e] x)."""
    graph_safe = False               # the rows of an expert are picked on the host's say

    def __init__(self, spec: TopOneSpec):
        self.spec = spec

    def weights(self):
        s = self.spec
        return {"router.weight": WeightDecl((s.n_experts, s.width)),
                "experts.w_in": WeightDecl((s.n_experts, s.inner, s.width)),
                "experts.w_out": WeightDecl((s.n_experts, s.width, s.inner))}

    def bind(self, tensors, ops, dtype):
        self.router = tensors["router.weight"].float()
        self.w_in, self.w_out = tensors["experts.w_in"], tensors["experts.w_out"]

    def forward(self, ctx, x):
        choice = (x.float() @ self.router.t()).argmax(dim=-1)
        out = torch.zeros_like(x)
        for e in range(self.spec.n_experts):
            rows = (choice == e).nonzero().flatten()
            if rows.numel():
                h = torch.relu(x[rows].float() @ self.w_in[e].float().t())
                out[rows] = (h @ self.w_out[e].float().t()).to(x.dtype)
        return out


@dataclass
class ClockSpec(PartSpec):
    rot_dim: int = 0
    max_position: int = 0
    step: float = 0.05


@register_position("clock")
class ClockPosition:
    """Pair j of the first rot_dim dims turns by position * (j + 1) * step."""

    def __init__(self, spec: ClockSpec):
        self.spec, self.rot_dim = spec, spec.rot_dim

    def angles(self):
        pos = torch.arange(self.spec.max_position, dtype=torch.float64)
        return pos[:, None] * (torch.arange(self.rot_dim // 2, dtype=torch.float64) + 1.0) * self.spec.step

    def tables(self, device):
        a = self.angles()
        return torch.cos(a).float().to(device), torch.sin(a).float().to(device)


def toys_spec(base_config):
    """The Llama model as data with layer 0's position encoding and layer 1's feed-forward
    replaced by the toys above."""
    spec = base_config.to_spec()
    spec.layers[0].mixer.position = ClockSpec(kind="clock", rot_dim=spec.layers[0].mixer.head_dim // 2,
                                              max_position=spec.max_position)
    spec.layers[1].feed_forward = TopOneSpec(kind="top1_experts", width=spec.width, inner=48, n_experts=3)
    spec.layers[1].prefixes["feed_forward"] = "model.layers.1.moe."
    return spec


def toys_oracle(cfg, weights, ids, step=0.05):
    """The same model through the plain functions, the two toys restated in numpy."""
    import numpy as np

    from plain import llama
    t = len(ids)
    x = llama.embedding(weights["model.embed_tokens.weight"], ids)
    positions = np.arange(t)
    # layer 0: attention with the clock rotation on the first half of every head
    p = "model.layers.0."
    h = llama.rms_norm(x, weights[p + "input_layernorm.weight"], cfg.eps)
    wqkv, _ = llama.fused_qkv(weights, p + "self_attn.")
    qkv = llama.linear(h, wqkv)
    qd, kd, hd = cfg.n_heads * cfg.head_dim, cfg.n_kv * cfg.head_dim, cfg.head_dim
    q = qkv[:, :qd].reshape(t, cfg.n_heads, hd)
    k = qkv[:, qd:qd + kd].reshape(t, cfg.n_kv, hd)
    v = qkv[:, qd + kd:].reshape(t, cfg.n_kv, hd)
    rot = hd // 2
    ang = positions[:, None] * (np.arange(rot // 2) + 1.0) * step
    cos, sin = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]

    def turn(a):
        a = a.copy()
        a1, a2 = a[..., :rot // 2].copy(), a[..., rot // 2:rot].copy()
        a[..., :rot // 2] = a1 * cos - a2 * sin
        a[..., rot // 2:rot] = a2 * cos + a1 * sin
        return a
    o = llama.attention(turn(q).transpose(1, 0, 2), turn(k).transpose(1, 0, 2), v.transpose(1, 0, 2), True)
    x = x + llama.linear(o.transpose(1, 0, 2).reshape(t, qd), weights[p + "self_attn.o_proj.weight"])
    x = x + llama.mlp(cfg, weights, 0, llama.rms_norm(x, weights[p + "post_attention_layernorm.weight"], cfg.eps))
    # layer 1: plain attention, routed feed-forward
    p = "model.layers.1."
    x = x + llama.attention_block(cfg, weights, 1, llama.rms_norm(x, weights[p + "input_layernorm.weight"], cfg.eps), positions)
    h = llama.rms_norm(x, weights[p + "post_attention_layernorm.weight"], cfg.eps)
    logits = h @ weights[p + "moe.router.weight"].T
    choice = logits.argmax(-1)
    margin = np.sort(logits, axis=-1)
    y = np.stack([weights[p + "moe.experts.w_out"][e] @ np.maximum(weights[p + "moe.experts.w_in"][e] @ row, 0.0)
                  for row, e in zip(h, choice)])
    x = x + y
    out = llama.lm_head(cfg, weights, llama.rms_norm(x, weights["model.norm.weight"], cfg.eps))
    return out, margin[:, -1] - margin[:, -2]


# ---------------------------------------------------------------------------------------------
# An output layer of another kind: logits capped smoothly, cap * tanh(h W^T / cap).
from libllm_amd.config.spec import HeadSpec  # noqa: E402
from libllm_amd.parts import register_head  # noqa: E402
from libllm_amd.parts.linear import Linear  # noqa: E402


@dataclass
class CappedHeadSpec(HeadSpec):
    cap: float = 30.0


@register_head("capped")
class CappedHead:
    graph_safe = True
    takes_normed = True

    def __init__(self, spec: CappedHeadSpec):
        self.cap = float(spec.cap)
        self.linear = Linear(spec.width, spec.vocab)

    def bind(self, weight, ops, dtype):
        self.linear.bind(weight, ops=ops)

    def forward(self, ctx, h):
        return self.cap * torch.tanh(self.linear(ctx, h, out_dtype=torch.float32) / self.cap)


# ---------------------------------------------------------------------------------------------
# A mixer that keeps one latent row per token in the cache's pages, in a plane of its own (no
# pair of keys and values, its own width and element type), and an input layer of another kind.
from libllm_amd.config.spec import EmbeddingSpec  # noqa: E402
from libllm_amd.parts import CacheNeed, Embedding, Stream, register_embedding, rows_plane  # noqa: E402


@dataclass
class LatentMixSpec(PartSpec):
    width: int = 0
    latent: int = 8


@register_mixer("latent_mix")
class LatentMix(Mixer):
    """z_t = W_z x_t is cached (one row of ``latent`` numbers a token, in float32 whatever the
    activations are); out_t = W_o sum_s softmax_s(q_t . z_s / sqrt(latent)) z_s over s <= t, with
    q_t = W_q x_t: the cached rows are what is scored and what is summed."""
    graph_safe = False               # walks the step's sequences on the host

    def __init__(self, spec: LatentMixSpec):
        self.width, self.latent = spec.width, spec.latent

    def weights(self):
        return {"z.weight": WeightDecl((self.latent, self.width)), "q.weight": WeightDecl((self.latent, self.width)),
                "o.weight": WeightDecl((self.width, self.latent))}

    def cache_need(self, page):
        return CacheNeed("full", (rows_plane("z", (self.latent,), page, torch.float32),))

    def bind(self, tensors, ops, dtype):
        self.wz, self.wq, self.wo = (tensors[n + ".weight"].float() for n in "zqo")

    def forward(self, ctx, x, entry):
        view = ctx.kv(entry.cache)
        pages, table, page = view.plane("z"), view.block_table, view.page_size
        z_new, q = x.float() @ self.wz.t(), x.float() @ self.wq.t()
        out = torch.empty_like(x)
        row = 0
        for slot, n, pos0 in zip(ctx.seq_slot_host, ctx.seq_lens, ctx.seq_pos0_host):
            if n == 0:
                continue
            pos = torch.arange(pos0 + n, device=x.device)
            where = table[slot].long()[pos // page]
            if entry.writes:
                pages[where[pos0:], pos[pos0:] % page] = z_new[row:row + n]
            z = pages[where, pos % page]                              # [pos0 + n, latent], the new rows among them
            s = q[row:row + n] @ z.t() / self.latent ** 0.5
            s = s.masked_fill(pos[None, :] > pos[pos0:, None], float("-inf"))
            out[row:row + n] = ((torch.softmax(s, dim=-1) @ z) @ self.wo.t()).to(x.dtype)
            row += n
        return out


@dataclass
class PositionedEmbeddingSpec(EmbeddingSpec):
    max_position: int = 0
    positions_tensor: str = "model.embed_positions.weight"


@register_embedding("lookup_plus_positions")
class PositionedEmbedding(Embedding):
    """x_t = table[token_t] * scale + positions[position_t]: learned absolute positions."""
    graph_safe = True                # index operations on device tensors only

    def __init__(self, spec: PositionedEmbeddingSpec):
        self.spec = spec

    def weights(self):
        s = self.spec
        return {s.tensor: WeightDecl((s.vocab, s.width)), s.positions_tensor: WeightDecl((s.max_position, s.width))}

    def bind(self, tensors, ops, dtype):
        self.table, self.positions = tensors[self.spec.tensor], tensors[self.spec.positions_tensor]

    def forward(self, ctx, then_norm=None):
        rows = self.table[ctx.tokens.long()].float() * self.spec.scale + self.positions[ctx.tok_pos.long()].float()
        return Stream(rows.contiguous())


def planes_spec(base_config, latent=8):
    """The Llama model as data with layer 0's mixer replaced by the latent mixer and the input
    layer by the one with learned positions."""
    spec = base_config.to_spec()
    spec.layers[0].mixer = LatentMixSpec(kind="latent_mix", width=spec.width, latent=latent)
    spec.layers[0].prefixes["mixer"] = "model.layers.0.latent."
    e = spec.embedding
    spec.embedding = PositionedEmbeddingSpec(e.vocab, e.width, e.tensor, e.scale, kind="lookup_plus_positions",
                                             max_position=spec.max_position)
    return spec


def planes_oracle(cfg, weights, ids, latent=8):
    """The same model through the plain functions, the two toys restated in numpy."""
    import numpy as np

    from plain import llama
    t = len(ids)
    x = llama.embedding(weights["model.embed_tokens.weight"], ids) + weights["model.embed_positions.weight"][:t]
    positions = np.arange(t)
    p = "model.layers.0."
    h = llama.rms_norm(x, weights[p + "input_layernorm.weight"], cfg.eps)
    z, q = h @ weights[p + "latent.z.weight"].T, h @ weights[p + "latent.q.weight"].T
    s = q @ z.T / np.sqrt(latent) + llama.causal_mask(t)
    x = x + (llama.softmax(s) @ z) @ weights[p + "latent.o.weight"].T
    x = x + llama.mlp(cfg, weights, 0, llama.rms_norm(x, weights[p + "post_attention_layernorm.weight"], cfg.eps))
    for layer in range(1, cfg.n_layers):
        x = llama.decode_layer(cfg, weights, layer, x, positions)
    return llama.lm_head(cfg, weights, llama.rms_norm(x, weights["model.norm.weight"], cfg.eps))


# ---------------------------------------------------------------------------------------------
# A norm of another kind (mean taken out, a bias added) and another arrangement of a block (the
# mixer and the feed-forward read the same normalised rows, one norm a block).
from libllm_amd.parts import Block, Norm, register_block, register_norm  # noqa: E402


@dataclass
class CenteredNormSpec(PartSpec):
    width: int = 0
    eps: float = 0.0


@register_norm("centered")
class CenteredNorm(Norm):
    """y = (x - mean(x)) * rsqrt(var(x) + eps) * weight + bias, in 32-bit, by library calls: it
    runs from the host, between the captured stretches of its neighbours."""
    graph_safe = False

    def __init__(self, spec: CenteredNormSpec):
        self.width, self.eps = spec.width, float(spec.eps)

    def weights(self):
        return {"weight": WeightDecl((self.width,), role="vector", init="ones"),
                "bias": WeightDecl((self.width,), role="vector", init="normal")}

    def bind(self, tensors, ops, dtype):
        self.weight, self.bias = tensors["weight"].float(), tensors["bias"].float()

    def add_norm(self, ctx, stream, rows=None, lazy=False):
        x = stream.settle()
        if rows is not None:
            x = x[rows.long()]
        x = x - x.mean(-1, keepdim=True)
        return (x * torch.rsqrt((x * x).mean(-1, keepdim=True) + self.eps) * self.weight + self.bias).to(ctx.dtype)


@register_block("parallel")
class ParallelBlock(Block):
    """x += mixer(norm(x)) + feed_forward(norm(x)): one norm, both parts read its rows, and their
    results go to the stream as two float32 matrices that the next norm adds in 32-bit."""

    def __init__(self, mixer, feed_forward, norms):
        assert len(norms) == 1
        super().__init__(mixer, feed_forward, norms)

    def entry_norm(self):
        return self.norms[0]

    def forward(self, ctx, stream, entry):
        h = self.norms[0].add_norm(ctx, stream)
        mixed = self.mixer.forward(ctx, h, entry)
        fed = self.feed_forward.forward(ctx, h)
        stream.put(torch.stack([mixed.float(), fed.float()]))


def arrangement_spec(base_config, eps=1e-3):
    """The Llama model as data with layer 0 arranged in parallel around its first RMS norm, and
    layer 1's two norms replaced by the centered one."""
    spec = base_config.to_spec()
    first, second = spec.layers[0], spec.layers[1]
    first.block, first.norms = "parallel", first.norms[:1]
    del first.prefixes["norm1"]
    second.norms = [CenteredNormSpec(kind="centered", width=spec.width, eps=eps) for _ in range(2)]
    second.prefixes["norm0"], second.prefixes["norm1"] = "model.layers.1.ln_a.", "model.layers.1.ln_b."
    return spec


def arrangement_oracle(cfg, weights, ids, eps=1e-3):
    """The same model through the plain functions, the two toys restated in numpy."""
    import numpy as np

    from plain import llama
    positions = np.arange(len(ids))
    x = llama.embedding(weights["model.embed_tokens.weight"], ids)
    h = llama.rms_norm(x, weights["model.layers.0.input_layernorm.weight"], cfg.eps)
    x = x + llama.attention_block(cfg, weights, 0, h, positions) + llama.mlp(cfg, weights, 0, h)

    def centered(x, name):
        c = x - x.mean(-1, keepdims=True)
        return c / np.sqrt((c * c).mean(-1, keepdims=True) + eps) * weights[name + "weight"] + weights[name + "bias"]
    x = x + llama.attention_block(cfg, weights, 1, centered(x, "model.layers.1.ln_a."), positions)
    x = x + llama.mlp(cfg, weights, 1, centered(x, "model.layers.1.ln_b."))
    return llama.lm_head(cfg, weights, llama.rms_norm(x, weights["model.norm.weight"], cfg.eps))
