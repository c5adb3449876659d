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
