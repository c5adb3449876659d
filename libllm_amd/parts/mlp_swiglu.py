"""SwiGLU feed-forward: down(silu(gate(x)) * up(x)); gate and up are one matrix product over the
stacked weight, gate rows first (src/libllm/llama.cc:81-98, tools/llama_exporter.py:73-78,
src/flint/cuda/swiglu.cu:44-49).  The record may name another activation for the gate, of those
the operations know (``ops.ACTIVATIONS``); the Llama configuration asks for SiLU only, as the
reference does (tools/llama_exporter.py:87-88)."""
from dataclasses import dataclass

import torch

from ..errors import ConfigError
from .base import PartSpec, FeedForward, StepContext, WeightDecl
from .linear import Linear
from .registry import register_feed_forward


@dataclass
class SwiGLUSpec(PartSpec):
    width: int = 0
    intermediate: int = 0
    activation: str = "silu"
    gate_name: str = "gate_proj"
    up_name: str = "up_proj"
    down_name: str = "down_proj"


ACTIVATIONS = ("silu", "gelu_tanh", "relu")


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True      # reads nothing from the host during a step
    takes_normed = True    # the input goes to a matrix product only
    adds_to_stream = True  # the output product can add into the residual stream

    def __init__(self, spec: SwiGLUSpec):
        if spec.activation not in ACTIVATIONS:
            raise ConfigError("feed-forward activation %r is not supported (known: %s)"
                              % (spec.activation, ", ".join(ACTIVATIONS)))
        if spec.width <= 0 or spec.intermediate <= 0:
            raise ConfigError("feed-forward sizes must be positive")
        self.spec = spec
        self.gate_up = Linear(spec.width, 2 * spec.intermediate)
        self.down = Linear(spec.intermediate, spec.width)

    def weights(self):
        s = self.spec
        return {
            s.gate_name + ".weight": WeightDecl((s.intermediate, s.width)),
            s.up_name + ".weight": WeightDecl((s.intermediate, s.width)),
            s.down_name + ".weight": WeightDecl((s.width, s.intermediate)),
        }

    def bind(self, tensors, ops, dtype):
        s = self.spec
        gate, up = tensors[s.gate_name + ".weight"], tensors[s.up_name + ".weight"]
        if gate.dtype != up.dtype:
            gate, up = gate.float(), up.float()
        self.gate_up.bind(torch.cat([gate, up], dim=0), ops=ops)
        self.down.bind(tensors[s.down_name + ".weight"], ops=ops)

    def forward(self, ctx: StepContext, x, residual=None):
        if self.spec.activation == "silu":
            h = ctx.ops.linear_swiglu(x, self.gate_up.prepared, ctx.dtype)
        else:
            h = ctx.ops.linear_swiglu(x, self.gate_up.prepared, ctx.dtype, self.spec.activation)
        return self.down(ctx, h, residual=residual)
