"""RMS norm: y = x * w * rsqrt(mean(x^2) + eps), computed in 32-bit
(src/flint/cuda/rms_norm.cu:45-76, src/flint/cpu/normalizations.cc:52-65)."""
from dataclasses import dataclass

import torch

from .base import PartSpec, Norm, Stream, StepContext, WeightDecl
from .registry import register_norm


@dataclass
class RMSNormSpec(PartSpec):
    width: int = 0
    eps: float = 0.0


@register_norm("rms")
class RMSNorm(Norm):
    graph_safe = True      # reads nothing from the host during a step

    def __init__(self, spec: RMSNormSpec):
        self.width = spec.width
        self.eps = float(spec.eps)
        self.weight = None

    def weights(self):
        return {"weight": WeightDecl((self.width,), role="vector", init="ones")}

    def bind(self, tensors, ops, dtype):
        self.weight = tensors["weight"]

    def rms_terms(self):
        return self.weight, self.eps

    def add_norm(self, ctx: StepContext, stream: Stream, rows=None, lazy=False) -> torch.Tensor:
        pre, stream.pre = stream.pre, None
        if lazy and stream.delta is None and hasattr(ctx.ops, "normed"):
            if pre is not None:
                return ctx.ops.normed(stream.res, self.weight, self.eps, rows, pre=pre)
            return ctx.ops.normed(stream.res, self.weight, self.eps, rows)
        out = ctx.ops.add_rmsnorm(stream.res, stream.delta, self.weight, self.eps, ctx.dtype, rows)
        stream.delta = None
        return out
