"""The output layer: logits = h W^T in float32, W the output matrix or, in a tied model, the
embedding table (src/libllm/llama.cc:305-308)."""
import torch

from .base import StepContext
from .linear import Linear
from .registry import register_head


@register_head("linear")
class LinearHead:
    graph_safe = True      # reads nothing from the host during a step
    takes_normed = True    # the input goes to a matrix product only

    def __init__(self, spec):
        self.spec = spec
        self.linear = Linear(spec.width, spec.vocab)

    def bind(self, weight: torch.Tensor, ops, dtype) -> None:
        """``weight``: the tensor the model's record names (the embedding table when tied)."""
        self.linear.bind(weight, ops=ops)

    def forward(self, ctx: StepContext, h) -> torch.Tensor:
        """``h``: the normalised wanted rows (a matrix or an ``ops.normed`` record).  Returns
        float32 logits ``[rows, vocab]``."""
        return self.linear(ctx, h, out_dtype=torch.float32)
