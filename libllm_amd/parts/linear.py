"""y = x W^T (+ b) with W stored [out, in] (src/libllm/layers.cc:56-92)."""
from typing import Optional

import torch


class Linear:
    def __init__(self, in_features: int, out_features: int):
        self.in_features = in_features
        self.out_features = out_features
        self.weight: Optional[torch.Tensor] = None
        self.prepared = None
        self.bias: Optional[torch.Tensor] = None

    def bind(self, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, ops=None, like=None):
        """``weight`` is the matrix; ``prepared`` is what the products are given: the matrix, or
        what ``ops.prepare_weight`` makes of it (with ``like``, the prepared form of a matrix of
        which this one is the leading rows)."""
        assert tuple(weight.shape) == (self.out_features, self.in_features)
        self.weight = weight if weight.stride(-1) == 1 else weight.contiguous()
        self.bias = bias
        self.prepared = self.weight
        if ops is not None and hasattr(ops, "prepare_weight"):
            self.prepared = ops.prepare_weight(self.weight, like=like)

    def __call__(self, ctx, x, out_dtype=None, residual=None):
        """``x``: a matrix or an ``ops.normed`` record.  With ``residual`` the result may be added
        into it, and None returned (or the record of a prepared norm: see ``Stream.put``)."""
        if residual is None:
            return ctx.ops.linear(x, self.prepared, self.bias, out_dtype or ctx.dtype)
        hint = getattr(ctx, "then_norm", None)
        if hint is not None and hint[0] is residual and getattr(ctx.ops, "folds_norms", False):
            # an RMS norm reads the stream next: the product may prepare it, and then returns a record
            return ctx.ops.linear(x, self.prepared, self.bias, out_dtype or ctx.dtype, residual=residual,
                                  then_norm=hint[1:])
        return ctx.ops.linear(x, self.prepared, self.bias, out_dtype or ctx.dtype, residual=residual)
