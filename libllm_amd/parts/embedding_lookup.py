"""The input layer: x[t] = table[token[t]] * scale, as the float32 residual stream
(src/libllm/layers.cc:43-47, src/libllm/llama.cc:294-296)."""
from .base import Embedding, Stream, StepContext, WeightDecl
from .registry import register_embedding


@register_embedding("lookup")
class LookupEmbedding(Embedding):
    graph_safe = True      # reads nothing from the host during a step

    def __init__(self, spec):
        self.spec = spec
        self.table = None

    def weights(self):
        s = self.spec
        return {s.tensor: WeightDecl((s.vocab, s.width))}

    def bind(self, tensors, ops, dtype) -> None:
        self.table = tensors[self.spec.tensor]

    def forward(self, ctx: StepContext, then_norm=None) -> Stream:
        s = self.spec
        if then_norm is not None and hasattr(ctx.ops, "embed_prepared"):
            # the kernel that gathers the rows may leave what that norm needs from them
            got = ctx.ops.embed_prepared(self.table, ctx.tokens, s.scale, then_norm[0], then_norm[1], ctx.dtype)
            if got is not None:
                stream = Stream(got[0])
                stream.pre = got[1]
                return stream
        return Stream(ctx.ops.embed(self.table, ctx.tokens, s.scale))
