"""Pre-norm residual block: x += mixer(norm0(x)); x += feed_forward(norm1(x))
(src/libllm/llama.cc:251-267).  The additions happen inside the following norm, in 32-bit."""
from ..errors import ConfigError
from .base import Block, Stream, StepContext
from .registry import register_block


@register_block("prenorm")
class PreNormBlock(Block):
    n_norms = 2

    def __init__(self, mixer, feed_forward, norms):
        if len(norms) != 2:
            raise ConfigError("a prenorm block needs two norms, got %d" % len(norms))
        super().__init__(mixer, feed_forward, norms)

    def forward(self, ctx: StepContext, stream: Stream, entry) -> None:
        h = self.norms[0].add_norm(ctx, stream)
        stream.delta = self.mixer.forward(ctx, h, entry)
        h = self.norms[1].add_norm(ctx, stream)
        stream.delta = self.feed_forward.forward(ctx, h)
