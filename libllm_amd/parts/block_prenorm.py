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

    def entry_norm(self):
        return self.norms[0]

    def forward(self, ctx: StepContext, stream: Stream, entry) -> None:
        mixer, ff = self.mixer, self.feed_forward
        after = ctx.norm_after_block
        h = self.norms[0].add_norm(ctx, stream, lazy=mixer.takes_normed)
        if mixer.adds_to_stream:
            self.announce(ctx, stream, self.norms[1])
            stream.put(mixer.forward(ctx, h, entry, residual=stream.res))
            self.announce(ctx, stream, None)
        else:
            stream.put(mixer.forward(ctx, h, entry))
        h = self.norms[1].add_norm(ctx, stream, lazy=ff.takes_normed)
        if ff.adds_to_stream:
            self.announce(ctx, stream, after)
            stream.put(ff.forward(ctx, h, residual=stream.res))
            self.announce(ctx, stream, None)
        else:
            stream.put(ff.forward(ctx, h))
