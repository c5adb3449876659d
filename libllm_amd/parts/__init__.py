"""Parts of a decoder layer.  Importing this package registers the built-in kinds."""
from . import attention, block_prenorm, head_linear, mlp_swiglu, norm_rms, rope  # noqa: F401
from .base import (Block, CacheNeed, FeedForward, KVView, Mixer, Norm, Part, StateNeed,  # noqa: F401
                   StepContext, Stream, WeightDecl)
from .registry import (build_block, build_feed_forward, build_head, build_mixer, build_norm,  # noqa: F401
                       build_position, register_block, register_feed_forward, register_head,
                       register_mixer, register_norm, register_position)
