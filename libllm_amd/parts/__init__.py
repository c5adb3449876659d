"""Parts of a decoder layer.  Importing this package registers the built-in kinds."""
from . import attention, block_prenorm, embedding_lookup, head_linear, mlp_swiglu, norm_rms, rope  # noqa: F401
from .base import (Block, CacheNeed, CacheView, Embedding, FeedForward, Mixer, Norm, Part, Plane, StateNeed,  # noqa: F401
                   StepContext, Stream, WeightDecl, rows_plane)
from .registry import (build_block, build_embedding, build_feed_forward, build_head, build_mixer, build_norm,  # noqa: F401
                       build_position, register_block, register_embedding, register_feed_forward, register_head,
                       register_mixer, register_norm, register_position)
