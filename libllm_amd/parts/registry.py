"""Registries from a record's ``kind`` to the class that implements the part.

A new part is added by defining its record and class anywhere (also outside this package) and
registering it here; nothing else in the framework has to change:

    @register_mixer("my_kind")
    class MyMixer(Mixer):
        def __init__(self, spec): ...
"""
from typing import Callable, Dict

from ..errors import ConfigError

_MIXERS: Dict[str, Callable] = {}
_FEED_FORWARDS: Dict[str, Callable] = {}
_NORMS: Dict[str, Callable] = {}
_POSITIONS: Dict[str, Callable] = {}
_BLOCKS: Dict[str, Callable] = {}
_HEADS: Dict[str, Callable] = {}
_EMBEDDINGS: Dict[str, Callable] = {}


def _register(table, what):
    def outer(kind):
        def inner(cls):
            table[kind] = cls
            return cls
        return inner
    return outer


def _build(table, what):
    def build(spec, *args):
        kind = spec if isinstance(spec, str) else spec.kind
        if kind not in table:
            raise ConfigError("unknown %s kind %r (registered: %s)"
                              % (what, kind, ", ".join(sorted(table)) or "none"))
        return table[kind](*args) if isinstance(spec, str) else table[kind](spec, *args)
    return build


register_mixer = _register(_MIXERS, "mixer")
register_feed_forward = _register(_FEED_FORWARDS, "feed-forward")
register_norm = _register(_NORMS, "norm")
register_position = _register(_POSITIONS, "position encoding")
register_block = _register(_BLOCKS, "block")
register_head = _register(_HEADS, "output layer")
register_embedding = _register(_EMBEDDINGS, "input layer")

build_mixer = _build(_MIXERS, "mixer")
build_feed_forward = _build(_FEED_FORWARDS, "feed-forward")
build_norm = _build(_NORMS, "norm")
build_position = _build(_POSITIONS, "position encoding")
build_block = _build(_BLOCKS, "block")
build_head = _build(_HEADS, "output layer")
build_embedding = _build(_EMBEDDINGS, "input layer")
