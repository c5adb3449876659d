"""Architecture-neutral description of a decoder, produced from a typed configuration.

A model is data: a list of layer records (each naming its mixer, feed-forward, norms and block
arrangement, with every size and constant), and a schedule that says in which order the layers
run and which cache entry each run uses.  Parts are built from these records alone; none of them
sees the configuration class or the architecture's name.

Each kind of part defines its own record type next to its implementation (for instance
``AttentionSpec`` beside the attention mixer); the records here are the ones every model has.
"""
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

from ..errors import ConfigError
from ..parts.base import PartSpec


@dataclass
class LayerSpec:
    block: str                          # arrangement of the parts, e.g. "prenorm"
    mixer: PartSpec
    feed_forward: PartSpec
    norms: List[PartSpec]               # as many as the arrangement needs, in its order
    prefixes: Dict[str, str]            # role ("mixer", "feed_forward", "norm0", ...) -> tensor-name prefix


@dataclass
class ScheduleEntry:
    """One run of a layer.  ``cache`` names the cache entry (keys/values and per-sequence state)
    that the run uses; ``writes`` is False when the run only reads an entry that an earlier run
    of the same step has filled."""
    layer: int
    cache: int
    writes: bool = True


@dataclass
class EmbeddingSpec:
    """The input layer.  ``kind`` names the registered class that turns a step's tokens into the
    residual stream ("lookup": a row of the table a token, times ``scale``); one that adds learned
    positions or normalises the rows is another kind with a record of its own that extends this
    one."""
    vocab: int
    width: int
    tensor: str                         # tensor name of the table
    scale: float = 1.0
    kind: str = "lookup"


@dataclass
class HeadSpec:
    """The output layer.  ``kind`` names the registered class that turns the normalised wanted
    rows into logits ("linear": a bare matrix product); one with a bias, a scale or a cap on the
    logits is another kind with a record of its own that extends this one."""
    vocab: int
    width: int
    tensor: str                         # tensor name of the output matrix (the table's, if tied)
    tied: bool = False
    kind: str = "linear"


@dataclass
class ModelSpec:
    name: str
    width: int
    vocab: int
    max_position: int
    embedding: EmbeddingSpec
    layers: List[LayerSpec]
    schedule: List[ScheduleEntry]
    final_norm: PartSpec
    final_norm_prefix: str
    head: HeadSpec
    stop_tokens: Tuple[int, ...] = ()
    bos_token: Optional[int] = None
    optional_tensors: Tuple[str, ...] = ()   # fnmatch patterns a file may hold; they are ignored

    def n_cache_entries(self) -> int:
        return (1 + max(e.cache for e in self.schedule)) if self.schedule else 0


def default_schedule(n_layers: int) -> List[ScheduleEntry]:
    """Every layer once, in order, each with a cache entry of its own."""
    return [ScheduleEntry(layer=i, cache=i, writes=True) for i in range(n_layers)]


def validate_schedule(spec: ModelSpec) -> None:
    written = set()
    for n, e in enumerate(spec.schedule):
        if not 0 <= e.layer < len(spec.layers):
            raise ConfigError("schedule entry %d names layer %d of %d"
                              % (n, e.layer, len(spec.layers)))
        if e.cache < 0:
            raise ConfigError("schedule entry %d has a negative cache entry" % n)
        if e.writes:
            if e.cache in written:
                raise ConfigError("cache entry %d is written by two runs of the schedule" % e.cache)
            written.add(e.cache)
        elif e.cache not in written:
            raise ConfigError("schedule entry %d reads cache entry %d before any run wrote it"
                              % (n, e.cache))
