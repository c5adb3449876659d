"""Interfaces that every part of a layer implements, and what a step hands to them.

A part is built from its record (sizes and constants), declares the tensors it needs by names
relative to a prefix, is bound to the loaded tensors, and then runs on packed rows: all tokens of
all sequences of a step lie one after another in a ``[tokens, width]`` matrix.  A part never
learns which model or architecture it belongs to.
"""
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch


@dataclass
class PartSpec:
    """Base of all part records.  ``kind`` is the key under which the part is registered; each
    kind of part defines its own record type, with its sizes and constants, beside its class."""
    kind: str


@dataclass
class WeightDecl:
    """A tensor a part expects in the weight file.

    role "matrix": kept in the model's dtype (bfloat16, or float32 when the file stores 32-bit
    or the whole model runs in 32-bit).  role "vector": small per-channel values (norm scales,
    biases) held in float32 on the device.  role "table": integer table held as int32.
    ``init`` says how the random-weights mode fills it: "normal", "ones" or "zeros".
    """
    shape: Tuple[int, ...]
    role: str = "matrix"
    init: str = "normal"


@dataclass(frozen=True)
class Plane:
    """One array that a mixer keeps per cached token: keys, values, a latent row, whatever its
    kernels read back.  The cache allocates ``[pages + 1, *page_shape]`` for it per cache entry
    and never looks inside a page: ``page_shape`` is the shape of one page (the cache's page size
    in positions, arranged as the mixer's kernels want them), ``layout`` a name for that
    arrangement, which whoever reads or writes the plane checks, and ``dtype`` the element type
    (None: the dtype of the activations)."""
    name: str
    page_shape: Tuple[int, ...]
    layout: str = "rows"
    dtype: Optional[torch.dtype] = None


def rows_plane(name: str, per_token: Tuple[int, ...], page: int, dtype=None) -> Plane:
    """The plain arrangement: a page is ``[page, *per_token]``, position after position."""
    return Plane(name, (page,) + tuple(per_token), "rows", dtype)


@dataclass
class CacheNeed:
    """What a mixer keeps per token: its planes, and which positions.  ``kind`` "full" keeps
    every position; "window" needs only the last ``window`` positions.  Cache entries with equal
    needs share a group of the cache, and each group has storage of its own."""
    kind: str
    planes: Tuple[Plane, ...]
    window: int = 0

    def key(self):
        return (self.kind, tuple(self.planes), self.window)

    def plane(self, name: str) -> Optional[Plane]:
        return next((p for p in self.planes if p.name == name), None)


@dataclass
class StateNeed:
    """Fixed-size state a mixer keeps per sequence (for instance a recurrent state)."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class CacheView:
    """One cache entry as a mixer sees it: its planes by name, each ``[pages, *page_shape]``, and
    the table that maps (slot, position // page_size) to a page."""

    def __init__(self, planes: Dict[str, torch.Tensor], block_table, page_size, need: CacheNeed):
        self.planes = dict(planes)
        self.block_table = block_table
        self.page_size = page_size
        self.need = need

    def plane(self, name: str) -> torch.Tensor:
        if name not in self.planes:
            raise KeyError("this cache entry has no plane %r (it has: %s)" % (name, ", ".join(sorted(self.planes)) or "none"))
        return self.planes[name]


class Stream:
    """The residual stream of a step: the 32-bit running sum and the output of the last part,
    which the next norm adds before it normalises (so the sum is formed once, in 32-bit)."""

    def __init__(self, res: torch.Tensor):
        self.res = res            # [tokens, width] float32
        self.delta = None         # what is still to be added: [tokens, width], or [n, tokens, width] float32, or None
        self.pre = None           # what a product that added into ``res`` has left for the next norm

    def put(self, out) -> None:
        """Takes what a mixer or feed-forward returned: rows still to be added (a matrix in the
        activation dtype, or a stack ``[n, tokens, width]`` of float32 matrices that are added
        one after another, in their order: the slices of K of a product, or the results of two
        parts that read the same rows), None (it added them itself), or the record
        ``ops.linear(..., then_norm=)`` returned when it added them and prepared the norm that
        comes next."""
        is_rows = out is None or isinstance(out, torch.Tensor)
        self.delta = out if is_rows else None
        self.pre = None if is_rows else out

    def settle(self) -> torch.Tensor:
        """Adds what is still to be added into the 32-bit sum, in the order the norm kernel
        adds it, and returns the sum: for a norm that has no kernel which adds and normalises
        in one pass (the RMS norm's does)."""
        delta, self.delta, self.pre = self.delta, None, None
        if delta is not None:
            for part in (delta if delta.dim() == 3 else [delta]):
                self.res.add_(part)
        return self.res


class StepContext:
    """Everything a part may look at during one step.

    Device tensors (int32): ``tokens`` [M], ``tok_pos`` [M] absolute position of each token,
    ``tok_seq`` [M] index of its sequence in this step, ``seq_start`` [B+1] offsets of the
    sequences in the packed rows, ``seq_slot`` [B], ``seq_pos0`` [B] tokens already cached
    before the step.  Host values: ``seq_lens``, ``seq_pos0_host`` and ``seq_slot_host`` (lists),
    ``max_new`` (largest number of new tokens of a sequence) and ``max_ctx`` (largest cached
    length after the step).

    ``captured`` says that the step runs over the fixed buffers of a captured shape.  Then
    ``max_new`` and ``max_ctx`` are upper bounds (kernels size their grids by them and read the
    true lengths from device memory), and the host lists describe the padded step: padding rows
    are sequences in the sink slot.  The lists are filled in before every run of the step, so a
    part that runs from the host (``graph_safe = False``) finds them valid, with ``captured`` set
    or not; a part whose work is recorded into a graph (``graph_safe = True``) must not read them
    at all, since what it read at the recording would be replayed for every later step.
    """

    def __init__(self, ops, dtype, n_tokens, n_seqs):
        self.ops = ops
        self.dtype = dtype
        self.n_tokens = n_tokens
        self.n_seqs = n_seqs
        self.tokens = None
        self.tok_pos = None
        self.tok_seq = None
        self.seq_start = None
        self.seq_slot = None
        self.seq_pos0 = None
        self.seq_lens: List[int] = []
        self.seq_pos0_host: List[int] = []
        self.seq_slot_host: List[int] = []
        self.max_new = 0
        self.max_ctx = 0
        self.decode = False        # every sequence brings exactly one token
        self.unequal = False       # a decode step whose sequences' cached lengths differ widely: work is then best dealt out by length, not by sequence
        # (stream tensor, weight, eps) while the next thing to read that stream is an RMS norm
        # with these, nothing else touching it in between: a product that adds into the stream
        # may then prepare that norm (``ops.linear(..., then_norm=)``).  Set by blocks.
        self.then_norm = None
        self.norm_after_block = None   # the norm that reads the stream first after the running block, if known
        self.captured = False      # the step runs over the fixed buffers of a captured shape (see above)
        self.want_all_rows = False  # the logits of every row are wanted, in order (a decode step): the last norm gathers nothing
        self._kv: Dict[int, CacheView] = {}
        self._state: Dict[int, torch.Tensor] = {}

    def kv(self, cache_entry: int) -> Optional[CacheView]:
        return self._kv.get(cache_entry)

    def state(self, cache_entry: int) -> Optional[torch.Tensor]:
        """Per-sequence state of a cache entry: ``[slots, *shape]``; row ``seq_slot[b]`` belongs
        to sequence b and is zero when the sequence starts."""
        return self._state.get(cache_entry)


class Part:
    """Common protocol: declare tensors, receive them."""

    def weights(self) -> Dict[str, WeightDecl]:
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor], ops, dtype) -> None:
        pass


class Embedding(Part):
    """The input layer: makes the residual stream of a step from its tokens.

    ``weights()`` names its tensors in full (an input layer has no prefix); ``forward(ctx,
    then_norm)`` returns a ``Stream`` whose ``res`` is the float32 matrix ``[tokens, width]``.
    ``then_norm`` = (weight, eps) says that a plain RMS norm with these reads the rows first; an
    input layer may prepare it in the same kernel (``Stream.pre``) or ignore the hint.  It reads
    ``ctx.tokens`` and, if it wants, ``ctx.tok_pos`` (learned positions); ``graph_safe`` as for
    the other parts."""
    graph_safe = False

    def forward(self, ctx: "StepContext", then_norm=None) -> "Stream":
        raise NotImplementedError


class Mixer(Part):
    """Mixes information between the tokens of a sequence (attention, a recurrence, ...).

    ``forward(ctx, x, entry)`` takes the normalised rows ``[M, width]`` in the activation dtype
    and returns rows of the same shape.  ``entry`` is the schedule entry of this run; the mixer
    reads what it keeps per token through ``ctx.kv(entry.cache)`` (a ``CacheView``) and its state through
    ``ctx.state(entry.cache)``, and writes them only if ``entry.writes``.

    Two optional abilities, off unless the class sets them (they apply to feed-forwards too):
    ``takes_normed = True``: ``x`` may be the record that ``ops.normed`` returns instead of a
    matrix; the part hands it to ``ops.linear`` / ``ops.linear_swiglu`` / ``ops.qkv_rope`` only,
    which decide how the norm is run (on which rows, in which dtype, in which kernel).
    ``adds_to_stream = True``: ``forward`` takes a keyword ``residual`` (the
    float32 stream) and may add its result into it, returning None.
    """
    takes_normed = False
    adds_to_stream = False

    def cache_need(self, page: int) -> Optional[CacheNeed]:
        """What the mixer keeps per token, for a cache whose pages hold ``page`` positions."""
        return None

    def state_need(self) -> Optional[StateNeed]:
        return None

    def forward(self, ctx: StepContext, x: torch.Tensor, entry) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """Row-wise transformation: ``forward(ctx, x [M, width]) -> [M, width]``."""
    takes_normed = False
    adds_to_stream = False

    def forward(self, ctx: StepContext, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Norm(Part):
    """``add_norm(ctx, stream, rows)``: adds ``stream.delta`` (if any) into ``stream.res`` in
    32-bit, then returns the normalised rows in the activation dtype.  With ``rows`` (int32
    indices) only those rows are normalised and returned, in that order.  With ``lazy`` a norm
    whose consumer ``takes_normed`` may return ``ctx.ops.normed(...)`` instead, when nothing is
    left to add: the record names the rows, and the product that takes it runs the norm."""

    def add_norm(self, ctx: StepContext, stream: Stream, rows=None, lazy=False) -> torch.Tensor:
        raise NotImplementedError

    def rms_terms(self):
        """(weight, eps) if this is a plain RMS norm, y = x * weight * rsqrt(mean(x^2) + eps),
        which a product before it may prepare; else None."""
        return None


class Block:
    """Arrangement of a mixer, a feed-forward and norms around the residual stream."""

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, norms: List[Norm]):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms

    def forward(self, ctx: StepContext, stream: Stream, entry) -> None:
        raise NotImplementedError

    def entry_norm(self) -> Optional[Norm]:
        """The norm that reads the stream first when this block runs, if nothing else touches
        the stream before it; else None."""
        return None

    @staticmethod
    def announce(ctx: StepContext, stream: Stream, norm: Optional[Norm]) -> None:
        """Says (or, with None, takes back) that ``norm`` reads the stream next."""
        terms = norm.rms_terms() if norm is not None else None
        ctx.then_norm = (stream.res,) + tuple(terms) if terms else None
