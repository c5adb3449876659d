"""The step function: runs the tokens it is given, as one batch, from the cache.

A step carries, for each of its requests, the next tokens of that request (a whole prompt, a part
of it, or one decoded token) and the places among them whose logits are wanted.  All rows of all
requests are packed one after another; no padding enters the model.  The reference has two entry
points for one sequence, prefill and decode (src/libllm/llama.cc:349-368); this is their
generalisation to unequal batches.
"""
import warnings
from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache import PAGE, SequenceCache
from ..errors import CacheError, ReplayMismatch, RequestError
from ..parts import StepContext
from .model import DecoderModel


@dataclass
class StepEntry:
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()          # indices into ``tokens`` whose logits are returned


class Engine:
    """Owns a bound model, its cache and the step function."""

    # batch sizes the decode graphs are captured for; a step runs in the smallest that holds it, its
    # spare rows pointing at the sink.  With powers of two alone a batch of 40 paid for 64 rows
    # (2.73 ms a step at the 1B shape against 2.43 in a graph of 48).  Beyond 256 rows a step is
    # queued kernel by kernel, which takes the host 4 to 5 ms at the 1B shape: less than the
    # device needs for that many rows unless the contexts are short.
    GRAPH_BATCHES = (1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64, 80, 96, 112, 128, 160, 192, 224, 256)
    GRAPH_MIN_CTX = 1024
    # A decode step whose longest sequence holds at least UNEQUAL_MIN tokens and UNEQUAL_RATIO times
    # the mean runs with ``ctx.unequal`` (a graph of its own): decode attention then deals its pages
    # out by length.  With the same number of blocks for every sequence, 63 sequences of 2,048
    # tokens beside one of 131,072 took 13.4 ms a step at the 1B shape.
    UNEQUAL_MIN = 4096
    UNEQUAL_RATIO = 2.0
    # Steps that bring whole prompts are captured too, padded to one of these numbers of rows and
    # of sequences (one sequence is always spare: it takes the padding rows, in the sink slot).  A
    # shape is captured when it comes the second time, so that a lone prompt does not pay for it.
    # Queued from the host a prompt of up to some hundred tokens waits for the host, not the device.
    # Up to 128 rows the steps are 16 apart, as the products' forms are: a prompt of 70 tokens in
    # a graph of 80 or 96 rows takes 1.47 ms where one of 128 rows takes 1.58 (1B shape; 5.34
    # against 5.85 at 8B).  Beyond, the vendor library's products run, whose time grows evenly with
    # the rows but for a few row counts at which its choice of kernel is poor: at exactly 192 rows
    # the four products of a layer take 153 us where they take 108 at 184 rows and 111 at 200 (3B
    # shape; 237 against 177 and 182 at 8B; 1B the same everywhere), and likewise at 160 rows of
    # the 8B shape.  Hence 176 and 224 between 128 and 256, and no 192.
    PROMPT_ROWS = (16, 32, 48, 64, 80, 96, 112, 128, 176, 224, 256, 384, 512, 768, 1024, 1536, 2048)
    PROMPT_SEQS = (2, 3, 5, 9, 17)
    PROMPT_SEEN = 2
    PROMPT_GRAPHS = 24      # prompt graphs kept; the one unused for longest goes first (each holds its activations)
    DECODE_GRAPHS = 64      # decode graphs kept, likewise (all twenty of one context length hold 2.8 GB at the 1B shape)

    def __init__(self, model: DecoderModel, ops, dtype: torch.dtype, max_tokens: int,
                 max_slots: Optional[int] = None, use_graphs: bool = True):
        self.model = model
        self.ops = ops
        self.dtype = dtype
        self.device = ops.device
        self.vocab = model.spec.vocab
        self.cache = SequenceCache(model.cache_needs(PAGE), model.state_needs(), max_tokens,
                                   model.spec.max_position, dtype, self.device, max_slots)
        # a part that reads the step's host-side data cannot be captured; the stretches of the
        # schedule around it still are (see _CapturedForward)
        self.use_graphs = bool(use_graphs) and ops.supports_graphs and not getattr(ops, "timing", False)
        self._graphs: Dict[tuple, "_DecodeGraph"] = {}     # (batch bucket, context bucket) -> graph
        self._prompt_graphs: Dict[tuple, "_PromptGraph"] = {}   # (rows, sequences) -> graph
        self._prompt_seen: Dict[tuple, int] = {}
        self._no_graph = set()         # shapes whose replays did not give the eager step's bits
        self.steps_run = 0

    # ---- requests
    def live_requests(self):
        return self.cache.slots.live()

    def room(self):
        """(free slots, free pages): what requests that start now can take; the pages of the
        group of layers that has the fewest left."""
        return self.cache.slots.n_free, min(g.pool.n_free for g in self.cache.groups)

    def end(self, requests) -> None:
        for r in requests:
            self.cache.release(r)

    def holds(self, request) -> bool:
        return self.cache.holds(request)

    def length(self, request) -> int:
        return self.cache.length(self.cache.slot_of(request))

    # ---- the step
    takes_device_tokens = True

    def step(self, entries: List[StepEntry], tokens_device: Optional[torch.Tensor] = None
             ) -> Optional[torch.Tensor]:
        """Returns float32 logits ``[wanted, vocab]`` in the order of the entries and of their
        ``want`` lists, or None if nothing is wanted.  The tensor may be a view of a captured
        graph's output buffer: it holds these logits until the next call of ``step``, which may
        overwrite it (on the same stream, so work already queued on it, such as sampling, still
        reads this step's values).  A caller that keeps logits across steps copies them;
        ``Model.step`` does.

        With ``tokens_device`` (int32 on the device, one per entry, for instance what the sampler
        just wrote) every entry brings exactly one token and that tensor holds it: the ids in the
        entries are placeholders, and the host need not know the tokens to start the step."""
        if not entries:
            raise RequestError("a step needs at least one entry")
        if tokens_device is not None:
            if (tokens_device.dtype != torch.int32 or tokens_device.device != self.device
                    or tuple(tokens_device.shape) != (len(entries),)):
                raise RequestError("tokens_device must be int32 on the device, one per entry")
            if any(len(e.tokens) != 1 for e in entries):
                raise RequestError("with tokens_device every entry brings exactly one token")
        seen = set()
        for e in entries:
            if e.request in seen:
                raise RequestError("request %r appears twice in one step" % (e.request,))
            seen.add(e.request)
            if len(e.tokens) == 0:
                raise RequestError("request %r brings no tokens" % (e.request,))
            if len(e.tokens) == 1 and type(e.tokens[0]) is int:          # a decode step's entry
                lo = hi = e.tokens[0]
            else:
                ids = np.asarray(e.tokens)
                if ids.ndim != 1 or ids.dtype.kind not in "iu":
                    raise RequestError("request %r: token ids are a flat list of integers" % (e.request,))
                lo, hi = int(ids.min()), int(ids.max())
            if tokens_device is None and (lo < 0 or hi >= self.vocab):
                raise RequestError("request %r has a token id outside [0, %d)" % (e.request, self.vocab))
            for w in e.want:
                if not 0 <= w < len(e.tokens):
                    raise RequestError("request %r wants row %d of %d" % (e.request, w, len(e.tokens)))
        cache = self.cache
        fresh = [e.request for e in entries if not cache.holds(e.request)]
        if len(fresh) > cache.slots.n_free:
            raise CacheError("no free slot: %d requests start, %d slots free"
                             % (len(fresh), cache.slots.n_free))
        plan = [(cache.slot_of(e.request) if cache.holds(e.request) else None,
                 cache.length(cache.slot_of(e.request)) if cache.holds(e.request) else 0,
                 len(e.tokens)) for e in entries]
        for slot, length, n_new in plan:
            if length + n_new > cache.max_position:
                raise CacheError("a sequence of %d tokens exceeds max_position_embeddings %d"
                                 % (length + n_new, cache.max_position))
        if not cache.can_reserve(plan):
            raise CacheError("the cache is full: this step needs more pages than are free "
                             "(max_tokens %d, %d tokens held)"
                             % (cache.n_pages * PAGE, cache.tokens_held()))
        slots = []
        for e in entries:
            slot = cache.slot_of(e.request) if cache.holds(e.request) else cache.admit(e.request)
            cache.reserve(slot, len(e.tokens))
            slots.append(slot)
        cache.flush()

        lens = [len(e.tokens) for e in entries]
        pos0 = [cache.length(s) for s in slots]
        want_all_single = all(n == 1 for n in lens) and all(list(e.want) == [0] for e in entries)
        graph = None
        if self.use_graphs and want_all_single and len(entries) <= self.GRAPH_BATCHES[-1] \
                and (graph := self._decode_graph(len(entries), pos0)) is not None:
            logits = graph.run([e.tokens[0] for e in entries], slots, pos0, tokens_device)
        elif self.use_graphs and tokens_device is None and not all(n == 1 for n in lens) \
                and (graph := self._prompt_graph(entries, lens)) is not None:
            logits = graph.run(entries, slots, lens, pos0)
        else:
            ctx, want_rows = self._context(entries, slots, lens, pos0)
            if tokens_device is not None:
                ctx.tokens = tokens_device.contiguous()
            logits = self.model.forward(ctx, want_rows)
        for s, n in zip(slots, lens):
            cache.commit(s, n)
        cache.flush()
        self.steps_run += 1
        return logits

    # ---- building the packed batch
    def _context(self, entries, slots, lens, pos0):
        b = len(entries)
        m = sum(lens)
        starts = np.zeros(b + 1, dtype=np.int64)
        starts[1:] = np.cumsum(lens)
        tokens = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries])
        tok_seq = np.repeat(np.arange(b, dtype=np.int64), lens)
        tok_pos = np.arange(m, dtype=np.int64) - starts[tok_seq] + np.asarray(pos0, dtype=np.int64)[tok_seq]
        want = [int(starts[i]) + int(w) for i, e in enumerate(entries) for w in e.want]
        packed = np.concatenate([tokens, tok_pos, tok_seq, starts, np.asarray(slots, dtype=np.int64),
                                 np.asarray(pos0, dtype=np.int64),
                                 np.asarray(want, dtype=np.int64)]).astype(np.int32)
        dev = self.ops.upload_int32(packed)
        ctx = StepContext(self.ops, self.dtype, m, b)
        o = 0
        ctx.tokens = dev[o:o + m]; o += m
        ctx.tok_pos = dev[o:o + m]; o += m
        ctx.tok_seq = dev[o:o + m]; o += m
        ctx.seq_start = dev[o:o + b + 1]; o += b + 1
        ctx.seq_slot = dev[o:o + b]; o += b
        ctx.seq_pos0 = dev[o:o + b]; o += b
        want_rows = dev[o:o + len(want)]
        ctx.seq_lens = list(lens)
        ctx.seq_pos0_host = list(pos0)
        ctx.seq_slot_host = list(slots)
        ctx.max_new = max(lens)
        ctx.max_ctx = max(p + n for p, n in zip(pos0, lens))
        ctx.decode = all(n == 1 for n in lens)
        ctx.unequal = ctx.decode and self._unequal(pos0)
        ctx.want_all_rows = want == list(range(m))
        self._attach_cache(ctx)
        return ctx, want_rows

    def _attach_cache(self, ctx):
        for entry in range(self.model.spec.n_cache_entries()):
            view = self.cache.kv_view(entry)
            if view is not None:
                ctx._kv[entry] = view
            if entry in self.cache.state:
                ctx._state[entry] = self.cache.state[entry]

    # ---- whole prompts through a captured graph
    def _prompt_graph(self, entries, lens):
        """The captured graph that holds this step, or None if the step runs from the host."""
        m, b = sum(lens), len(entries)
        wanted = sum(len(e.want) for e in entries)
        if m > self.PROMPT_ROWS[-1] or b + 1 > self.PROMPT_SEQS[-1]:
            return None
        rows = next(r for r in self.PROMPT_ROWS if r >= m)
        seqs = next(q for q in self.PROMPT_SEQS if q >= b + 1)
        # the spare sequence may take all rows but one, at positions 0..: they must lie within a
        # row of the page table and within the position encoding's tables (the position limit
        # need not be a multiple of a page); the wanted rows must fit the places the graph has
        if rows > min(self.cache.pages_per_seq * PAGE, self.cache.max_position) or wanted > seqs:
            return None
        key = (rows, seqs)
        if ("prompt",) + key in self._no_graph:
            return None
        graph = self._prompt_graphs.pop(key, None)
        if graph is None:
            seen = self._prompt_seen.get(key, 0) + 1
            self._prompt_seen[key] = seen
            if seen < self.PROMPT_SEEN:
                return None
            while len(self._prompt_graphs) >= max(1, self.PROMPT_GRAPHS):
                del self._prompt_graphs[next(iter(self._prompt_graphs))]     # dicts keep the order of insertion
            graph = self._checked(("prompt",) + key, lambda: _PromptGraph(self, rows, seqs))
            if graph is None:
                return None
        self._prompt_graphs[key] = graph                                      # the last used lies last
        return graph

    def _checked(self, key, make):
        """The graph that ``make`` captures, or None if its replays do not give what the same
        step gives queued kernel by kernel: steps of that shape then run from the host, and a
        warning says so once."""
        try:
            return make()
        except ReplayMismatch as e:
            self._no_graph.add(key)
            warnings.warn("libllm_amd: %s; steps of this shape run without a captured graph" % e)
            return None

    # ---- decoding one token per sequence through a captured graph
    def _unequal(self, pos0) -> bool:
        longest, total = max(pos0) + 1, sum(pos0) + len(pos0)
        return len(pos0) > 1 and longest >= self.UNEQUAL_MIN and longest * len(pos0) >= self.UNEQUAL_RATIO * total

    def _decode_graph(self, b, pos0):
        """The captured graph for a decode step of ``b`` sequences, or None if there is none."""
        bucket = next(g for g in self.GRAPH_BATCHES if g >= b)
        # the longest context a graph serves is part of its key: kernels size their grids by it
        limit = self.cache.pages_per_seq * PAGE
        ctx_bucket = self.GRAPH_MIN_CTX
        while ctx_bucket < max(pos0) + 1:
            ctx_bucket *= 2
        ctx_bucket = min(ctx_bucket, limit)
        unequal = self._unequal(pos0)
        key = (bucket, ctx_bucket, unequal)
        graph = self._graphs.pop(key, None)
        if graph is None and ("decode",) + key not in self._no_graph:
            while len(self._graphs) >= max(1, self.DECODE_GRAPHS):
                del self._graphs[next(iter(self._graphs))]                  # dicts keep the order of insertion
            graph = self._checked(("decode",) + key, lambda: _DecodeGraph(self, bucket, ctx_bucket, unequal))
        if graph is not None:
            self._graphs[key] = graph                                       # the last used lies last
        return graph


class _CapturedForward:
    """``model.forward`` over fixed device buffers, ready to be run again and again: the stretches
    of units whose parts read nothing from the host are captured HIP graphs, the units between
    them (a part with ``graph_safe = False``) run from the host each time, on the same stream.

    What passes from one stretch to the next is the residual stream: its 32-bit sum, which the
    parts change in place, and the rows still to be added.  A captured stretch leaves them at
    fixed addresses; what a host-run unit returns lies somewhere new each time and is copied to
    a buffer that the next captured stretch was captured with (a prepared norm that such a unit
    may leave is dropped: the next norm then works from the sum itself).  The state of the stream
    object at every border is kept from set-up, since a replayed graph runs no Python.

    With ``check``, the captured step is replayed ``CHECK_REPLAYS`` times over the buffers it was
    captured with before it serves, and must give, every time, the logits that the same step gave
    queued kernel by kernel, or ReplayMismatch is raised: work may be recorded into a graph that
    does not replay (see ``HipOps.capture``).  This asks for a step that gives the same bits
    whenever it runs: a decode step of padding alone does (every row is the same token at
    position 0 of the sink slot), a prompt step of padding alone does not (its rows a page apart
    write to the same places of the sink page), and a model whose parts keep state of their own
    per sequence does not either, since running a step again moves that state on."""

    CHECK_REPLAYS = 2

    def __init__(self, model, ops, ctx, want_rows, check=False):
        self.model, self.ctx, self.want_rows = model, ctx, want_rows
        self.stream = self.logits = None
        reference = None
        check = check and self.CHECK_REPLAYS > 0 and all(need is None for need in model.state_needs())
        if check:
            # the same step from the host, cut where the captured one is cut: after a stretch
            # that runs from the host the next norm works from the sum itself, here too
            for safe, units in model.stretches():
                self._run(units)
                if not safe:
                    self.stream.pre = None
            reference = None if self.logits is None else self.logits.clone()
            self.stream = self.logits = None
        self.pieces = []                 # (graph or None, units, border state after the piece)
        self.stream = None
        self.logits = None
        last = model.n_units() - 1
        for safe, units in model.stretches():
            before = self.pieces[-1][2] if self.pieces else None
            if safe:
                # (the capture runs its body twice, once to warm up: each run starts from the
                # stream as the piece before left it)
                graph = ops.capture(lambda units=units, before=before: self._run(units, before))
                graph.replay()           # its results are real for the host-run unit that may follow
                self.pieces.append((graph, units, self._border()))
            else:
                self._run(units, before)
                static = None
                if self.stream.delta is not None:
                    static = self.stream.delta.clone()
                self.stream.delta, self.stream.pre = static, None
                self.pieces.append((None, units, self._border()))
        self.n_graphs = sum(1 for g, _, _ in self.pieces if g is not None)
        self.n_host_pieces = len(self.pieces) - self.n_graphs
        self.last_unit = last
        if check and self.n_graphs:
            for replay in range(self.CHECK_REPLAYS):
                if not self._same(self.run(), reference):
                    raise ReplayMismatch("replay %d of a captured step of %d rows differs from the step queued "
                                         "kernel by kernel" % (replay + 1, ctx.n_tokens))

    @staticmethod
    def _same(out, reference) -> bool:
        if out is None or reference is None:
            return out is None and reference is None
        # bit for bit, so that a NaN equals itself
        return out.shape == reference.shape and torch.equal(out.view(torch.int32), reference.view(torch.int32))

    def _run(self, units, before=None):
        if before is not None:
            self.stream.res, self.stream.delta, self.stream.pre = before
        for unit in units:
            out = self.model.run_unit(unit, self.ctx, self.stream, self.want_rows)
            if unit == 0:
                self.stream = out
            elif unit == self.model.n_units() - 1:
                self.logits = out

    def _border(self):
        return (self.stream.res, self.stream.delta, self.stream.pre)

    def run(self):
        """Runs the step that the buffers hold; returns the logits (None if no row is wanted)."""
        before = None
        for graph, units, border in self.pieces:
            if graph is not None:
                graph.replay()
            else:
                self._run(units, before)
                res, delta, _ = border
                if self.stream.res is not res:
                    res.copy_(self.stream.res)
                if (self.stream.delta is None) != (delta is None):
                    raise RequestError("a part that runs from the host changed what it returns between steps")
                if delta is not None:
                    delta.copy_(self.stream.delta)
            before = border
        return self.logits


class _DecodeGraph:
    """One captured decode step for a batch of exactly ``bucket`` rows whose sequences hold at
    most ``max_ctx`` tokens after the step (``unequal``: of widely different lengths).  Rows beyond the live sequences point at the cache's
    sink slot and page, so they change nothing that is read."""

    RING = 4

    def __init__(self, engine: Engine, bucket: int, max_ctx: int, unequal: bool = False):
        # no reference back to the engine: an engine that is dropped then goes at once, with its
        # graphs, and not whenever the collector of cycles next runs
        self.model = engine.model
        self.sink_slot = engine.cache.sink_slot
        self.bucket = bucket
        ops = engine.ops
        b = bucket
        # pinned host copies, so that an upload does not wait for the device; a ring of them, as
        # the device may run several steps behind the host and each upload reads its copy late
        self.ring = [torch.zeros(7 * b + 1, dtype=torch.int32, pin_memory=True) for _ in range(self.RING)]
        self.ring_done = [None] * self.RING
        self.turn = 0
        self.static = self.ring[0].to(ops.device)
        ctx = StepContext(ops, engine.dtype, b, b)
        o = 0
        ctx.tokens = self.static[o:o + b]; o += b
        ctx.tok_pos = self.static[o:o + b]; o += b
        ctx.tok_seq = self.static[o:o + b]; o += b
        ctx.seq_start = self.static[o:o + b + 1]; o += b + 1
        ctx.seq_slot = self.static[o:o + b]; o += b
        ctx.seq_pos0 = self.static[o:o + b]; o += b
        self.want_rows = self.static[o:o + b]
        ctx.max_new = 1
        ctx.max_ctx = max_ctx
        ctx.decode = True
        ctx.unequal = unequal
        ctx.captured = True
        ctx.want_all_rows = True       # the graph's wanted rows are all its rows, in order
        engine._attach_cache(ctx)
        self.ctx = ctx
        self._fill([0] * b, [engine.cache.sink_slot] * b, [0] * b)
        self.forward = _CapturedForward(self.model, ops, ctx, self.want_rows, check=True)

    def _fill(self, tokens, slots, pos0):
        b = self.bucket
        n = len(tokens)
        sink = self.sink_slot
        # for the parts that run from the host: the padding rows are sequences in the sink slot
        self.ctx.seq_lens = [1] * b
        self.ctx.seq_slot_host = list(slots) + [sink] * (b - n)
        self.ctx.seq_pos0_host = list(pos0) + [0] * (b - n)
        self.turn = (self.turn + 1) % self.RING
        if self.ring_done[self.turn] is not None:
            self.ring_done[self.turn].synchronize()        # its last upload has been read
        h = self.ring[self.turn].numpy()
        h[0:b] = 0
        h[0:n] = tokens
        h[b:2 * b] = 0
        h[b:b + n] = pos0
        h[2 * b:3 * b] = np.arange(b)
        h[3 * b:4 * b + 1] = np.arange(b + 1)
        h[4 * b + 1:5 * b + 1] = sink
        h[4 * b + 1:4 * b + 1 + n] = slots
        h[5 * b + 1:6 * b + 1] = 0
        h[5 * b + 1:5 * b + 1 + n] = pos0
        h[6 * b + 1:7 * b + 1] = np.arange(b)
        self.static.copy_(self.ring[self.turn], non_blocking=True)
        done = torch.cuda.Event()
        done.record()
        self.ring_done[self.turn] = done

    def run(self, tokens, slots, pos0, tokens_device=None):
        self._fill(tokens, slots, pos0)
        if tokens_device is not None:
            self.static[:len(tokens)].copy_(tokens_device, non_blocking=True)
        return self.forward.run()[:len(tokens)]


class _PromptGraph:
    """One captured step of exactly ``rows`` tokens in ``seqs`` sequences, any of which may hold
    past tokens.  The live sequences come first; the next one takes the rows that are left over,
    at positions 0.. of the sink slot, whose every page is the sink page; the others are empty.
    ``seqs`` places hold the wanted rows; spare ones ask for row 0.  Kernels read offsets, slots
    and lengths from device memory; their grids are sized for one sequence of all the rows."""

    RING = 4

    def __init__(self, engine: Engine, rows: int, seqs: int):
        self.model, self.sink_slot = engine.model, engine.cache.sink_slot     # and no reference back
        self.rows, self.seqs = rows, seqs
        ops = engine.ops
        t, b = rows, seqs
        self.size = 3 * t + (b + 1) + 3 * b
        self.ring = [torch.zeros(self.size, dtype=torch.int32, pin_memory=True) for _ in range(self.RING)]
        self.ring_done = [None] * self.RING
        self.turn = 0
        self.static = self.ring[0].to(ops.device)
        ctx = StepContext(ops, engine.dtype, t, b)
        o = 0
        ctx.tokens = self.static[o:o + t]; o += t
        ctx.tok_pos = self.static[o:o + t]; o += t
        ctx.tok_seq = self.static[o:o + t]; o += t
        ctx.seq_start = self.static[o:o + b + 1]; o += b + 1
        ctx.seq_slot = self.static[o:o + b]; o += b
        ctx.seq_pos0 = self.static[o:o + b]; o += b
        self.want_rows = self.static[o:o + b]
        ctx.max_new = t
        ctx.max_ctx = engine.cache.pages_per_seq * PAGE
        ctx.decode = False
        ctx.captured = True
        engine._attach_cache(ctx)
        self.ctx = ctx
        self._fill([], [], [], [], [])
        self.forward = _CapturedForward(self.model, ops, ctx, self.want_rows)

    def _fill(self, tokens, slots, lens, pos0, want):
        t, b = self.rows, self.seqs
        n, m = len(lens), len(tokens)
        sink = self.sink_slot
        # for the parts that run from the host: the spare sequence holds the rows left over, in
        # the sink slot, and the sequences after it are empty
        self.ctx.seq_lens = list(lens) + [t - m] + [0] * (b - n - 1)
        self.ctx.seq_slot_host = list(slots) + [sink] * (b - n)
        self.ctx.seq_pos0_host = list(pos0) + [0] * (b - n)
        self.turn = (self.turn + 1) % self.RING
        if self.ring_done[self.turn] is not None:
            self.ring_done[self.turn].synchronize()        # its last upload has been read
        h = self.ring[self.turn].numpy()
        starts = np.zeros(n + 1, dtype=np.int64)
        starts[1:] = np.cumsum(lens)
        tok_seq = np.repeat(np.arange(n, dtype=np.int64), lens)
        o = 0
        h[o:o + t] = 0
        h[o:o + m] = tokens; o += t
        h[o + m:o + t] = np.arange(t - m)                   # the spare sequence counts from 0
        if m:
            h[o:o + m] = np.arange(m) - starts[tok_seq] + np.asarray(pos0, dtype=np.int64)[tok_seq]
        o += t
        h[o:o + m] = tok_seq
        h[o + m:o + t] = n; o += t
        h[o:o + n + 1] = starts
        h[o + n + 1:o + b + 1] = t; o += b + 1               # the spare one ends at the last row, the rest are empty
        h[o:o + b] = sink
        h[o:o + n] = slots; o += b
        h[o:o + b] = 0
        h[o:o + n] = pos0; o += b
        h[o:o + b] = 0
        h[o:o + len(want)] = want
        self.static.copy_(self.ring[self.turn], non_blocking=True)
        done = torch.cuda.Event()
        done.record()
        self.ring_done[self.turn] = done

    def run(self, entries, slots, lens, pos0):
        starts = np.concatenate([[0], np.cumsum(lens)])
        want = [int(starts[i]) + int(w) for i, e in enumerate(entries) for w in e.want]
        tokens = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries])
        self._fill(tokens, slots, lens, pos0, want)
        logits = self.forward.run()
        return logits[:len(want)] if want else None
