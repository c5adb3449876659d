"""A decoder assembled from a ModelSpec: embedding, scheduled blocks, final norm, output matrix.

This class is the same for every architecture; what differs between architectures is the
ModelSpec their configuration produces (src/libllm/llama.cc:273-312 is the reference's fixed
counterpart for Llama).
"""
from typing import Dict, Optional

import torch

from ..config.spec import ModelSpec, validate_schedule
from ..errors import ConfigError
from ..parts import (Stream, StepContext, WeightDecl, build_block, build_embedding, build_feed_forward,
                     build_head, build_mixer, build_norm)


def _build_layers(spec: ModelSpec):
    blocks = []
    for ls in spec.layers:
        mixer = build_mixer(ls.mixer)
        ff = build_feed_forward(ls.feed_forward)
        norms = [build_norm(n) for n in ls.norms]
        blocks.append(build_block(ls.block, mixer, ff, norms))
    return blocks


def _layer_decls(block, ls):
    out = {}
    groups = [("mixer", block.mixer), ("feed_forward", block.feed_forward)]
    groups += [("norm%d" % i, n) for i, n in enumerate(block.norms)]
    for role, part in groups:
        decls = part.weights()
        if decls and role not in ls.prefixes:
            raise ConfigError("layer record has no tensor-name prefix for %r" % role)
        for rel, decl in decls.items():
            out[ls.prefixes[role] + rel] = (part, rel, decl)
    return out


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        validate_schedule(spec)
        self.spec = spec
        self.embedding = build_embedding(spec.embedding)
        self.blocks = _build_layers(spec)
        self.final_norm = build_norm(spec.final_norm)
        self.head = build_head(spec.head)
        self._decls = None

    # ---- weights
    def _collect(self):
        if self._decls is None:
            s = self.spec
            d = {}
            for name, decl in self.embedding.weights().items():      # an input layer names its tensors in full
                d[name] = (self.embedding, name, decl)
            if not s.head.tied:
                if s.head.tensor in d:
                    raise ConfigError("tensor %r is declared by two parts" % s.head.tensor)
                d[s.head.tensor] = (None, "head", WeightDecl((s.head.vocab, s.head.width)))
            elif s.head.tensor not in d or tuple(d[s.head.tensor][2].shape) != (s.head.vocab, s.head.width):
                raise ConfigError("the output layer is tied to %r, which the input layer does not declare as a "
                                  "[%d, %d] matrix" % (s.head.tensor, s.head.vocab, s.head.width))
            for block, ls in zip(self.blocks, s.layers):
                for name, item in _layer_decls(block, ls).items():
                    if name in d:
                        raise ConfigError("tensor %r is declared by two parts" % name)
                    d[name] = item
            for rel, decl in self.final_norm.weights().items():
                d[s.final_norm_prefix + rel] = (self.final_norm, rel, decl)
            self._decls = d
        return self._decls

    def declared(self) -> Dict[str, WeightDecl]:
        return {name: item[2] for name, item in self._collect().items()}

    def bind(self, tensors: Dict[str, torch.Tensor], ops, dtype) -> None:
        s = self.spec
        per_part: Dict[int, Dict[str, torch.Tensor]] = {}
        parts = {}
        for name, (part, rel, _decl) in self._collect().items():
            if part is None:
                continue
            per_part.setdefault(id(part), {})[rel] = tensors[name]
            parts[id(part)] = part
        for pid, part in parts.items():
            part.bind(per_part[pid], ops, dtype)
        for block in self.blocks:                       # parts without tensors still get ops
            for part in [block.mixer, block.feed_forward] + list(block.norms):
                if id(part) not in parts:
                    part.bind({}, ops, dtype)
        if id(self.embedding) not in parts:
            self.embedding.bind({}, ops, dtype)
        self.head.bind(tensors[s.head.tensor], ops, dtype)      # the input layer's table, if tied

    # ---- what the cache has to hold
    def cache_needs(self, page: int):
        """What every cache entry keeps per token, for a cache whose pages hold ``page`` positions."""
        needs = [None] * self.spec.n_cache_entries()
        for e in self.spec.schedule:
            if e.writes:
                needs[e.cache] = self.blocks[e.layer].mixer.cache_need(page)
        return needs

    def state_needs(self):
        needs = [None] * self.spec.n_cache_entries()
        for e in self.spec.schedule:
            if e.writes:
                needs[e.cache] = self.blocks[e.layer].mixer.state_need()
        return needs

    def graph_safe(self) -> bool:
        """True if no part reads host-side step data, so a whole step can be captured."""
        return all(safe for safe, _ in self.stretches()) and len(self.stretches()) == 1

    # ---- one step over packed rows, in units: the embedding, every run of the schedule, the output
    def n_units(self) -> int:
        return len(self.spec.schedule) + 2

    def unit_is_graph_safe(self, unit: int) -> bool:
        """Whether a unit reads nothing from the host while it runs (so it can be captured)."""
        n = len(self.spec.schedule)
        if unit == 0:
            return getattr(self.embedding, "graph_safe", False)
        if unit == n + 1:
            return getattr(self.final_norm, "graph_safe", False) and getattr(self.head, "graph_safe", False)
        block = self.blocks[self.spec.schedule[unit - 1].layer]
        return all(getattr(part, "graph_safe", False)
                   for part in [block.mixer, block.feed_forward] + list(block.norms))

    def stretches(self):
        """The units of a step cut into runs of neighbours that are all graph-safe or all not:
        [(safe, [units])].  A model whose parts all are gives one stretch."""
        out = []
        for unit in range(self.n_units()):
            safe = self.unit_is_graph_safe(unit)
            if out and out[-1][0] == safe:
                out[-1][1].append(unit)
            else:
                out.append((safe, [unit]))
        return out

    def run_unit(self, unit: int, ctx: StepContext, stream: Optional[Stream], want_rows):
        """Runs one unit.  Unit 0 returns the stream it has made from the tokens; the last unit
        returns float32 logits (None if no row is wanted); the others return None."""
        s = self.spec
        n = len(s.schedule)
        if unit == 0:
            # if a plain RMS norm reads the rows first, the input layer may prepare it
            first = self.blocks[s.schedule[0].layer].entry_norm() if n else self.final_norm
            terms = first.rms_terms() if first is not None and (n or ctx.want_all_rows) else None
            return self.embedding.forward(ctx, terms)
        if unit == n + 1:
            ctx.norm_after_block = None
            if want_rows is None or want_rows.numel() == 0:
                return None
            # every row wanted, in order: no gather, and the product before may have prepared the norm
            rows = None if ctx.want_all_rows else want_rows
            h = self.final_norm.add_norm(ctx, stream, rows=rows,
                                         lazy=getattr(self.head, "takes_normed", False))
            return self.head.forward(ctx, h)
        i = unit - 1
        entry = s.schedule[i]
        # the block is told which norm reads the stream after it, so that its last product
        # may prepare that norm (the final norm gathers rows and is left alone)
        nxt = s.schedule[i + 1] if i + 1 < n else None
        if nxt is not None:
            ctx.norm_after_block = self.blocks[nxt.layer].entry_norm()
        else:
            ctx.norm_after_block = self.final_norm if ctx.want_all_rows else None
        self.blocks[entry.layer].forward(ctx, stream, entry)
        return None

    def forward(self, ctx: StepContext, want_rows: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        """Runs every token of the step through the schedule; returns float32 logits
        ``[len(want_rows), vocab]`` (None if no row is wanted)."""
        stream = self.run_unit(0, ctx, None, want_rows)
        for unit in range(1, self.n_units() - 1):
            self.run_unit(unit, ctx, stream, want_rows)
        return self.run_unit(self.n_units() - 1, ctx, stream, want_rows)


def declared_weights(spec: ModelSpec) -> Dict[str, WeightDecl]:
    return DecoderModel(spec).declared()
