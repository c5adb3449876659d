"""Grouped-query causal attention over the paged cache.

The reference's order (src/libllm/llama.cc:178-225): one stacked q|k|v product, split, rotate q
and k at absolute positions, append k and v to the past, softmax(q k^T / sqrt(hd)) v with query
head h reading kv head h // (n_heads / n_kv_heads) (src/flint/operators.cc:43-56,100-127), merge
heads, output product.  Here the rotation and the cache write are one kernel, and attention reads
keys and values from the cache for whole prompts and single tokens alike.
"""
from dataclasses import dataclass
from typing import Optional

import torch

from ..errors import ConfigError
from .base import PartSpec, Mixer, StepContext, WeightDecl
from .kv_pages import kv_need
from .linear import Linear
from .registry import build_position, register_mixer


@dataclass
class AttentionSpec(PartSpec):
    width: int = 0
    n_heads: int = 0
    n_kv_heads: int = 0
    head_dim: int = 0
    position: PartSpec = None
    qkv_bias: bool = False
    window: int = 0                   # 0: every earlier key; n: only the last n keys
    scale: Optional[float] = None     # None: head_dim ** -0.5
    q_name: str = "q_proj"
    k_name: str = "k_proj"
    v_name: str = "v_proj"
    o_name: str = "o_proj"


@register_mixer("attention")
class Attention(Mixer):
    graph_safe = True      # reads nothing from the host during a step
    takes_normed = True    # the input goes to a matrix product only
    adds_to_stream = True  # the output product can add into the residual stream

    def __init__(self, spec: AttentionSpec):
        if min(spec.width, spec.n_heads, spec.n_kv_heads, spec.head_dim) <= 0:
            raise ConfigError("attention sizes must be positive")
        if spec.n_heads % spec.n_kv_heads:
            raise ConfigError("num_attention_heads (%d) is not a multiple of num_key_value_heads (%d)"
                              % (spec.n_heads, spec.n_kv_heads))
        if spec.window < 0:
            raise ConfigError("attention window must not be negative")
        self.spec = spec
        self.q_dim = spec.n_heads * spec.head_dim
        self.kv_dim = spec.n_kv_heads * spec.head_dim
        self.scale = float(spec.scale) if spec.scale is not None else float(spec.head_dim) ** -0.5
        self.position = build_position(spec.position)
        if self.position.rot_dim > spec.head_dim:
            raise ConfigError("rotary dimension %d exceeds head_dim %d"
                              % (self.position.rot_dim, spec.head_dim))
        self.qkv = Linear(spec.width, self.q_dim + 2 * self.kv_dim)
        self.q_only = Linear(spec.width, self.q_dim)
        self.out = Linear(self.q_dim, spec.width)
        self.cos = self.sin = None
        self.bias = None
        self.adjacent = False

    def cache_need(self, page):
        s = self.spec
        return kv_need(s.n_kv_heads, s.head_dim, s.window, page)

    def weights(self):
        s = self.spec
        decl = {
            s.q_name + ".weight": WeightDecl((self.q_dim, s.width)),
            s.k_name + ".weight": WeightDecl((self.kv_dim, s.width)),
            s.v_name + ".weight": WeightDecl((self.kv_dim, s.width)),
            s.o_name + ".weight": WeightDecl((s.width, self.q_dim)),
        }
        if s.qkv_bias:
            decl[s.q_name + ".bias"] = WeightDecl((self.q_dim,), role="vector", init="normal")
            decl[s.k_name + ".bias"] = WeightDecl((self.kv_dim,), role="vector", init="normal")
            decl[s.v_name + ".bias"] = WeightDecl((self.kv_dim,), role="vector", init="normal")
        return decl

    def bind(self, tensors, ops, dtype):
        s = self.spec
        parts = [tensors[n + ".weight"] for n in (s.q_name, s.k_name, s.v_name)]
        if len({p.dtype for p in parts}) > 1:
            parts = [p.float() for p in parts]
        bias = None
        if s.qkv_bias:
            bias = torch.cat([tensors[n + ".bias"] for n in (s.q_name, s.k_name, s.v_name)]).contiguous()
        w = torch.cat(parts, dim=0)                      # q rows, then k, then v
        # A position encoding pairs dims (j, j + rot_dim/2) ("half", the default) or neighbours
        # (2j, 2j+1) ("interleaved").  Kernels that rotate inside the projection want the two dims
        # of a pair side by side: for "half" the output rows of q and k (and the bias) are
        # reordered once; scores do not change, since queries and keys are reordered alike.
        pairing = getattr(self.position, "pairing", "half")
        rotates = self.position.rot_dim > 0
        if pairing == "interleaved" and rotates:
            if not getattr(ops, "prefers_adjacent_pairs", False):
                raise ConfigError("these kernels rotate the halves of a head only (pairing 'interleaved')")
            self.adjacent = True
        else:
            self.adjacent = bool(getattr(ops, "prefers_adjacent_pairs", False)) and rotates
            if self.adjacent:
                order = self._pair_order(w.device)
                w = w[order]
                if bias is not None:
                    bias = bias[order].contiguous()
        self.qkv.bind(w, ops=ops)
        self.q_only.bind(self.qkv.weight[:self.q_dim], ops=ops, like=self.qkv.prepared)    # the same storage
        self.bias = bias                                 # added inside the rotation kernel
        self.out.bind(tensors[s.o_name + ".weight"], ops=ops)
        self.cos, self.sin = self.position.tables(w.device)

    def _pair_order(self, device):
        """Row order of the stacked projection with rotating pairs side by side: in every q and
        k head dims (j, j + rot_dim/2) move to (2j, 2j+1); other dims and v stay."""
        s, rot = self.spec, self.position.rot_dim
        head = torch.arange(s.head_dim)
        head[0:rot:2] = torch.arange(rot // 2)
        head[1:rot:2] = torch.arange(rot // 2) + rot // 2
        n_rot = s.n_heads + s.n_kv_heads
        qk = (torch.arange(n_rot)[:, None] * s.head_dim + head[None, :]).reshape(-1)
        v = torch.arange(n_rot * s.head_dim, (n_rot + s.n_kv_heads) * s.head_dim)
        return torch.cat([qk, v]).to(device)

    def forward(self, ctx: StepContext, x, entry, residual=None):
        s = self.spec
        kv = ctx.kv(entry.cache)
        proj = self.qkv if entry.writes else self.q_only
        if hasattr(ctx.ops, "qkv_rope"):
            qkv = ctx.ops.qkv_rope(x, proj.prepared, self.bias, s.n_heads, s.n_kv_heads, s.head_dim,
                                   self.cos, self.sin, self.position.rot_dim, ctx, kv, entry.writes,
                                   self.adjacent, ctx.dtype)
        else:
            qkv = proj(ctx, x)
            ctx.ops.rope_kv_write(qkv, self.bias, s.n_heads, s.n_kv_heads, s.head_dim, self.cos,
                                  self.sin, self.position.rot_dim, ctx, kv, entry.writes,
                                  **({"adjacent": True} if self.adjacent else {}))
        o = ctx.ops.attention(qkv, s.n_heads, s.n_kv_heads, s.head_dim, ctx, kv,
                              self.scale, s.window)
        return self.out(ctx, o, residual=residual)
