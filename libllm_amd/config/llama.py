"""Typed configuration of the Llama decoder, read from the architecture's own config.json keys.

The reference reads the same values from an ini section that its exporter fills from the
config.json (src/libllm/llama.cc:53-75, tools/llama_exporter.py:90-100): hidden_size,
num_attention_heads, num_key_value_heads (default: the number of heads), intermediate_size,
rms_norm_eps, num_hidden_layers, vocab_size, max_position_embeddings; the exporter asserts
hidden_act == "silu" (tools/llama_exporter.py:87-88).  Keys the reference bakes into its
exported rotary table are read here directly: rope_theta, rope_scaling, head_dim,
tie_word_embeddings.
"""
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..errors import ConfigError
from ..parts.attention import AttentionSpec
from ..parts.mlp_swiglu import SwiGLUSpec
from ..parts.norm_rms import RMSNormSpec
from ..parts.rope import RotarySpec
from .spec import (EmbeddingSpec, HeadSpec, LayerSpec, ModelSpec, default_schedule,
                   validate_schedule)


def _get(d, key, typ, default=None, required=False):
    if key not in d or d[key] is None:
        if required:
            raise ConfigError("config.json: required key %r is missing" % key)
        return default
    v = d[key]
    if typ is float and isinstance(v, int) and not isinstance(v, bool):
        v = float(v)
    if typ is int and isinstance(v, bool) or not isinstance(v, typ):
        raise ConfigError("config.json: key %r must be %s, got %r" % (key, typ.__name__, v))
    return v


@dataclass
class LlamaConfig:
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    num_hidden_layers: int
    vocab_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: Optional[Dict[str, Any]]
    tie_word_embeddings: bool
    attention_bias: bool
    hidden_act: str
    bos_token_id: Optional[int]
    eos_token_ids: Tuple[int, ...]
    model_type: str = "llama"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LlamaConfig":
        hidden = _get(d, "hidden_size", int, required=True)
        heads = _get(d, "num_attention_heads", int, required=True)
        if hidden <= 0 or heads <= 0:
            raise ConfigError("config.json: hidden_size and num_attention_heads must be positive")
        kv_heads = _get(d, "num_key_value_heads", int, default=heads)
        head_dim = _get(d, "head_dim", int)
        if head_dim is None:
            if hidden % heads:
                raise ConfigError("config.json: hidden_size %d is not a multiple of "
                                  "num_attention_heads %d and head_dim is not given" % (hidden, heads))
            head_dim = hidden // heads
        if kv_heads <= 0 or heads % kv_heads:
            raise ConfigError("config.json: num_attention_heads %d is not a multiple of "
                              "num_key_value_heads %d" % (heads, kv_heads))
        if head_dim <= 0 or head_dim % 2:
            raise ConfigError("config.json: head_dim %d must be positive and even" % head_dim)
        act = _get(d, "hidden_act", str, default="silu")
        if act != "silu":
            raise ConfigError("config.json: hidden_act %r is not supported (silu only)" % act)
        if _get(d, "mlp_bias", bool, default=False):
            raise ConfigError("config.json: mlp_bias true is not supported")
        if _get(d, "pretraining_tp", int, default=1) != 1:
            raise ConfigError("config.json: pretraining_tp must be 1")
        scaling = d.get("rope_scaling")
        if scaling is not None and not isinstance(scaling, dict):
            raise ConfigError("config.json: rope_scaling must be an object or null")
        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids = ()
        elif isinstance(eos, int) and not isinstance(eos, bool):
            eos_ids = (eos,)
        elif isinstance(eos, list) and all(isinstance(e, int) for e in eos):
            eos_ids = tuple(eos)
        else:
            raise ConfigError("config.json: eos_token_id must be an integer or a list of integers")
        cfg = cls(
            hidden_size=hidden,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=_get(d, "intermediate_size", int, required=True),
            num_hidden_layers=_get(d, "num_hidden_layers", int, required=True),
            vocab_size=_get(d, "vocab_size", int, required=True),
            max_position_embeddings=_get(d, "max_position_embeddings", int, required=True),
            rms_norm_eps=_get(d, "rms_norm_eps", float, required=True),
            rope_theta=_get(d, "rope_theta", float, default=10000.0),
            rope_scaling=dict(scaling) if scaling else None,
            tie_word_embeddings=_get(d, "tie_word_embeddings", bool, default=False),
            attention_bias=_get(d, "attention_bias", bool, default=False),
            hidden_act=act,
            bos_token_id=_get(d, "bos_token_id", int),
            eos_token_ids=eos_ids,
            model_type=_get(d, "model_type", str, default="llama"),
        )
        for key in ("intermediate_size", "num_hidden_layers", "vocab_size", "max_position_embeddings"):
            if getattr(cfg, key) <= 0:
                raise ConfigError("config.json: %s must be positive" % key)
        if not cfg.rms_norm_eps > 0:
            raise ConfigError("config.json: rms_norm_eps must be positive")
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        d = {
            "model_type": self.model_type,
            "architectures": ["LlamaForCausalLM"],
            "hidden_size": self.hidden_size,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": self.rope_scaling,
            "tie_word_embeddings": self.tie_word_embeddings,
            "attention_bias": self.attention_bias,
            "hidden_act": self.hidden_act,
            "bos_token_id": self.bos_token_id,
            "eos_token_id": (None if not self.eos_token_ids else
                             self.eos_token_ids[0] if len(self.eos_token_ids) == 1
                             else list(self.eos_token_ids)),
        }
        return d

    def build_prompt(self, messages):
        """The messages of a chat in this architecture's format, as blocks of text and control
        tokens (src/libllm/llama.cc:406-442)."""
        from ..prompt import llama3_prompt
        return llama3_prompt(messages)

    # the control token that ends a turn in that format: a reply stops there, beside the stop
    # tokens that config.json names (the reference reads its id from the exported model,
    # src/libllm/llama.cc:342,390-392)
    chat_stop_tokens = ("<|eot_id|>",)

    def to_spec(self) -> ModelSpec:
        """The decoder as data: every layer a prenorm block of grouped-query attention with
        rotary positions and a SwiGLU feed-forward (src/libllm/llama.cc:231-312); tensor names
        are the ones the exporter reads (tools/llama_exporter.py:35-78)."""
        h = self.hidden_size
        rotary = RotarySpec(kind="rotary", rot_dim=self.head_dim, theta=self.rope_theta,
                            max_position=self.max_position_embeddings, scaling=self.rope_scaling)
        layers = []
        for i in range(self.num_hidden_layers):
            p = "model.layers.%d." % i
            layers.append(LayerSpec(
                block="prenorm",
                mixer=AttentionSpec(kind="attention", width=h, n_heads=self.num_attention_heads,
                                    n_kv_heads=self.num_key_value_heads, head_dim=self.head_dim,
                                    position=rotary, qkv_bias=self.attention_bias),
                feed_forward=SwiGLUSpec(kind="swiglu", width=h, intermediate=self.intermediate_size,
                                        activation=self.hidden_act),
                norms=[RMSNormSpec(kind="rms", width=h, eps=self.rms_norm_eps),
                       RMSNormSpec(kind="rms", width=h, eps=self.rms_norm_eps)],
                prefixes={"mixer": p + "self_attn.", "feed_forward": p + "mlp.",
                          "norm0": p + "input_layernorm.", "norm1": p + "post_attention_layernorm."},
            ))
        embed_name = "model.embed_tokens.weight"
        spec = ModelSpec(
            name=self.model_type,
            width=h,
            vocab=self.vocab_size,
            max_position=self.max_position_embeddings,
            embedding=EmbeddingSpec(self.vocab_size, h, embed_name),
            layers=layers,
            schedule=default_schedule(self.num_hidden_layers),
            final_norm=RMSNormSpec(kind="rms", width=h, eps=self.rms_norm_eps),
            final_norm_prefix="model.norm.",
            head=HeadSpec(self.vocab_size, h,
                          embed_name if self.tie_word_embeddings else "lm_head.weight",
                          tied=self.tie_word_embeddings),
            stop_tokens=self.eos_token_ids,
            bos_token=self.bos_token_id,
            # rotary buffers some files carry, and the duplicate head of a tied model
            optional_tensors=("*.rotary_emb.inv_freq",) + (("lm_head.weight",) if self.tie_word_embeddings else ()),
        )
        validate_schedule(spec)
        return spec
