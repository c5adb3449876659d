"""Rotary position encoding: the frequency table and its scaling rules.

The reference stores a cos/sin table that its exporter obtains from an external rotary module
and rounds to half precision (tools/llama_exporter.py:54-62, tools/model_exporter.py:168-171);
here the table is computed from the configuration's constants in float64 and held in float32.
Row p of the table holds cos/sin of ``p * inv_freq[j]`` for j < rot_dim/2; the rotate-half
application (src/libllm/llama.cc:151-176) pairs dimension j with j + rot_dim/2.
"""
import math
from dataclasses import dataclass
from typing import Dict, Optional

import torch

from ..errors import ConfigError
from .base import PartSpec
from .registry import register_position


@dataclass
class RotarySpec(PartSpec):
    rot_dim: int = 0                   # leading head dimensions that rotate (even)
    theta: float = 10000.0
    max_position: int = 0
    scaling: Optional[Dict] = None     # {"rope_type": "llama3", "factor": ..., ...} or None
    pairing: str = "half"              # "half": dims (j, j + rot_dim/2) rotate together; "interleaved": (2j, 2j + 1)


@dataclass
class NoPositionSpec(PartSpec):
    pass


def scaled_inv_freq(rot_dim: int, theta: float, scaling: Optional[Dict]) -> torch.Tensor:
    """float64 inverse frequencies, one per rotating pair."""
    j = torch.arange(0, rot_dim, 2, dtype=torch.float64)
    inv = 1.0 / (torch.tensor(theta, dtype=torch.float64) ** (j / rot_dim))
    if not scaling:
        return inv
    kind = scaling.get("rope_type", scaling.get("type"))
    if kind in (None, "default"):
        return inv
    if kind == "linear":
        return inv / float(_need(scaling, "factor"))
    if kind == "llama3":
        factor = float(_need(scaling, "factor"))
        low = float(_need(scaling, "low_freq_factor"))
        high = float(_need(scaling, "high_freq_factor"))
        orig = float(_need(scaling, "original_max_position_embeddings"))
        if not high > low:
            raise ConfigError("rope_scaling: high_freq_factor must exceed low_freq_factor")
        wavelen = 2.0 * math.pi / inv
        smooth = (orig / wavelen - low) / (high - low)
        blended = (1.0 - smooth) * inv / factor + smooth * inv
        out = torch.where(wavelen > orig / low, inv / factor, blended)
        out = torch.where(wavelen < orig / high, inv, out)
        return out
    raise ConfigError("unsupported rope_scaling type %r (supported: default, linear, llama3)" % (kind,))


def _need(d, key):
    if key not in d:
        raise ConfigError("rope_scaling: key %r is missing" % key)
    return d[key]


@register_position("rotary")
class RotaryPosition:
    def __init__(self, spec: RotarySpec):
        if spec.rot_dim <= 0 or spec.rot_dim % 2:
            raise ConfigError("rotary dimension must be positive and even, got %d" % spec.rot_dim)
        if spec.pairing not in ("half", "interleaved"):
            raise ConfigError("unsupported rotary pairing %r (half or interleaved)" % (spec.pairing,))
        if spec.max_position <= 0:
            raise ConfigError("rotary position encoding needs max_position > 0")
        self.spec = spec
        self.rot_dim = spec.rot_dim
        self.pairing = spec.pairing
        self._tables = {}

    def inv_freq(self) -> torch.Tensor:
        return scaled_inv_freq(self.spec.rot_dim, self.spec.theta, self.spec.scaling)

    def tables(self, device):
        """(cos, sin), each float32 ``[max_position, rot_dim/2]`` on ``device``."""
        key = str(device)
        if key not in self._tables:
            pos = torch.arange(self.spec.max_position, dtype=torch.float64)
            ang = pos[:, None] * self.inv_freq()[None, :]
            self._tables[key] = (torch.cos(ang).float().contiguous().to(device),
                                 torch.sin(ang).float().contiguous().to(device))
        return self._tables[key]


@register_position("none")
class NoPosition:
    """No rotation: keys and queries go to the cache and the scores unchanged."""
    rot_dim = 0

    def __init__(self, spec=None):
        self.spec = spec

    def tables(self, device):
        return None, None
