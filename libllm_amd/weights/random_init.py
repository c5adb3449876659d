"""Random-weights mode: fills every tensor a model declares from a seed, and writes a model
folder (config.json, model.safetensors) that loads like any other.

Matrices are normal with the given standard deviation; norm scales are 1 (plus an optional
normal jitter, so that tests can tell a scale from no scale); each tensor has a generator of its
own, keyed by the seed and the tensor's name, so its values do not depend on the others.
"""
import json
import os
import zlib
from typing import Dict

import torch

from ..parts.base import WeightDecl
from .safetensors_io import write_safetensors


def _generator(seed: int, name: str, device) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed((int(seed) * 1000003 + zlib.crc32(name.encode("utf-8"))) % (2**63 - 1))
    return g


def random_tensors(expected: Dict[str, WeightDecl], seed: int, std: float = 0.02,
                   norm_std: float = 0.0, dtype: torch.dtype = torch.bfloat16,
                   device="cpu") -> Dict[str, torch.Tensor]:
    out = {}
    for name in sorted(expected):
        decl = expected[name]
        g = _generator(seed, name, device)
        shape = tuple(decl.shape)
        if decl.role == "table":
            t = torch.zeros(shape, dtype=torch.int32, device=device)
        elif decl.init == "ones":
            t = torch.ones(shape, dtype=torch.float32, device=device)
            if norm_std:
                t = t + norm_std * torch.randn(shape, generator=g, dtype=torch.float32, device=device)
        elif decl.init == "zeros":
            t = torch.zeros(shape, dtype=torch.float32, device=device)
        else:
            t = torch.empty(shape, dtype=torch.float32, device=device).normal_(0.0, std, generator=g)
        out[name] = t if decl.role == "table" else t.to(dtype)
    return out


def write_random_model(model_dir: str, config, seed: int, std: float = 0.02,
                       norm_std: float = 0.0, dtype: torch.dtype = torch.bfloat16) -> None:
    """``config`` is a typed configuration (for instance ``LlamaConfig``)."""
    from ..engine.model import declared_weights
    expected = declared_weights(config.to_spec())
    tensors = random_tensors(expected, seed, std=std, norm_std=norm_std, dtype=dtype)
    os.makedirs(model_dir, exist_ok=True)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config.to_dict(), f, indent=2)
    write_safetensors(os.path.join(model_dir, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": seed})
