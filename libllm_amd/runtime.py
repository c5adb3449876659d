"""From a model folder to an engine: configuration, model as data, weights, cache, step function."""
from typing import Optional

import torch

from .config import config_from_dir
from .engine.model import DecoderModel
from .engine.step import Engine
from .errors import ConfigError
from .weights import load_tensors, random_tensors
from .weights.loader import place

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
           "float32": torch.float32, "fp32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ConfigError("dtype must be bfloat16 or float32")
        return name
    if name not in _DTYPES:
        raise ConfigError("dtype must be bfloat16 or float32, got %r" % (name,))
    return _DTYPES[name]


def default_ops():
    """The kernels of the product path.  Raises KernelError without a GPU or the built library."""
    from .hip import HipOps
    return HipOps()


def load_engine(model_dir: str, dtype="bfloat16", max_tokens: int = 8192, ops=None,
                max_slots: Optional[int] = None, use_graphs: bool = True,
                keep_float32: bool = False, tiled_weights: bool = True) -> Engine:
    """Reads config.json, chooses the architecture by its ``model_type``, loads the tensors by
    name and returns an engine whose cache holds ``max_tokens`` tokens.  ``keep_float32``: in
    bfloat16 mode a matrix that the file stores in 32-bit stays float32 (true 32-bit products
    for it) instead of becoming bfloat16.  ``tiled_weights=False``: no second, tiled copy of the
    bfloat16 matrices (half the weight memory; decoding is 5 to 11 % slower)."""
    config = config_from_dir(model_dir)
    tdtype = parse_dtype(dtype)
    spec = config.to_spec()
    model = DecoderModel(spec)
    ops = ops if ops is not None else default_ops()
    if not tiled_weights:
        ops.pack_weights = False
    tensors = load_tensors(model_dir, model.declared(), spec.optional_tensors, tdtype, ops.device,
                           keep_float32)
    model.bind(tensors, ops, tdtype)
    engine = Engine(model, ops, tdtype, max_tokens, max_slots=max_slots, use_graphs=use_graphs)
    engine.config = config
    return engine


def random_engine(config, seed: int = 0, dtype="bfloat16", max_tokens: int = 8192, ops=None,
                  max_slots: Optional[int] = None, use_graphs: bool = True, std: float = 0.02,
                  stored: torch.dtype = torch.bfloat16, tiled_weights: bool = True) -> Engine:
    """The random-weights mode without a file: every tensor the model declares is drawn on the
    device from ``seed`` (matrices normal with ``std``, norm scales 1) and bound as a loaded file
    would be that stores ``stored`` (float32: full significands for the 32-bit path).  ``config``
    is a typed configuration."""
    tdtype = parse_dtype(dtype)
    spec = config.to_spec()
    model = DecoderModel(spec)
    ops = ops if ops is not None else default_ops()
    if not tiled_weights:
        ops.pack_weights = False
    declared = model.declared()
    tensors = {}
    for name in sorted(declared):
        t = random_tensors({name: declared[name]}, seed, std=std, dtype=stored,
                           device=ops.device)[name]
        tensors[name] = place(t, declared[name], tdtype, ops.device)
    model.bind(tensors, ops, tdtype)
    engine = Engine(model, ops, tdtype, max_tokens, max_slots=max_slots, use_graphs=use_graphs)
    engine.config = config
    return engine
