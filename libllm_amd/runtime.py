"""From a model folder to an engine: configuration, model as data, weights, cache, step function."""
from typing import Optional

import torch

from .config import config_from_dir
from .engine.model import DecoderModel
from .engine.step import Engine
from .errors import ConfigError
from .weights import load_tensors

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
                max_slots: Optional[int] = None, use_graphs: bool = True) -> Engine:
    """Reads config.json, chooses the architecture by its ``model_type``, loads the tensors by
    name and returns an engine whose cache holds ``max_tokens`` tokens."""
    config = config_from_dir(model_dir)
    tdtype = parse_dtype(dtype)
    spec = config.to_spec()
    model = DecoderModel(spec)
    ops = ops if ops is not None else default_ops()
    tensors = load_tensors(model_dir, model.declared(), spec.optional_tensors, tdtype, ops.device)
    model.bind(tensors, ops, tdtype)
    engine = Engine(model, ops, tdtype, max_tokens, max_slots=max_slots, use_graphs=use_graphs)
    engine.config = config
    return engine
