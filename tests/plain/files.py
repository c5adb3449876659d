"""Minimal reader for a model folder (config.json + model.safetensors) for the plain oracle.

The safetensors container: 8 bytes little-endian header length, a JSON header mapping each
tensor name to ``{"dtype", "shape", "data_offsets"}``, then the raw little-endian bytes.
"""
import json
import os
import struct

import numpy as np


def _bf16_to_f32(raw: np.ndarray) -> np.ndarray:
    # bfloat16 is the upper half of an IEEE float32.
    return (raw.astype(np.uint32) << 16).view(np.float32)


_DECODERS = {
    "F32": lambda b: np.frombuffer(b, dtype="<f4"),
    "F16": lambda b: np.frombuffer(b, dtype="<f2").astype(np.float32),
    "BF16": lambda b: _bf16_to_f32(np.frombuffer(b, dtype="<u2")),
    "F64": lambda b: np.frombuffer(b, dtype="<f8"),
    "I32": lambda b: np.frombuffer(b, dtype="<i4"),
    "I64": lambda b: np.frombuffer(b, dtype="<i8"),
}


def read_safetensors(path, dtype=np.float64):
    """Returns {name: ndarray}; floating tensors are widened to ``dtype`` (exactly)."""
    with open(path, "rb") as f:
        blob = f.read()
    (hlen,) = struct.unpack("<Q", blob[:8])
    header = json.loads(blob[8:8 + hlen].decode("utf-8"))
    base = 8 + hlen
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        lo, hi = meta["data_offsets"]
        arr = _DECODERS[meta["dtype"]](blob[base + lo:base + hi]).reshape(meta["shape"])
        if arr.dtype.kind == "f":
            arr = arr.astype(dtype)
        out[name] = arr
    return out


def read_model_dir(path, dtype=np.float64):
    with open(os.path.join(path, "config.json"), "r", encoding="utf-8") as f:
        config = json.load(f)
    weights = read_safetensors(os.path.join(path, "model.safetensors"), dtype=dtype)
    return config, weights
