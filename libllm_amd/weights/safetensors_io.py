"""Reading and writing the safetensors container.

Layout: 8 bytes little-endian header length N, N bytes of JSON mapping each tensor name to
``{"dtype", "shape", "data_offsets": [begin, end]}`` (offsets relative to the end of the header),
then the raw little-endian data.  Tensors are memory-mapped and handed out one at a time, so a
large file is never held in host memory whole.
"""
import json
import os
import struct
from typing import Dict, Optional

import numpy as np
import torch

from ..errors import WeightError

_DTYPES = {
    "F64": (torch.float64, 8), "F32": (torch.float32, 4), "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}
_MAX_HEADER = 100 * 1024 * 1024


class TensorEntry:
    __slots__ = ("name", "dtype", "shape", "begin", "end", "file")

    def __init__(self, name, dtype, shape, begin, end, file):
        self.name, self.dtype, self.shape = name, dtype, tuple(shape)
        self.begin, self.end, self.file = begin, end, file


class SafetensorsFile:
    """One file: validated header, tensors fetched by name."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        with open(path, "rb") as f:
            head = f.read(8)
            if len(head) < 8:
                raise WeightError("%s: too short to be a safetensors file" % path)
            (hlen,) = struct.unpack("<Q", head)
            if hlen > _MAX_HEADER or 8 + hlen > size:
                raise WeightError("%s: header length %d exceeds the file" % (path, hlen))
            raw = f.read(hlen)
        try:
            header = json.loads(raw.decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightError("%s: header is not valid JSON (%s)" % (path, e))
        if not isinstance(header, dict):
            raise WeightError("%s: header is not an object" % path)
        self.data_start = 8 + hlen
        self.metadata = header.pop("__metadata__", None)
        self.entries: Dict[str, TensorEntry] = {}
        for name, meta in header.items():
            try:
                dtype, shape = meta["dtype"], list(meta["shape"])
                begin, end = meta["data_offsets"]
            except (KeyError, TypeError, ValueError):
                raise WeightError("%s: malformed entry for tensor %r" % (path, name))
            if dtype not in _DTYPES:
                raise WeightError("%s: tensor %r has unsupported dtype %s" % (path, name, dtype))
            numel = 1
            for s in shape:
                if not isinstance(s, int) or s < 0:
                    raise WeightError("%s: tensor %r has an invalid shape %r" % (path, name, shape))
                numel *= s
            if begin < 0 or end < begin or self.data_start + end > size:
                raise WeightError("%s: tensor %r points outside the file (offsets %d..%d, data "
                                  "section of %d bytes)" % (path, name, begin, end, size - self.data_start))
            if end - begin != numel * _DTYPES[dtype][1]:
                raise WeightError("%s: tensor %r: %d bytes of data do not match shape %r of %s"
                                  % (path, name, end - begin, shape, dtype))
            self.entries[name] = TensorEntry(name, dtype, shape, begin, end, self)
        self._map = None

    def tensor(self, name: str) -> torch.Tensor:
        """CPU tensor viewing the mapped file (copy-on-write; do not keep it for long)."""
        e = self.entries[name]
        if self._map is None:
            self._map = np.memmap(self.path, dtype=np.uint8, mode="c")
        tdtype, isize = _DTYPES[e.dtype]
        if e.end == e.begin:
            return torch.empty(e.shape, dtype=tdtype)
        buf = self._map[self.data_start + e.begin:self.data_start + e.end]
        return torch.frombuffer(buf, dtype=tdtype).reshape(e.shape)

    def close(self):
        self._map = None


def open_model_files(model_dir: str) -> Dict[str, TensorEntry]:
    """All tensors of a model folder: ``model.safetensors``, or the shards that
    ``model.safetensors.index.json`` lists."""
    single = os.path.join(model_dir, "model.safetensors")
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.isfile(single):
        files = [single]
    elif os.path.isfile(index):
        try:
            with open(index, "r", encoding="utf-8") as f:
                weight_map = json.load(f)["weight_map"]
        except (json.JSONDecodeError, KeyError, TypeError) as e:
            raise WeightError("%s: not a valid shard index (%s)" % (index, e))
        files = sorted({os.path.join(model_dir, v) for v in weight_map.values()})
    else:
        raise WeightError("no model.safetensors (or model.safetensors.index.json) in %s" % model_dir)
    entries: Dict[str, TensorEntry] = {}
    for path in files:
        if not os.path.isfile(path):
            raise WeightError("shard %s is listed in the index but does not exist" % path)
        for name, e in SafetensorsFile(path).entries.items():
            if name in entries:
                raise WeightError("tensor %r appears in two files" % name)
            entries[name] = e
    return entries


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor],
                      metadata: Optional[Dict[str, str]] = None) -> None:
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise WeightError("cannot store tensor %r of dtype %s" % (name, t.dtype))
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * (-len(raw) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(raw)))
        f.write(raw)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    os.replace(tmp, path)
