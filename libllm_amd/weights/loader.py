"""Fetching a model's tensors by name, with one error that says everything that is wrong.

The reference asks its tensor dictionary for each name with the expected shape and fails at the
first mismatch (src/libllm/var_builder.cc:113-125, src/flint/tensor.cc:228-272).  Here the model
first declares every tensor it needs; the file is compared with the declaration as a whole.

Storage on the device: with dtype bfloat16 every matrix becomes bfloat16, whatever float type the
file stores (the reference casts every float tensor to its device's float type,
src/libllm/var_builder.cc:113-125), so that every product runs on the matrix cores and a 32-bit
file costs no more memory than a 16-bit one; small per-channel vectors (norm scales, biases) are
held in float32, which is how a vector stored in 32-bit stays so; integer tables become int32.
With ``keep_float32`` a matrix stored in 32-bit or wider stays float32 in bfloat16 mode too, and
its products then run in true 32-bit.  With dtype float32 every floating tensor is widened to
32-bit and nothing is rounded on the way.
"""
import fnmatch
from typing import Dict, Iterable

import torch

from ..errors import WeightError
from ..parts.base import WeightDecl
from .safetensors_io import TensorEntry, open_model_files

_FLOAT = {"F64", "F32", "F16", "BF16"}
_INT = {"I64", "I32", "I16", "I8", "U8"}
_LIST_LIMIT = 24


def _listing(names):
    names = sorted(names)
    shown = ", ".join(names[:_LIST_LIMIT])
    if len(names) > _LIST_LIMIT:
        shown += ", ... and %d more" % (len(names) - _LIST_LIMIT)
    return shown


def check_tensors(entries: Dict[str, TensorEntry], expected: Dict[str, WeightDecl],
                  optional: Iterable[str] = ()) -> None:
    optional = tuple(optional)
    missing = [n for n in expected if n not in entries]
    unexpected = [n for n in entries if n not in expected
                  and not any(fnmatch.fnmatchcase(n, p) for p in optional)]
    shapes, dtypes = [], []
    for n, decl in expected.items():
        e = entries.get(n)
        if e is None:
            continue
        if tuple(e.shape) != tuple(decl.shape):
            shapes.append("%s: expected %s, found %s" % (n, tuple(decl.shape), tuple(e.shape)))
        ok = e.dtype in (_INT if decl.role == "table" else _FLOAT)
        if not ok:
            dtypes.append("%s: %s" % (n, e.dtype))
    if not (missing or unexpected or shapes or dtypes):
        return
    lines = ["the weight file does not match the model:"]
    if missing:
        lines.append("  missing tensors (%d): %s" % (len(missing), _listing(missing)))
    if unexpected:
        lines.append("  unexpected tensors (%d): %s" % (len(unexpected), _listing(unexpected)))
    if shapes:
        lines.append("  wrong shapes (%d): %s" % (len(shapes), "; ".join(sorted(shapes)[:_LIST_LIMIT])))
    if dtypes:
        lines.append("  wrong dtypes (%d): %s" % (len(dtypes), "; ".join(sorted(dtypes)[:_LIST_LIMIT])))
    err = WeightError("\n".join(lines))
    err.missing, err.unexpected = sorted(missing), sorted(unexpected)
    err.wrong_shapes, err.wrong_dtypes = sorted(shapes), sorted(dtypes)
    raise err


def device_dtype(decl: WeightDecl, stored: torch.dtype, model_dtype: torch.dtype,
                 keep_float32: bool = False) -> torch.dtype:
    if decl.role == "table":
        return torch.int32
    if decl.role == "vector" or model_dtype == torch.float32:
        return torch.float32
    if keep_float32 and stored in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


def place(t: torch.Tensor, decl: WeightDecl, model_dtype: torch.dtype, device,
          keep_float32: bool = False) -> torch.Tensor:
    target = device_dtype(decl, t.dtype, model_dtype, keep_float32)
    if decl.role == "table" and t.numel() and (int(t.max()) > 2**31 - 1 or int(t.min()) < -2**31):
        raise WeightError("an integer table holds values outside the int32 range")
    return t.to(device=device, dtype=target, copy=True).contiguous()


def load_tensors(model_dir: str, expected: Dict[str, WeightDecl], optional: Iterable[str],
                 model_dtype: torch.dtype, device, keep_float32: bool = False) -> Dict[str, torch.Tensor]:
    entries = open_model_files(model_dir)
    check_tensors(entries, expected, optional)
    out = {}
    for name, decl in expected.items():
        e = entries[name]
        out[name] = place(e.file.tensor(name), decl, model_dtype, device, keep_float32)
    for f in {e.file for e in entries.values()}:
        f.close()
    return out
