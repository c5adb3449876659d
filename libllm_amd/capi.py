"""The Python side of the C API (csrc/capi/llm.h): JSON text in, JSON text out.

The C functions keep handles to the objects made here and pass every argument as JSON text, in
the manner of the reference's C API (src/libllm/llm.h:52-72, src/libllm/llm.cc:178-349): a model is
loaded from ``{"filename": ..., "device": ...}``, a completion is started from ``{"messages": [...],
"temperature": ..., "top_k": ..., "top_p": ...}`` with the reference's defaults and its strict check
of keys, and chunks come back as ``{"text": ...}``.  Beside the reference's keys a few of this
library's own are taken (they are listed where they are read).
"""
import json
from typing import Iterator, Optional

from .errors import ConfigError, RequestError

_LOAD_KEYS = {"filename", "device", "dtype", "max_tokens", "max_batch"}
_COMPLETE_KEYS = {"messages", "token_ids", "temperature", "top_k", "top_p", "max_new_tokens", "seed"}


def parse(text: str) -> str:
    """Checks that ``text`` is JSON and returns it in canonical form."""
    return json.dumps(json.loads(text))


def load(kwargs_json: str):
    """``filename``: the model folder or its config.json; ``device``: cpu, cuda or auto
    (src/libllm/llm.cc:154-168, 206-236).  Ours: ``dtype``, ``max_tokens``, ``max_batch``."""
    from .api import Device, Model
    kw = json.loads(kwargs_json)
    if not isinstance(kw, dict):
        raise ConfigError("kwargs must be a JSON object")
    for key in kw:
        if key not in _LOAD_KEYS:
            raise ConfigError("unexpected key in kwargs: %s" % key)
    if "filename" not in kw:
        raise ConfigError("key \"filename\" is required")
    device = str(kw.get("device", "auto")).lower()
    if device not in ("cpu", "cuda", "auto"):
        raise ConfigError("invalid device: %s" % device)
    dev = {"cpu": Device.CPU, "cuda": Device.CUDA, "auto": Device.AUTO}[device]
    return Model(kw["filename"], dev, dtype=kw.get("dtype", "bfloat16"),
                 max_tokens=int(kw.get("max_tokens", 8192)), max_batch=int(kw.get("max_batch", 64)))


def info(model) -> str:
    """``{"name": ...}`` as the reference gives (src/libllm/llm.cc:238-250), and the sizes."""
    spec = model.engine.model.spec
    return json.dumps({"name": model.name, "vocab_size": spec.vocab, "max_position": spec.max_position,
                       "stop_tokens": list(spec.stop_tokens)})


def complete(model, kwargs_json: str) -> Iterator:
    """Starts a completion.  ``messages`` is a list of ``{"role", "content"}`` as in the reference
    (src/libllm/llm.cc:98-123); since tokenisation lies outside this library the contents are
    joined as the command line joins them.  Ours: ``token_ids`` in place of ``messages``,
    ``max_new_tokens``, ``seed``.  Defaults: temperature 1.0, top_k 50, top_p 0.8
    (src/libllm/llm.cc:125-132)."""
    kw = json.loads(kwargs_json)
    if not isinstance(kw, dict):
        raise RequestError("kwargs must be a JSON object")
    for key in kw:
        if key not in _COMPLETE_KEYS:
            raise RequestError("unexpected key in kwargs: %s" % key)
    if ("messages" in kw) == ("token_ids" in kw):
        raise RequestError("exactly one of \"messages\" and \"token_ids\" is required")
    if "token_ids" in kw:
        prompt = [int(t) for t in kw["token_ids"]]
    else:
        parts = []
        for m in kw["messages"]:
            if not isinstance(m, dict) or "role" not in m or "content" not in m:
                raise RequestError("a message needs \"role\" and \"content\"")
            parts.append("%s: %s\n" % (m["role"], m["content"]))
        prompt = "".join(parts) + "assistant: "
    completion = model.complete(prompt, top_k=int(kw.get("top_k", 50)), top_p=float(kw.get("top_p", 0.8)),
                                temperature=float(kw.get("temperature", 1.0)),
                                max_new_tokens=int(kw.get("max_new_tokens", 256)), seed=int(kw.get("seed", 0)))
    return iter(completion)


def next_chunk(chunks: Iterator) -> Optional[str]:
    """The next chunk as ``{"text": ..., "token_id": ...}``, or None at the end."""
    for chunk in chunks:
        return json.dumps({"text": chunk.text, "token_id": chunk.token_id})
    return None
