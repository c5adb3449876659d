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

_LOAD_KEYS = {"filename", "device", "dtype", "max_tokens", "max_batch", "random_weights", "seed"}
_GENERATE_KEYS = {"prompts", "max_new_tokens", "temperature", "top_k", "top_p", "seed", "stop_tokens"}
_STEP_KEYS = {"step", "entries", "end"}
_COMPLETE_KEYS = {"messages", "token_ids", "temperature", "top_k", "top_p", "max_new_tokens", "seed", "stop_ids"}


def parse(text: str) -> str:
    """Checks that ``text`` is JSON and returns it in canonical form."""
    return json.dumps(json.loads(text))


def load(kwargs_json: str):
    """``filename``: the model folder or its config.json; ``device``: cpu, cuda or auto
    (src/libllm/llm.cc:154-168, 206-236).  Ours: ``dtype``, ``max_tokens``, ``max_batch``, and
    ``random_weights`` with ``seed`` (only config.json is then read)."""
    from .api import Model, parse_device
    kw = json.loads(kwargs_json)
    if not isinstance(kw, dict):
        raise ConfigError("kwargs must be a JSON object")
    for key in kw:
        if key not in _LOAD_KEYS:
            raise ConfigError("unexpected key in kwargs: %s" % key)
    if "filename" not in kw:
        raise ConfigError("key \"filename\" is required")
    return Model(kw["filename"], parse_device(str(kw.get("device", "auto"))), dtype=kw.get("dtype", "bfloat16"),
                 max_tokens=int(kw.get("max_tokens", 8192)), max_batch=int(kw.get("max_batch", 64)),
                 random_weights=bool(kw.get("random_weights", False)), seed=int(kw.get("seed", 0)))


def info(model) -> str:
    """``{"name": ...}`` as the reference gives (src/libllm/llm.cc:238-250), and the sizes."""
    spec = model.engine.model.spec
    return json.dumps({"name": model.name, "vocab_size": spec.vocab, "max_position": spec.max_position,
                       "stop_tokens": list(spec.stop_tokens)})


def complete(model, kwargs_json: str) -> Iterator:
    """Starts a completion.  ``messages`` is a list of ``{"role", "content"}`` as in the reference
    (src/libllm/llm.cc:98-123), put into the architecture's chat format where the tokenizer beside
    the model knows its control tokens (``Model.build_prompt``).  Ours: ``token_ids`` in place of ``messages``,
    ``max_new_tokens``, ``seed``, ``stop_ids`` (beside the model's own).  Defaults: temperature 1.0, top_k 50, top_p 0.8
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
        prompt = model.build_prompt(kw["messages"])
        kw["stop_ids"] = list(kw.get("stop_ids") or []) + model.chat_stop_ids()
    completion = model.complete(prompt, top_k=int(kw.get("top_k", 50)), top_p=float(kw.get("top_p", 0.8)),
                                temperature=float(kw.get("temperature", 1.0)),
                                max_new_tokens=int(kw.get("max_new_tokens", 256)), seed=int(kw.get("seed", 0)),
                                stop_ids=kw.get("stop_ids"))
    return iter(completion)


def next_chunk(chunks: Iterator) -> Optional[str]:
    """The next chunk as ``{"text": ..., "token_id": ...}``, or None at the end."""
    for chunk in chunks:
        return json.dumps({"text": chunk.text, "token_id": chunk.token_id})
    return None


def generate(model, kwargs_json: str) -> str:
    """Batches of prompts of token ids, as ``Model.generate``: ``{"prompts": [[...], ...]}`` with
    ``max_new_tokens``, ``temperature``, ``top_k``, ``top_p``, ``seed``, ``stop_tokens``; returns
    ``{"tokens": [[...], ...]}``.  No counterpart in the reference's C API."""
    kw = json.loads(kwargs_json)
    if not isinstance(kw, dict) or "prompts" not in kw:
        raise RequestError("key \"prompts\" is required")
    for key in kw:
        if key not in _GENERATE_KEYS:
            raise RequestError("unexpected key in kwargs: %s" % key)
    prompts = [[int(t) for t in p] for p in kw["prompts"]]
    out = model.generate(prompts, max_new_tokens=int(kw.get("max_new_tokens", 256)),
                         temperature=float(kw.get("temperature", 1.0)), top_k=int(kw.get("top_k", 50)),
                         top_p=float(kw.get("top_p", 0.8)), seed=int(kw.get("seed", 0)),
                         stop_tokens=kw.get("stop_tokens"))
    return json.dumps({"tokens": out})


def step(model, kwargs_json: str, address: int, capacity: int) -> int:
    """One call of the step function, in the words of a trace line: ``{"entries": [{"id", "tokens",
    "want"}], "end": [...]}``.  The float32 logits at the wanted places, [wanted, vocab], are
    written to ``capacity`` floats at ``address``; returns the number of wanted rows, or minus
    the number of floats needed if they do not fit (nothing has run then).  No counterpart in the
    reference's C API."""
    import ctypes
    from .engine import StepEntry
    kw = json.loads(kwargs_json)
    if not isinstance(kw, dict) or "entries" not in kw:
        raise RequestError("key \"entries\" is required")
    for key in kw:
        if key not in _STEP_KEYS:
            raise RequestError("unexpected key in kwargs: %s" % key)
    entries = [StepEntry(e["id"], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])])
               for e in kw["entries"]]
    wanted = sum(len(e.want) for e in entries)
    vocab = model.engine.vocab
    if wanted * vocab > capacity:
        return -(wanted * vocab)
    logits = model.step(entries) if entries else None     # a line may only end requests
    if wanted:
        host = logits.float().cpu().contiguous().numpy()
        ctypes.memmove(address, host.ctypes.data, host.nbytes)
    if kw.get("end"):
        model.end(list(kw["end"]))
    return wanted
