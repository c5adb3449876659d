"""Trace replay: feeds given token ids through the engine step by step and writes logits.

It samples nothing and has no model code of its own: each input line becomes one call of the
engine's step function.  Input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["a"]}

For a step that wants logits, ``<out>/<step>.f32`` receives them as little-endian float32
``[wanted, vocab]`` in the order of the entries and of their ``want`` lists; after every step a
line ``done <step>`` is printed and flushed.
"""
import json
import os
import sys

from ..errors import RequestError
from .step import StepEntry


def replay(engine, lines, out_dir: str, log=sys.stdout) -> int:
    os.makedirs(out_dir, exist_ok=True)
    n = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        try:
            obj = json.loads(line)
            step = obj["step"]
            entries = [StepEntry(e["id"], [int(t) for t in e["tokens"]],
                                 [int(w) for w in e.get("want", [])]) for e in obj["entries"]]
            ended = list(obj.get("end", []))
        except (ValueError, KeyError, TypeError) as e:
            raise RequestError("bad trace line %r: %s" % (line[:200], e))
        logits = engine.step(entries) if entries else None
        if logits is not None and logits.shape[0] > 0:
            arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            tmp = os.path.join(out_dir, "%s.f32.tmp" % step)
            arr.tofile(tmp)
            os.replace(tmp, os.path.join(out_dir, "%s.f32" % step))
        if ended:
            engine.end(ended)
        print("done %s" % step, file=log, flush=True)
        n += 1
    return n
