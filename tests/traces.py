"""Traces for the replay tests: the same requests cut into steps in different ways, and the
bookkeeping that maps the logits a replay wrote back to (request, position)."""
import json
import os

import numpy as np


def whole(requests):
    """Each request alone, all its tokens in one step, logits at every position."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks,
                                                       "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def tail_one_by_one(requests, tail=32):
    """Each request alone: all but the last ``tail`` tokens in one step, then one token a step."""
    steps = []
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[:head],
                                                       "want": list(range(head))}], "end": []})
        for i in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}],
                          "end": [rid] if i == len(toks) - 1 else []})
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def batches(groups, decode=None):
    """groups: list of {id: tokens}.  Every group starts together: the first step brings each
    request's prompt (all but its last ``decode[id]`` tokens, default a third), later steps one
    token for every request that still has some; a request ends with its last token, so shorter
    ones leave the batch earlier.  The groups follow one another."""
    steps = []
    for group in groups:
        left = {}
        entries = []
        for rid, toks in group.items():
            d = (decode or {}).get(rid, len(toks) // 3)
            head = max(1, len(toks) - d)
            entries.append({"id": rid, "tokens": toks[:head], "want": list(range(head))})
            left[rid] = list(toks[head:])
        steps.append({"step": len(steps), "entries": entries,
                      "end": [r for r in group if not left[r]]})
        while any(left.values()):
            entries, ended = [], []
            for rid in group:
                if left[rid]:
                    entries.append({"id": rid, "tokens": [left[rid].pop(0)], "want": [0]})
                    if not left[rid]:
                        ended.append(rid)
            steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def lines(steps):
    return [json.dumps(s) for s in steps]


def max_tokens_needed(steps, page=64):
    """Largest number of tokens the live requests hold at any time, each rounded up to pages."""
    held, peak = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum((n + page - 1) // page * page for n in held.values()))
        for r in s["end"]:
            held.pop(r)
    return peak


def collect(steps, out_dir, vocab):
    """{request: {position: logits}} from the files a replay wrote."""
    got, pos0 = {}, {}
    for s in steps:
        n_want = sum(len(e["want"]) for e in s["entries"])
        path = os.path.join(out_dir, "%s.f32" % s["step"])
        if n_want == 0:
            assert not os.path.exists(path)
            data = None
        else:
            data = np.fromfile(path, dtype="<f4").reshape(n_want, vocab)
        row = 0
        for e in s["entries"]:
            base = pos0.get(e["id"], 0)
            for w in e["want"]:
                got.setdefault(e["id"], {})[base + w] = data[row]
                row += 1
            pos0[e["id"]] = base + len(e["tokens"])
        for r in s["end"]:
            pos0.pop(r)
    return got
