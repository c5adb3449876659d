"""Plain sampling and generation: the order of src/libllm/generator.cc, in float64.

logits * (1/temperature) -> softmax -> top-k (sorted, largest first) -> nucleus (shortest prefix
whose probabilities sum to top_p or more) -> draw r = u * sum(selected), first index whose
running sum exceeds r (generator.cc:47-113, 197-214).  Ties in the sort go to the lower index.
The uniform number comes from a counter hash keyed by (seed, stream, counter), restated here.
"""
import numpy as np

from . import llama

_M64 = (1 << 64) - 1


def uniform(seed, stream, counter):
    """splitmix64 finaliser over a linear mix of the three keys; 24 random bits in [0, 1)."""
    x = (seed * 0x9E3779B97F4A7C15 + stream * 0xBF58476D1CE4E5B9
         + counter * 0x94D049BB133111EB + 0x2545F4914F6CDD1D) & _M64
    x ^= x >> 30
    x = (x * 0xBF58476D1CE4E5B9) & _M64
    x ^= x >> 27
    x = (x * 0x94D049BB133111EB) & _M64
    x ^= x >> 31
    return (x >> 40) / float(1 << 24)


def candidates(logits, temperature, top_k, top_p):
    """Returns (labels, cumulative sums) of the nucleus, in drawing order."""
    x = np.asarray(logits, dtype=np.float64)
    if temperature != 1.0:
        x = x * (1.0 / temperature)
    p = llama.softmax(x)
    v = p.shape[0]
    if top_k <= 0 or top_k >= v:
        if top_p < 1.0:
            order = np.argsort(-p, kind="stable")
        else:
            order = np.arange(v)                      # nothing cut: plain index order
    else:
        order = np.argsort(-p, kind="stable")[:top_k]   # generator.cc:66-90
    acc, labels, run = [], [], 0.0
    for lab in order:                                   # generator.cc:47-64
        run += p[lab]
        labels.append(int(lab))
        acc.append(run)
        if top_p < 1.0 and run >= top_p:
            break
    return labels, acc


def sample(logits, temperature, top_k, top_p, u):
    """One draw (generator.cc:92-113).  temperature 0 is arg-max (lowest index wins)."""
    if temperature == 0.0 or top_k == 1:
        return int(np.argmax(logits))
    labels, acc = candidates(logits, temperature, top_k, top_p)
    r = u * acc[-1]
    for lab, a in zip(labels, acc):
        if r < a:
            return lab
    return labels[-1]


def margin(logits, temperature, top_k, top_p, u):
    """Distance of the draw from the nearest boundary of the running sum, relative to its
    total: a draw closer than rounding error may legitimately fall either way."""
    if temperature == 0.0 or top_k == 1:
        s = np.sort(np.asarray(logits, dtype=np.float64))
        return float(s[-1] - s[-2])
    _, acc = candidates(logits, temperature, top_k, top_p)
    r = u * acc[-1]
    return float(np.min(np.abs(np.asarray(acc) - r)) / acc[-1])


def generate(cfg, weights, prompt, max_new_tokens, temperature=0.0, top_k=0, top_p=1.0,
             seed=0, stream=0, stop=None):
    """Greedy / sampled generation by re-running the whole sequence for each new token
    (src/libllm/generator.cc:140-156: the stop token ends the sequence and is not emitted)."""
    stop = cfg.stop if stop is None else set(stop)
    ids = list(prompt)
    out = []
    for step in range(max_new_tokens):
        logits = llama.logits_all(cfg, weights, ids)[-1]
        u = uniform(seed, stream, step)
        tok = sample(logits, temperature, top_k, top_p, u)
        if tok in stop:
            break
        out.append(tok)
        ids.append(tok)
    return out
