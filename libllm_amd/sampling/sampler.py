"""Choosing the next token from logits.

The reference's order (src/libllm/generator.cc:197-214, 47-113): logits * (1/temperature), softmax,
the top_k most probable tokens sorted from the largest, the shortest prefix of them whose
probabilities reach top_p, then one draw in proportion to the probabilities kept.  It has no
greedy class; top_k == 1 is arg-max (src/flint/cuda/test.cc:385-392).  Here temperature 0 and
top_k 1 are arg-max (lowest index wins a tie), top_k 0 means no limit (with top_p below 1 the
nucleus is then taken over the whole vocabulary), and the uniform number of a
draw comes from a counter hash of (seed, stream, counter): the same request draws the same tokens
whatever else is in its batch.
"""
from dataclasses import dataclass
from typing import List, Sequence

import torch

from ..errors import RequestError

TOP_K_MAX = 1024     # the sampling kernel sorts its candidates in shared memory


@dataclass
class SamplingParams:
    """Defaults are the reference API's (src/libllm/llm.cc:125-132)."""
    temperature: float = 1.0
    top_k: int = 50
    top_p: float = 0.8
    seed: int = 0

    def validate(self, vocab: int) -> "SamplingParams":
        if not self.temperature >= 0.0:
            raise RequestError("temperature must not be negative")
        if self.top_k < 0:
            raise RequestError("top_k must not be negative (0 means no limit)")
        if not 0.0 < self.top_p <= 1.0:
            raise RequestError("top_p must lie in (0, 1]")
        k = 0 if self.top_k >= vocab else self.top_k       # the reference aborts here; we clamp
        if self.greedy:
            return SamplingParams(self.temperature, k, self.top_p, self.seed)
        if k > TOP_K_MAX:
            raise RequestError("top_k above %d is not supported (0 means no limit)" % TOP_K_MAX)
        # k == 0 with top_p < 1: the nucleus over the whole vocabulary, however many tokens it takes
        return SamplingParams(self.temperature, k, self.top_p, self.seed)

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0 or self.top_k == 1


class PendingTokens:
    """Tokens the sampler wrote on the device, on their way to the host.  The copy is queued on
    the stream of the sampling itself, at once, so behind it and before whatever the caller queues
    next: the device goes on with that work while the host waits only for the copy.  (On a stream
    of its own the copy can end up behind the next step all the same, since streams share few
    hardware queues, each of which runs its commands in order; the host then sees every token a
    step late and the device idles while the host queues the step after.)  ``device`` is the
    int32 tensor; ``tokens()`` waits and returns the list."""

    def __init__(self, device: torch.Tensor):
        self.device = device
        self._host = torch.empty(device.shape, dtype=device.dtype, pin_memory=True)
        self._host.copy_(device, non_blocking=True)
        self._done = torch.cuda.Event()
        self._done.record()
        self._list = None

    def tokens(self) -> List[int]:
        if self._list is None:
            self._done.synchronize()
            self._list = [int(t) for t in self._host.tolist()]
        return self._list

    def rows(self, index: Sequence[int]) -> torch.Tensor:
        """The device tokens of the given rows, in that order."""
        if list(index) == list(range(self.device.shape[0])):
            return self.device
        idx = torch.tensor(list(index), dtype=torch.long).pin_memory().to(self.device.device, non_blocking=True)
        return self.device.index_select(0, idx)


class Sampler:
    def __init__(self, ops, vocab: int):
        self.ops = ops
        self.vocab = vocab

    @property
    def samples_ahead(self) -> bool:
        """True if ``sample_device`` can leave the tokens on a GPU."""
        return getattr(self.ops.device, "type", "cpu") == "cuda"

    def sample_device(self, logits: torch.Tensor, params: SamplingParams, streams: Sequence[int],
                      counters: Sequence[int]) -> PendingTokens:
        """As ``sample``, but returns at once: the tokens stay on the device, and their copy to
        the host is queued behind the sampling."""
        p = params.validate(self.vocab)
        if logits.shape[0] != len(streams) or len(streams) != len(counters):
            raise RequestError("one stream and one counter per row of logits are needed")
        if p.greedy:
            out = self.ops.argmax(logits)
        else:
            out = self.ops.sample(logits, p.temperature, p.top_k, p.top_p, p.seed,
                                  list(streams), list(counters))
        return PendingTokens(out)

    def sample(self, logits: torch.Tensor, params: SamplingParams, streams: Sequence[int],
               counters: Sequence[int]) -> List[int]:
        """logits float32 ``[rows, vocab]``; ``streams[i]`` identifies the request of row i and
        ``counters[i]`` how many tokens it has drawn before."""
        p = params.validate(self.vocab)
        if logits.shape[0] != len(streams) or len(streams) != len(counters):
            raise RequestError("one stream and one counter per row of logits are needed")
        if p.greedy:
            out = self.ops.argmax(logits)
        else:
            out = self.ops.sample(logits, p.temperature, p.top_k, p.top_p, p.seed,
                                  list(streams), list(counters))
        return [int(t) for t in out.tolist()]
