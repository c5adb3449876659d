"""The generation loop above the step function.

The reference generates for one sequence: prefill, then decode token by token, ending when the
sampled token is a stop token, which is not emitted (src/libllm/generator.cc:140-156).  Here many
requests are served: they are cut into batches that fit the cache, each batch starts together with
prompts of unequal lengths in one step, goes on one token per live sequence, sequences that end
leave the batch and give their slot back, and batches follow one another until all are served.
"""
from dataclasses import dataclass, field
from typing import Callable, Iterable, List, Optional, Sequence

import torch

from ..errors import CacheError, RequestError
from ..sampling import SamplingParams
from .step import StepEntry


def plan_batches(prompt_lens: Sequence[int], max_new_tokens: int, max_batch: int,
                 page_budget: int, page: int, max_position: int) -> List[List[int]]:
    """Cuts request indices into consecutive batches: at most ``max_batch`` requests each, and
    the pages every request may grow to (prompt plus ``max_new_tokens``, capped by
    ``max_position``) fit ``page_budget`` together."""
    if max_batch <= 0:
        raise RequestError("max_batch must be positive")
    batches, cur, used = [], [], 0
    for i, n in enumerate(prompt_lens):
        if n <= 0:
            raise RequestError("request %d has an empty prompt" % i)
        if n > max_position:
            raise RequestError("request %d: a prompt of %d tokens exceeds max_position_embeddings %d"
                               % (i, n, max_position))
        need = (min(n + max_new_tokens, max_position) + page - 1) // page
        if need > page_budget:
            raise RequestError("request %d needs %d cache pages but the cache has %d"
                               % (i, need, page_budget))
        if cur and (len(cur) >= max_batch or used + need > page_budget):
            batches.append(cur)
            cur, used = [], 0
        cur.append(i)
        used += need
    if cur:
        batches.append(cur)
    return batches


def plan_prompt_steps(prompt_lens: Sequence[int], max_rows: int) -> List[List[tuple]]:
    """Cuts the prompts of a batch into steps of at most ``max_rows`` rows, which bounds the
    activations a step needs: a list of steps, each a list of (sequence, first token, end).  The
    sequences come in their order; a prompt that does not fit what is left of a step goes on in
    the next one (a step's entries then hold parts of different prompts, which the step function
    takes as they are).  Prompts that fit together make one step."""
    if max_rows <= 0:
        raise RequestError("the rows of a prompt step must be positive")
    steps, cur, room = [], [], max_rows
    for i, n in enumerate(prompt_lens):
        start = 0
        while start < n:
            take = min(n - start, room)
            cur.append((i, start, start + take))
            start += take
            room -= take
            if room == 0:
                steps.append(cur)
                cur, room = [], max_rows
    if cur:
        steps.append(cur)
    return steps


@dataclass
class SequenceState:
    index: int                       # position of the request among all requests
    prompt_len: int
    output: List[int] = field(default_factory=list)
    finished: bool = False
    reason: str = ""

    def accept(self, token: int, stop: set, max_new_tokens: int, max_position: int) -> bool:
        """Takes the token sampled for this sequence; returns True if the sequence goes on.
        A stop token ends it and is not emitted; so does the token budget or the position limit."""
        if token in stop:
            self.finished, self.reason = True, "stop"
            return False
        self.output.append(token)
        if len(self.output) >= max_new_tokens:
            self.finished, self.reason = True, "length"
            return False
        if self.prompt_len + len(self.output) >= max_position:
            self.finished, self.reason = True, "max_position"
            return False
        return True


class _Rows:
    """Some rows of tokens that are still on their way to the host."""

    def __init__(self, pending, index):
        self._pending, self._index = pending, list(index)

    def tokens(self):
        all_tokens = self._pending.tokens()
        return [all_tokens[i] for i in self._index]

    def rows(self, index):
        return self._pending.rows([self._index[i] for i in index])


class Generator:
    """``engine`` needs ``step(entries)`` and ``end(requests)``; ``sampler`` needs
    ``sample(logits, params, streams, counters)``."""

    def __init__(self, engine, sampler, stop_tokens: Iterable[int], max_position: int,
                 page_budget: int, page: int, max_batch: int = 64, max_prompt_rows: int = 16384):
        """``max_prompt_rows``: the most rows one prompt step brings; a batch whose prompts hold
        more starts with several steps (see ``plan_prompt_steps``)."""
        self.max_prompt_rows = max_prompt_rows
        self.engine = engine
        self.sampler = sampler
        self.stop_tokens = set(stop_tokens)
        self.max_position = max_position
        self.page_budget = page_budget
        self.page = page
        self.max_batch = max_batch
        self._serial = 0

    def generate(self, prompts: Sequence[Sequence[int]], params: SamplingParams,
                 max_new_tokens: int = 256, stop_tokens: Optional[Iterable[int]] = None,
                 on_token: Optional[Callable[[int, int], None]] = None) -> List[List[int]]:
        """Tokens generated for each prompt, in the order of the prompts.  ``on_token(index,
        token)`` is called for every emitted token as soon as it is known."""
        results: List[List[int]] = [[] for _ in prompts]
        for index, token in self.stream(prompts, params, max_new_tokens, stop_tokens):
            results[index].append(token)
            if on_token is not None:
                on_token(index, token)
        return results

    def stream(self, prompts: Sequence[Sequence[int]], params: SamplingParams,
               max_new_tokens: int = 256, stop_tokens: Optional[Iterable[int]] = None):
        """Yields ``(prompt index, token)`` for every emitted token, step by step."""
        if max_new_tokens <= 0:
            return
        stop = self.stop_tokens if stop_tokens is None else set(stop_tokens)
        lens = [len(p) for p in prompts]
        batches = plan_batches(lens, max_new_tokens, self.max_batch, self.page_budget, self.page,
                               self.max_position)
        room = getattr(self.engine, "room", None)
        todo = [i for batch in batches for i in batch]
        while todo:
            # The plan above holds where the whole cache is free (and refuses what can never fit).
            # Other requests may hold a part of it (a completion that its caller has not
            # finished): each batch is cut, by the same rule, to what is free when it starts.
            slots, pages = room() if room is not None else (self.max_batch, self.page_budget)
            if slots <= 0:
                raise CacheError("no free slot: other requests hold every slot of the cache")
            head = todo[:self.max_batch]
            try:
                first = plan_batches([lens[i] for i in head], max_new_tokens, min(self.max_batch, slots),
                                     min(self.page_budget, pages), self.page, self.max_position)[0]
            except RequestError:
                raise CacheError("the cache is full: request %d needs more pages than the %d that other "
                                 "requests leave free" % (todo[0], pages)) from None
            batch, todo = head[:len(first)], todo[len(first):]
            yield from self._run_batch(batch, prompts, params, max_new_tokens, stop)

    def _run_batch(self, batch, prompts, params, max_new_tokens, stop):
        """One batch from its prompt step to its last token.

        Where the engine takes tokens from the device and the sampler can leave them there, the
        next step is queued before the host has seen the tokens it continues from: only a stop
        token is news to the host, and a sequence that drew one has then run one step in vain,
        whose result is dropped.  Everything else that ends a sequence (the token budget, the
        position limit) is known from lengths alone, and such a sequence is not queued again."""
        self._serial += 1
        states = [SequenceState(i, len(prompts[i])) for i in batch]
        name = {st.index: ("gen", self._serial, st.index) for st in states}
        live = list(states)
        ahead = (getattr(self.sampler, "samples_ahead", False)
                 and getattr(self.engine, "takes_device_tokens", False))
        try:
            logits = self._prompt_steps(live, prompts, name)
            pending = self._draw(logits, params, live, 0, ahead)
            while True:
                queued = None
                if ahead:
                    # sequences that go on unless their token turns out to be a stop token
                    cand = [st for st in live if len(st.output) + 1 < max_new_tokens
                            and st.prompt_len + len(st.output) + 1 < self.max_position]
                    if cand:
                        place = {id(st): i for i, st in enumerate(live)}     # (a search per sequence would compare records field by field)
                        rows = pending.rows([place[id(st)] for st in cand])
                        logits = self.engine.step([StepEntry(name[st.index], [0], [0]) for st in cand],
                                                  tokens_device=rows)
                        queued = (cand, self._draw(logits, params, cand, 1, True))
                tokens = pending.tokens() if ahead else pending
                ended, going, emitted = [], [], []
                for st, tok in zip(live, tokens):
                    n_before = len(st.output)
                    (going if st.accept(tok, stop, max_new_tokens, self.max_position) else ended).append(st)
                    if len(st.output) > n_before:
                        emitted.append((st.index, tok))
                if ended:
                    self.engine.end([name[st.index] for st in ended])
                live = going
                for item in emitted:
                    yield item
                if not live:
                    break
                if queued is not None:
                    cand, drawn = queued
                    place = {id(st): i for i, st in enumerate(cand)}
                    pending = _Rows(drawn, [place[id(st)] for st in live])
                else:
                    logits = self.engine.step([StepEntry(name[st.index], [st.output[-1]], [0])
                                               for st in live])
                    pending = self._draw(logits, params, live, 0, ahead)
        finally:
            held = [name[st.index] for st in live if self._holds(name[st.index])]
            if held:
                self.engine.end(held)

    def _prompt_steps(self, live, prompts, name):
        """The prompts of a batch through the step function; returns the logits of every
        sequence's last prompt token, in the order of ``live``."""
        plan = plan_prompt_steps([st.prompt_len for st in live], self.max_prompt_rows)
        rows = []
        for step in plan:
            entries = []
            for i, start, end in step:
                st = live[i]
                entries.append(StepEntry(name[st.index], list(prompts[st.index][start:end]),
                                         [end - start - 1] if end == st.prompt_len else []))
            logits = self.engine.step(entries)
            if len(plan) == 1:
                return logits
            if logits is not None:
                rows.append(logits.clone())        # the next step may overwrite what it returned
        return torch.cat(rows, dim=0)

    def _draw(self, logits, params, seqs, lead, ahead):
        """Samples one token for each sequence; ``lead`` counts tokens that are drawn but not yet
        in ``output``."""
        streams = [st.index for st in seqs]
        counters = [len(st.output) + lead for st in seqs]
        if ahead:
            return self.sampler.sample_device(logits, params, streams, counters)
        return self.sampler.sample(logits, params, streams, counters)

    def _holds(self, request) -> bool:
        holds = getattr(self.engine, "holds", None)
        return True if holds is None else holds(request)
