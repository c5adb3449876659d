"""The generation loop's decisions, with a scripted engine and sampler: batching, stop tokens,
sequences that end earlier, token budgets, slots given back."""
import pytest
import torch

from libllm_amd import RequestError
from libllm_amd.engine import Generator, SequenceState, plan_batches, plan_prompt_steps
from libllm_amd.sampling import Sampler, SamplingParams


class ScriptedEngine:
    """Records the steps; its 'logits' are the token each request is scripted to produce next."""

    def __init__(self, scripts):
        self.scripts = scripts              # prompt index -> list of tokens to emit
        self.steps, self.ended, self.live = [], [], set()
        self.cursor = {}

    def step(self, entries):
        self.steps.append([(e.request[2], list(e.tokens), list(e.want)) for e in entries])
        out = []
        for e in entries:
            i = e.request[2]
            self.live.add(e.request)
            if not e.want:                  # a part of a prompt: nothing comes back for it
                continue
            n = self.cursor.get(i, 0)
            out.append(self.scripts[i][n])
            self.cursor[i] = n + 1
        return torch.tensor(out).reshape(-1, 1)

    def end(self, requests):
        for r in requests:
            assert r in self.live, "a request is ended that is not live"
            self.live.remove(r)
            self.ended.append(r[2])

    def holds(self, request):
        return request in self.live


class ScriptedSampler:
    def __init__(self):
        self.calls = []

    def sample(self, logits, params, streams, counters):
        self.calls.append((list(streams), list(counters)))
        return [int(v) for v in logits[:, 0]]


def make(scripts, max_batch=64, pages=1000, stop=(99,), max_position=10000):
    eng, smp = ScriptedEngine(scripts), ScriptedSampler()
    return eng, smp, Generator(eng, smp, stop, max_position, pages, 64, max_batch=max_batch)


def test_stop_token_ends_one_sequence_while_others_continue():
    scripts = {0: [5, 6, 99, 1, 1], 1: [7, 99], 2: [8, 9, 10, 11, 12]}
    eng, smp, gen = make(scripts)
    out = gen.generate([[1, 2, 3], [4], [5, 6]], SamplingParams(0.0), max_new_tokens=4)
    assert out == [[5, 6], [7], [8, 9, 10, 11]]            # the stop token is not emitted
    # one prompt step with all prompts and the last row wanted, then one token per live sequence
    assert eng.steps[0] == [(0, [1, 2, 3], [2]), (1, [4], [0]), (2, [5, 6], [1])]
    assert eng.steps[1] == [(0, [5], [0]), (1, [7], [0]), (2, [8], [0])]
    assert eng.steps[2] == [(0, [6], [0]), (2, [9], [0])]   # sequence 1 has left
    assert eng.steps[3] == [(2, [10], [0])]
    assert len(eng.steps) == 4                              # the budget ends 2 without another step
    assert sorted(eng.ended) == [0, 1, 2] and not eng.live
    assert smp.calls[0] == ([0, 1, 2], [0, 0, 0]) and smp.calls[2] == ([0, 2], [2, 2])


def test_batches_follow_one_another():
    scripts = {i: [10 + i, 99] for i in range(5)}
    eng, _, gen = make(scripts, max_batch=2)
    out = gen.generate([[1]] * 5, SamplingParams(0.0), max_new_tokens=8)
    assert out == [[10], [11], [12], [13], [14]]
    firsts = [s for s in eng.steps if s[0][1] == [1]]
    assert [[i for i, _, _ in s] for s in firsts] == [[0, 1], [2, 3], [4]]
    assert eng.ended == [0, 1, 2, 3, 4]


def test_on_token_streams_in_order_and_custom_stop():
    scripts = {0: [5, 6, 7], 1: [8, 42, 9]}
    eng, _, gen = make(scripts)
    seen = []
    out = gen.generate([[1], [2]], SamplingParams(0.0), 3, stop_tokens=[42], on_token=lambda i, t: seen.append((i, t)))
    assert out == [[5, 6, 7], [8]] and seen == [(0, 5), (1, 8), (0, 6), (0, 7)]


def test_an_error_gives_the_slots_back():
    class Failing(ScriptedEngine):
        def step(self, entries):
            if len(self.steps) == 2:
                raise RuntimeError("boom")
            return super().step(entries)
    eng = Failing({0: [1, 2, 3], 1: [4, 5, 6]})
    gen = Generator(eng, ScriptedSampler(), (), 1000, 100, 64)
    with pytest.raises(RuntimeError):
        gen.generate([[1], [2]], SamplingParams(0.0), 5)
    assert not eng.live


def test_plan_batches():
    assert plan_batches([10, 20, 30], 5, 2, 100, 64, 4096) == [[0, 1], [2]]
    # 64-token pages: 60+10 -> 2 pages, 100+10 -> 2, 10+10 -> 1; a budget of 4 pages
    assert plan_batches([60, 100, 10, 10], 10, 8, 4, 64, 4096) == [[0, 1], [2, 3]]
    assert plan_batches([60, 100], 10, 8, 3, 64, 4096) == [[0], [1]]
    assert plan_batches([100], 1000, 8, 2, 64, 128) == [[0]]             # growth is capped by max_position
    for bad in (([0], 5, 2, 10), ([300], 5, 2, 2), ([200], 5, 2, 10)):
        with pytest.raises(RequestError):
            plan_batches(bad[0], bad[1], bad[2], bad[3], 64, 128)
    with pytest.raises(RequestError):
        plan_batches([1], 1, 0, 10, 64, 128)


def test_sequence_state():
    st = SequenceState(0, prompt_len=5)
    assert st.accept(3, {9}, 3, 100) and st.accept(4, {9}, 3, 100)
    assert not st.accept(5, {9}, 3, 100) and st.reason == "length" and st.output == [3, 4, 5]
    st = SequenceState(0, prompt_len=5)
    assert not st.accept(9, {9}, 3, 100) and st.reason == "stop" and st.output == []
    st = SequenceState(0, prompt_len=5)
    assert st.accept(1, set(), 10, 7) and not st.accept(2, set(), 10, 7) and st.reason == "max_position"


def test_sampling_params():
    v = 1000
    assert SamplingParams().validate(v) == SamplingParams(1.0, 50, 0.8, 0)   # src/libllm/llm.cc:125-132
    assert SamplingParams(0.0, 50, 0.8).greedy and SamplingParams(1.0, 1, 0.8).greedy
    assert SamplingParams(1.0, 5000, 1.0).validate(v).top_k == 0             # clamped, not an abort
    assert SamplingParams(1.0, 0, 0.5).validate(v).top_k == 0                # a nucleus with no limit on its size
    assert SamplingParams(1.0, 0, 0.9).validate(128256) == SamplingParams(1.0, 0, 0.9, 0)
    for bad in (SamplingParams(-1.0), SamplingParams(1.0, -1), SamplingParams(1.0, 5, 0.0),
                SamplingParams(1.0, 5, 1.5), SamplingParams(1.0, 2000, 0.9)):
        with pytest.raises(RequestError):
            bad.validate(128256)

    class Ops:
        def argmax(self, logits):
            return torch.argmax(logits, -1)
    assert Sampler(Ops(), 4).sample(torch.tensor([[0.0, 2.0, 1.0, 2.0]]), SamplingParams(0.0), [0], [0]) == [1]
    with pytest.raises(RequestError):
        Sampler(Ops(), 4).sample(torch.zeros((2, 4)), SamplingParams(0.0), [0], [0])


class AheadEngine(ScriptedEngine):
    """Takes the tokens of a step from a 'device' tensor: the host's ids are placeholders."""
    takes_device_tokens = True

    def step(self, entries, tokens_device=None):
        if tokens_device is not None:
            assert len(tokens_device) == len(entries) and all(list(e.tokens) == [0] for e in entries)
            entries = [type(e)(e.request, [int(t)], e.want) for e, t in zip(entries, tokens_device)]
        return super().step(entries)


class AheadSampler(ScriptedSampler):
    samples_ahead = True

    class Pending:
        def __init__(self, toks):
            self.toks, self.read = toks, False

        def tokens(self):
            self.read = True
            return list(self.toks)

        def rows(self, index):
            assert not self.read, "the next step is queued before the host reads the tokens"
            return [self.toks[i] for i in index]

    def sample_device(self, logits, params, streams, counters):
        return self.Pending(self.sample(logits, params, streams, counters))


def test_steps_are_queued_ahead_and_a_stop_token_costs_one_step():
    scripts = {0: [5, 6, 99, 1, 1], 1: [7, 99, 3], 2: [8, 9, 10, 11, 12]}
    eng, smp = AheadEngine(scripts), AheadSampler()
    gen = Generator(eng, smp, (99,), 10000, 1000, 64)
    out = gen.generate([[1, 2, 3], [4], [5, 6]], SamplingParams(0.0), max_new_tokens=4)
    assert out == [[5, 6], [7], [8, 9, 10, 11]]            # the same tokens as step by step
    assert eng.steps[1] == [(0, [5], [0]), (1, [7], [0]), (2, [8], [0])]
    # sequence 1 drew its stop token in step 1; step 2 was queued before the host saw it
    assert eng.steps[2] == [(0, [6], [0]), (1, [99], [0]), (2, [9], [0])]
    assert eng.steps[3] == [(0, [99], [0]), (2, [10], [0])]
    assert len(eng.steps) == 4                              # the budget is known ahead: no step in vain
    assert sorted(eng.ended) == [0, 1, 2] and not eng.live
    # counters of the draws: the tokens drawn before, whether the host has seen them or not
    assert smp.calls[1] == ([0, 1, 2], [1, 1, 1]) and smp.calls[2] == ([0, 1, 2], [2, 2, 2])
    assert smp.calls[3] == ([0, 2], [3, 3])


def test_queued_ahead_respects_the_position_limit():
    eng, smp = AheadEngine({0: [5, 6, 7, 8, 9]}), AheadSampler()
    gen = Generator(eng, smp, (99,), 5, 1000, 64)           # prompt 3 + 2 tokens reach the limit
    assert gen.generate([[1, 2, 3]], SamplingParams(0.0), max_new_tokens=10) == [[5, 6]]
    assert [s[0][1] for s in eng.steps] == [[1, 2, 3], [5]]  # no step beyond the limit


def test_prompt_steps_are_bounded():
    """The prompts of a batch come in steps of at most ``max_prompt_rows`` rows: prompts that fit
    together share a step, a long one is cut, and the last token's logits are wanted where a
    prompt ends.  The tokens that follow are the same as with one big step."""
    assert plan_prompt_steps([3, 2, 4], 100) == [[(0, 0, 3), (1, 0, 2), (2, 0, 4)]]
    assert plan_prompt_steps([3, 2, 4], 4) == [[(0, 0, 3), (1, 0, 1)], [(1, 1, 2), (2, 0, 3)], [(2, 3, 4)]]
    assert plan_prompt_steps([9], 4) == [[(0, 0, 4)], [(0, 4, 8)], [(0, 8, 9)]]
    with pytest.raises(RequestError):
        plan_prompt_steps([1], 0)
    scripts = {0: [5, 6, 99], 1: [7, 99], 2: [8, 9, 99]}
    prompts = [[1, 2, 3], [4, 5], [6, 7, 8, 9]]
    eng, smp, gen = make(scripts)
    gen.max_prompt_rows = 4
    out = gen.generate(prompts, SamplingParams(0.0), max_new_tokens=8)
    assert out == [[5, 6], [7], [8, 9]]
    assert eng.steps[0] == [(0, [1, 2, 3], [2]), (1, [4], [])]
    assert eng.steps[1] == [(1, [5], [0]), (2, [6, 7, 8], [])]
    assert eng.steps[2] == [(2, [9], [0])]
    assert eng.steps[3] == [(0, [5], [0]), (1, [7], [0]), (2, [8], [0])]
    assert smp.calls[0] == ([0, 1, 2], [0, 0, 0])
    assert sorted(eng.ended) == [0, 1, 2] and not eng.live
