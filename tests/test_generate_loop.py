"""Decisions of the generation loop, with a stepper that needs no GPU."""
import pytest

from transformer_amd.engine.generate import GenerationError, plan_batches, run_batches
from transformer_amd.sampling.args import InvalidSampleArgs, SampleArgs
from transformer_amd.sampling.sampler import uniform


class Script:
    """Next token of request i after g generated tokens = script[i][g]."""

    def __init__(self, script, slots=4):
        self.script, self.free_slots, self.live = script, list(range(slots)), {}
        self.calls, self.used = [], []

    def alloc(self):
        h = self.free_slots.pop(0)
        self.live[h] = 0
        self.used.append(h)
        return h

    def free(self, h):
        assert h in self.live, "slot freed twice"
        del self.live[h]
        self.free_slots.insert(0, h)

    def step(self, items):
        self.calls.append([(h, i, list(t)) for h, i, g, t in items])
        out = []
        for h, i, g, toks in items:
            assert h in self.live
            self.live[h] += len(toks)
            out.append(self.script[i][g])
        return out


def test_prompts_in_one_step_then_one_token_each_and_early_leavers():
    st = Script({0: [5, 6, 99, 0], 1: [7, 99, 0, 0], 2: [8, 9, 10, 11]})
    r = run_batches(st, [[1, 2, 3], [4], [5, 6]], max_new_tokens=4, stop_ids=[99])
    assert r.tokens == [[5, 6], [7], [8, 9, 10, 11]]                  # the stop token is not emitted
    assert r.finish == ["stop", "stop", "length"]
    assert [len(c) for c in st.calls] == [3, 3, 2, 1]                 # the batch shrinks
    assert st.calls[0] == [(0, 0, [1, 2, 3]), (1, 1, [4]), (2, 2, [5, 6])]
    assert st.calls[1] == [(0, 0, [5]), (1, 1, [7]), (2, 2, [8])]     # only the new token is fed
    assert st.calls[3] == [(2, 2, [10])]
    assert st.live == {}                                              # every slot came back
    assert r.timing.prefill_tokens == 6 and r.timing.decode_tokens == 6
    assert r.timing.decode_steps == 3


def test_batches_follow_each_other_in_reused_slots():
    st = Script({i: [i + 10] * 3 for i in range(5)}, slots=2)
    r = run_batches(st, [[1]] * 5, max_new_tokens=2, max_batch=2)
    assert r.batches == [[0, 1], [2, 3], [4]]
    assert r.tokens == [[i + 10] * 2 for i in range(5)]
    assert len(st.used) == 5 and set(st.used) == {0, 1} and st.live == {}   # two slots serve five requests
    # no request of a later batch joins before the earlier batch is done
    seen = [sorted({i for _, i, _ in c}) for c in st.calls]
    assert seen == [[0, 1], [0, 1], [2, 3], [2, 3], [4], [4]]


def test_batches_are_cut_by_cache_capacity():
    # 100+28 -> 128 tokens each: two fit 256; 10+28 -> 64 more does not
    assert plan_batches([100, 100, 10, 90], 29, capacity_tokens=256, max_batch=8) == [[0, 1], [2, 3]]
    with pytest.raises(GenerationError, match="cache holds"):
        plan_batches([300], 29, capacity_tokens=256, max_batch=8)
    assert plan_batches([100, 100, 10], 29, capacity_tokens=320, max_batch=8) == [[0, 1, 2]]
    with pytest.raises(GenerationError, match="at least one token"):
        plan_batches([0], 4, 1024, 8)


def test_nothing_to_do():
    st = Script({})
    assert run_batches(st, [], 5).tokens == []
    assert run_batches(st, [[1]], 0).tokens == [[]] and st.calls == []


def test_slots_come_back_when_a_step_fails():
    class Boom(Script):
        def step(self, items):
            raise RuntimeError("kernel failed")
    st = Boom({}, slots=2)
    with pytest.raises(RuntimeError):
        run_batches(st, [[1], [2]], 3)
    assert st.live == {}


def test_sample_args_defaults_and_ranges():
    a = SampleArgs()
    assert (a.temperature, a.top_p, a.top_k) == (0.0, 1.0, None) and a.greedy
    assert SampleArgs(0.8).greedy is False and SampleArgs(0.8, top_k=1).greedy
    for bad in (dict(temperature=-0.1), dict(top_p=1.5), dict(top_p=-0.1), dict(top_k=0),
                dict(temperature=float("nan")), dict(top_k=2.5)):
        with pytest.raises(InvalidSampleArgs):
            SampleArgs(**bad)


def test_uniform_is_a_function_of_its_keys():
    us = [uniform(3, s, n) for s in range(50) for n in range(50)]
    assert all(0.0 <= u < 1.0 for u in us) and len(set(us)) > 2400
    assert uniform(3, 4, 5) == uniform(3, 4, 5) != uniform(4, 4, 5)
    assert abs(sum(us) / len(us) - 0.5) < 0.02


class AheadScript(Script):
    """The same script behind the protocol of a stepper that is driven one step ahead: a
    step hands back something whose tokens can be asked for later; the step after it takes
    its tokens from there by position."""

    class Pending:
        def __init__(self, tokens, log):
            self.tokens, self.log, self.asked = tokens, log, False

        def result(self):
            self.asked = True
            self.log.append("result")
            return list(self.tokens)

    def __init__(self, script, slots=4):
        super().__init__(script, slots)
        self.log = []

    def step_async(self, items, previous=None, take=None):
        self.log.append("start")
        if previous is not None:
            assert not previous.asked, "the earlier step's tokens were already on the host"
            assert all(t is None for _, _, _, t in items)
            items = [(h, i, g, [previous.tokens[k]]) for (h, i, g, _), k in zip(items, take)]
        return self.Pending(self.step(items), self.log)


def test_one_step_ahead_gives_the_same_tokens_and_drops_the_step_too_many():
    script = {0: [5, 6, 99, 0, 0], 1: [7, 99, 0, 0, 0], 2: [8, 9, 10, 11, 12]}
    st = AheadScript(script)
    seen = []
    r = run_batches(st, [[1, 2, 3], [4], [5, 6]], max_new_tokens=4, stop_ids=[99],
                    on_token=lambda i, t: seen.append((i, t)))
    assert r.tokens == [[5, 6], [7], [8, 9, 10, 11]] and r.finish == ["stop", "stop", "length"]
    assert seen == [(0, 5), (1, 7), (2, 8), (0, 6), (2, 9), (2, 10), (2, 11)]
    # request 1 stops with its second token, known only after the third step has started: it
    # is stepped once too often; request 2 is never started beyond its four tokens
    assert [sorted(i for _, i, _ in c) for c in st.calls] == [[0, 1, 2], [0, 1, 2], [0, 1, 2], [0, 2]]
    assert st.calls[2] == [(0, 0, [6]), (1, 1, [99]), (2, 2, [9])]    # fed from the step before
    assert st.calls[3] == [(0, 0, [99]), (2, 2, [10])]
    # the prompts' step is read before the first single-token step starts (its time is the time
    # to the first token); from then on a step starts before the last one is read
    assert st.log[:6] == ["start", "result", "start", "start", "result", "start"]
    assert st.live == {}
    assert r.timing.prefill_tokens == 6 and r.timing.decode_steps == 3


def test_one_step_ahead_over_batches_in_reused_slots():
    st = AheadScript({i: [i + 10] * 3 for i in range(5)}, slots=2)
    r = run_batches(st, [[1]] * 5, max_new_tokens=2, max_batch=2)
    assert r.tokens == [[i + 10] * 2 for i in range(5)]
    assert set(st.used) == {0, 1} and st.live == {}
    assert [sorted({i for _, i, _ in c}) for c in st.calls] == [[0, 1], [0, 1], [2, 3], [2, 3], [4], [4]]


def test_a_sequence_that_stops_with_its_first_token_is_not_stepped_again():
    st = AheadScript({0: [99, 0, 0], 1: [5, 6, 7]})
    r = run_batches(st, [[1, 2], [3]], max_new_tokens=3, stop_ids=[99])
    assert r.tokens == [[], [5, 6, 7]] and r.finish == ["stop", "length"]
    assert [sorted(i for _, i, _ in c) for c in st.calls] == [[0, 1], [1], [1]]
    assert r.timing.prefill_tokens == 3 and r.timing.decode_tokens == 2 and st.live == {}
