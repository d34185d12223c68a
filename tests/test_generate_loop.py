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
