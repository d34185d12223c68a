"""The integer tables of a step: positions, row offsets, wanted rows, page tables."""
import numpy as np
import pytest

from transformer_amd.engine.batch import Entry, StepError, check_entries, layout_step


def test_layout_of_an_unequal_batch():
    entries = [Entry(4, [7, 8, 9], [0, 2]), Entry(1, [5], []), Entry(2, list(range(70)), [69])]
    lengths = [0, 130, 60]
    pages = [[[3], [9, 2, 5], [6, 0, 1]]]
    packed, off, s = layout_step(entries, lengths, pages)

    def get(n):
        return packed[off[n][0]:off[n][1]]

    assert s["nt"] == 74 and s["batch"] == 3 and s["max_qlen"] == 70 and s["max_kv_len"] == 131
    assert get("tokens")[:4].tolist() == [7, 8, 9, 5]
    assert get("positions")[:5].tolist() == [0, 1, 2, 130, 60]
    assert get("cu_q").tolist() == [0, 3, 4, 74] and get("pos0").tolist() == lengths
    assert get("slots").tolist() == [4, 1, 2]
    assert get("want").tolist() == [0, 2, 4 + 69]            # rows in the order of entries, then of want
    table = get("table0").reshape(s["shapes"]["table0"])
    assert table.shape == (3, 3)
    assert table[0].tolist() == [3, 0, 0] and table[1].tolist() == [9, 2, 5]
    dest = get("dest0")
    assert dest[:3].tolist() == [3 * 64, 3 * 64 + 1, 3 * 64 + 2]
    assert dest[3] == 5 * 64 + 2                              # position 130 -> third page, offset 2
    assert dest[4] == 6 * 64 + 60 and dest[4 + 4] == 0 * 64 + 0   # position 64 starts the next page
    assert dest[-1] == 1 * 64 + 1                             # position 129


def test_entries_are_checked_before_anything_runs():
    with pytest.raises(StepError, match="twice"):
        check_entries([Entry(0, [1]), Entry(0, [2])], 10)
    with pytest.raises(StepError, match="at least one token"):
        check_entries([Entry(0, [])], 10)
    with pytest.raises(StepError, match="vocabulary"):
        check_entries([Entry(0, [10])], 10)
    with pytest.raises(StepError, match="outside"):
        check_entries([Entry(0, [1, 2], [2])], 10)
    with pytest.raises(StepError, match="ascend"):
        check_entries([Entry(0, [1, 2], [1, 0])], 10)


def test_units_of_work_cover_every_page_once_and_are_about_equal():
    import random
    from transformer_amd import kernels
    rnd = random.Random(3)
    for trial in range(300):
        B = rnd.randint(1, 40)
        lens = [rnd.choice([1, 63, 64, 65, rnd.randint(1, 5000)]) for _ in range(B)]
        n_units = kernels.key_unit_count(B, rnd.choice([1, 2, 8]))
        assert n_units >= B
        units, seq = kernels.plan_key_units(lens, n_units)
        assert units.shape == (n_units, 8) and seq.shape == (B, 2) and units.dtype == np.int32
        used = 0
        order = sorted(range(B), key=lambda b: seq[b][0])
        assert sorted(int(seq[b][0]) for b in range(B)) == list(np.cumsum([0] + [int(seq[b][1]) for b in order[:-1]]))
        for b, n in enumerate(lens):
            first, count = seq[b]
            assert count >= 1
            pages = -(-n // 64)
            at = 0
            for u in units[first:first + count]:
                assert u[0] == b and u[1] == at and u[2] >= 1 and u[3] == n and u[6] == count
                at += u[2]
            assert at == pages                                   # every page, in order, once
            sizes = units[first:first + count, 2]
            assert sizes.max() - sizes.min() <= 1
            assert count == 1 or sizes.min() >= 2                # no cut makes runs shorter than two pages
            used += count
        assert (units[used:, 2] == 0).all()                      # spare units hold nothing
        # sequences with the longest runs come first (their workgroups start first)
        runs = [-(-lens[b] // 64) / int(seq[b][1]) for b in order]
        assert all(x >= y for x, y in zip(runs, runs[1:]))
        # the longest run is as short as the number of units allows
        longest = units[:, 2].max()
        if used < n_units:
            b = int(units[np.argmax(units[:, 2]), 0])
            assert -(-lens[b] // 64) < 2 * (seq[b, 1] + 1)
    with pytest.raises(kernels.KernelError, match="cannot hold"):
        kernels.plan_key_units([5, 5, 5], 2)
    u, s = kernels.uniform_key_units([130, 64], 2)
    assert u[:, :4].tolist() == [[0, 0, 2, 130], [0, 2, 1, 130], [1, 0, 1, 64]] and s.tolist() == [[0, 2], [2, 1]]
    assert u[:, 6].tolist() == [2, 2, 1]


def test_a_step_of_single_tokens_carries_what_its_mixers_planners_work_out():
    """The step's layout knows no attention kernel: a group's planners are asked for named
    tables, which travel with the page tables. The attention mixer's own planner cuts the
    sequences into units of work; its table sizes follow from the batch size alone."""
    from transformer_amd import kernels
    from transformer_amd.parts.attention import KeyUnitPlanner

    class EightUnits:
        def tables(self, kv_lens, table):
            units, seq_units = kernels.plan_key_units(kv_lens, 8, tables=table)
            return {"units": units, "seq_units": seq_units}

    class Doubled:                                   # any other part's plan rides along
        def tables(self, kv_lens, table):
            return {"twice": 2 * np.asarray(kv_lens)}

    entries = [Entry(0, [5], [0]), Entry(1, [6], [0])]
    packed, off, s = layout_step(entries, [700, 3], [[list(range(11)), [40]]], 16, planners=[[EightUnits(), Doubled()]])
    a, b = off["plan0.0.units"]
    units = packed[a:b].reshape(s["shapes"]["plan0.0.units"])
    # 11 pages in runs of at least two: 3, 2, 2, 2, 2; then the sequence of one page
    assert units[:, 2].tolist() == [3, 2, 2, 2, 2, 1, 0, 0] and units[:6, 0].tolist() == [0, 0, 0, 0, 0, 1]
    assert units[:6, 4].tolist() == [0, 3, 5, 7, 9, 40]                                     # the first two pages
    assert units[:6, 5].tolist() == [1, 4, 6, 8, 10, 40]                                    # of each run
    a, b = off["plan0.0.seq_units"]
    assert packed[a:b].tolist() == [0, 5, 5, 1]
    a, b = off["plan0.1.twice"]
    assert packed[a:b].tolist() == [1402, 8]                     # lengths with this step's token
    _, off2, _ = layout_step([Entry(0, [5, 6], [1])], [700], [[list(range(11))]], 16, planners=[[EightUnits()]])
    assert not any(n.startswith("plan") for n in off2)           # only steps of single tokens
    for nkv in (1, 2, 8):
        planner = KeyUnitPlanner(nkv)
        assert planner == KeyUnitPlanner(nkv) and hash(planner) == hash(KeyUnitPlanner(nkv))
        for batch in (1, 5, 64):
            t = planner.tables([100] * batch, np.zeros((batch, 2), dtype=np.int32))
            assert sum(a.size for a in t.values()) == planner.ints(batch)


def test_positions_past_the_models_limit_are_refused():
    from transformer_amd.engine.batch import PositionPastLimit, check_positions
    entries = [Entry(0, [1, 2, 3]), Entry(1, [4])]
    check_positions(entries, [5, 7], 8)             # positions 5..7 and 7: the last one allowed
    check_positions(entries, [500, 700], None)      # no limit given
    with pytest.raises(PositionPastLimit, match="slot 1"):
        check_positions(entries, [5, 8], 8)
    with pytest.raises(PositionPastLimit, match="slot 0"):
        check_positions(entries, [6, 0], 8)


def test_choice_of_the_prompt_attention_kernel():
    """Short prompts read their operands directly; heads above 128 share pages through LDS
    without overlap; everything else takes the kernel that overlaps by half pages."""
    from transformer_amd.kernels import rows_kernel
    assert rows_kernel(40, 32, 8, 128) == 0                 # 160 rows
    assert rows_kernel(64, 32, 8, 128) == 2
    assert rows_kernel(255, 8, 8, 64) == 0 and rows_kernel(256, 8, 8, 64) == 2
    assert rows_kernel(16384, 32, 8, 128) == 2
    assert rows_kernel(4096, 4, 4, 256) == 1 and rows_kernel(4096, 5, 5, 160) == 1
    assert rows_kernel(100, 4, 4, 256) == 0
