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
