"""The cache's bookkeeping: no slot or page lost, held twice or freed twice."""
import random

import pytest

from transformer_amd.cache.pool import CacheError, CacheFull, PagePool, SlotPool


def test_pages_are_handed_out_once_and_come_back():
    p = PagePool(5)
    a = p.take(3)
    b = p.take(2)
    assert sorted(a + b) == [0, 1, 2, 3, 4]
    with pytest.raises(CacheFull):
        p.take(1)
    p.give(a)
    with pytest.raises(CacheError, match="twice"):
        p.give(a[:1])
    assert sorted(p.take(3)) == sorted(a)
    p.check()


def test_slots_are_reused_and_double_free_is_refused():
    s = SlotPool(2, 64, {0: 8})
    a, b = s.alloc(), s.alloc()
    assert {a, b} == {0, 1}
    with pytest.raises(CacheFull):
        s.alloc()
    s.free(a)
    with pytest.raises(CacheError, match="twice"):
        s.free(a)
    assert s.alloc() == a                     # the slot that was given back is used again
    with pytest.raises(CacheError, match="not in use"):
        SlotPool(2, 64, {0: 8}).length(1)
    s.check()


def test_reserve_rounds_up_to_pages_and_is_all_or_nothing():
    s = SlotPool(3, 64, {"full": 4, "other": 4})
    a, b = s.alloc(), s.alloc()
    s.reserve({a: 65})                        # 2 pages in each group
    s.advance(a, 65)
    assert len(s.pages(a, 0)) == 2 and len(s.pages(a, 1)) == 2 and s.held_tokens() == 128
    before = [p.free_count for p in s.pools]
    with pytest.raises(CacheFull, match="pages"):
        s.reserve({a: 1, b: 129})             # a fits, b needs 3 pages: only 2 are free
    assert [p.free_count for p in s.pools] == before and s.pages(b, 0) == []
    s.reserve({a: 63})                        # still inside the second page
    assert [p.free_count for p in s.pools] == before
    with pytest.raises(CacheError, match="past its reserved"):
        s.advance(b, 1)
    s.free(a)
    assert all(p.free_count == 4 for p in s.pools)
    s.check()


def test_random_traffic_keeps_the_invariants():
    rnd = random.Random(7)
    s = SlotPool(6, 64, {0: 40})
    live = {}
    for _ in range(3000):
        op = rnd.random()
        if op < 0.25 and s.free_slots:
            live[s.alloc()] = 0
        elif op < 0.45 and live:
            i = rnd.choice(list(live))
            s.free(i)
            del live[i]
        elif live:
            picks = rnd.sample(list(live), rnd.randint(1, len(live)))
            wants = {i: rnd.randint(1, 200) for i in picks}
            try:
                s.reserve(wants)
            except CacheFull:
                continue
            for i, n in wants.items():
                s.advance(i, n)
                live[i] += n
        for i, n in live.items():
            assert s.length(i) == n and len(s.pages(i, 0)) >= -(-n // 64)
        s.check()
    for i in list(live):
        s.free(i)
    s.check()
    assert s.pools[0].free_count == 40 and s.free_slots == 6


def test_reset_keeps_the_slot_and_returns_its_pages():
    s = SlotPool(2, 64, {0: 4})
    a = s.alloc()
    s.reserve({a: 200})
    s.advance(a, 200)
    s.reset(a)
    assert s.length(a) == 0 and s.pages(a, 0) == [] and s.pools[0].free_count == 4
    s.reserve({a: 10})
    s.advance(a, 10)
    s.check()


def test_pages_that_left_a_window_go_back_early_and_only_once():
    """Two groups: group 0 keeps everything, group 1 serves layers with a window of 100."""
    from transformer_amd.cache.pool import RELEASED
    s = SlotPool(2, 64, {0: 8, 1: 4})
    a = s.alloc()
    s.reserve({a: 200})
    s.advance(a, 200)                              # pages 0..3 of each group
    assert s.release_before(a, 1, 200 + 1 - 100) == 1        # positions < 101: page 0 only
    assert s.release_before(a, 1, 200 + 1 - 100) == 0        # asking again gives nothing back
    assert s.pages(a, 1)[0] == RELEASED and all(p >= 0 for p in s.pages(a, 1)[1:])
    assert all(p >= 0 for p in s.pages(a, 0))
    assert s.held_pages(1) == 3 and s.held_pages(0) == 4
    s.check()
    s.reserve({a: 64})                             # the page that came back serves position 256..319
    s.advance(a, 64)
    assert len(s.pages(a, 1)) == 5 and s.held_pages(1) == 4
    with pytest.raises(CacheFull, match="group 1"):
        s.reserve({a: 64})                         # group 1 is full until the window moves on
    assert s.release_before(a, 1, 264 + 1 - 100) == 1
    s.reserve({a: 64})
    s.check()
    assert s.release_before(a, 1, 10 ** 6) == 2    # never past the slot's own length
    assert s.pages(a, 1)[:4] == [RELEASED] * 4
    s.free(a)                                      # released places are not given back twice
    s.check()
    assert s.pools[0].free_count == 8 and s.pools[1].free_count == 4


def test_random_traffic_with_windows_keeps_the_invariants():
    rnd = random.Random(11)
    window = 150
    s = SlotPool(5, 64, {0: 60, 1: 5 * (window // 64 + 3) + 200 // 64})
    live = {}
    for _ in range(3000):
        op = rnd.random()
        if op < 0.2 and s.free_slots:
            live[s.alloc()] = 0
        elif op < 0.35 and live:
            i = rnd.choice(list(live))
            (s.free if rnd.random() < 0.7 else s.reset)(i)
            if s.slots[i].live:
                live[i] = 0
            else:
                del live[i]
        elif live:
            picks = rnd.sample(list(live), rnd.randint(1, len(live)))
            total = 200
            wants = {}
            for i in picks:
                wants[i] = rnd.randint(1, max(1, total // len(picks)))
            try:
                s.reserve(wants)
            except CacheFull as e:
                assert "group 0" in str(e)         # the windowed group is sized never to be the one
                continue
            for i, n in wants.items():
                s.advance(i, n)
                live[i] += n
                s.release_before(i, 1, live[i] + 1 - window)
                first = max(0, live[i] + 1 - window) // 64
                assert all(p >= 0 for p in s.pages(i, 1)[first:-(-live[i] // 64)])
                assert all(p < 0 for p in s.pages(i, 1)[:first])
        s.check()
    for i in list(live):
        s.free(i)
    s.check()
    assert s.pools[0].free_count == 60 and s.pools[1].free_count == s.pools[1].num_pages
