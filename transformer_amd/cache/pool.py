"""Host-side bookkeeping of the cache: slots for sequences, pages for tokens.

A *slot* stands for one live sequence: its length, the pages it holds in each
group of layers, and a row in every table of fixed-size state. A *page* holds
``page_size`` consecutive tokens of one sequence for all layers of one group.
Nothing here touches the GPU, so the invariants (no slot or page lost, held
twice or freed twice) are tested without one.

The reference gives each request one cache tensor of fixed capacity that the
caller carries along with ``pos`` (models/llama/common/src/
args.rs:19-25, lib.rs:98-111); here the pool owns both.
"""
from __future__ import annotations

from typing import Dict, List


class CacheError(RuntimeError):
    pass


class CacheFull(CacheError):
    """No free slot, or not enough free pages; nothing was changed."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise CacheError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = num_pages
        # pop() hands out low numbers first
        self._free: List[int] = list(range(num_pages - 1, -1, -1))
        self._held = [False] * num_pages

    @property
    def free_count(self) -> int:
        return len(self._free)

    def take(self, n: int) -> List[int]:
        if n < 0:
            raise CacheError("cannot take a negative number of pages")
        if n > len(self._free):
            raise CacheFull(f"{n} pages wanted, {len(self._free)} of {self.num_pages} free")
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            if self._held[p]:
                raise CacheError(f"page {p} was on the free list while held")
            self._held[p] = True
        return out

    def give(self, pages) -> None:
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise CacheError(f"page {p} does not exist")
            if not self._held[p]:
                raise CacheError(f"page {p} freed twice")
        for p in pages:
            self._held[p] = False
            self._free.append(p)

    def check(self) -> None:
        """Every page is either free or held, exactly once."""
        if len(set(self._free)) != len(self._free):
            raise CacheError("a page is on the free list twice")
        for p in range(self.num_pages):
            if self._held[p] == (p in set(self._free)):
                raise CacheError(f"page {p} is {'both held and free' if self._held[p] else 'lost'}")


RELEASED = -1      # stands in a slot's page list for a page that was given back early


class Slot:
    __slots__ = ("index", "length", "pages", "released", "live")

    def __init__(self, index: int, num_groups: int):
        self.index = index
        self.length = 0
        # pages[g][i] holds positions [i * page_size, (i + 1) * page_size) in group g
        self.pages: List[List[int]] = [[] for _ in range(num_groups)]
        self.released = [0] * num_groups      # leading entries of pages[g] that are RELEASED
        self.live = False


class SlotPool:
    """Slots and, per page group, the pages they hold.

    page_groups: {group key: number of pages}; every group pages the same token
    positions of a sequence but has storage, and therefore a pool, of its own.
    """

    def __init__(self, max_slots: int, page_size: int, page_groups: Dict[object, int]):
        if max_slots <= 0:
            raise CacheError(f"a cache needs at least one slot, got {max_slots}")
        self.page_size = page_size
        self.group_keys = list(page_groups)
        self.pools = [PagePool(n) for n in page_groups.values()]
        self.slots = [Slot(i, len(self.pools)) for i in range(max_slots)]
        self._free = list(range(max_slots - 1, -1, -1))

    # ------------------------------------------------------------------ slots
    @property
    def free_slots(self) -> int:
        return len(self._free)

    def live_slots(self) -> List[int]:
        return [s.index for s in self.slots if s.live]

    def alloc(self) -> int:
        if not self._free:
            raise CacheFull(f"all {len(self.slots)} slots are in use")
        s = self.slots[self._free.pop()]
        if s.live:
            raise CacheError(f"slot {s.index} was on the free list while live")
        s.live, s.length = True, 0
        return s.index

    def _slot(self, index: int) -> Slot:
        if not 0 <= index < len(self.slots):
            raise CacheError(f"slot {index} does not exist")
        s = self.slots[index]
        if not s.live:
            raise CacheError(f"slot {index} is not in use")
        return s

    def free(self, index: int) -> None:
        if not 0 <= index < len(self.slots):
            raise CacheError(f"slot {index} does not exist")
        s = self.slots[index]
        if not s.live:
            raise CacheError(f"slot {index} freed twice")
        self._drop_pages(s)
        s.live, s.length = False, 0
        self._free.append(index)

    def _drop_pages(self, s: Slot) -> None:
        for g, pool in enumerate(self.pools):
            pool.give(s.pages[g][s.released[g]:])
            s.pages[g] = []
            s.released[g] = 0

    def reset(self, index: int) -> None:
        """The slot stays with its owner but forgets its tokens and gives its pages back."""
        s = self._slot(index)
        self._drop_pages(s)
        s.length = 0

    def length(self, index: int) -> int:
        return self._slot(index).length

    # ------------------------------------------------------------------ pages
    def pages_for(self, tokens: int) -> int:
        return -(-tokens // self.page_size)

    def reserve(self, wants: Dict[int, int]) -> None:
        """Make room for ``wants[slot]`` more tokens in each named slot, in every
        group. Either all of it succeeds or nothing changes."""
        need = [0] * len(self.pools)
        plan = []
        for index, extra in wants.items():
            s = self._slot(index)
            if extra < 0:
                raise CacheError("cannot reserve a negative number of tokens")
            total = self.pages_for(s.length + extra)
            for g in range(len(self.pools)):
                more = max(0, total - len(s.pages[g]))
                need[g] += more
                plan.append((s, g, more))
        for g, pool in enumerate(self.pools):
            if need[g] > pool.free_count:
                raise CacheFull(
                    f"cache group {self.group_keys[g]!r}: {need[g]} more pages of "
                    f"{self.page_size} tokens needed, {pool.free_count} of {pool.num_pages} free")
        for s, g, more in plan:
            s.pages[g].extend(self.pools[g].take(more))

    def advance(self, index: int, tokens: int) -> None:
        s = self._slot(index)
        if any(self.pages_for(s.length + tokens) > len(s.pages[g]) for g in range(len(self.pools))):
            raise CacheError(f"slot {index}: advancing by {tokens} tokens past its reserved pages")
        s.length += tokens

    def release_before(self, index: int, group: int, position: int) -> int:
        """Gives back the pages of one group that lie wholly before ``position``: a group
        whose layers read a window of keys never looks at them again. Their places in the
        slot's page list keep RELEASED, so that a position still finds its page by index.
        Returns the number of pages given back."""
        s = self._slot(index)
        upto = min(max(position, 0), s.length) // self.page_size
        first = s.released[group]
        if upto <= first:
            return 0
        self.pools[group].give(s.pages[group][first:upto])
        s.pages[group][first:upto] = [RELEASED] * (upto - first)
        s.released[group] = upto
        return upto - first

    def pages(self, index: int, group: int) -> List[int]:
        """Page of every 64 positions of the slot, RELEASED where it was given back early."""
        return self._slot(index).pages[group]

    def held_pages(self, group: int) -> int:
        return self.pools[group].num_pages - self.pools[group].free_count

    def held_tokens(self) -> int:
        """Tokens held by live slots, each rounded up to whole pages."""
        return sum(self.pages_for(s.length) * self.page_size for s in self.slots if s.live)

    def check(self) -> None:
        for pool in self.pools:
            pool.check()
        if len(set(self._free)) != len(self._free):
            raise CacheError("a slot is on the free list twice")
        for s in self.slots:
            if s.live == (s.index in self._free):
                raise CacheError(f"slot {s.index} is {'both live and free' if s.live else 'lost'}")
            if not s.live and any(s.pages[g] for g in range(len(self.pools))):
                raise CacheError(f"free slot {s.index} still holds pages")
        for g, pool in enumerate(self.pools):
            seen = set()
            for s in self.slots:
                if any(p != RELEASED for p in s.pages[g][:s.released[g]]) or \
                        any(p == RELEASED for p in s.pages[g][s.released[g]:]):
                    raise CacheError(f"slot {s.index}: released pages of group "
                                     f"{self.group_keys[g]!r} are out of place")
                for p in s.pages[g][s.released[g]:]:
                    if p in seen:
                        raise CacheError(f"page {p} of group {self.group_keys[g]!r} is held twice")
                    seen.add(p)
            if len(seen) + pool.free_count != pool.num_pages:
                raise CacheError(f"group {self.group_keys[g]!r}: pages lost")
