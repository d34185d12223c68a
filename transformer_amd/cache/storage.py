"""Device storage of the cache, grouped by what the layers need.

A mixer declares its need per cache layer: ``KVNeed`` (keys and values of all
positions, or of a window of them) or ``StateNeed`` (one block of fixed size per
sequence). Layers with the same need form a group; a group has storage of its
own and, for keys and values, a page pool and page tables of its own:

    keys   : [layers of the group][pages][kv heads][PAGE][head size]
    values : [layers of the group][pages][kv heads][value size][PAGE]
    state  : [layers of the group][slots + 1][*shape]

so one head of one page is one contiguous block that the attention kernels
stream; value pages are transposed because the matrix cores want runs of
consecutive keys for one output column. The reference's layout is one tensor per request,
[buf, nblk, 2, nkvh, dh] (models/llama/common/src/lib.rs:98-107).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from .pool import CacheError, CacheFull, SlotPool

from ..kernels import PAGE   # tokens per cache page: one constant, checked against the kernel library


@dataclass(frozen=True)
class KVNeed:
    """Keys and values of every position (or of a window of them). ``value_dim``: width of a
    value row where it differs from the key's (None: the same; 0: keys only, for a mixer that
    keeps one row per token and derives both from it)."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None     # None: every earlier position is read
    value_dim: Optional[int] = None

    def __post_init__(self):
        if self.value_dim is None:
            object.__setattr__(self, "value_dim", self.head_dim)


@dataclass(frozen=True)
class StateNeed:
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class SequenceCache:
    """Slots, pages and the tensors behind them.

    needs: one entry per cache layer (None for a layer that keeps nothing).
    A mixer that needs several things names them in a list; each is a cache layer of its own.
    max_tokens: tokens that live sequences may hold together, each sequence
    rounded up to whole pages. max_slots: sequences alive at once.
    max_step_tokens: the most tokens that one step brings, all sequences together. A group
    whose layers read a window gives pages that have left the window back after every step;
    with this bound its storage is sized for the windows of all slots plus one step
    instead of for max_tokens (a larger step then fails with CacheFull before it runs).
    planners: one entry per cache layer (or None): what the layer's mixer wants worked out on
    the host for every step of single tokens, beside the page tables of its group (see
    ``engine.batch.plan_step``); the distinct planners of a group are asked once per step.
    """

    def __init__(self, needs: Sequence[object], max_tokens: int, max_slots: int,
                 dtype: torch.dtype, device, max_step_tokens: Optional[int] = None,
                 planners: Optional[Sequence[object]] = None):
        if max_tokens <= 0:
            raise CacheError(f"max_tokens must be positive, got {max_tokens}")
        self.dtype, self.device = dtype, torch.device(device)
        self.num_pages = -(-max_tokens // PAGE)
        self.max_slots = max_slots
        self.kv_groups: List[KVNeed] = []
        self.state_groups: List[StateNeed] = []
        self._where: List[Optional[Tuple[str, int, int]]] = []   # layer -> (kind, group, index)
        counts_kv: List[int] = []
        counts_st: List[int] = []
        self.group_planners: List[List[object]] = []
        if planners is not None and len(planners) != len(needs):
            raise CacheError("one planner (or None) per cache layer")
        for i, need in enumerate(needs):
            if need is None:
                self._where.append(None)
            elif isinstance(need, KVNeed):
                if need not in self.kv_groups:
                    self.kv_groups.append(need)
                    self.group_planners.append([])
                    counts_kv.append(0)
                g = self.kv_groups.index(need)
                self._where.append(("kv", g, counts_kv[g]))
                counts_kv[g] += 1
                if planners is not None and planners[i] is not None and \
                        planners[i] not in self.group_planners[g]:
                    self.group_planners[g].append(planners[i])
            elif isinstance(need, StateNeed):
                if need not in self.state_groups:
                    self.state_groups.append(need)
                    counts_st.append(0)
                g = self.state_groups.index(need)
                self._where.append(("state", g, counts_st[g]))
                counts_st[g] += 1
            else:
                raise CacheError(f"unknown cache need {need!r}")
        self.group_pages = [self.num_pages] * len(self.kv_groups)
        if max_step_tokens is not None:
            for g, need in enumerate(self.kv_groups):
                if need.window is not None:
                    # a slot holds at most the pages that touch its window and its share of
                    # the step: (window + n - 1) / PAGE + 2
                    bound = max_slots * (need.window // PAGE + 3) + max_step_tokens // PAGE
                    self.group_pages[g] = max(1, min(self.num_pages, bound))
        self.pool = SlotPool(max_slots, PAGE, dict(enumerate(self.group_pages)))
        self.keys, self.values = [], []
        # one page more than the pool hands out: rows that a step only carries to fill a
        # recorded launch shape store their key and value there, where nothing reads them
        self.spare_page = list(self.group_pages)
        # steps that the model has recorded against this cache's tensors (HIP graphs), and
        # the model that recorded them
        self.graphs: Dict[tuple, object] = {}
        self.graphs_checked = set()          # (batch, wanted rows) whose recording has been tried
        self.graphs_failed = set()           # (batch, wanted rows) that run eagerly for good
        self.graph_owner = None
        for need, n, pages in zip(self.kv_groups, counts_kv, self.group_pages):
            kshape = (n, pages + 1, need.num_kv_heads, PAGE, need.head_dim)
            vshape = (n, pages + 1, need.num_kv_heads, need.value_dim, PAGE)
            self.keys.append(torch.empty(kshape, dtype=dtype, device=self.device))
            self.values.append(torch.empty(vshape, dtype=dtype, device=self.device))
        # one row more than there are slots, as there is a spare page: the rows that fill a
        # recorded step carry this slot, so that a mixer's update of "its" state lands nowhere
        self.spare_slot = max_slots
        self.states = [torch.zeros((n, max_slots + 1, *need.shape), dtype=need.dtype, device=self.device)
                       for need, n in zip(self.state_groups, counts_st)]

    # ------------------------------------------------------------------ slots
    def alloc_slot(self) -> int:
        slot = self.pool.alloc()
        for s in self.states:           # fixed-size state starts from zero
            s[:, slot].zero_()
        return slot

    def free_slot(self, slot: int) -> None:
        self.pool.free(slot)

    def reset_slot(self, slot: int) -> None:
        """Back to an empty sequence: no tokens, no pages, fixed-size state zero."""
        self.pool.reset(slot)
        for s in self.states:
            s[:, slot].zero_()

    def length(self, slot: int) -> int:
        return self.pool.length(slot)

    def release_outside_windows(self, slot: int) -> None:
        """After a step: the next token of the slot sits at position ``length`` and a layer
        with window w reads keys from ``length + 1 - w`` on; earlier pages go back."""
        n = self.pool.length(slot)
        for g, need in enumerate(self.kv_groups):
            if need.window is not None:
                self.pool.release_before(slot, g, n + 1 - need.window)

    def bytes(self) -> int:
        n = sum(t.numel() * t.element_size() for t in self.keys + self.values + self.states)
        return n

    # ------------------------------------------------------------------ views
    def layer_kv(self, layer: int):
        """(keys [pages, kv heads, PAGE, head size], values [pages, kv heads, head size,
        PAGE], group) of a cache layer."""
        w = self._where[layer]
        if w is None or w[0] != "kv":
            raise CacheError(f"cache layer {layer} holds no keys and values")
        return self.keys[w[1]][w[2]], self.values[w[1]][w[2]], w[1]

    def layer_state(self, layer: int) -> torch.Tensor:
        """State of a cache layer for every slot: [slots + 1, *shape]; the last row belongs to
        nobody (rows that only fill a recorded step name it as their slot)."""
        w = self._where[layer]
        if w is None or w[0] != "state":
            raise CacheError(f"cache layer {layer} holds no fixed-size state")
        return self.states[w[1]][w[2]]
