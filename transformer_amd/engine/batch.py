"""What one step knows about its batch, on the host and on the device.

The tokens of all sequences are concatenated without padding (nt = sum of the
sequences' new tokens), as in the reference's step
(models/llama/common/src/compute.rs:188-201: positions are
pos..pos+seq_len per request, the row split is the list of seq_len). All
integer tables of a step travel to the device in one copy.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache.storage import PAGE, SequenceCache
from ..parts.linear import Workspace


class StepError(ValueError):
    pass


class PositionPastLimit(StepError):
    """A step would place a token at a position the model's configuration does not allow."""


@dataclass
class Entry:
    """One sequence's share of a step: its slot, its next tokens, and the places
    among these tokens whose logits are wanted."""
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class GroupTables:
    block_table: torch.Tensor    # int32 [B, max_blocks]: pages of each sequence, in order
    dest: torch.Tensor           # int32 [nt]: page * PAGE + offset where each new token is stored
    # steps of single tokens: what the planners of the group's mixers worked out on the host,
    # {planner: {name: int32 tensor}}; empty otherwise. A planner is any hashable object with
    #   ints(batch) -> int32 values its tables hold for a step of ``batch`` single tokens (a
    #       function of the batch size alone, so that a recorded step keeps its buffers), and
    #   tables(kv_lens, block_table) -> {name: int32 numpy array} from the sequences' lengths
    #       with this step's token and the group's page table (numpy, [batch, width]);
    # a mixer offers its planner as ``step_planner()`` and reads ``plans.get(planner)``.
    plans: Dict[object, Dict[str, torch.Tensor]] = field(default_factory=dict)


class Uploader:
    """Pinned staging buffers used in turn; a buffer is reused only after the copy
    that read it has finished."""

    def __init__(self, device, depth: int = 4):
        self.device = torch.device(device)
        self.depth = depth
        self._host: List[Optional[torch.Tensor]] = [None] * depth
        self._events: List[Optional[torch.cuda.Event]] = [None] * depth
        self._dev: List[Optional[torch.Tensor]] = [None] * depth
        self._turn = 0

    def upload(self, arr: np.ndarray, into: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Copies ``arr`` to the device: into this uploader's own buffer of the turn,
        or into ``into`` (a fixed device buffer that a captured graph reads)."""
        i = self._turn
        self._turn = (i + 1) % self.depth
        n = int(arr.size)
        if self._events[i] is not None:
            self._events[i].synchronize()
        if self._host[i] is None or self._host[i].numel() < n:
            cap = max(1024, 1 << (n - 1).bit_length())
            self._host[i] = torch.empty(cap, dtype=torch.int32, pin_memory=True)
            self._dev[i] = torch.empty(cap, dtype=torch.int32, device=self.device)
        self._host[i][:n].numpy()[:] = arr
        dst = self._dev[i][:n] if into is None else into[:n]
        dst.copy_(self._host[i][:n], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._events[i] = ev
        return dst


class StepContext:
    """Built by ``plan_step``; handed to every part of the model."""

    def __init__(self):
        self.nt = 0
        self.batch = 0
        self.max_qlen = 0
        self.max_kv_len = 0
        self.all_single = False
        self.slots_host: List[int] = []
        self.seq_lens: List[int] = []
        self.tokens = self.positions = self.cu_q = self.pos0 = self.slots = None
        self.want_rows: Optional[torch.Tensor] = None
        self.n_want = 0
        self.kv: List[GroupTables] = []
        self.ws: Optional[Workspace] = None
        self.shared = {}     # what parts compute once per step and share (cleared by every run)
        self.timers = None   # parts.base.PartTimers while the model collects times per kind of part
        self.real_batch = 0  # sequences of the caller; the rest of ``batch`` only fills a launch shape
        self.real_want = 0


def check_entries(entries: Sequence[Entry], vocab: int) -> None:
    if not entries:
        raise StepError("a step needs at least one sequence")
    seen = set()
    for e in entries:
        if e.slot in seen:
            raise StepError(f"slot {e.slot} appears twice in one step")
        seen.add(e.slot)
        n = len(e.tokens)
        if n == 0:
            raise StepError(f"slot {e.slot}: a step needs at least one token per sequence")
        if n > 16:                       # a prompt: one pass in numpy instead of a loop over its tokens
            arr = np.asarray(e.tokens)
            if arr.dtype.kind not in "iu":
                arr = np.asarray([int(t) for t in e.tokens])
            bad = (arr < 0) | (arr >= vocab)
            if bad.any():
                raise StepError(f"slot {e.slot}: token {int(arr[int(np.argmax(bad))])} is outside "
                                f"the vocabulary [0, {vocab})")
        else:
            for t in e.tokens:
                if not 0 <= int(t) < vocab:
                    raise StepError(f"slot {e.slot}: token {t} is outside the vocabulary [0, {vocab})")
        last = -1
        for w in e.want:
            if not 0 <= int(w) < n:
                raise StepError(f"slot {e.slot}: wanted place {w} is outside its {n} tokens")
            if int(w) <= last:
                raise StepError(f"slot {e.slot}: wanted places must ascend without repeats")
            last = int(w)


def layout_step(entries: Sequence[Entry], lengths: Sequence[int], pages: Sequence[Sequence[Sequence[int]]],
                table_width: int = 0, planners: Optional[Sequence[Sequence[object]]] = None):
    """Pure host part: the integer tables of a step.

    lengths[i]: tokens already cached for entry i. pages[g][i]: pages that entry i
    holds in group g (enough for lengths[i] + len(tokens)); a negative entry is a page that
    was given back because no layer of the group reads it any more, and its place in the
    table reads 0. table_width: the page
    tables get at least this many columns (a captured graph wants a fixed width).
    planners[g]: the planners of group g (see ``GroupTables.plans``), asked when every
    sequence brings one token; their tables are packed as "plan{g}.{k}.{name}".
    Returns (packed int32 array, offsets dict, summary dict).
    """
    B = len(entries)
    seq = [len(e.tokens) for e in entries]
    nt = sum(seq)
    if nt == B:
        tokens = np.fromiter((int(e.tokens[0]) for e in entries), dtype=np.int32, count=nt)
    else:
        tokens = np.concatenate([np.asarray(e.tokens, dtype=np.int64).astype(np.int32) for e in entries])
    positions = np.concatenate([np.arange(l, l + n, dtype=np.int32) for l, n in zip(lengths, seq)])
    cu = np.zeros(B + 1, dtype=np.int32)
    cu[1:] = np.cumsum(seq)
    pos0 = np.asarray(lengths, dtype=np.int32)
    slots = np.asarray([e.slot for e in entries], dtype=np.int32)
    want = np.asarray([cu[i] + int(w) for i, e in enumerate(entries) for w in e.want],
                      dtype=np.int32)
    parts = [tokens, positions, cu, pos0, slots, want]
    names = ["tokens", "positions", "cu_q", "pos0", "slots", "want"]
    shapes = {}
    for g, group_pages in enumerate(pages):
        need = [-(-(l + n) // PAGE) for l, n in zip(lengths, seq)]
        max_blocks = max(max(need), table_width)
        table = np.zeros((B, max_blocks), dtype=np.int32)
        dest = np.empty(nt, dtype=np.int32)
        for i in range(B):
            pg = np.asarray(group_pages[i][:need[i]], dtype=np.int32)
            if len(pg) < need[i]:
                raise StepError(f"entry {i} holds {len(pg)} pages, needs {need[i]}")
            table[i, :need[i]] = np.maximum(pg, 0)
            p = positions[cu[i]:cu[i + 1]]
            if (pg[p // PAGE] < 0).any():
                raise StepError(f"entry {i} would store into a page that it has given back")
            dest[cu[i]:cu[i + 1]] = pg[p // PAGE] * PAGE + p % PAGE
        parts += [table.reshape(-1), dest]
        names += [f"table{g}", f"dest{g}"]
        shapes[f"table{g}"] = (B, max_blocks)
        if planners is not None and max(seq) == 1:
            for k, planner in enumerate(planners[g]):
                for nme, arr in planner.tables([l + 1 for l in lengths], table).items():
                    arr = np.ascontiguousarray(arr, dtype=np.int32)
                    parts.append(arr.reshape(-1))
                    names.append(f"plan{g}.{k}.{nme}")
                    shapes[names[-1]] = tuple(arr.shape)
    offsets, off = {}, 0
    for nme, a in zip(names, parts):
        offsets[nme] = (off, off + a.size)
        off += a.size
    packed = np.concatenate(parts) if parts else np.zeros(0, dtype=np.int32)
    summary = dict(nt=nt, batch=B, seq=seq, max_qlen=max(seq),
                   max_kv_len=max(l + n for l, n in zip(lengths, seq)), shapes=shapes)
    return packed, offsets, summary


def table_ints(batch: int, n_want: int, table_width: int, cache: SequenceCache) -> int:
    """int32 values that the tables of a step of ``batch`` single tokens hold together."""
    n = 5 * batch + 1 + n_want
    for g in range(len(cache.kv_groups)):
        n += batch * table_width + batch + sum(p.ints(batch) for p in cache.group_planners[g])
    return n


def check_positions(entries: Sequence[Entry], lengths: Sequence[int], max_position: Optional[int]) -> None:
    """Positions run from 0 to max_position - 1 (the configuration's context length, nctx of
    models/llama/common/src/lib.rs:27): a step that would go past it is refused whole."""
    if max_position is None:
        return
    for e, l in zip(entries, lengths):
        if l + len(e.tokens) > max_position:
            raise PositionPastLimit(f"slot {e.slot}: {l} cached + {len(e.tokens)} new tokens reach "
                                    f"position {l + len(e.tokens) - 1}, the model allows positions "
                                    f"below {max_position} (max_position_embeddings)")


def plan_step(entries: Sequence[Entry], cache: SequenceCache, vocab: int, uploader: Uploader,
              ws: Workspace, table_width: int = 0, into: Optional[torch.Tensor] = None,
              max_position: Optional[int] = None, pad_to: int = 0) -> StepContext:
    """Checks the entries, reserves cache pages (raising before anything runs when
    they do not fit) and uploads the step's tables.

    pad_to: a step of single tokens is filled up to this many sequences with rows that
    belong to nobody (token 0 at position 0, stored into the cache's spare page, their slot
    the spare row of every table of fixed-size state), so that
    steps of several batch sizes share one recorded launch shape; when every sequence wants
    its logits, the filling rows are wanted too and the caller drops their logits."""
    check_entries(entries, vocab)
    check_positions(entries, [cache.pool.length(e.slot) for e in entries], max_position)
    cache.pool.reserve({e.slot: len(e.tokens) for e in entries})
    lengths = [cache.pool.length(e.slot) for e in entries]
    pages = [[cache.pool.pages(e.slot, g) for e in entries] for g in range(len(cache.kv_groups))]
    real_batch, real_want = len(entries), sum(len(e.want) for e in entries)
    if pad_to > len(entries):
        if any(len(e.tokens) != 1 for e in entries):
            raise StepError("only steps of single tokens are filled up")
        all_wanted = all(len(e.want) == 1 for e in entries)
        fill = pad_to - len(entries)
        entries = list(entries) + [Entry(cache.spare_slot, (0,), (0,) if all_wanted else ())] * fill
        lengths = lengths + [0] * fill
        pages = [pg + [[cache.spare_page[g]]] * fill for g, pg in enumerate(pages)]
    packed, off, s = layout_step(entries, lengths, pages, table_width, cache.group_planners)
    if into is not None and into.numel() < packed.size:
        raise StepError("the fixed table buffer is too small for this step")
    dev = uploader.upload(packed, into)
    ctx = StepContext()
    ctx.nt, ctx.batch, ctx.seq_lens = s["nt"], s["batch"], s["seq"]
    ctx.max_qlen, ctx.max_kv_len = s["max_qlen"], s["max_kv_len"]
    ctx.all_single = s["max_qlen"] == 1
    ctx.slots_host = [e.slot for e in entries]
    ctx.real_batch, ctx.real_want = real_batch, real_want

    def view(name):
        a, b = off[name]
        return dev[a:b]

    ctx.tokens, ctx.positions = view("tokens"), view("positions")
    ctx.cu_q, ctx.pos0, ctx.slots = view("cu_q"), view("pos0"), view("slots")
    ctx.want_rows = view("want")
    ctx.n_want = ctx.want_rows.numel()
    for g in range(len(cache.kv_groups)):
        tables = GroupTables(view(f"table{g}").view(*s["shapes"][f"table{g}"]), view(f"dest{g}"))
        for k, planner in enumerate(cache.group_planners[g]):
            pre = f"plan{g}.{k}."
            found = {n[len(pre):]: view(n).view(*s["shapes"][n]) for n in off if n.startswith(pre)}
            if found:
                tables.plans[planner] = found
        ctx.kv.append(tables)
    ctx.ws = ws
    return ctx
