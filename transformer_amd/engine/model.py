"""The decoder as the engine sees it: an embedding table, blocks run in the
order of a schedule, a final norm, an output matrix, and ONE step function.

``step`` is the reference's ``LlamaWorker::launch``
(models/llama/common/src/compute.rs:139-366) with the embedding
gather (models/llama/cuda/src/infer.rs:98-104), the position
build and the cache handling taken inside: it runs exactly the tokens it is
given, as one batch, against what earlier steps left in the cache, and returns
float32 logits at the wanted places, in the order of the entries and of their
``want`` lists (compute.rs:341-356 packs the rows of the requests in that order).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from .. import kernels
from ..cache.storage import SequenceCache
from ..config.spec import ModelSpec
from ..parts.base import build_part
from ..parts.linear import Workspace, linear
from ..weights.loader import Param
from .batch import Entry, Uploader, plan_step, table_ints
from .params import declared_params  # noqa: F401

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16,
           "fp32": torch.float32, "bf16": torch.bfloat16}


def engine_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.float32, torch.bfloat16):
            raise ValueError(f"the engine computes in float32 or bfloat16, not {name}")
        return name
    try:
        return _DTYPES[str(name)]
    except KeyError:
        raise ValueError(f"dtype must be one of {sorted(_DTYPES)}, got {name!r}") from None


class DecoderModel:
    def __init__(self, spec: ModelSpec, dtype, device="cuda:0"):
        spec.validate()
        self.spec = spec
        self.dtype = engine_dtype(dtype)
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError(f"the engine runs on the GPU only; device {self.device} was asked for")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible to torch; the engine has no CPU path")
        kernels.library()          # fail now, not at the first step, if the kernels are missing
        self.blocks = [build_part(b, self.dtype, self.device) for b in spec.blocks]
        self.final_norm = build_part(spec.final_norm, self.dtype, self.device)
        # cache layers: one per schedule entry that owns one
        self.cache_layer: List[Optional[int]] = []
        self.cache_needs: List[object] = []
        for i, run in enumerate(spec.schedule):
            need = self.blocks[run.block].cache_need()
            if need is None:
                self.cache_layer.append(None)
            elif run.cache_of is None:
                self.cache_layer.append(len(self.cache_needs))
                self.cache_needs.append(need)
            else:
                lender = spec.schedule[run.cache_of]
                if self.blocks[lender.block].cache_need() != need:
                    raise ValueError(f"schedule[{i}] borrows the cache of entry {run.cache_of}, "
                                     f"whose layout differs")
                self.cache_layer.append(self.cache_layer[run.cache_of])
        self.w: Dict[str, torch.Tensor] = {}
        self.ws = Workspace(self.device)
        self.uploader = Uploader(self.device)
        # single-token steps are replayed from recorded HIP graphs when every block
        # says that its work is a fixed sequence of kernels on fixed buffers
        self.use_graphs = True
        self._graph_safe = all(getattr(b, "graph_safe", False) for b in self.blocks)

    # ------------------------------------------------------------------ parameters
    def all_params(self) -> Dict[str, Param]:
        s = self.spec
        out = {"embed.weight": Param((s.vocab, s.hidden), "matrix")}
        for i, b in enumerate(self.blocks):
            out.update(b.all_params(f"blocks.{i}."))
        out.update(self.final_norm.all_params("final_norm."))
        out["head.weight"] = Param((s.vocab, s.hidden), "matrix")
        return out

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        want = self.all_params()
        missing = sorted(set(want) - set(tensors))
        if missing:
            raise ValueError(f"parameters not given: {', '.join(missing)}")
        for i, b in enumerate(self.blocks):
            b.bind_all(tensors, f"blocks.{i}.")
        self.final_norm.bind_all(tensors, "final_norm.")
        for n in ("embed.weight", "head.weight"):
            if tuple(tensors[n].shape) != tuple(want[n].shape):
                raise ValueError(f"parameter {n} has shape {tuple(tensors[n].shape)}, "
                                 f"expected {tuple(want[n].shape)}")
        self.w = {"embed": tensors["embed.weight"], "head": tensors["head.weight"]}

    def weight_bytes(self) -> int:
        """Bytes of every distinct parameter tensor (a shared table counts once)."""
        seen, total = set(), 0

        def visit(part):
            nonlocal total
            for t in getattr(part, "w", {}).values():
                if t.data_ptr() not in seen:
                    seen.add(t.data_ptr())
                    total += t.numel() * t.element_size()
            for c in part.children().values():
                visit(c)

        for b in self.blocks:
            visit(b)
        visit(self.final_norm)
        for t in self.w.values():
            if t.data_ptr() not in seen:
                seen.add(t.data_ptr())
                total += t.numel() * t.element_size()
        return total

    # ------------------------------------------------------------------ cache
    def new_cache(self, max_tokens: int, max_slots: Optional[int] = None,
                  max_step_tokens: Optional[int] = None) -> SequenceCache:
        """A cache for sequences that together hold at most ``max_tokens`` tokens
        (each rounded up to pages of 64). ``max_step_tokens``: a promise that no step brings
        more tokens than this; layers that read a window then get less storage."""
        pages = -(-max_tokens // kernels.PAGE)
        if max_slots is None:
            max_slots = max(1, min(pages, 1024))
        return SequenceCache(self.cache_needs, max_tokens, max_slots, self.dtype, self.device,
                             max_step_tokens)

    # ------------------------------------------------------------------ the step
    def _forward(self, ctx, cache: SequenceCache) -> torch.Tensor:
        """Everything a step does on the GPU, given its uploaded tables."""
        s = self.spec
        ctx.shared.clear()
        x = kernels.embed(self.w["embed"], ctx.tokens,
                          self.ws.take("model.x", (ctx.nt, s.hidden), torch.float32))
        pending = (None, None)
        for i, run in enumerate(s.schedule):
            block = self.blocks[run.block]
            kw = {}
            if getattr(block, "folds_norms", False) and i + 1 < len(s.schedule):
                kw["after"] = self.blocks[s.schedule[i + 1].block]    # it may prepare that block's norm
            pending = block.run(x, pending, ctx, cache, self.cache_layer[i],
                                writes_cache=run.cache_of is None, **kw)
        logits = self.ws.take("model.logits", (ctx.n_want, s.vocab), torch.float32)
        if ctx.n_want:
            hn = self.ws.take("model.hn", (ctx.n_want, s.hidden), self.dtype)
            self.final_norm.run(x, hn, pending[0], pending[1], rows=ctx.want_rows)
            linear(hn, self.w["head"], logits)
        return logits

    def step(self, cache: SequenceCache, entries: Sequence[Entry],
             device_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Runs the entries' tokens as one batch. Returns float32 logits
        [wanted places, vocab]; the tensor is scratch that the next step reuses.

        device_tokens (int32 on the GPU, one per token of the step, in the entries'
        order) replaces the token values of the entries, whose count alone is used then:
        a caller that chose the tokens on the GPU can start the next step without first
        bringing them to the host.

        A step in which every sequence brings one token is the launch-bound inner
        loop of generation: its kernels are recorded once into a HIP graph per
        (batch size, wanted rows, page-table width) and replayed afterwards; only
        the integer tables change between replays."""
        if not self.w:
            raise RuntimeError("the model has no weights bound")
        with torch.cuda.device(self.device):
            if device_tokens is not None:
                nt = sum(len(e.tokens) for e in entries)
                if device_tokens.dtype != torch.int32 or device_tokens.device != self.device or \
                        device_tokens.numel() != nt:
                    raise ValueError(f"device_tokens must be {nt} int32 values on {self.device}")
            if self.use_graphs and self._graph_safe and all(len(e.tokens) == 1 for e in entries):
                logits = self._step_graph(cache, entries, device_tokens)
            else:
                ctx = plan_step(entries, cache, self.spec.vocab, self.uploader, self.ws)
                if device_tokens is not None:
                    ctx.tokens.copy_(device_tokens.reshape(-1))
                logits = self._forward(ctx, cache)
            for e in entries:
                cache.pool.advance(e.slot, len(e.tokens))
                # later steps run after this one on the same stream, so a page that is given
                # back here is not written before this step has read it
                cache.release_outside_windows(e.slot)
        return logits

    # a page table of a graph is this many pages wide, rounded up: the graph is
    # recorded again only when the longest sequence grows past a multiple of it
    GRAPH_TABLE_STEP = 16
    MAX_GRAPHS = 12

    def _step_graph(self, cache: SequenceCache, entries: Sequence[Entry],
                    device_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        need = max(-(-(cache.pool.length(e.slot) + 1) // kernels.PAGE) for e in entries)
        width = -(-need // self.GRAPH_TABLE_STEP) * self.GRAPH_TABLE_STEP
        n_want = sum(len(e.want) for e in entries)
        graphs = cache.__dict__.setdefault("_graphs", {})
        if cache.__dict__.setdefault("_graph_owner", self) is not self:
            raise RuntimeError("a cache is stepped by the model that made it")
        key = (len(entries), n_want, width)
        rec = graphs.get(key)
        stamp = (self.ws.generation, kernels.scratch_generation())
        if rec is not None and rec[4] != stamp:      # a buffer the graph points at has moved
            graphs.clear()
            rec = None
        if rec is None:
            ints = torch.empty(table_ints(len(entries), n_want, width, cache), dtype=torch.int32,
                               device=self.device)
            ctx = plan_step(entries, cache, self.spec.vocab, self.uploader, self.ws, width, ints)
            ctx.max_kv_len = width * kernels.PAGE       # launch shapes must not follow the lengths
            if device_tokens is not None:
                ctx.tokens.copy_(device_tokens.reshape(-1))
            logits = self._forward(ctx, cache)          # this step's result; also warms every buffer
            torch.cuda.synchronize(self.device)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                captured = self._forward(ctx, cache)
            if captured.data_ptr() != logits.data_ptr():
                raise RuntimeError("scratch memory moved while the step was recorded")
            if len(graphs) >= self.MAX_GRAPHS:
                graphs.pop(next(iter(graphs)))
            graphs[key] = (graph, ints, ctx, captured, (self.ws.generation, kernels.scratch_generation()))
            return logits
        graph, ints, ctx, logits, _ = rec
        new = plan_step(entries, cache, self.spec.vocab, self.uploader, self.ws, width, ints)
        if new.nt != ctx.nt or new.n_want != ctx.n_want or \
                [t.block_table.shape for t in new.kv] != [t.block_table.shape for t in ctx.kv]:
            raise RuntimeError("a recorded step was replayed with other shapes")
        if device_tokens is not None:
            new.tokens.copy_(device_tokens.reshape(-1))
        graph.replay()
        return logits
