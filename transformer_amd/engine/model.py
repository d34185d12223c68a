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
from ..parts.base import build_part, span
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
        self.after_embed = build_part(spec.after_embed, self.dtype, self.device) \
            if spec.after_embed is not None else None
        self.on_logits = build_part(spec.on_logits, self.dtype, self.device) \
            if spec.on_logits is not None else None
        # dump(name, tensor): called with the step's intermediate tensors when set (the
        # reference's Operators::debug, models/llama/common/src/compute.rs:31-33); steps
        # run eagerly while it is set
        self.dump = None
        # timers: a ``parts.base.PartTimers`` collects GPU time per kind of part while set;
        # steps run eagerly meanwhile
        self.timers = None
        # cache layers: a schedule entry owns one per need of its block (none, one, or, where
        # the block names several needs in a list, a tuple of them in that order)
        self.cache_layer: List[object] = []
        self.cache_needs: List[object] = []
        self.cache_planners: List[object] = []
        for i, run in enumerate(spec.schedule):
            block = self.blocks[run.block]
            need = block.cache_need()
            if need is None or (isinstance(need, (list, tuple)) and not need):
                self.cache_layer.append(None)
            elif run.cache_of is None:
                several = isinstance(need, (list, tuple))
                planner = getattr(block, "step_planner", lambda: None)()
                layers = []
                for one in (need if several else [need]):
                    layers.append(len(self.cache_needs))
                    self.cache_needs.append(one)
                    self.cache_planners.append(planner)
                self.cache_layer.append(tuple(layers) if several else layers[0])
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
        self._graph_safe = all(getattr(b, "graph_safe", False) for b in
                               [*self.blocks, *self._extras().values()])

    def _extras(self):
        return {n: p for n, p in (("after_embed", self.after_embed), ("on_logits", self.on_logits))
                if p is not None}

    # ------------------------------------------------------------------ parameters
    def all_params(self) -> Dict[str, Param]:
        s = self.spec
        out = {"embed.weight": Param((s.vocab, s.hidden), "matrix")}
        for i, b in enumerate(self.blocks):
            out.update(b.all_params(f"blocks.{i}."))
        out.update(self.final_norm.all_params("final_norm."))
        for n, p in self._extras().items():
            out.update(p.all_params(n + "."))
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
        for n, p in self._extras().items():
            p.bind_all(tensors, n + ".")
        for n in ("embed.weight", "head.weight"):
            if tuple(tensors[n].shape) != tuple(want[n].shape):
                raise ValueError(f"parameter {n} has shape {tuple(tensors[n].shape)}, "
                                 f"expected {tuple(want[n].shape)}")
        self.w = {"embed": tensors["embed.weight"], "head": tensors["head.weight"]}
        self.tensors = {n: tensors[n] for n in want}     # every parameter by its declared name

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

        for b in [*self.blocks, self.final_norm, *self._extras().values()]:
            visit(b)
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
                             max_step_tokens, planners=self.cache_planners)

    # ------------------------------------------------------------------ the step
    def _forward(self, ctx, cache: SequenceCache) -> torch.Tensor:
        """Everything a step does on the GPU, given its uploaded tables."""
        s = self.spec
        ctx.shared.clear()
        ctx.timers = self.timers
        with span(ctx, "embed"):
            x = kernels.embed(self.w["embed"], ctx.tokens,
                              self.ws.take("model.x", (ctx.nt, s.hidden), torch.float32))
            if self.after_embed is not None:
                self.after_embed.run(x, ctx)
        if self.dump is not None:
            self.dump("embed", x)
        pending = (None, None)
        for i, run in enumerate(s.schedule):
            block = self.blocks[run.block]
            kw = {}
            if getattr(block, "folds_norms", False) and i + 1 < len(s.schedule):
                kw["after"] = self.blocks[s.schedule[i + 1].block]    # it may prepare that block's norm
            pending = block.run(x, pending, ctx, cache, self.cache_layer[i],
                                writes_cache=run.cache_of is None, **kw)
            if self.dump is not None:
                self.dump(f"run.{i}", self._stream_with(x, pending))
        logits = self.ws.take("model.logits", (ctx.n_want, s.vocab), torch.float32)
        if ctx.n_want:
            hn = self.ws.take("model.hn", (ctx.n_want, s.hidden), self.dtype)
            with span(ctx, "norm"):
                self.final_norm.run(x, hn, pending[0], pending[1], rows=ctx.want_rows)
            if self.dump is not None:
                self.dump("final_norm", hn)
            with span(ctx, "head"):
                linear(hn, self.w["head"], logits)
                if self.on_logits is not None:
                    self.on_logits.run(logits, ctx)
        if self.dump is not None:
            self.dump("logits", logits)
        return logits

    @staticmethod
    def _stream_with(x, pending) -> torch.Tensor:
        """The residual stream with what a block has left to be added (debugging only: the
        engine itself lets the next norm do the add)."""
        if isinstance(pending, kernels.RowScale):
            return x.clone()                      # the block's last product has added itself
        delta, bias = pending
        full = x.clone()
        if delta is not None:
            full += delta.float().sum(0) if delta.dim() == 3 else delta.float()
        if bias is not None:
            full += bias
        return full

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
            logits = None
            if self.use_graphs and self._graph_safe and self.dump is None and self.timers is None and \
                    all(len(e.tokens) == 1 for e in entries):
                logits = self._step_graph(cache, entries, device_tokens)   # None: this shape runs eagerly
            if logits is None:
                ctx = plan_step(entries, cache, self.spec.vocab, self.uploader, self.ws,
                                max_position=self.spec.max_position)
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
    # recorded again only when the longest sequence grows past a multiple of it (4,096 tokens;
    # recording costs an eager step and the capture, about three steps' time: with tables of 16
    # pages a run of 50 steps at batch 64 whose longest sequence crossed 2,048 tokens measured
    # 6.5 ms per step where the steps themselves take 6.06)
    GRAPH_TABLE_STEP = 64
    MAX_GRAPHS = 24
    check_recordings = True     # replay every new recording twice against its eager step
    # batch sizes that steps are recorded at; a step of another size is filled up to the
    # next of them with rows that belong to nobody, so a batch that shrinks sequence by
    # sequence records a dozen graphs and not one per size. The sizes sit at the row counts
    # where the products change kernels (8, 16, 32, 64).
    GRAPH_BATCHES = (1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64)

    @classmethod
    def graph_batch(cls, n: int) -> int:
        for b in cls.GRAPH_BATCHES:
            if n <= b:
                return b
        return -(-n // 32) * 32

    def _step_graph(self, cache: SequenceCache, entries: Sequence[Entry],
                    device_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        need = max(-(-(cache.pool.length(e.slot) + 1) // kernels.PAGE) for e in entries)
        width = -(-need // self.GRAPH_TABLE_STEP) * self.GRAPH_TABLE_STEP
        n, n_want = len(entries), sum(len(e.want) for e in entries)
        batch = self.graph_batch(n)
        if n_want == n:
            want_rows = batch                        # the filling rows are wanted too
        elif batch == n:
            want_rows = n_want
        else:
            batch, want_rows = n, n_want             # some sequences want nothing: recorded as it is
        graphs = cache.graphs
        if cache.graph_owner is None:
            cache.graph_owner = self
        if cache.graph_owner is not self:
            raise RuntimeError("a cache is stepped by the model that made it")
        if (batch, want_rows) in cache.graphs_failed:    # its recording replayed wrongly once
            return None
        key = (batch, want_rows, width)
        rec = graphs.get(key)
        stamp = (self.ws.generation, kernels.scratch_generation())
        if rec is not None and rec[4] != stamp:      # a buffer the graph points at has moved
            graphs.clear()
            rec = None
        if rec is None:
            ints = torch.empty(table_ints(batch, want_rows, width, cache), dtype=torch.int32,
                               device=self.device)
            ctx = plan_step(entries, cache, self.spec.vocab, self.uploader, self.ws, width, ints,
                            self.spec.max_position, pad_to=batch)
            ctx.max_kv_len = width * kernels.PAGE       # launch shapes must not follow the lengths
            if device_tokens is not None:
                ctx.tokens[:n].copy_(device_tokens.reshape(-1))
            check = self.check_recordings and n_want > 0 and (batch, want_rows) not in cache.graphs_checked
            # keys and values are written to the same effect however often a step runs;
            # fixed-size state is not, so a recording that is tried starts from what the
            # state was before the step every time
            before = [t.clone() for t in cache.states] if check else []
            logits = self._forward(ctx, cache)          # this step's result; also warms every buffer
            torch.cuda.synchronize(self.device)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                captured = self._forward(ctx, cache)
            if captured.data_ptr() != logits.data_ptr():
                raise RuntimeError("scratch memory moved while the step was recorded")
            if len(graphs) >= self.MAX_GRAPHS:
                graphs.pop(next(iter(graphs)))
            stamp = (self.ws.generation, kernels.scratch_generation())
            # The recording is tried before it is trusted: replayed twice on the same inputs (a
            # step writes the same keys and values again, nothing accumulates), each replay has
            # to give the eager step's logits. A library product inside the graph may clear its
            # workspace through a recorded memset, and such nodes have gone wrong from the second
            # replay on; a shape that fails runs eagerly from then on, whatever becomes of the
            # recorded graphs (they are dropped when a buffer moves and when too many are kept).
            if check:
                cache.graphs_checked.add((batch, want_rows))     # a wider table changes no kernel
                eager = logits[:n_want].clone()
                bound = 1e-3 * (1.0 + float(eager.abs().max()))
                for replay in range(2):
                    for t, b in zip(cache.states, before):
                        t.copy_(b)
                    graph.replay()
                    if not float((logits[:n_want] - eager).abs().max()) <= bound:    # also false for NaN
                        import warnings
                        warnings.warn(f"a recorded step of {batch} sequences differs from the eager step on "
                                      f"replay {replay + 1}: steps of this shape run eagerly", stacklevel=3)
                        cache.graphs_failed.add((batch, want_rows))
                        # the bad replay has written this step's keys, values and states last:
                        # the eager step writes all of them, and the logits, again
                        for t, b in zip(cache.states, before):
                            t.copy_(b)
                        return self._forward(ctx, cache)[:n_want]
            graphs[key] = (graph, ints, ctx, captured, stamp)
            return logits[:n_want]
        graph, ints, ctx, logits, _ = rec
        new = plan_step(entries, cache, self.spec.vocab, self.uploader, self.ws, width, ints,
                        self.spec.max_position, pad_to=batch)
        if new.nt != ctx.nt or new.n_want != ctx.n_want or \
                [t.block_table.shape for t in new.kv] != [t.block_table.shape for t in ctx.kv]:
            raise RuntimeError("a recorded step was replayed with other shapes")
        if device_tokens is not None:
            new.tokens[:n].copy_(device_tokens.reshape(-1))
        graph.replay()
        return logits[:n_want]
