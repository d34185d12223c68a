"""The decoder as the engine sees it: an embedding table, blocks run in the
order of a schedule, a final norm, an output matrix, and ONE step function.

``step`` is the reference's ``LlamaWorker::launch``
(/root/reference/models/llama/common/src/compute.rs:139-366) with the embedding
gather (/root/reference/models/llama/cuda/src/infer.rs:98-104), the position
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
from .batch import Entry, Uploader, plan_step
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
    def new_cache(self, max_tokens: int, max_slots: Optional[int] = None) -> SequenceCache:
        """A cache for sequences that together hold at most ``max_tokens`` tokens
        (each rounded up to pages of 64)."""
        pages = -(-max_tokens // kernels.PAGE)
        if max_slots is None:
            max_slots = max(1, min(pages, 1024))
        return SequenceCache(self.cache_needs, max_tokens, max_slots, self.dtype, self.device)

    # ------------------------------------------------------------------ the step
    def step(self, cache: SequenceCache, entries: Sequence[Entry]) -> torch.Tensor:
        """Runs the entries' tokens as one batch. Returns float32 logits
        [wanted places, vocab]; the tensor is scratch that the next step reuses."""
        if not self.w:
            raise RuntimeError("the model has no weights bound")
        s = self.spec
        with torch.cuda.device(self.device):
            ctx = plan_step(entries, cache, s.vocab, self.uploader, self.ws)
            x = kernels.embed(self.w["embed"], ctx.tokens,
                              self.ws.take("model.x", (ctx.nt, s.hidden), torch.float32))
            pending = (None, None)
            for i, run in enumerate(s.schedule):
                pending = self.blocks[run.block].run(x, pending, ctx, cache, self.cache_layer[i],
                                                     writes_cache=run.cache_of is None)
            logits = self.ws.take("model.logits", (ctx.n_want, s.vocab), torch.float32)
            if ctx.n_want:
                hn = self.ws.take("model.hn", (ctx.n_want, s.hidden), self.dtype)
                self.final_norm.run(x, hn, pending[0], pending[1], rows=ctx.want_rows)
                linear(hn, self.w["head"], logits)
            for e in entries:
                cache.pool.advance(e.slot, len(e.tokens))
        return logits
