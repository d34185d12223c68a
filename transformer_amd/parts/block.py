"""Arrangement of parts in a block.

"prenorm": x += mixer(norm1(x)); x += ffn(norm2(x)), the reference's block
(models/llama/common/src/compute.rs:204-292). The adds are
carried as a pending (delta, bias) pair and folded into the next norm, so the
float32 residual stream is read and written once per norm.
"""
from __future__ import annotations

import torch

from .. import kernels
from .base import Part, build_part, register_part, span


class PreNormBlock(Part):
    def __init__(self, spec, dtype, device):
        self.dtype = dtype
        self.norm1 = build_part(spec.norm1, dtype, device)
        self.mixer = build_part(spec.mixer, dtype, device)
        self.norm2 = build_part(spec.norm2, dtype, device)
        self.ffn = build_part(spec.ffn, dtype, device)

    def children(self):
        return {"norm1": self.norm1, "mixer": self.mixer, "norm2": self.norm2, "ffn": self.ffn}

    def cache_need(self):
        return self.mixer.cache_need()

    def step_planner(self):
        """What the mixer wants planned on the host for steps of single tokens, or None."""
        f = getattr(self.mixer, "step_planner", None)
        return f() if f is not None else None

    @property
    def graph_safe(self) -> bool:
        """True when a step of this block is a fixed sequence of kernel launches on
        fixed buffers (no host decisions that depend on the data)."""
        return all(getattr(p, "graph_safe", False) for p in (self.norm1, self.mixer, self.norm2, self.ffn))

    # Single-token steps of a bfloat16 engine: a few-rows product in front of a norm adds to the
    # residual stream and prepares the norm itself, and the product behind it applies the
    # rows' factors, so the norm needs no kernel of its own. Both neighbours have to offer
    # it (``can_fold`` / ``takes_scaled``); any other part gets the norm's own kernel.
    folds_norms = True

    def _fusable(self, nt: int) -> bool:
        return self.dtype == torch.bfloat16 and 0 < nt <= kernels.SKINNY_MAX_ROWS

    @staticmethod
    def _offers(part, what: str, nt: int) -> bool:
        f = getattr(part, what, None)
        return f is not None and bool(f(nt))

    def entry_fold(self, x, ctx):
        """What the last product of the block in front needs to take over norm1, or None."""
        if not (self._fusable(x.shape[0]) and self._offers(self.mixer, "takes_scaled", x.shape[0])
                and hasattr(self.norm1, "fold")):
            return None
        return self.norm1.fold(x, ctx.ws.take("block.h", x.shape, self.dtype), ctx)

    def run(self, x, pending, ctx, cache, layer, writes_cache=True, after=None):
        """x: float32 residual stream [nt, hidden]; pending: (delta, bias) not yet added to
        x, (None, None), or the ``RowScale`` of an ``entry_fold`` that the block in front has
        served. after: the block that runs next, if any. Returns the new pending."""
        nt = x.shape[0]
        h = ctx.ws.take("block.h", x.shape, self.dtype)
        kw = {}
        if isinstance(pending, kernels.RowScale):
            kw["scale"] = pending                  # h already holds the rows, not yet scaled
        else:
            with span(ctx, "norm"):
                self.norm1.run(x, h, pending[0], pending[1])
        fusable = self._fusable(nt)
        if (fusable and hasattr(self.norm2, "fold") and self._offers(self.mixer, "can_fold", nt)
                and self._offers(self.ffn, "takes_scaled", nt)):
            kw["fold"] = self.norm2.fold(x, h, ctx)
        # with many rows a part whose last product can add itself to the stream is given it
        # (``can_add`` / ``into``); it returns no delta then, and the next norm only reads
        if "fold" not in kw and self._offers(self.mixer, "can_add", nt):
            kw["into"] = x
        with span(ctx, "mixer"):
            pending = self.mixer.run(h, ctx, cache, layer, writes_cache, **kw)
        kw2 = {}
        if "fold" in kw:
            kw2["scale"] = kw["fold"].scale()
        else:
            with span(ctx, "norm"):
                self.norm2.run(x, h, pending[0], pending[1])
        handover = None
        if fusable and after is not None and self._offers(self.ffn, "can_fold", nt):
            entry = getattr(after, "entry_fold", None)
            handover = entry(x, ctx) if entry is not None else None
        if handover is not None:
            with span(ctx, "ffn"):
                self.ffn.run(h, ctx, fold=handover, **kw2)
            return handover.scale()
        if self._offers(self.ffn, "can_add", nt):
            kw2["into"] = x
        with span(ctx, "ffn"):
            return self.ffn.run(h, ctx, **kw2)


register_part("prenorm", PreNormBlock)
