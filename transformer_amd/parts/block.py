"""Arrangement of parts in a block.

"prenorm": x += mixer(norm1(x)); x += ffn(norm2(x)), the reference's block
(/root/reference/models/llama/common/src/compute.rs:204-292). The adds are
carried as a pending (delta, bias) pair and folded into the next norm, so the
float32 residual stream is read and written once per norm.
"""
from __future__ import annotations

from .base import Part, build_part, register_part


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

    @property
    def graph_safe(self) -> bool:
        """True when a step of this block is a fixed sequence of kernel launches on
        fixed buffers (no host decisions that depend on the data)."""
        return all(getattr(p, "graph_safe", False) for p in (self.norm1, self.mixer, self.norm2, self.ffn))

    def run(self, x, pending, ctx, cache, layer, writes_cache=True):
        """x: float32 residual stream [nt, hidden]; pending: (delta, bias) not yet
        added to x, or (None, None). Returns the new pending pair."""
        h = ctx.ws.take("block.h", x.shape, self.dtype)
        self.norm1.run(x, h, pending[0], pending[1])
        pending = self.mixer.run(h, ctx, cache, layer, writes_cache)
        self.norm2.run(x, h, pending[0], pending[1])
        return self.ffn.run(h, ctx)


register_part("prenorm", PreNormBlock)
