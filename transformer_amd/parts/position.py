"""Position encodings of the attention mixer.

Interface: ``encode_and_store(qkv, ctx, nq, nkv, dest, kcache, vcache, bias)``
transforms the q and k heads of the packed qkv rows for the absolute positions
of the step (``ctx.positions``) and stores the step's k and v into the cache layer. Both happen in
one kernel because each touches every k element once.

Rotary: pair (u, v) of a head becomes (u cos a - v sin a, u sin a + v cos a) with
a = position * theta^(-2j/head_dim); the angle, sine and cosine are float32.
The reference rotates q and k in place before the cache write and hands theta to
the operator (models/llama/common/src/compute.rs:232-233,
:457-488); positions of a request are pos .. pos+seq_len (:188-198).
"""
from __future__ import annotations

import numpy as np
import torch

from .. import kernels
from .base import Part, PartError, register_part


class Rotary(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        if spec.head_dim % 2:
            raise PartError(f"rotary head size {spec.head_dim} must be even")
        if spec.style not in ("half", "interleaved"):
            raise PartError(f"unknown rotary pairing {spec.style!r}")
        self.head_dim = spec.head_dim
        self.interleaved = spec.style == "interleaved"
        j = np.arange(spec.head_dim // 2, dtype=np.float64)
        inv = float(spec.theta) ** (-2.0 * j / spec.head_dim)
        self.inv_freq = torch.tensor(inv.astype(np.float32), device=device)
        self.key = ("rope", spec.head_dim, float(spec.theta))

    def angles(self, ctx):
        """(cos, sin) of every token of the step, computed once per step and shared
        by all layers that rotate with the same frequencies."""
        table = ctx.shared.get(self.key)
        if table is None:
            out = ctx.ws.take(f"rope.angles.{self.head_dim}.{self.key[2]}",
                              (ctx.nt, self.head_dim // 2, 2), torch.float32)
            table = kernels.rope_table(ctx.positions, self.inv_freq, out)
            ctx.shared[self.key] = table
        return table

    def encode_and_store(self, qkv, ctx, nq, nkv, dest=None, kcache=None, vcache=None, bias=None):
        return kernels.rope_kv_write(qkv, nq, nkv, self.head_dim, self.angles(ctx),
                                     self.interleaved, dest, kcache, vcache, bias)

    def rotation_of(self, ctx):
        """(angle table, interleaved) for a kernel that rotates q and k itself. A position
        part without this method is always run through ``encode_and_store``."""
        return self.angles(ctx), self.interleaved


class NoPosition(Part):
    """Leaves q and k as they are; only the cache write happens."""
    graph_safe = True

    def __init__(self, spec, dtype, device):
        self.head_dim = spec.head_dim

    def encode_and_store(self, qkv, ctx, nq, nkv, dest=None, kcache=None, vcache=None, bias=None):
        return kernels.rope_kv_write(qkv, nq, nkv, self.head_dim, None, False, dest, kcache,
                                     vcache, bias)

    def rotation_of(self, ctx):
        return None, False


register_part("rope", Rotary)
register_part("none", NoPosition)
