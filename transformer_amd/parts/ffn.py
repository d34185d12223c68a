"""The dense SwiGLU feed-forward.

gate_up = h @ Wgu^T with the gate rows first and the up rows second
(models/llama/common/src/lib.rs:154-157, split at
compute.rs:286); act = silu(gate) * up (:286-288); the down projection is
added to the residual (:290-292).
"""
from __future__ import annotations

import torch

from .. import kernels
from ..weights.loader import Param
from .base import Part, register_part
from .linear import adds_in_place, linear, linear_delta


class SwiGLU(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        self.spec, self.dtype = spec, dtype

    def params(self):
        s = self.spec
        p = {"gate_up.weight": Param((2 * s.intermediate, s.hidden), "matrix"),
             "down.weight": Param((s.hidden, s.intermediate), "matrix")}
        if s.bias:
            p["gate_up.bias"] = Param((2 * s.intermediate,), "vector")
            p["down.bias"] = Param((s.hidden,), "vector")
        return p

    def takes_scaled(self, nt: int) -> bool:
        return kernels.skinny_takes(nt, self.w["gate_up.weight"])

    def can_fold(self, nt: int) -> bool:
        return kernels.skinny_folds(nt, self.w["down.weight"])

    def can_add(self, nt: int) -> bool:
        return adds_in_place(nt, self.w["down.weight"])

    def run(self, h, ctx, scale=None, fold=None, into=None):
        """h: [nt, hidden] engine dtype -> (delta float32 [nt, hidden], bias row or None);
        None with ``fold``, which has then taken the result; (None, bias) with ``into``, the
        residual stream that the down projection has then added itself to. ``scale``: the rows
        of h still lack their norm's factor."""
        s, nt = self.spec, h.shape[0]
        act = ctx.ws.take("swiglu.act", (nt, s.intermediate), self.dtype)
        if scale is not None or kernels.skinny_wins(h, self.w["gate_up.weight"]):
            # few rows: the product applies the activation itself and [nt, 2*di] is never stored
            kernels.gemm_skinny(h, self.w["gate_up.weight"], act, swiglu=True,
                                bias=self.w.get("gate_up.bias"), scale=scale)
        elif h.dtype == torch.bfloat16 and kernels.mid_takes(nt, self.w["gate_up.weight"]):
            # up to 64 rows the product of our own applies the activation itself: 44 to 54 us on
            # the 8B shape where the vendor library's product and the activation's kernel take 55
            kernels.gemm_mid(h, self.w["gate_up.weight"], act, swiglu=True, bias=self.w.get("gate_up.bias"))
        else:
            gu = linear(h, self.w["gate_up.weight"],
                        ctx.ws.take("swiglu.gate_up", (nt, 2 * s.intermediate), self.dtype))
            kernels.swiglu(gu, act, self.w.get("gate_up.bias"))
        if fold is not None:
            kernels.gemm_skinny(act, self.w["down.weight"], None, bias=self.w.get("down.bias"), fold=fold)
            return None
        return (linear_delta(act, self.w["down.weight"], ctx.ws, "swiglu.delta", into=into),
                self.w.get("down.bias"))


register_part("swiglu", SwiGLU)
