"""RMS norm, fused with the pending add into the float32 residual stream.

y = v / sqrt(mean(v^2) + eps) * w with v = x + delta (+ delta_bias); the sum of
squares and the product are float32 and the result is rounded once. The
reference calls its norm before attention, before the feed-forward and on the
gathered output rows (models/llama/common/src/compute.rs:206-207,
:274-275, :358-363) and keeps x for the residual (:169, x1 is a separate buffer).
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import kernels
from ..weights.loader import Param
from .base import Part, register_part


class RMSNorm(Part):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        self.size, self.eps, self.dtype = spec.size, float(spec.eps), dtype

    def params(self):
        return {"weight": Param((self.size,), "vector", init="around_one")}

    def run(self, x: torch.Tensor, out: torch.Tensor, delta: Optional[torch.Tensor] = None,
            delta_bias: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None):
        """x: float32 [nt, size], updated in place by the pending delta unless
        ``rows`` selects the rows to normalise. out: engine dtype."""
        return kernels.add_rmsnorm(x, self.w["weight"], self.eps, out, delta, delta_bias, rows)

    def fold(self, x: torch.Tensor, out: torch.Tensor, ctx) -> "kernels.NormFold":
        """For the few-rows product in front of this norm, which then does the add and the
        sums of squares itself; ``.scale()`` of the result goes to the product behind it."""
        parts = ctx.ws.take("norm.parts", kernels.NormFold.parts_shape(self.size), torch.float32)
        return kernels.NormFold(x, self.w["weight"], self.eps, out, parts)


register_part("rmsnorm", RMSNorm)
