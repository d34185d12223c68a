"""Sampling options with the reference's names, defaults and ranges:
temperature 0 (= argmax), top_p 1, top_k unlimited
(test-utils/src/lib.rs:78-80; ranges [0, inf), [0, 1], [1, inf]
in docs/user-guide/doc.md:156-158). Invalid values are refused,
as ``SampleArgs::new(..).expect("invalid sample args")`` does
(models/llama/cuda/src/infer.rs:44).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional


class InvalidSampleArgs(ValueError):
    pass


@dataclass(frozen=True)
class SampleArgs:
    temperature: float = 0.0
    top_p: float = 1.0
    top_k: Optional[int] = None      # None: unlimited

    def __post_init__(self):
        t, p, k = self.temperature, self.top_p, self.top_k
        if not isinstance(t, (int, float)) or isinstance(t, bool) or math.isnan(t) or t < 0 \
                or math.isinf(t):
            raise InvalidSampleArgs(f"temperature must be a finite number >= 0, got {t!r}")
        if not isinstance(p, (int, float)) or isinstance(p, bool) or math.isnan(p) or not 0 <= p <= 1:
            raise InvalidSampleArgs(f"top_p must lie in [0, 1], got {p!r}")
        if k is not None and (isinstance(k, bool) or not isinstance(k, int) or k < 1):
            raise InvalidSampleArgs(f"top_k must be an integer >= 1 (or None), got {k!r}")

    @property
    def greedy(self) -> bool:
        """Argmax: temperature 0, or a kept set of one token."""
        return self.temperature == 0 or self.top_k == 1 or self.top_p == 0
