"""Architecture-neutral descriptions of a decoder, as plain data.

A model is a list of blocks plus a schedule. Every block names its parts
(norms, mixer, feed-forward) with all their sizes and constants, so two
blocks of one model may differ in any of them. The schedule is the order in
which blocks run; it may name a block twice or let a run read the cache that
an earlier run wrote.

Each spec class carries a ``kind`` string. ``transformer_amd.parts.registry``
maps that string to the class that executes it, so a new part is a new spec
class plus a registered executor; nothing in this file changes.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


class ConfigError(ValueError):
    """A configuration that cannot be built; the message names the key."""


@dataclass(frozen=True)
class NormSpec:
    size: int
    eps: float
    kind: str = "rmsnorm"


@dataclass(frozen=True)
class PositionSpec:
    """Rotation of (q, k) pairs by position * theta^(-2j/head_dim).

    style "half" pairs element j with j + head_dim/2, "interleaved" pairs 2j
    with 2j + 1. kind "none" leaves q and k as they are.
    """
    head_dim: int
    theta: float = 10000.0
    style: str = "half"
    kind: str = "rope"


@dataclass(frozen=True)
class AttentionSpec:
    """Causal grouped-query attention over the per-sequence key/value cache.

    window: a query at position p reads keys in (p - window, p]; None = all.
    """
    hidden: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float
    position: PositionSpec
    window: Optional[int] = None
    qkv_bias: bool = False
    out_bias: bool = False
    kind: str = "attention"


@dataclass(frozen=True)
class SwiGLUSpec:
    hidden: int
    intermediate: int
    bias: bool = False
    kind: str = "swiglu"


@dataclass(frozen=True)
class BlockSpec:
    """x += mixer(norm1(x)); x += ffn(norm2(x))  (kind "prenorm")."""
    norm1: object
    mixer: object
    norm2: object
    ffn: object
    kind: str = "prenorm"


@dataclass(frozen=True)
class RunSpec:
    """One entry of the schedule.

    block: index into ModelSpec.blocks.
    cache_of: None = this run owns a cache layer of its own (if its mixer
    needs one); an int names an EARLIER schedule entry whose cache layer this
    run reads instead of writing one.
    """
    block: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    vocab: int
    hidden: int
    blocks: Tuple[BlockSpec, ...]
    schedule: Tuple[RunSpec, ...]
    final_norm: object
    tie_embeddings: Optional[bool] = None  # None: decided by the weight file
    max_position: Optional[int] = None
    stop_ids: Tuple[int, ...] = field(default_factory=tuple)
    # Optional parts around the blocks, for architectures that scale or shift the embedded
    # rows or transform the logits: specs of registered kinds whose executors offer
    # ``run(t, ctx)`` and change the float32 tensor in place ([nt, hidden] after the
    # embedding, [wanted, vocab] for the logits). The Llama decoder has neither.
    after_embed: object = None
    on_logits: object = None

    def validate(self) -> None:
        if self.vocab <= 0 or self.hidden <= 0:
            raise ConfigError("vocab and hidden must be positive")
        if not self.blocks or not self.schedule:
            raise ConfigError("a model needs at least one block and one schedule entry")
        for i, run in enumerate(self.schedule):
            if not 0 <= run.block < len(self.blocks):
                raise ConfigError(f"schedule[{i}] names block {run.block}, "
                                  f"model has {len(self.blocks)}")
            if run.cache_of is not None:
                if not 0 <= run.cache_of < i:
                    raise ConfigError(f"schedule[{i}].cache_of={run.cache_of} must name an "
                                      f"earlier schedule entry")
                if self.schedule[run.cache_of].cache_of is not None:
                    raise ConfigError(f"schedule[{i}].cache_of={run.cache_of} names an entry "
                                      f"that itself borrows a cache")
