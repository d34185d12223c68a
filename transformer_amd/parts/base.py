"""What every part of a block has in common, and the registry of part kinds.

A part is built from its spec alone (all sizes and constants are in the spec),
declares the parameters it wants by relative name, is bound to device tensors,
and is then run by the block it sits in. It never learns which model, layer
index or architecture it belongs to.

Interfaces (duck-typed; the classes below document them):

  Norm         run(x, out, delta, delta_bias, rows) -> out
  Mixer        cache_need() -> KVNeed | StateNeed | None, or a list of them (``layer`` of
               ``run`` is then a tuple of cache layers, one per need)
               run(h, ctx, cache, layer, writes_cache) -> (delta, delta_bias)
               optional step_planner() -> what it wants planned on the host for steps of
               single tokens (engine/batch.py, ``GroupTables.plans``)
  FeedForward  run(h, ctx) -> (delta, delta_bias)
  Block        run(x, pending, ctx, cache, layer, writes_cache) -> pending

``delta`` is what the part adds to the float32 residual stream; the add itself
is fused into the next norm, so a part returns it (with an optional float32 bias
row still to be added) instead of touching the stream.
"""
from __future__ import annotations

from typing import Callable, Dict

import torch

from ..weights.loader import Param


class PartError(ValueError):
    pass


class PartTimers:
    """Time per kind of part, from GPU events around each part's work: set ``model.timers =
    PartTimers()`` and steps run eagerly with a pair of events around the embedding, every norm,
    mixer and feed-forward, the final norm and the output matrix (the reference keeps such
    timers behind a flag of its operators). ``table()`` waits for the GPU and returns
    {name: (calls, milliseconds)}; the product path without timers records no event."""

    def __init__(self):
        self._spans = {}

    class _Span:
        def __init__(self, pairs):
            self.pairs = pairs

        def __enter__(self):
            self.start = torch.cuda.Event(enable_timing=True)
            self.start.record()

        def __exit__(self, *exc):
            end = torch.cuda.Event(enable_timing=True)
            end.record()
            self.pairs.append((self.start, end))
            return False

    def span(self, name: str):
        return self._Span(self._spans.setdefault(name, []))

    def table(self):
        torch.cuda.synchronize()
        return {n: (len(p), sum(a.elapsed_time(b) for a, b in p)) for n, p in self._spans.items()}

    def reset(self):
        self._spans.clear()


class _NoSpan:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SPAN = _NoSpan()


def span(ctx, name: str):
    """``with span(ctx, "mixer"):`` times the block when the step has timers, else does nothing."""
    t = getattr(ctx, "timers", None)
    return t.span(name) if t is not None else _NO_SPAN


_KINDS: Dict[str, Callable] = {}


def register_part(kind: str, builder: Callable) -> None:
    """builder(spec, dtype, device) -> part. Registering a kind again replaces it."""
    _KINDS[kind] = builder


def build_part(spec, dtype: torch.dtype, device):
    try:
        builder = _KINDS[spec.kind]
    except KeyError:
        raise PartError(f"no part registered for kind {spec.kind!r}; known: "
                        f"{', '.join(sorted(_KINDS))}") from None
    return builder(spec, dtype, device)


class Part:
    """Base class: parameter declaration and binding."""

    def params(self) -> Dict[str, Param]:
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        """tensors: relative name -> device tensor, exactly the names of params()."""
        want = self.params()
        for name, p in want.items():
            if name not in tensors:
                raise PartError(f"{type(self).__name__}: parameter {name} was not given")
            if tuple(tensors[name].shape) != tuple(p.shape):
                raise PartError(f"{type(self).__name__}: parameter {name} has shape "
                                f"{tuple(tensors[name].shape)}, expected {tuple(p.shape)}")
        self.w = dict(tensors)

    def children(self) -> Dict[str, "Part"]:
        return {}

    def all_params(self, prefix: str = "") -> Dict[str, Param]:
        out = {prefix + n: p for n, p in self.params().items()}
        for cname, child in self.children().items():
            out.update(child.all_params(prefix + cname + "."))
        return out

    def bind_all(self, tensors: Dict[str, torch.Tensor], prefix: str = "") -> None:
        self.bind({n: tensors[prefix + n] for n in self.params()})
        for cname, child in self.children().items():
            child.bind_all(tensors, prefix + cname + ".")
