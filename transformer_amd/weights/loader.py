"""Binds the parameters that a model's parts declare to tensors of a weight file.

The parts say which parameters exist (name, shape, role); the architecture
entry says where each is found in the file (one tensor, or several that are
concatenated by rows, e.g. q/k/v into one qkv matrix in the reference's order
models/llama/common/src/lib.rs:132-137). All problems of a
file are reported together in one ``WeightsError``.

Storage rule: a "matrix" takes the engine's dtype (bfloat16 or float32), a
"vector" (norm weight, bias) is kept in float32 whatever the file holds, and a
"table" of integers is int32. Nothing is ever narrowed below bfloat16.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch


@dataclass(frozen=True)
class Param:
    shape: Tuple[int, ...]
    role: str = "matrix"        # "matrix" | "vector" | "table"


@dataclass(frozen=True)
class Piece:
    name: str                   # tensor name in the file
    shape: Tuple[int, ...]


@dataclass(frozen=True)
class Source:
    """Where a parameter comes from.

    options: ways to assemble it; each is a tuple of pieces concatenated along
    axis 0. The first option whose pieces are all in the file is taken.
    stand_in: another parameter that is shared when no option is in the file
    (an output matrix tied to the embedding table).
    ignored: file tensors that belong to this parameter but are not read (a
    stored copy of a tied matrix); they are not reported as unexpected.
    """
    options: Tuple[Tuple[Piece, ...], ...]
    stand_in: Optional[str] = None
    ignored: Tuple[str, ...] = ()


class WeightsError(ValueError):
    def __init__(self, where, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.wrong_shape = sorted(wrong_shape)
        self.wrong_dtype = sorted(wrong_dtype)
        lines = [f"weights of {where} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): "
                         + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n} is {list(got)}, model needs {list(want)}" for n, got, want in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  unsupported dtypes ({len(self.wrong_dtype)}): " + "; ".join(
                f"{n} is {dt}" for n, dt in self.wrong_dtype))
        super().__init__("\n".join(lines))


_FLOATS = (torch.float64, torch.float32, torch.float16, torch.bfloat16)
_INTS = (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8)


def storage_dtype(role: str, engine_dtype: torch.dtype, file_dtypes=()) -> torch.dtype:
    """What a parameter is kept as: matrices in the engine's dtype, except that a matrix
    whose file tensors are all stored in 32 bits (or more) stays float32; vectors (norm
    weights, biases) float32 whatever the file holds; integer tables int32."""
    if role == "matrix":
        wide = (torch.float32, torch.float64)
        if file_dtypes and all(dt in wide for dt in file_dtypes):
            return torch.float32
        return engine_dtype
    if role == "vector":
        return torch.float32
    if role == "table":
        return torch.int32
    raise ValueError(f"unknown parameter role {role!r}")


def plan_binding(params: Dict[str, Param], sources: Dict[str, Source], file, where="model"):
    """Decide, without reading data, which option feeds each parameter.

    Returns {param: tuple of pieces | ("=", other param)}. Raises WeightsError
    listing every missing, unexpected and mis-shaped tensor.
    """
    missing, wrong_shape, wrong_dtype = set(), set(), set()
    used = set()
    chosen = {}
    for pname, param in params.items():
        src = sources.get(pname)
        if src is None:
            raise KeyError(f"architecture gives no source for parameter {pname}")
        pick = None
        for opt in src.options:
            if all(p.name in file for p in opt):
                pick = opt
                break
        if pick is None:
            if src.stand_in is not None:
                chosen[pname] = ("=", src.stand_in)
                continue
            # report what the first option lacks (its names are the canonical ones)
            first = src.options[0] if src.options else ()
            missing.update(p.name for p in first if p.name not in file)
            used.update(p.name for opt in src.options for p in opt if p.name in file)
            continue
        rows = 0
        for p in pick:
            used.add(p.name)
            got = tuple(file.shape(p.name))
            if got != tuple(p.shape):
                wrong_shape.add((p.name, got, tuple(p.shape)))
            dt = file.dtype(p.name)
            ok = dt in (_INTS if param.role == "table" else _FLOATS)
            if not ok:
                wrong_dtype.add((p.name, str(dt)))
            rows += p.shape[0] if p.shape else 0
        if pick and tuple(param.shape) and rows != param.shape[0] and not wrong_shape:
            raise AssertionError(f"source of {pname} assembles {rows} rows, parameter has "
                                 f"{param.shape[0]}")
        chosen[pname] = pick
    for pname, c in chosen.items():
        if c and c[0] == "=" and c[1] not in params:
            raise KeyError(f"parameter {pname} stands in for unknown parameter {c[1]}")
    unexpected = set(file.names()) - used
    # a tensor that an unchosen option names (e.g. an output matrix beside a tied
    # table) is known to the model, not unexpected
    known = {p.name for s in sources.values() for opt in s.options for p in opt}
    known |= {n for s in sources.values() for n in s.ignored}
    unexpected -= known
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightsError(where, missing, unexpected, wrong_shape, wrong_dtype)
    return chosen


def load_parameters(params: Dict[str, Param], sources: Dict[str, Source], file,
                    engine_dtype: torch.dtype, device, where="model", progress=None):
    """{param name: device tensor}. Tensors are streamed one by one."""
    chosen = plan_binding(params, sources, file, where)
    out: Dict[str, torch.Tensor] = {}
    for pname, pick in chosen.items():
        if pick and pick[0] == "=":
            continue
        param = params[pname]
        dst = torch.empty(param.shape, device=device,
                          dtype=storage_dtype(param.role, engine_dtype, [file.dtype(p.name) for p in pick]))
        row = 0
        for piece in pick:
            src = file.read(piece.name)
            if len(pick) == 1:
                dst.copy_(src)
            else:
                dst[row:row + piece.shape[0]].copy_(src)
                row += piece.shape[0]
        out[pname] = dst
        if progress is not None:
            progress(pname)
    for pname, pick in chosen.items():
        if pick and pick[0] == "=":
            out[pname] = out[pick[1]]
    return out
