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
    """A parameter as its part declares it. ``init`` says how the random-weights mode draws
    it: "normal" = N(0, std) (matrices, biases), "around_one" = 1 + N(0, norm_std) (the
    weight of a norm), "zero". The part knows what its parameter means; nobody guesses it
    from the name."""
    shape: Tuple[int, ...]
    role: str = "matrix"        # "matrix" | "vector" | "table"
    init: str = "normal"        # "normal" | "around_one" | "zero"


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


ALIGN = 256                      # every parameter starts on a multiple of this in the arena
CHUNK_BYTES = 32 << 20           # one staging buffer; the ring holds RING of them
RING = 4


def plan_placement(params: Dict[str, Param], chosen, file, engine_dtype: torch.dtype):
    """Where every parameter that is read from the file lies in ONE allocation: returns
    ({name: (byte offset, storage dtype)}, total bytes); offsets are multiples of ALIGN.
    The reference lays its weights out the same way before it copies anything
    (common/src/lib.rs:91-113, models/llama/cuda/src/lib.rs:85-101)."""
    place, off = {}, 0
    for pname, pick in chosen.items():
        if pick and pick[0] == "=":
            continue
        param = params[pname]
        dt = storage_dtype(param.role, engine_dtype, [file.dtype(p.name) for p in pick])
        n = 1
        for d in param.shape:
            n *= int(d)
        place[pname] = (off, dt)
        off += -(-(n * torch.empty((), dtype=dt).element_size()) // ALIGN) * ALIGN
    return place, off


class _Stager:
    """Brings file bytes to the device through a small ring of pinned buffers: a buffer is
    filled from the mapped file (each page of the file is touched once), copied without
    waiting, and used again only after the event behind its copy has passed. The host never
    holds more than RING * CHUNK_BYTES of a model, whatever its size (the reference pools
    its pinned buffers the same way, models/llama/cuda/src/lib.rs:102-141). Bytes whose type
    differs from what is kept arrive in a device buffer of the same ring and are converted
    there by a kernel."""

    def __init__(self, device, chunk_bytes=CHUNK_BYTES, ring=RING):
        self.device = torch.device(device)
        self.gpu = self.device.type == "cuda"
        self.chunk, self.ring = int(chunk_bytes), int(ring)
        self.host = [None] * self.ring
        self.events = [None] * self.ring
        self.stage = [None] * self.ring
        self.turn = 0
        self.bytes_moved = 0

    def _slot(self):
        i = self.turn
        self.turn = (i + 1) % self.ring
        if self.host[i] is None:
            self.host[i] = torch.empty(self.chunk, dtype=torch.uint8, pin_memory=True)
        if self.events[i] is not None:
            self.events[i].synchronize()
        return i

    def _sent(self, i):
        ev = torch.cuda.Event()
        ev.record()
        self.events[i] = ev

    def move(self, src: torch.Tensor, dst: torch.Tensor) -> None:
        """dst (a contiguous range of the arena, any floating or integer type) = src (a CPU
        tensor that views the mapped file), converted if the types differ."""
        src = src.reshape(-1)
        dst = dst.reshape(-1)
        if src.numel() != dst.numel():
            raise ValueError(f"{src.numel()} values for a place of {dst.numel()}")
        if not self.gpu:
            dst.copy_(src)
            return
        from .. import kernels
        same = src.dtype == dst.dtype
        on_device = not same and kernels.convert_takes(src.dtype, dst.dtype)
        # a chunk holds whole elements of both types
        wire = src.dtype if (same or on_device) else dst.dtype
        per = self.chunk // max(src.element_size(), dst.element_size())
        for a in range(0, src.numel(), per):
            b = min(a + per, src.numel())
            i = self._slot()
            staged = self.host[i][:(b - a) * torch.empty((), dtype=wire).element_size()].view(wire)
            staged.copy_(src[a:b])          # same type: a memcpy; else the host converts (rare types)
            if same or not on_device:
                dst[a:b].copy_(staged, non_blocking=True)
            else:
                if self.stage[i] is None:
                    self.stage[i] = torch.empty(self.chunk, dtype=torch.uint8, device=self.device)
                onto = self.stage[i][:staged.numel() * staged.element_size()].view(wire)
                onto.copy_(staged, non_blocking=True)
                kernels.convert(onto, dst[a:b])
            self._sent(i)
            self.bytes_moved += (b - a) * staged.element_size()

    def finish(self):
        if self.gpu:
            torch.cuda.synchronize(self.device)


def load_parameters(params: Dict[str, Param], sources: Dict[str, Source], file,
                    engine_dtype: torch.dtype, device, where="model", progress=None,
                    chunk_bytes: int = CHUNK_BYTES):
    """{param name: device tensor}. All parameters are views of one allocation (aligned
    ranges, ``plan_placement``); the file's bytes stream through a bounded ring of pinned
    buffers (``_Stager``) and the mapped pages of a tensor are given back once it is copied."""
    chosen = plan_binding(params, sources, file, where)
    place, total = plan_placement(params, chosen, file, engine_dtype)
    device = torch.device(device)
    out: Dict[str, torch.Tensor] = {}
    ctx = torch.cuda.device(device) if device.type == "cuda" else _Nothing()
    with ctx:
        arena = torch.empty(max(total, 1), dtype=torch.uint8, device=device)
        stager = _Stager(device, chunk_bytes)
        for pname, pick in chosen.items():
            if pick and pick[0] == "=":
                continue
            param = params[pname]
            off, dt = place[pname]
            n = 1
            for d in param.shape:
                n *= int(d)
            dst = arena[off:off + n * torch.empty((), dtype=dt).element_size()].view(dt).view(param.shape)
            row = 0
            for piece in pick:
                src = file.read(piece.name)
                if len(pick) == 1:
                    stager.move(src, dst)
                else:
                    stager.move(src, dst[row:row + piece.shape[0]])
                    row += piece.shape[0]
                del src
                release = getattr(file, "release", None)
                if release is not None:
                    release(piece.name)
            out[pname] = dst
            if progress is not None:
                progress(pname)
        stager.finish()
    for pname, pick in chosen.items():
        if pick and pick[0] == "=":
            out[pname] = out[pick[1]]
    wide = sorted(n for n, t in out.items() if params[n].role == "matrix" and t.dtype != engine_dtype)
    if wide:
        # stored in 32 bits, so kept in 32 bits: right, and far slower than the engine's own type
        import warnings
        warnings.warn(f"{where}: {len(wide)} matrices are stored in 32 bits and stay so although the "
                      f"engine runs in {engine_dtype} (first: {wide[0]}); their products take the "
                      f"32-bit kernels. Convert the file to use the fast ones.", stacklevel=2)
    return out


class _Nothing:
    def __enter__(self):
        return self

    def __exit__(self, *a):
        return False
