"""A minimal reader and writer of GGUF version 3 files.

The reference reads its models from GGUF through an external parser
(gguf/src/lib.rs:74-126): metadata key/values and tensors by
name, 32-bit and 16-bit float payloads being the ones it guarantees
(docs/user-guide/doc.md:126). This module reads the container
itself: header, key/value table, tensor table, aligned data. Tensors of type
F32, F16 and BF16 can be loaded; any other (quantised) type is listed by the
loader as unsupported.

Layout: "GGUF", version u32, tensor count u64, key/value count u64; key/values
(key string, type u32, value); tensor infos (name, n_dims u32, dims u64[n_dims]
with the contiguous axis first, type u32, offset u64 into the data section);
padding to ``general.alignment`` (default 32); data. Shapes are reported
row-major, i.e. with the file's dims reversed.
"""
from __future__ import annotations

import mmap
import struct
import warnings
from pathlib import Path
from typing import Dict, List, Tuple

import torch

MAGIC = b"GGUF"
_SCALARS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q",
            11: "<q", 12: "<d"}
T_STRING, T_ARRAY = 8, 9
GGML_F32, GGML_F16, GGML_BF16 = 0, 1, 30
_TENSOR_DTYPES = {GGML_F32: torch.float32, GGML_F16: torch.float16, GGML_BF16: torch.bfloat16}
_TENSOR_CODES = {v: k for k, v in _TENSOR_DTYPES.items()}


class GGUFError(ValueError):
    pass


class _Cursor:
    def __init__(self, buf, pos=0):
        self.buf, self.pos = buf, pos

    def take(self, fmt):
        size = struct.calcsize(fmt)
        if self.pos + size > len(self.buf):
            raise GGUFError("file ends inside its header")
        (v,) = struct.unpack_from(fmt, self.buf, self.pos)
        self.pos += size
        return v

    def string(self) -> str:
        n = self.take("<Q")
        if self.pos + n > len(self.buf):
            raise GGUFError("file ends inside a string")
        s = bytes(self.buf[self.pos:self.pos + n]).decode("utf-8", errors="replace")
        self.pos += n
        return s

    def value(self, typ):
        if typ in _SCALARS:
            return self.take(_SCALARS[typ])
        if typ == T_STRING:
            return self.string()
        if typ == T_ARRAY:
            inner, count = self.take("<I"), self.take("<Q")
            return [self.value(inner) for _ in range(count)]
        raise GGUFError(f"unknown metadata value type {typ}")


class GGUFFile:
    format = "gguf"

    def __init__(self, path):
        self.path = Path(path)
        self._f = open(self.path, "rb")
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        c = _Cursor(self._mm)
        if len(self._mm) < 24 or bytes(self._mm[:4]) != MAGIC:
            raise GGUFError(f"{self.path}: not a GGUF file")
        c.pos = 4
        version = c.take("<I")
        if version not in (2, 3):
            raise GGUFError(f"{self.path}: GGUF version {version} is not supported (2 or 3)")
        n_tensors, n_kv = c.take("<Q"), c.take("<Q")
        self.metadata: Dict[str, object] = {}
        for _ in range(n_kv):
            key = c.string()
            typ = c.take("<I")
            if key in self.metadata:
                raise GGUFError(f"{self.path}: metadata key {key} appears twice")
            self.metadata[key] = c.value(typ)
        infos: List[Tuple[str, Tuple[int, ...], int, int]] = []
        for _ in range(n_tensors):
            name = c.string()
            nd = c.take("<I")
            dims = tuple(c.take("<Q") for _ in range(nd))
            typ, off = c.take("<I"), c.take("<Q")
            infos.append((name, tuple(reversed(dims)), typ, off))
        align = int(self.metadata.get("general.alignment", 32))
        self._data = -(-c.pos // align) * align
        self.entries: Dict[str, Tuple[Tuple[int, ...], int, int]] = {}
        for name, shape, typ, off in infos:
            if name in self.entries:
                raise GGUFError(f"{self.path}: tensor {name} appears twice")
            self.entries[name] = (shape, typ, off)

    def names(self):
        return self.entries.keys()

    def __contains__(self, name):
        return name in self.entries

    def shape(self, name):
        return self.entries[name][0]

    def dtype(self, name):
        typ = self.entries[name][1]
        return _TENSOR_DTYPES.get(typ, f"ggml type {typ} (quantised or unknown)")

    def read(self, name) -> torch.Tensor:
        shape, typ, off = self.entries[name]
        if typ not in _TENSOR_DTYPES:
            raise GGUFError(f"{self.path}: tensor {name} has ggml type {typ}; only F32, F16 and "
                            f"BF16 tensors can be loaded")
        dt = _TENSOR_DTYPES[typ]
        n = 1
        for s in shape:
            n *= s
        start = self._data + off
        if start + n * torch.empty((), dtype=dt).element_size() > len(self._mm):
            raise GGUFError(f"{self.path}: tensor {name} reaches past the end of the file")
        if n == 0:
            return torch.empty(shape, dtype=dt)
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)
            t = torch.frombuffer(self._mm, dtype=dt, count=n, offset=start)
        return t.reshape(shape)

    def release(self, name) -> None:
        """The mapped pages of this tensor are not needed again (see safetensors_io)."""
        from .safetensors_io import release_pages
        shape, typ, off = self.entries[name]
        if typ not in _TENSOR_DTYPES:
            return
        n = 1
        for s in shape:
            n *= s
        start = self._data + off
        release_pages(self._mm, start, start + n * torch.empty((), dtype=_TENSOR_DTYPES[typ]).element_size())

    def close(self):
        self._f.close()


# ------------------------------------------------------------------ writing
def _pack_string(s: str) -> bytes:
    b = s.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _pack_value(v) -> bytes:
    if isinstance(v, bool):
        return struct.pack("<I", 7) + struct.pack("<?", v)
    if isinstance(v, int):
        return struct.pack("<I", 4) + struct.pack("<I", v) if 0 <= v < 2 ** 32 else \
            struct.pack("<I", 11) + struct.pack("<q", v)
    if isinstance(v, float):
        return struct.pack("<I", 6) + struct.pack("<f", v)
    if isinstance(v, str):
        return struct.pack("<I", T_STRING) + _pack_string(v)
    if isinstance(v, (list, tuple)):
        if all(isinstance(x, str) for x in v):
            body = b"".join(_pack_string(x) for x in v)
            return struct.pack("<I", T_ARRAY) + struct.pack("<IQ", T_STRING, len(v)) + body
        if all(isinstance(x, int) and not isinstance(x, bool) for x in v):
            body = b"".join(struct.pack("<i", x) for x in v)
            return struct.pack("<I", T_ARRAY) + struct.pack("<IQ", 5, len(v)) + body
        if all(isinstance(x, (int, float)) for x in v):
            body = b"".join(struct.pack("<f", float(x)) for x in v)
            return struct.pack("<I", T_ARRAY) + struct.pack("<IQ", 6, len(v)) + body
    raise GGUFError(f"cannot store metadata value {v!r}")


def write_gguf(path, metadata: Dict[str, object], tensors: Dict[str, torch.Tensor],
               alignment: int = 32) -> None:
    head = bytearray(MAGIC + struct.pack("<IQQ", 3, len(tensors), len(metadata)))
    for k, v in metadata.items():
        head += _pack_string(k) + _pack_value(v)
    off = 0
    blobs = []
    for name, t in tensors.items():
        if t.dtype not in _TENSOR_CODES:
            raise GGUFError(f"cannot store dtype {t.dtype} of {name}")
        t = t.detach().cpu().contiguous()
        head += _pack_string(name) + struct.pack("<I", t.dim())
        for dim in reversed(t.shape):
            head += struct.pack("<Q", dim)
        head += struct.pack("<IQ", _TENSOR_CODES[t.dtype], off)
        raw = t.reshape(-1).view(torch.uint8).numpy().tobytes() if t.numel() else b""
        pad = (-len(raw)) % alignment
        blobs.append(raw + b"\0" * pad)
        off += len(raw) + pad
    head += b"\0" * ((-len(head)) % alignment)
    with open(path, "wb") as f:
        f.write(head)
        for b in blobs:
            f.write(b)
