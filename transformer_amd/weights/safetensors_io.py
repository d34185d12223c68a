"""Reader and writer of the safetensors container.

Layout: 8-byte little-endian header length, a JSON header mapping each tensor
name to {dtype, shape, data_offsets}, then the raw little-endian data. The
file is memory-mapped; a tensor is a zero-copy view until it is cast or moved
to the device, so a large model is never held twice on the host.

A folder may hold one ``model.safetensors`` or shards listed by
``model.safetensors.index.json`` ({"weight_map": {tensor name: file name}}).
"""
from __future__ import annotations

import json
import mmap
import struct
import warnings
from pathlib import Path
from typing import Dict, Tuple

import torch

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    def __init__(self, path):
        self.path = Path(path)
        self._f = open(self.path, "rb")
        size = self.path.stat().st_size
        if size < 8:
            raise SafetensorsError(f"{self.path}: too short for a safetensors header")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if 8 + hlen > size:
            raise SafetensorsError(f"{self.path}: header length {hlen} exceeds the file")
        try:
            header = json.loads(self._f.read(hlen))
        except json.JSONDecodeError as e:
            raise SafetensorsError(f"{self.path}: header is not JSON ({e})") from None
        self.metadata = header.pop("__metadata__", {})
        self._base = 8 + hlen
        self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size else None
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        for name, info in header.items():
            dt, shape = info["dtype"], tuple(info["shape"])
            lo, hi = info["data_offsets"]
            if dt not in _DTYPES:
                raise SafetensorsError(f"{self.path}: tensor {name} has unsupported dtype {dt}")
            n = 1
            for s in shape:
                n *= s
            if hi - lo != n * torch.empty((), dtype=_DTYPES[dt]).element_size() or \
                    self._base + hi > size:
                raise SafetensorsError(f"{self.path}: tensor {name} has inconsistent offsets")
            self.entries[name] = (dt, shape, lo, hi)

    def names(self):
        return self.entries.keys()

    def shape(self, name):
        return self.entries[name][1]

    def dtype(self, name) -> torch.dtype:
        return _DTYPES[self.entries[name][0]]

    def read(self, name) -> torch.Tensor:
        """A CPU tensor viewing the mapped file (read-only memory: copy before writing)."""
        dt, shape, lo, hi = self.entries[name]
        if hi == lo:
            return torch.empty(shape, dtype=_DTYPES[dt])
        with warnings.catch_warnings():
            warnings.simplefilter("ignore", UserWarning)   # the map is read-only on purpose
            t = torch.frombuffer(self._mm, dtype=_DTYPES[dt], count=(hi - lo) // _itemsize(dt),
                                 offset=self._base + lo)
        return t.reshape(shape)

    def release(self, name) -> None:
        """Tells the system that the mapped pages of this tensor are not needed again (the
        loader has copied them): a large model then never stays resident on the host."""
        _, _, lo, hi = self.entries[name]
        release_pages(self._mm, self._base + lo, self._base + hi)

    def close(self):
        # views handed out by read() keep the map alive; dropping our handle is enough
        self._mm = None
        self._f.close()


def release_pages(mm, lo: int, hi: int) -> None:
    """madvise(DONTNEED) over the whole pages inside [lo, hi) of a read-only file map."""
    if mm is None or not hasattr(mm, "madvise") or not hasattr(mmap, "MADV_DONTNEED"):
        return
    page = mmap.PAGESIZE
    a, b = -(-lo // page) * page, hi // page * page
    if b > a:
        try:
            mm.madvise(mmap.MADV_DONTNEED, a, b - a)
        except (OSError, ValueError):
            pass                      # advice only


def _itemsize(dt: str) -> int:
    return torch.empty((), dtype=_DTYPES[dt]).element_size()


class TensorFolder:
    """All tensors of a model folder, whichever shard holds them."""

    format = "safetensors"

    def __init__(self, folder):
        folder = Path(folder)
        index = folder / "model.safetensors.index.json"
        single = folder / "model.safetensors"
        self.files = []
        if index.exists():
            wm = json.loads(index.read_text()).get("weight_map", {})
            for fn in sorted(set(wm.values())):
                self.files.append(SafetensorsFile(folder / fn))
        elif single.exists():
            self.files.append(SafetensorsFile(single))
        else:
            raise SafetensorsError(f"{folder}: neither model.safetensors nor "
                                   f"model.safetensors.index.json")
        self._where = {}
        for f in self.files:
            for n in f.names():
                if n in self._where:
                    raise SafetensorsError(f"tensor {n} appears in {self._where[n].path.name} "
                                           f"and in {f.path.name}")
                self._where[n] = f

    def names(self):
        return self._where.keys()

    def __contains__(self, name):
        return name in self._where

    def shape(self, name):
        return self._where[name].shape(name)

    def dtype(self, name):
        return self._where[name].dtype(name)

    def read(self, name):
        return self._where[name].read(name)

    def release(self, name):
        self._where[name].release(name)

    def close(self):
        for f in self.files:
            f.close()


def write_safetensors(path, tensors: Dict[str, torch.Tensor], metadata=None) -> None:
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    off = 0
    order = []
    for name, t in tensors.items():
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"cannot store dtype {t.dtype} of {name}")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [off, off + nbytes]}
        off += nbytes
        order.append(name)
    h = json.dumps(header, separators=(",", ":")).encode()
    h += b" " * ((8 - len(h) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)))
        f.write(h)
        for name in order:
            # a tensor may live on the GPU: it comes over in pieces, so the host never holds
            # more than one piece of a model that is being saved
            t = tensors[name].detach().contiguous().reshape(-1)
            per = max(1, (64 << 20) // max(1, t.element_size()))
            for a in range(0, t.numel(), per):
                f.write(t[a:a + per].cpu().view(torch.uint8).numpy().tobytes())
