"""Reading and writing of safetensors files, by tensor name, without copying.

Container: 8-byte little-endian header length, a JSON object
``{name: {"dtype", "shape", "data_offsets"}}`` (``__metadata__`` skipped), then the
data section.  Checked as the reference checks it
(``crates/mach-model/src/loader.rs:28, 59-152, 289-314``): header cap of 64 MiB,
duplicate names rejected, offsets inside the data section, byte span equal to the
element count times the element size.  The file is memory-mapped; a tensor is a view
into the map until it is copied to the device.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, Tuple

import torch

HEADER_CAP = 64 << 20

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


def _no_duplicates(pairs):
    out = {}
    for k, v in pairs:
        if k in out:
            raise SafetensorsError(f"duplicate tensor name {k!r} in header")
        out[k] = v
    return out


class SafetensorsFile:
    """One memory-mapped file.  ``entries[name] = (dtype, shape, begin, end)``."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: truncated (no header length)")
        self._f = open(path, "rb")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if hlen > HEADER_CAP:
            raise SafetensorsError(f"{path}: header of {hlen} bytes exceeds the cap of {HEADER_CAP}")
        if 8 + hlen > size:
            raise SafetensorsError(f"{path}: truncated header ({hlen} bytes announced, {size - 8} present)")
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"), object_pairs_hook=_no_duplicates)
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not valid JSON ({e})") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: header must be an object")
        self._base = 8 + hlen
        data_len = size - self._base
        self.entries: Dict[str, Tuple[torch.dtype, Tuple[int, ...], int, int]] = {}
        for name, info in header.items():
            if name == "__metadata__":
                continue
            try:
                dt, shape, (b, e) = info["dtype"], tuple(int(s) for s in info["shape"]), info["data_offsets"]
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError(f"{path}: malformed entry for {name!r}") from None
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: {name}: unsupported dtype {dt}")
            n = 1
            for s in shape:
                n *= s
            if not (0 <= b <= e <= data_len):
                raise SafetensorsError(f"{path}: {name}: data_offsets [{b}, {e}) outside the data section "
                                       f"of {data_len} bytes")
            if e - b != n * _DTYPES[dt].itemsize:
                raise SafetensorsError(f"{path}: {name}: {e - b} bytes for shape {list(shape)} of {dt}")
            self.entries[name] = (_DTYPES[dt], shape, b, e)
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def tensor(self, name: str) -> torch.Tensor:
        dtype, shape, b, e = self.entries[name]
        if e == b:
            return torch.empty(shape, dtype=dtype)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the map is read-only; the view is never written
            flat = torch.frombuffer(self._map, dtype=dtype, count=(e - b) // dtype.itemsize, offset=self._base + b)
        return flat.view(shape)


def write_safetensors(path: str, plan: Iterable[Tuple[str, Tuple[int, ...], torch.dtype]], produce) -> None:
    """Stream a file: ``plan`` lists (name, shape, dtype) in file order, ``produce(name)``
    returns that tensor when its turn comes, so the whole model is never held at once."""
    plan = list(plan)
    header, off = {}, 0
    for name, shape, dtype in plan:
        n = 1
        for s in shape:
            n *= s
        nbytes = n * dtype.itemsize
        header[name] = {"dtype": _NAMES[dtype], "shape": list(shape), "data_offsets": [off, off + nbytes]}
        off += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * (-len(blob) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, shape, dtype in plan:
            t = produce(name)
            if tuple(t.shape) != tuple(shape) or t.dtype != dtype:
                raise SafetensorsError(f"{name}: produced {tuple(t.shape)} {t.dtype}, planned {tuple(shape)} {dtype}")
            t = t.contiguous().cpu()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
