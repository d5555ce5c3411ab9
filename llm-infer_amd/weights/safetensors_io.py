"""Reader and writer for safetensors files.

Layout: 8 bytes little-endian header length, a JSON header with ``dtype``,
``shape`` and ``data_offsets`` for each tensor (and an optional ``__metadata__``),
then the tensors' bytes.  The checks follow the reference's reader
(src/safetensors.cpp:108-193): header length bounds, valid JSON, known dtypes,
offsets that tile the data section without gap or overlap, sizes that match the
shapes, and a file exactly as long as the header says.  Tensors are views into a
memory map; nothing is copied until a tensor is moved to the device.
"""
from __future__ import annotations

import json
import mmap
import struct

import torch

from ..tensor import Tensor

MAX_HEADER = 100_000_000            # src/safetensors.cpp:11

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


def _itemsize(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


class SafetensorsFile:
    """An open safetensors file: ``names()``, ``info(name)`` and ``tensor(name)``."""

    def __init__(self, path: str):
        self.path = path
        with open(path, "rb") as f:
            self._map = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_COPY)
        size = len(self._map)
        if size < 8:
            raise SafetensorsError(f"{path}: Header too small")
        (n,) = struct.unpack("<Q", self._map[:8])
        if n > MAX_HEADER:
            raise SafetensorsError(f"{path}: Header too large ({n} bytes)")
        if 8 + n > size:
            raise SafetensorsError(f"{path}: Invalid header length {n} for a file of {size} bytes")
        try:
            header = json.loads(self._map[8:8 + n].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: Invalid JSON in header: {e}") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: Invalid JSON in header: not an object")
        self.metadata = header.pop("__metadata__", {})
        self._data_start = 8 + n
        self._info = {}
        for name, entry in header.items():
            try:
                dtype, shape, (lo, hi) = entry["dtype"], tuple(int(s) for s in entry["shape"]), entry["data_offsets"]
            except (KeyError, TypeError, ValueError):
                raise SafetensorsError(f"{path}: Invalid tensor info for {name!r}") from None
            if dtype not in _DTYPES:
                raise SafetensorsError(f"{path}: Unknown dtype {dtype!r} of tensor {name!r}")
            self._info[name] = (_DTYPES[dtype], shape, int(lo), int(hi))
        self._validate(size)

    def _validate(self, size: int) -> None:
        end = 0
        for name, (dtype, shape, lo, hi) in sorted(self._info.items(), key=lambda kv: kv[1][2]):
            if lo != end or hi < lo:
                raise SafetensorsError(f"{self.path}: Invalid offset for tensor {name!r}: [{lo}, {hi}) after {end}")
            count = 1
            for s in shape:
                count *= s
            if count * _itemsize(dtype) != hi - lo:
                raise SafetensorsError(f"{self.path}: Invalid tensor info - size mismatch for {name!r}: "
                                       f"shape {list(shape)} of {dtype} is not {hi - lo} bytes")
            end = hi
        if self._data_start + end != size:
            raise SafetensorsError(f"{self.path}: Metadata incomplete buffer: tensors end at "
                                   f"{self._data_start + end}, the file has {size} bytes")

    def names(self) -> list:
        return list(self._info)

    def info(self, name: str):
        """(dtype, shape) of a tensor."""
        if name not in self._info:
            raise SafetensorsError(f"{self.path}: Tensor not found: {name}")
        dtype, shape, _, _ = self._info[name]
        return dtype, shape

    def tensor(self, name: str) -> Tensor:
        """The tensor as a view into the file's mapping (owner "borrowed": nothing is copied)."""
        if name not in self._info:
            raise SafetensorsError(f"{self.path}: Tensor not found: {name}")
        dtype, shape, lo, hi = self._info[name]
        count = (hi - lo) // _itemsize(dtype)
        if count == 0:
            return Tensor.wrap(torch.empty(shape, dtype=dtype))
        flat = torch.frombuffer(self._map, dtype=dtype, count=count, offset=self._data_start + lo)
        return Tensor.borrow(flat.view(shape), keeps=self._map)


def write_safetensors(path: str, tensors: dict, metadata: dict | None = None) -> None:
    """Write CPU tensors under their names, in the given order, tightly packed."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    for name, t in tensors.items():
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"cannot store dtype {t.dtype} of tensor {name!r}")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * (-len(blob) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for t in tensors.values():
            t = t.detach().cpu().contiguous()
            f.write(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"")
