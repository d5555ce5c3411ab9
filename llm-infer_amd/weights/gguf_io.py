"""Reader (and a writer for tests and the random-weights mode) for GGUF files with
unquantized tensors.

Layout (docs/gguf.md of the reference; its reader is src/gguf.cpp:8-85 and 173-257): the magic
``GGUF``, a u32 version (2 or 3), the u64 numbers of tensors and of metadata pairs;
then the pairs, each a string key (u64 length + bytes), a u32 value type and the
value; then for each tensor its name, a u32 number of dimensions, the u64 dimensions
with the fastest first, a u32 tensor type and a u64 offset into the data section,
which starts at the next multiple of ``general.alignment`` (32 if absent,
src/gguf.cpp:231-236).  Value types: 0..7 u8 i8 u16 i16 u32 i32 f32 bool, 8 string,
9 array (u32 item type, u64 count, items), 10..12 u64 i64 f64.

Tensor types 0 (F32), 1 (F16) and 30 (BF16) are read; a quantized type is refused by
name.  Shapes are reported slowest dimension first, as safetensors and the rest of
this library have them.  Tensors are views into a memory map.
"""
from __future__ import annotations

import mmap
import struct

import numpy as np
import torch

from ..tensor import Tensor

MAGIC = b"GGUF"
_SCALARS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}
T_STRING, T_ARRAY = 8, 9
_TENSOR_TYPES = {0: (torch.float32, 4), 1: (torch.float16, 2), 30: (torch.bfloat16, 2)}
_TYPE_OF = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 30}
_QUANTIZED = {2: "Q4_0", 3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 8: "Q8_0", 9: "Q8_1", 10: "Q2_K", 11: "Q3_K", 12: "Q4_K",
              13: "Q5_K", 14: "Q6_K", 15: "Q8_K"}


class GGUFError(ValueError):
    pass


class _Cursor:
    def __init__(self, buf, path):
        self.buf, self.at, self.path = buf, 0, path

    def take(self, fmt: str):
        n = struct.calcsize(fmt)
        if self.at + n > len(self.buf):
            raise GGUFError(f"{self.path}: file ends inside its header (at byte {self.at})")
        (v,) = struct.unpack_from(fmt, self.buf, self.at)
        self.at += n
        return v

    def string(self) -> str:
        n = self.take("<Q")
        if self.at + n > len(self.buf):
            raise GGUFError(f"{self.path}: a string of {n} bytes runs past the end of the file")
        s = bytes(self.buf[self.at:self.at + n]).decode("utf-8", errors="replace")
        self.at += n
        return s

    def value(self, vtype: int):
        if vtype in _SCALARS:
            return self.take(_SCALARS[vtype])
        if vtype == T_STRING:
            return self.string()
        if vtype == T_ARRAY:
            item, count = self.take("<I"), self.take("<Q")
            if item in _SCALARS and item != 7:
                fmt = _SCALARS[item]
                n = struct.calcsize(fmt) * count
                if self.at + n > len(self.buf):
                    raise GGUFError(f"{self.path}: an array of {count} items runs past the end of the file")
                arr = np.frombuffer(self.buf, dtype=np.dtype(fmt), count=count, offset=self.at)
                self.at += n
                return arr
            return [self.value(item) for _ in range(count)]
        raise GGUFError(f"{self.path}: unknown metadata value type {vtype}")


class GGUFFile:
    """An open GGUF file: ``metadata`` (key -> value), ``names()``, ``info(name)``, ``tensor(name)``."""

    def __init__(self, path: str):
        self.path = path
        with open(path, "rb") as f:
            if f.seek(0, 2) == 0:
                raise GGUFError(f"{path}: not a GGUF file (it is empty)")
            self._map = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_COPY)
        c = _Cursor(self._map, path)
        if len(self._map) < 4 or bytes(self._map[:4]) != MAGIC:
            raise GGUFError(f"{path}: not a GGUF file (magic {bytes(self._map[:4])!r})")
        c.at = 4
        self.version = c.take("<I")
        if self.version not in (2, 3):
            raise GGUFError(f"{path}: GGUF version {self.version} is not supported (2 and 3 are)")
        n_tensors, n_pairs = c.take("<Q"), c.take("<Q")
        self.metadata = {}
        for _ in range(n_pairs):
            key = c.string()
            self.metadata[key] = c.value(c.take("<I"))
        self._info = {}
        for _ in range(n_tensors):
            name = c.string()
            n_dims = c.take("<I")
            if n_dims > 8:
                raise GGUFError(f"{path}: tensor {name!r} claims {n_dims} dimensions")
            dims = [c.take("<Q") for _ in range(n_dims)]
            ttype, offset = c.take("<I"), c.take("<Q")
            self._info[name] = (ttype, tuple(reversed(dims)), offset)
        align = int(self.metadata.get("general.alignment", 32))
        if align <= 0 or align & (align - 1):
            raise GGUFError(f"{path}: general.alignment {align} is no power of two")
        self._data_start = (c.at + align - 1) // align * align
        for name, (ttype, shape, offset) in self._info.items():
            if ttype not in _TENSOR_TYPES:
                continue
            count = 1
            for s in shape:
                count *= s
            end = self._data_start + offset + count * _TENSOR_TYPES[ttype][1]
            if offset % align or end > len(self._map):
                raise GGUFError(f"{path}: tensor {name!r} at offset {offset} does not lie inside the file")

    def names(self) -> list:
        return list(self._info)

    def info(self, name: str):
        ttype, shape, _ = self._info[name]
        if ttype not in _TENSOR_TYPES:
            what = _QUANTIZED.get(ttype, f"type {ttype}")
            raise GGUFError(f"{self.path}: tensor {name!r} is stored as {what}; only F32, F16 and BF16 tensors "
                            "are read (quantized weights are not supported)")
        return _TENSOR_TYPES[ttype][0], shape

    def tensor(self, name: str) -> Tensor:
        dtype, shape = self.info(name)
        _, _, offset = self._info[name]
        count = 1
        for s in shape:
            count *= s
        raw = np.frombuffer(self._map, dtype=np.uint8, count=count * _TENSOR_TYPES[self._info[name][0]][1],
                            offset=self._data_start + offset)
        return Tensor.borrow(torch.from_numpy(raw).view(dtype).reshape(shape), keeps=self._map)


# ---------------------------------------------------------------------------
# writer
# ---------------------------------------------------------------------------
def _pack_string(s: str) -> bytes:
    b = s.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _pack_value(v) -> bytes:
    """(value type, bytes) chosen by the Python type: bool, int (u32 if it fits, else u64; negative
    i64), float (f32), str, list of str / int / float; numpy.uint64 and numpy.float64 force u64 / f64."""
    if isinstance(v, np.uint64):
        return struct.pack("<IQ", 10, int(v))
    if isinstance(v, np.float64):
        return struct.pack("<Id", 12, float(v))
    if isinstance(v, bool):
        return struct.pack("<I?", 7, v)
    if isinstance(v, int):
        if v < 0:
            return struct.pack("<Iq", 11, v)
        return struct.pack("<II", 4, v) if v < (1 << 32) else struct.pack("<IQ", 10, v)
    if isinstance(v, float):
        return struct.pack("<If", 6, v)
    if isinstance(v, str):
        return struct.pack("<I", T_STRING) + _pack_string(v)
    if isinstance(v, (list, tuple)):
        if all(isinstance(x, str) for x in v):
            return struct.pack("<IIQ", T_ARRAY, T_STRING, len(v)) + b"".join(_pack_string(x) for x in v)
        if all(isinstance(x, int) and not isinstance(x, bool) for x in v):
            return struct.pack("<IIQ", T_ARRAY, 5, len(v)) + struct.pack(f"<{len(v)}i", *v)
        if all(isinstance(x, (int, float)) for x in v):
            return struct.pack("<IIQ", T_ARRAY, 6, len(v)) + struct.pack(f"<{len(v)}f", *v)
    raise GGUFError(f"cannot write a metadata value of type {type(v).__name__}")


def write_gguf(path: str, metadata: dict, tensors: dict, alignment: int = 32, version: int = 3) -> None:
    """``tensors``: name -> torch tensor (float32, float16 or bfloat16), written in the given order."""
    meta = dict(metadata)
    if alignment != 32:
        meta["general.alignment"] = alignment
    head = [MAGIC, struct.pack("<IQQ", version, len(tensors), len(meta))]
    for k, v in meta.items():
        head.append(_pack_string(k) + _pack_value(v))
    offset, infos, blobs = 0, [], []
    for name, t in tensors.items():
        if t.dtype not in _TYPE_OF:
            raise GGUFError(f"tensor {name!r}: dtype {t.dtype} cannot be written (float32, float16, bfloat16 can)")
        t = t.detach().cpu().contiguous()
        data = t.view(torch.uint8).numpy().tobytes() if t.numel() else b""
        infos.append(_pack_string(name) + struct.pack("<I", t.dim())
                     + b"".join(struct.pack("<Q", s) for s in reversed(t.shape))
                     + struct.pack("<IQ", _TYPE_OF[t.dtype], offset))
        pad = (-len(data)) % alignment
        blobs.append(data + b"\0" * pad)
        offset += len(data) + pad
    header = b"".join(head) + b"".join(infos)
    with open(path, "wb") as f:
        f.write(header)
        f.write(b"\0" * ((-len(header)) % alignment))
        for b in blobs:
            f.write(b)
