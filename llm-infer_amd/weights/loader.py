"""Weights by tensor name.

A model states which tensors it needs (``ParamSpec`` for each name); the loader
compares that table with what a checkpoint folder holds and raises ONE error that
lists every missing tensor, every unexpected tensor and every wrong shape
(the reference stops at the first: include/model/tensor.hpp:18-24, 112-137).

Kept dtypes: matrices in the compute dtype (bfloat16 or float16; float32 in the
32-bit path), norm vectors in float32 (the reference requires F32 norm weights,
src/model/block.cpp:81-83), integer tables as int32, and a tensor that is stored
in 32-bit stays 32-bit.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass

import torch

from ..tensor import Tensor
from .safetensors_io import SafetensorsFile


class WeightError(ValueError):
    pass


@dataclass(frozen=True)
class ParamSpec:
    shape: tuple
    kind: str = "matrix"        # "matrix" | "vector" | "int"
    init: str = "normal"        # random-weights mode: "normal" N(0, 0.02) | "ones" 1 + N(0, 0.01)


class Checkpoint:
    """The tensors of a model folder: one ``model.safetensors`` or the shards that
    ``model.safetensors.index.json`` names."""

    def __init__(self, folder: str):
        self.folder = folder
        single = os.path.join(folder, "model.safetensors")
        index = os.path.join(folder, "model.safetensors.index.json")
        self._where = {}
        self._files = {}
        if os.path.isfile(single):
            self._files[single] = SafetensorsFile(single)
        elif os.path.isfile(index):
            with open(index) as f:
                for name, shard in json.load(f)["weight_map"].items():
                    path = os.path.join(folder, shard)
                    if path not in self._files:
                        self._files[path] = SafetensorsFile(path)
        else:
            raise WeightError(f"no model.safetensors (or model.safetensors.index.json) in {folder}")
        for path, f in self._files.items():
            for name in f.names():
                self._where[name] = f

    def names(self) -> list:
        return list(self._where)

    def info(self, name: str):
        return self._where[name].info(name)

    def tensor(self, name: str) -> torch.Tensor:
        return self._where[name].tensor(name)


class GGUFCheckpoint:
    """The tensors of a GGUF file under the names this library uses: ``rename`` maps a name of
    the model's table to the name in the file (the configuration class knows it)."""

    def __init__(self, path: str, needed, rename):
        from .gguf_io import GGUFFile
        self.file = GGUFFile(path)
        self._to_file = {n: rename(n) for n in needed}
        back = {v: k for k, v in self._to_file.items()}
        self._names = [back.get(n, n) for n in self.file.names()]
        self._to_file.update({n: n for n in self._names if n not in self._to_file})

    def names(self) -> list:
        return list(self._names)

    def info(self, name: str):
        return self.file.info(self._to_file[name])

    def tensor(self, name: str) -> torch.Tensor:
        return self.file.tensor(self._to_file[name])


def read_checkpoint(folder: str, needed=(), config=None):
    """A folder with safetensors, or a GGUF file (or the folder that holds one)."""
    from ..registry import find_gguf
    has_st = os.path.isdir(folder) and (os.path.isfile(os.path.join(folder, "model.safetensors")) or
                                        os.path.isfile(os.path.join(folder, "model.safetensors.index.json")))
    gguf = None if has_st else find_gguf(folder)
    if gguf is not None:
        rename = getattr(config, "gguf_tensor_name", None) or (lambda n: n)
        return GGUFCheckpoint(gguf, needed, rename)
    return Checkpoint(folder)


def check_tensors(needed: dict, found, ignorable=()) -> None:
    """``needed``: name -> ParamSpec; ``found``: object with names() and info(name).
    Raises one WeightError listing all that is missing, unexpected or misshapen."""
    have = set(found.names())
    missing = [n for n in needed if n not in have]
    unexpected = sorted(n for n in have if n not in needed and n not in ignorable)
    wrong = []
    for n, spec in needed.items():
        if n in have:
            dtype, shape = found.info(n)
            if tuple(shape) != tuple(spec.shape):
                wrong.append(f"{n}: expected {list(spec.shape)}, got {list(shape)}")
            elif spec.kind == "int" and dtype.is_floating_point:
                wrong.append(f"{n}: expected an integer table, got {dtype}")
            elif spec.kind != "int" and not dtype.is_floating_point:
                wrong.append(f"{n}: expected floating point, got {dtype}")
    if missing or unexpected or wrong:
        parts = ["the checkpoint does not fit the model:"]
        if missing:
            parts.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            parts.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            parts.append(f"  wrong shapes or types ({len(wrong)}): " + "; ".join(wrong))
        raise WeightError("\n".join(parts))


def kept_dtype(stored: torch.dtype, kind: str, compute: torch.dtype) -> torch.dtype:
    if kind == "int":
        return torch.int32
    if kind == "vector" or compute == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32                      # stored in 32-bit stays so
    return compute


def place_tensor(t: torch.Tensor, kind: str, compute: torch.dtype, device) -> Tensor:
    """One tensor as the engine keeps it: a device-owned copy in its kept dtype (a borrowed view of a file's
    mapping is read once on the way)."""
    if not isinstance(t, Tensor):
        t = Tensor.wrap(t)
    return t.on_device(device, kept_dtype(t.dtype, kind, compute))


_DTYPE_NAMES = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}


def stored_matrix_dtype(needed: dict, found) -> torch.dtype | None:
    """The type in which a checkpoint stores its matrices: the widest among the matrices of the model's
    table that the checkpoint holds (the reference reads it off blk.0.attn_q/k/v and ffn_up and rejects
    a mix, src/model/config.cpp:36-70)."""
    have = set(found.names())
    seen = set()
    for n, spec in needed.items():
        if spec.kind == "matrix" and n in have:
            try:
                dtype = found.info(n)[0]
            except ValueError:
                continue                 # a tensor type that is not read: the check of the table says so
            if dtype.is_floating_point:
                seen.add(dtype)
    if not seen:
        return None
    return next(iter(seen)) if len(seen) == 1 else torch.float32      # a mix: the type that holds them all


def choose_dtype(requested, config_dtype: str | None, stored: torch.dtype | None, say=None) -> torch.dtype:
    """The compute dtype of an engine.  ``requested`` None: what the model's own files say, ``torch_dtype``
    of config.json first, else the type its matrices are stored in (a GGUF file has no other word on
    it), else bfloat16; a float32 model so runs the 32-bit path (the reference takes the type from the
    file in the same way and knows float32 and float16, src/model/config.cpp:119-129).  When the
    result narrows what is stored, or turns one 16-bit type into the other, ``say`` gets one line."""
    if requested is not None and not isinstance(requested, torch.dtype):
        if requested not in _DTYPE_NAMES and requested not in ("bf16", "fp16", "fp32"):
            raise ValueError(f"dtype {requested!r}: one of bfloat16, float16, float32")
        requested = {**_DTYPE_NAMES, "bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[requested]
    if requested is not None:
        chosen, by = requested, "as asked for"
    elif config_dtype is not None:
        if config_dtype not in _DTYPE_NAMES:
            raise ValueError(f"Unsupported torch_dtype: {config_dtype}")
        chosen, by = _DTYPE_NAMES[config_dtype], "by the configuration's torch_dtype"
    elif stored is not None:
        chosen, by = (torch.float32 if stored == torch.float64 else stored), "as stored"
    else:
        chosen, by = torch.bfloat16, "by default"
    if say is not None and stored is not None and chosen != stored:
        name = lambda d: str(d).replace("torch.", "")
        if stored in (torch.float32, torch.float64) and chosen != torch.float32:
            say(f"the matrices are stored in {name(stored)} and run in {name(chosen)} ({by}): they are rounded")
        elif stored == torch.float16 and chosen == torch.bfloat16:
            say(f"the matrices are stored in float16 and run in bfloat16 ({by}): three bits of every mantissa are lost")
        elif stored == torch.bfloat16 and chosen == torch.float16:
            say(f"the matrices are stored in bfloat16 and run in float16 ({by}): values beyond 65504 become infinite, "
                "tiny ones lose bits")
    return chosen


def load_into(model, folder: str, config=None, ckpt=None) -> None:
    """Check the folder's tensors against ``model.params()`` and hand each part its tensors."""
    needed = model.params()
    if ckpt is None:
        ckpt = read_checkpoint(folder, needed, config)
    ignorable = list(model.ignorable_names())
    if isinstance(ckpt, GGUFCheckpoint):
        ignorable += list(getattr(config, "gguf_ignorable", ()))     # the configuration class names them
    check_tensors(needed, ckpt, ignorable)
    model.bind(OnDemand(lambda name: place_tensor(ckpt.tensor(name), needed[name].kind, model.dtype, model.device)))


class OnDemand:
    """A mapping name -> tensor that makes the tensor when it is asked for and keeps nothing: a model
    binds its parts one after the other, so the device never holds a whole checkpoint twice (once as
    read and once as the parts keep it: fused, interleaved, tiled)."""

    def __init__(self, make):
        self._make = make

    def __getitem__(self, name: str):
        return self._make(name)
