"""The library's tensor: what a weight, a cache pool, a staging buffer or a kernel operand is.

The reference's model-side tensor is a pointer with an element type and an ownership
{Reference, CPUOwned, CUDAOwned} and no shape (include/model/tensor.hpp:26-106); its ``tensor/``
library adds shapes and is not used by the model.  Here the same notions sit on one type:

* element type and shape: float32, float16, bfloat16, int32, int64; contiguous, last index fastest;
* ``layout``: ``"rows"`` (the shape is the storage's own) or ``"tiled"`` (a 16-bit matrix [n, k] kept
  in the order in which the matrix cores take it, csrc/gemm.hip "Tiled weights": the storage is flat
  and ``logical`` holds (n, k));
* ``owner``: ``"borrowed"`` (a view into memory that someone else owns, the mapping of a checkpoint
  file; ``keeps`` holds that owner alive), ``"host"``, ``"pinned"`` (page-locked host memory that the
  device copies from and to without a staging copy) or ``"device"``.

torch stays behind it as the allocator (and as stream owner and graph recorder elsewhere): a
``Tensor`` is a ``torch.Tensor`` whose memory torch allocated or mapped, so every torch operation
works on it and gives a plain ``torch.Tensor`` back; the kernels' C interface gets pointer, element
type and sizes from it (kernels/ops.py).  The host side stays Python on purpose: tests must be able to
add parts and whole architectures from outside, and none of this is on the device's critical path.
"""
from __future__ import annotations

import torch

LAYOUTS = ("rows", "tiled")
OWNERS = ("borrowed", "host", "pinned", "device")
DTYPES = (torch.float32, torch.float16, torch.bfloat16, torch.int32, torch.int64)


class Tensor(torch.Tensor):
    layout: str = "rows"
    owner: str = "host"
    logical: tuple | None = None
    keeps = None

    # results of torch operations are plain tensors: what an operation makes is new memory, whose
    # layout and owner this type cannot know
    __torch_function__ = torch._C._disabled_torch_function_impl

    @staticmethod
    def wrap(t: torch.Tensor, layout: str = "rows", logical=None, owner: str | None = None, keeps=None) -> "Tensor":
        """``t``'s memory as a ``Tensor`` (no copy).  ``owner`` None: read off where the memory lies."""
        if layout not in LAYOUTS:
            raise ValueError(f"layout {layout!r}: one of {LAYOUTS}")
        if t.dtype not in DTYPES:
            raise ValueError(f"element type {t.dtype} is not one of this library's")
        if not t.is_contiguous():
            raise ValueError("a Tensor is contiguous")
        if layout == "tiled":
            if logical is None or len(logical) != 2 or t.dim() != 1 or t.dtype not in (torch.float16, torch.bfloat16):
                raise ValueError("a tiled Tensor is a flat 16-bit storage with its logical shape (n, k)")
            n, k = logical
            if k % 32 != 0 or t.numel() != (n + 15) // 16 * 16 * k:
                raise ValueError(f"tiled storage of {t.numel()} elements does not hold [{n}, {k}]")
        if owner is None:
            owner = "device" if t.is_cuda else ("pinned" if t.is_pinned() else "host")
        if owner not in OWNERS:
            raise ValueError(f"owner {owner!r}: one of {OWNERS}")
        if (owner == "device") != t.is_cuda:
            raise ValueError(f"owner {owner!r} for memory on {t.device}")
        out = torch.Tensor._make_subclass(Tensor, t.detach(), False)
        out.layout, out.owner, out.keeps = layout, owner, keeps
        out.logical = tuple(logical) if logical is not None else tuple(t.shape)
        return out

    # -- making one ------------------------------------------------------------
    @classmethod
    def empty(cls, shape, dtype, device) -> "Tensor":
        """Device-owned (or host-owned for device "cpu") memory of this shape, not initialised."""
        return cls.wrap(torch.empty(tuple(shape), dtype=dtype, device=device))

    @classmethod
    def zeros(cls, shape, dtype, device) -> "Tensor":
        return cls.wrap(torch.zeros(tuple(shape), dtype=dtype, device=device))

    @classmethod
    def pinned(cls, shape, dtype) -> "Tensor":
        """Page-locked host memory, allocated as such (memory that exists already cannot be registered here)."""
        return cls.wrap(torch.zeros(tuple(shape), dtype=dtype, pin_memory=True), owner="pinned")

    @classmethod
    def borrow(cls, view: torch.Tensor, keeps) -> "Tensor":
        """A view into memory that ``keeps`` owns (a file's mapping); nothing is copied."""
        return cls.wrap(view, owner="borrowed", keeps=keeps)

    # -- what it is -------------------------------------------------------------
    @property
    def nbytes_stored(self) -> int:
        return self.numel() * self.element_size()

    def plain(self) -> torch.Tensor:
        """The same memory as a plain torch tensor (rows layout only: tiled storage has no meaning to torch)."""
        if self.layout != "rows":
            raise ValueError("a tiled Tensor has no torch view; ops.untile gives the matrix back")
        return self.as_subclass(torch.Tensor)

    def on_device(self, device, dtype=None) -> "Tensor":
        """A device-owned copy in ``dtype`` (default: its own); the borrowed or host memory is read once."""
        if self.layout != "rows":
            raise ValueError("tiled storage is made on the device (ops.tile_weight)")
        t = self.plain().to(device=device, dtype=dtype or self.dtype).contiguous()
        return Tensor.wrap(t)

    def prefix(self, rows: int) -> "Tensor":
        """The matrix of the first ``rows`` rows, sharing the storage (tiled: a multiple of 16 rows)."""
        n, k = self.logical if self.layout == "tiled" else self.shape
        if self.layout == "tiled":
            if rows % 16 != 0 or not 0 < rows <= n:
                raise ValueError("a tiled weight is cut at multiples of 16 rows")
            return Tensor.wrap(self.as_subclass(torch.Tensor)[: rows * k], "tiled", (rows, k), self.owner, self.keeps or self)
        return Tensor.wrap(self.plain()[:rows], owner=self.owner, keeps=self.keeps or self)

    def describe(self) -> str:
        shape = list(self.logical)
        return f"{str(self.dtype).replace('torch.', '')}{shape} {self.layout}, {self.owner}"
