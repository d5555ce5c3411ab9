from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import register_norm
from ..weights.loader import ParamSpec
from .base import Part


@register_norm("rmsnorm")
class RMSNorm(Part):
    """out = x / sqrt(mean(x^2) + eps) * weight, in float32; the weight is kept in float32
    (include/kernels_cpu.hpp:43-54, src/model/block.cpp:81-83)."""
    can_be_lazy = True          # forward takes ``lazy``

    def __init__(self, *, size: int, eps: float, prefix: str, dtype, device):
        self.size, self.eps, self.prefix, self.dtype, self.device = size, float(eps), prefix, dtype, device
        self.weight = None

    def params(self):
        return {"weight": ParamSpec((self.size,), "vector", "ones")}

    def bind(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, x: torch.Tensor, rows: torch.Tensor | None = None, lazy: bool = False):
        """The normed rows in the compute dtype.  ``lazy``: the caller hands the result to parts that pass
        it on to ``ops.linear`` untouched (``takes_lazy_norm``); then, where the product before has prepared
        this norm (a decode step), an ``ops.LazyNorm`` is returned and the product that reads it finishes it."""
        if lazy and rows is None:
            deferred = ops.lazy_rmsnorm(x, self.weight, self.eps, self.dtype)
            if deferred is not None:
                return deferred
        if rows is None:
            ready = ops.prepared_rmsnorm(x, self.weight, self.eps, self.dtype)    # taken by the product before
            if ready is not None:
                return ready
        return ops.rmsnorm(x, self.weight, self.eps, self.dtype, rows)
