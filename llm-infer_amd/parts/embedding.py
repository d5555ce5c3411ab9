from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import register_embedding, register_head
from ..weights.loader import ParamSpec
from .base import Part


@register_embedding("embedding")
class Embedding(Part):
    """x = float32(table[token]), unscaled (src/model/model.cpp:101-118)."""

    def __init__(self, *, vocab_size, hidden_size, prefix, dtype, device):
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.weight = None

    def params(self):
        return {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def bind(self, tensors):
        self.weight = tensors["weight"]

    def forward(self, ctx):
        """The residual stream's first value for the step's tokens, float32 [T, hidden].  ``ctx`` is the
        step (``token_ids``, and ``pos`` for an embedding that adds positions)."""
        return ops.embed(self.weight, ctx.token_ids)


@register_head("lm_head")
class LMHead(Part):
    """logits = h W^T in float32 (src/model/model.cpp:93-98).  ``tied``: W is the embedding
    table (the reference has no tied models: it requires output.weight, model.cpp:35-38)."""

    def __init__(self, *, vocab_size, hidden_size, tied, prefix, dtype, device):
        self.vocab_size, self.hidden_size, self.tied = vocab_size, hidden_size, tied
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.weight = None

    def params(self):
        return {} if self.tied else {"weight": ParamSpec((self.vocab_size, self.hidden_size))}

    def ignorable(self):
        return [self.prefix + "weight"] if self.tied else []

    def bind(self, tensors):
        if not self.tied:
            self.weight = ops.prepare_weight(tensors["weight"])

    def tie(self, table):
        # the embedding gathers rows, the head streams the whole matrix: it keeps a tiled copy
        self.weight = ops.prepare_weight(table)

    def forward(self, h):
        return ops.linear(h, self.weight, out_dtype=torch.float32)
