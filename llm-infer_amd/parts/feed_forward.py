from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import register_feed_forward
from ..weights.loader import ParamSpec
from .base import Part


@register_feed_forward("gated_mlp")
class GatedMLP(Part):
    """down(act(gate(x)) * up(x)) added into the residual stream; act is silu, x / (1 + exp(-x)), or
    gelu in the tanh form the reference computes (src/model/block.cpp:200-222,
    include/kernels_cpu.hpp:179-186).

    Gate and up rows are interleaved into one matrix (row 2j = gate_j, row 2j+1 = up_j),
    so that one product yields both and its epilogue applies the activation before
    anything is written; each row's sum is what it would be alone.
    """

    takes_lazy_norm = True      # the normed input goes to ops.linear as it comes

    def __init__(self, *, hidden_size, intermediate_size, activation="silu", prefix, dtype, device):
        if activation not in ("silu", "gelu"):
            raise ValueError(f"gated_mlp: activation {activation!r} is not built (silu and gelu are)")
        self.mode = ops.EPI_SWIGLU if activation == "silu" else ops.EPI_GEGLU
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.w_gate_up = self.w_down = None

    def params(self):
        f, d = self.intermediate_size, self.hidden_size
        return {"gate_proj.weight": ParamSpec((f, d)), "up_proj.weight": ParamSpec((f, d)),
                "down_proj.weight": ParamSpec((d, f))}

    def bind(self, tensors):
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        gu = torch.stack([g, u], dim=1).reshape(2 * self.intermediate_size, self.hidden_size).contiguous()
        self.w_gate_up = ops.prepare_weight(gu)
        self.w_down = ops.prepare_weight(tensors["down_proj.weight"])

    def forward(self, h, residual):
        t = ops.linear(h, self.w_gate_up, self.mode, out_dtype=self.dtype)
        ops.linear(t, self.w_down, ops.EPI_ADD, out=residual)
