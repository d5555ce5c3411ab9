from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import register_position
from .base import Part


@register_position("rope")
class RotaryPosition(Part):
    """Rotation of q and k by position: angle = pos * theta^(-i / rotary_dim) for the pair
    that starts at dimension i (include/kernels_cpu.hpp:82-100).  ``pairing`` "adjacent"
    rotates (i, i+1) as the reference does; "half" rotates (i/2, i/2 + rotary_dim/2).

    A position encoding is a part like the others: it may own tensors (``params`` under its
    ``prefix``, handed over by ``bind``); this one owns none.  It keeps a table of one frequency per
    rotated pair; another encoding of this family (scaled, interpolated, with learned factors) only
    fills the table differently.  Layers whose position specs are equal share one instance.  Its one
    duty towards a mixer is ``rotate_store``: rotate q and k of the step's tokens, write k and v into
    the layer's pages, and return q.
    """

    def __init__(self, *, theta: float, rotary_dim: int, head_dim: int, pairing: str = "adjacent", prefix: str = "",
                 dtype, device):
        self.rotary_dim, self.head_dim, self.pairing, self.theta = rotary_dim, head_dim, pairing, float(theta)
        self.prefix = prefix
        i = torch.arange(0, rotary_dim, 2, dtype=torch.float32)
        # 1 / powf(theta, i / rotary_dim) in float32, as kernels_cpu.hpp:87
        inv = 1.0 / torch.pow(torch.tensor(float(theta), dtype=torch.float32), i / float(rotary_dim))
        self.inv_freq = inv.to(device) if device is not None else inv
        self.dtype = dtype

    def rotate_store(self, qkv, ctx, kv_view, n_heads, n_kv_heads, head_dim):
        k = v = table = stride = None
        if n_kv_heads > 0:
            k, v, table, stride = kv_view.k, kv_view.v, kv_view.page_table, kv_view.page_stride
        return ops.rope_store(qkv, self.inv_freq, self.rotary_dim, self.pairing == "half", ctx.pos, ctx.tok_slot,
                              table, stride, k, v, n_heads, n_kv_heads, head_dim, self.dtype,
                              kv_round=getattr(kv_view, "round_to", None))

    def project_rotate_store(self, h, w, ctx, kv_view, n_heads, n_kv_heads, head_dim):
        """q, k, v = h W^T, rotated and stored; with adjacent pairing and 16-bit storage the rotation
        and the cache write happen in the product's epilogue."""
        return _project(self, h, w, ctx, kv_view, n_heads, n_kv_heads, head_dim, self.inv_freq, self.rotary_dim,
                        self.pairing == "adjacent", self._table(ctx))

    def _table(self, ctx):
        """cos and sin of every token's angles, computed once per step and shared by all layers that
        rotate with the same frequencies."""
        if self.rotary_dim == 0 or self.pairing != "adjacent" or self.dtype == torch.float32:
            return None
        # keyed by the frequencies themselves: two encodings that fill them differently never share a table
        return ctx.shared(("rope_table", self.inv_freq.data_ptr(), self.rotary_dim),
                          lambda: ops.rope_table(self.inv_freq, ctx.pos, ctx.n_tokens))


def _project(part, h, w, ctx, kv_view, n_heads, n_kv_heads, head_dim, inv_freq, rotary_dim, fusable, table=None):
    if fusable and part.dtype != torch.float32 and h.dtype == part.dtype:
        k = v = ptab = stride = None
        if n_kv_heads > 0:
            k, v, ptab, stride = kv_view.k, kv_view.v, kv_view.page_table, kv_view.page_stride
        return ops.linear_rope_store(h, w, inv_freq, rotary_dim, ctx.pos, ctx.tok_slot, ptab, stride, k, v,
                                     n_heads, n_kv_heads, head_dim, part.dtype, cos_sin=table)
    qkv = ops.linear(h, w, out_dtype=torch.float32)
    return part.rotate_store(qkv, ctx, kv_view, n_heads, n_kv_heads, head_dim)


@register_position("none")
class NoPosition(Part):
    """No position encoding: q passes unrotated, k and v are written as they are."""

    def __init__(self, *, prefix: str = "", dtype, device, **_):
        self.dtype, self.prefix = dtype, prefix

    def rotate_store(self, qkv, ctx, kv_view, n_heads, n_kv_heads, head_dim):
        k = v = table = stride = None
        if n_kv_heads > 0:
            k, v, table, stride = kv_view.k, kv_view.v, kv_view.page_table, kv_view.page_stride
        return ops.rope_store(qkv, None, 0, False, ctx.pos, ctx.tok_slot, table, stride, k, v, n_heads, n_kv_heads,
                              head_dim, self.dtype, kv_round=getattr(kv_view, "round_to", None))

    def project_rotate_store(self, h, w, ctx, kv_view, n_heads, n_kv_heads, head_dim):
        return _project(self, h, w, ctx, kv_view, n_heads, n_kv_heads, head_dim, None, 0, True)
