from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import register_position
from .base import Part


@register_position("rope")
class RotaryPosition(Part):
    """Rotation of q and k by position: angle = pos * theta^(-i / rotary_dim) for the pair
    that starts at dimension i (include/kernels_cpu.hpp:82-100).  ``pairing`` "adjacent"
    rotates (i, i+1) as the reference does; "half" rotates (i/2, i/2 + rotary_dim/2), the order of
    a checkpoint whose q and k rows were never permuted for the reference (docs/gguf.md:487-493).

    The kernels rotate adjacent pairs only.  A half-paired model runs on them unchanged because a
    score is a sum over the dimensions of a head and does not care about their order: the mixer asks
    ``head_row_order`` once, when it binds its weights, and puts the rows of every q and k head into
    that order (row 2j <- row j, row 2j+1 <- row j + rotary_dim/2), after which pair j sits in
    (2j, 2j+1) with the same frequency as before.  Values and the output projection are untouched.

    A position encoding is a part like the others: it may own tensors (``params`` under its
    ``prefix``, handed over by ``bind``); this one owns none.  It keeps a table of one frequency per
    rotated pair; another encoding of this family (scaled, interpolated, with learned factors) only
    fills the table differently.  Layers whose position specs are equal share one instance.  Its
    duties towards a mixer: ``head_row_order`` (the order it wants the rows of a q or k head in, or
    None) and ``project_rotate_store`` / ``rotate_store``: rotate q and k of the step's tokens, write
    k and v into the layer's pages, and return q.
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

    def head_row_order(self, head_dim: int):
        """The order in which a mixer must keep the rows of each q and k head (new row i holds the
        checkpoint's row ``order[i]``), or None for the checkpoint's own order."""
        if self.pairing != "half" or self.rotary_dim == 0:
            return None
        half = self.rotary_dim // 2
        order = list(range(head_dim))
        for j in range(half):
            order[2 * j], order[2 * j + 1] = j, j + half
        return order

    def rotate_store(self, qkv, ctx, kv_view, n_heads, n_kv_heads, head_dim):
        k = v = table = stride = None
        if n_kv_heads > 0:
            k, v, table, stride = kv_view.k, kv_view.v, kv_view.page_table, kv_view.page_stride
        return ops.rope_store(qkv, self.inv_freq, self.rotary_dim, False, ctx.pos, ctx.tok_slot,
                              table, stride, k, v, n_heads, n_kv_heads, head_dim, self.dtype,
                              kv_round=getattr(kv_view, "round_to", None))

    def project_rotate_store(self, h, w, ctx, kv_view, n_heads, n_kv_heads, head_dim):
        """q, k, v = h W^T, rotated and stored (the rows of W's q and k heads in ``head_row_order``); with
        16-bit storage the rotation and the cache write happen in the product's epilogue."""
        return _project(self, h, w, ctx, kv_view, n_heads, n_kv_heads, head_dim, self.inv_freq, self.rotary_dim,
                        True, self._table(ctx))

    def step_table(self):
        """(key, frequencies) of the table of angles that this part will ask a step for, or None.  Whoever
        builds a step and knows its positions early (the recorded decode step's bookkeeping kernel) may fill
        the table itself and leave it in the step under that key."""
        if self.rotary_dim == 0 or self.dtype == torch.float32:
            return None
        # keyed by the frequencies themselves: two encodings that fill them differently never share a table
        return ("rope_table", self.inv_freq.data_ptr(), self.rotary_dim), self.inv_freq

    def _table(self, ctx):
        """cos and sin of every token's angles, computed once per step and shared by all layers that
        rotate with the same frequencies."""
        wanted = self.step_table()
        if wanted is None:
            return None
        return ctx.shared(wanted[0], lambda: ops.rope_table(self.inv_freq, ctx.pos, ctx.n_tokens))


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
