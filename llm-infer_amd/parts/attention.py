from __future__ import annotations

import torch

from ..cache.specs import KVSpec
from ..kernels import ops
from ..registry import register_mixer
from ..weights.loader import ParamSpec
from .base import Part


@register_mixer("attention")
class Attention(Part):
    """Causal grouped-query attention over the cache (src/model/block.cpp:121-172):
    q, k, v projections without bias, rotation of q and k by the position part, keys and
    values into the cache, softmax(q.k * scale) over the keys a token may see, output
    projection added into the residual stream.  Query head h reads KV head h // (H // K).

    The three projections are one matrix product against the rows [Wq; Wk; Wv]; the sum
    for each row is unchanged by that.

    The attention kernels take head sizes in steps of 16 up to 256.  Any other head size (the reference's
    CPU path takes any, include/kernels_cpu.hpp:140-167) runs as the next multiple of 16: when the
    weights are bound every head gets zero rows in Wq, Wk and Wv and zero columns in Wo, so the
    dimensions added hold zeros in q, k and v, add nothing to a score and nothing to the output;
    ``scale`` and the rotated dimensions stay those of the true head size.
    """

    takes_lazy_norm = True      # the normed input goes to ops.linear as it comes
    prefill_recordable = True   # nothing here is planned on the host from a step's lengths but the tile list,
                                # which a recorded step brings along (ops.PREFILL_TILES_KEY)

    def __init__(self, *, hidden_size, n_heads, n_kv_heads, head_dim, scale, window=None, position=None,
                 prefix, dtype, device):
        if n_heads % n_kv_heads != 0:
            raise ValueError("n_heads must be a multiple of n_kv_heads")
        if not 1 <= head_dim <= 256:
            raise ValueError(f"head size {head_dim}: the attention kernels take head sizes up to 256")
        self.hidden_size, self.n_heads, self.n_kv_heads, self.head_dim = hidden_size, n_heads, n_kv_heads, head_dim
        self.padded_head_dim = (head_dim + 15) // 16 * 16        # what the kernels and the cache see
        self.scale, self.window, self.position = float(scale), window, position
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.wqkv = self.wo = None

    def params(self):
        h, k, hd, d = self.n_heads, self.n_kv_heads, self.head_dim, self.hidden_size
        return {"q_proj.weight": ParamSpec((h * hd, d)), "k_proj.weight": ParamSpec((k * hd, d)),
                "v_proj.weight": ParamSpec((k * hd, d)), "o_proj.weight": ParamSpec((d, h * hd))}

    def _pad_rows(self, w, heads, order=None):
        """[heads * hd, d] -> [heads * padded, d]: the rows of each head in ``order`` (the position part's
        wish for q and k heads, see ``RotaryPosition.head_row_order``), zero rows after each head's own."""
        hd, pad = self.head_dim, self.padded_head_dim
        if order is not None:
            index = torch.as_tensor(order, dtype=torch.long, device=w.device)
            w = w.view(heads, hd, w.shape[1])[:, index].reshape(heads * hd, w.shape[1])
        if pad == hd:
            return w
        out = torch.zeros((heads, pad, w.shape[1]), dtype=w.dtype, device=w.device)
        out[:, :hd] = w.view(heads, hd, w.shape[1])
        return out.view(heads * pad, w.shape[1])

    def bind(self, tensors):
        H, K, hd, pad = self.n_heads, self.n_kv_heads, self.head_dim, self.padded_head_dim
        wants = getattr(self.position, "head_row_order", None)
        order = wants(hd) if wants else None
        wqkv = torch.cat([self._pad_rows(tensors["q_proj.weight"], H, order),
                          self._pad_rows(tensors["k_proj.weight"], K, order),
                          self._pad_rows(tensors["v_proj.weight"], K)], 0)
        self.wqkv = ops.prepare_weight(wqkv)
        self.wq = self.wqkv.prefix(H * pad) if ops.is_tiled(self.wqkv) else self.wqkv[:H * pad]
        wo = tensors["o_proj.weight"]
        if pad != hd:                               # zero columns after each head's own
            full = torch.zeros((wo.shape[0], H, pad), dtype=wo.dtype, device=wo.device)
            full[:, :, :hd] = wo.view(wo.shape[0], H, hd)
            wo = full.view(wo.shape[0], H * pad)
        self.wo = ops.prepare_weight(wo)

    def cache_spec(self):
        return KVSpec(self.n_kv_heads, self.padded_head_dim, self.window)

    def forward(self, h, ctx, cache_view, residual, owns_cache=True):
        H, K, hd = self.n_heads, self.n_kv_heads, self.padded_head_dim
        if owns_cache:
            q = self.position.project_rotate_store(h, self.wqkv, ctx, cache_view, H, K, hd)
        else:                                   # reads another layer's keys and values
            q = self.position.project_rotate_store(h, self.wq, ctx, None, H, 0, hd)
        kv = cache_view.as_tuple()
        if self.dtype == torch.float32:
            a = ops.attention_f32(q, kv, ctx.pos, ctx.tok_slot, H, K, hd, self.scale, self.window)
        elif ctx.is_decode:
            a = ops.attention_decode(q, kv, ctx.seq_slot, ctx.seq_ctx, ctx.n_seqs, H, K, hd, self.scale,
                                     self.window, ctx.decode_splits(K, H))
        else:
            a = ops.attention_prefill(q, kv, ops.prefill_meta(ctx), H, K, hd, self.scale, self.window)
        ops.linear(a.view(a.shape[0], H * hd), self.wo, ops.EPI_ADD, out=residual)
