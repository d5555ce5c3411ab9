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
    """

    def __init__(self, *, hidden_size, n_heads, n_kv_heads, head_dim, scale, window=None, position=None,
                 prefix, dtype, device):
        if n_heads % n_kv_heads != 0:
            raise ValueError("n_heads must be a multiple of n_kv_heads")
        if head_dim % 16 != 0 or not 16 <= head_dim <= 256:
            raise ValueError(f"head size {head_dim}: the attention kernels take multiples of 16 up to 256")
        self.hidden_size, self.n_heads, self.n_kv_heads, self.head_dim = hidden_size, n_heads, n_kv_heads, head_dim
        self.scale, self.window, self.position = float(scale), window, position
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.wqkv = self.wo = None

    def params(self):
        h, k, hd, d = self.n_heads, self.n_kv_heads, self.head_dim, self.hidden_size
        return {"q_proj.weight": ParamSpec((h * hd, d)), "k_proj.weight": ParamSpec((k * hd, d)),
                "v_proj.weight": ParamSpec((k * hd, d)), "o_proj.weight": ParamSpec((d, h * hd))}

    def bind(self, tensors):
        wqkv = torch.cat([tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]], 0)
        self.wqkv = ops.prepare_weight(wqkv)
        self.wq = self.wqkv.prefix(self.n_heads * self.head_dim) if isinstance(self.wqkv, ops.TiledWeight) \
            else self.wqkv[:self.n_heads * self.head_dim]
        self.wo = ops.prepare_weight(tensors["o_proj.weight"])

    def cache_spec(self):
        return KVSpec(self.n_kv_heads, self.head_dim, self.window)

    def forward(self, h, ctx, cache_view, residual, owns_cache=True):
        H, K, hd = self.n_heads, self.n_kv_heads, self.head_dim
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
