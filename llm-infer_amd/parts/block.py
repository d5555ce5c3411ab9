from __future__ import annotations

from ..registry import register_block
from .base import Part


@register_block("pre_norm")
class PreNormBlock(Part):
    """x += mixer(norm(x)); x += feed_forward(norm(x))   (src/model/block.cpp:106-224)."""

    def __init__(self, mixer_norm, mixer, feed_forward_norm, feed_forward):
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.feed_forward_norm, self.feed_forward = feed_forward_norm, feed_forward

    def children(self):
        return [self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward]

    def forward(self, x, ctx, cache_view, owns_cache=True):
        self.mixer.forward(self.mixer_norm.forward(x), ctx, cache_view, x, owns_cache)
        self.feed_forward.forward(self.feed_forward_norm.forward(x), x)
