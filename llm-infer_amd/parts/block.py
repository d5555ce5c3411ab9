from __future__ import annotations

from ..kernels import ops
from ..registry import register_block
from .base import Part


class SubLayer:
    """A built sub-layer: its part, what the part is to the engine ("mixer" or "feed_forward"), the norm
    on its input and the norm on its output (either may be None)."""

    def __init__(self, role: str, part, norm=None, post_norm=None):
        self.role, self.part, self.norm, self.post_norm = role, part, norm, post_norm

    def parts(self) -> list:
        return [p for p in (self.norm, self.part, self.post_norm) if p is not None]


class Block(Part):
    """An arrangement of sub-layers.  A block class is built from the list of its ``SubLayer``s and runs
    them on the float32 residual stream ``x`` [T, hidden] in place: ``forward(x, ctx, cache_views,
    owns_cache)``, where ``cache_views`` holds one view for each mixer of the layer, in their order."""

    def __init__(self, sublayers):
        self.sublayers = list(sublayers)

    def children(self):
        return [p for s in self.sublayers for p in s.parts()]

    def first_norm(self):
        """The norm that reads the residual stream first in this layer (None: the first part takes it raw)."""
        return self.sublayers[0].norm

    # the first of each kind, for layers of the common shape
    def _first(self, role):
        for s in self.sublayers:
            if s.role == role:
                return s
        return None

    @property
    def mixer(self):
        s = self._first("mixer")
        return s.part if s else None

    @property
    def mixer_norm(self):
        s = self._first("mixer")
        return s.norm if s else None

    @property
    def feed_forward(self):
        s = self._first("feed_forward")
        return s.part if s else None

    @property
    def feed_forward_norm(self):
        s = self._first("feed_forward")
        return s.norm if s else None


@register_block("pre_norm")
class PreNormBlock(Block):
    """x += part(norm(x)) for each sub-layer in turn; for the Llama layer: x += mixer(norm(x));
    x += feed_forward(norm(x))   (src/model/block.cpp:106-224)."""
    takes_next_norm = True          # forward accepts ``next_norm``

    def __init__(self, sublayers):
        super().__init__(sublayers)
        for s in self.sublayers:
            if s.norm is None or s.post_norm is not None:
                raise ValueError("a pre_norm block has one norm before each part and none after it")

    def forward(self, x, ctx, cache_views, owns_cache=True, next_norm=None):
        """``next_norm``: the norm that reads ``x`` after this layer, if the caller knows it."""
        views = iter(cache_views)
        for i, s in enumerate(self.sublayers):
            # a part that only passes its input on to ops.linear may get a norm whose last step is taken
            # inside that product (ops.LazyNorm)
            if getattr(s.part, "takes_lazy_norm", False) and getattr(s.norm, "can_be_lazy", False):
                h = s.norm.forward(x, lazy=True)
            else:
                h = s.norm.forward(x)
            # and the product that completes the rows of x may prepare the norm that reads them next
            after = self.sublayers[i + 1].norm if i + 1 < len(self.sublayers) else next_norm
            lazy_after = getattr(after, "can_be_lazy", False)
            ops.expect_norm(x, after.weight if lazy_after else None, after.eps if lazy_after else None)
            if s.role == "mixer":
                s.part.forward(h, ctx, next(views), x, owns_cache)
            else:
                s.part.forward(h, x)
