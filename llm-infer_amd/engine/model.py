"""A decoder model assembled from a ``ModelSpec``: embedding, layers in the order of
the schedule, final norm, output head (src/model/model.cpp:60-99 is the reference's
single-token forward)."""
from __future__ import annotations

import torch

from .. import parts as _parts  # noqa: F401  (registers the built-in parts)
from ..config.spec import ModelSpec
from ..parts.base import Part, collect_params
from ..registry import lookup


def _make(table: str, spec, dtype, device, **extra):
    return lookup(table, spec.kind)(**spec.params, prefix=spec.prefix, dtype=dtype, device=device, **extra)


class DecoderModel(Part):
    def __init__(self, spec: ModelSpec, dtype=torch.bfloat16, device="cuda", allocate: bool = True):
        spec.validate()
        self.spec, self.dtype = spec, dtype
        self.device = device if allocate else None
        dev = self.device
        self.embedding = _make("embedding", spec.embedding, dtype, dev)
        self.layers = []
        for ls in spec.layers:
            position = None
            if ls.position is not None:
                position = lookup("position", ls.position.kind)(**ls.position.params, dtype=dtype, device=dev)
            mixer = _make("mixer", ls.mixer, dtype, dev, position=position)
            ffn = _make("feed_forward", ls.feed_forward, dtype, dev)
            n1 = _make("norm", ls.mixer_norm, dtype, dev)
            n2 = _make("norm", ls.feed_forward_norm, dtype, dev)
            self.layers.append(lookup("block", ls.block)(n1, mixer, n2, ffn))
        self.final_norm = _make("norm", spec.final_norm, dtype, dev)
        self.head = _make("head", spec.head, dtype, dev)
        self.schedule = list(spec.schedule)
        self._table = collect_params(self)

    # -- weights -----------------------------------------------------------
    def children(self):
        return [self.embedding, *self.layers, self.final_norm, self.head]

    def recordable(self) -> bool:
        """True if every part's forward pass can be recorded into a graph."""
        stack = list(self.children())
        while stack:
            part = stack.pop()
            if not getattr(part, "recordable", True):
                return False
            stack += list(part.children()) if hasattr(part, "children") else []
        return True

    def params(self) -> dict:
        """Full tensor name -> ParamSpec of everything the model needs."""
        return {name: spec for name, (_, _, spec) in getattr(self, "_table", {}).items()}

    def ignorable_names(self) -> list:
        out = []
        stack = [self]
        while stack:
            p = stack.pop()
            out.extend(p.ignorable())
            stack.extend(p.children())
        return out

    def bind(self, tensors) -> None:
        """``tensors``: full tensor name -> tensor.  They are asked for part by part, so a mapping that
        makes each tensor when it is asked for (``weights.loader.OnDemand``) never holds more than one
        part's tensors beside what the parts keep."""
        per_part: dict = {}
        for name, (part, local, _) in self._table.items():
            per_part.setdefault(id(part), (part, []))[1].append((local, name))
        for part, names in per_part.values():
            part.bind({local: tensors[name] for local, name in names})
        if getattr(self.head, "tied", False):
            self.head.tie(self.embedding.weight)

    # -- cache -------------------------------------------------------------
    def cache_specs(self) -> list:
        """For each schedule entry what its mixer asks of the cache (None: reads another's)."""
        return [None if e.cache_from is not None else self.layers[e.layer].mixer.cache_spec()
                for e in self.schedule]

    # -- the forward pass of one step ---------------------------------------
    def forward(self, ctx, cache) -> torch.Tensor:
        """Runs the step's tokens through the schedule; returns float32 logits [n_want, vocab]."""
        x = self.embedding.forward(ctx.token_ids)
        for i, e in enumerate(self.schedule):
            owner = i if e.cache_from is None else e.cache_from
            self.layers[e.layer].forward(x, ctx, cache.view(owner), e.cache_from is None)
        if ctx.n_want == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=x.device)
        h = self.final_norm.forward(x, ctx.want_rows)
        return self.head.forward(h)
