"""A decoder model assembled from a ``ModelSpec``: embedding, layers in the order of
the schedule, final norm, output head (src/model/model.cpp:60-99 is the reference's
single-token forward)."""
from __future__ import annotations

import torch

from .. import parts as _parts  # noqa: F401  (registers the built-in parts)
from ..config.spec import ModelSpec
from ..parts.base import Part, collect_params
from ..parts.block import SubLayer
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
        self.positions = {}            # layers whose position specs are equal share one part
        self.layers = []
        self.layer_mixers = []         # for each layer its mixers, in the order in which they run
        for ls in spec.layers:
            position = self._position(ls.position, dtype, dev)
            subs, mixers = [], []
            for sub in ls.sublayers:
                if sub.role == "mixer":
                    part = _make("mixer", sub.part, dtype, dev, position=position)
                    mixers.append(part)
                else:
                    part = _make("feed_forward", sub.part, dtype, dev)
                subs.append(SubLayer(sub.role, part,
                                     None if sub.norm is None else _make("norm", sub.norm, dtype, dev),
                                     None if sub.post_norm is None else _make("norm", sub.post_norm, dtype, dev)))
            self.layers.append(lookup("block", ls.block)(subs))
            self.layer_mixers.append(mixers)
        self.final_norm = _make("norm", spec.final_norm, dtype, dev)
        self.head = _make("head", spec.head, dtype, dev)
        self.schedule = list(spec.schedule)
        # what the cache keeps is counted in units: one for each mixer of each run of a layer
        self._unit, n = {}, 0
        for i, e in enumerate(self.schedule):
            if e.cache_from is not None and (len(self.layer_mixers[e.layer]) !=
                                             len(self.layer_mixers[self.schedule[e.cache_from].layer])):
                raise ValueError(f"schedule entry {i} reads the cache of entry {e.cache_from}, whose layer has "
                                 "another number of mixers")
            for k in range(len(self.layer_mixers[e.layer])):
                self._unit[i, k] = n
                n += 1
        self._table = collect_params(self)

    def _position(self, spec, dtype, dev):
        if spec is None:
            return None
        key = (spec.kind, spec.prefix, repr(sorted(spec.params.items())))
        if key not in self.positions:
            self.positions[key] = _make("position", spec, dtype, dev)
        return self.positions[key]

    # -- weights -----------------------------------------------------------
    def children(self):
        return [self.embedding, *self.positions.values(), *self.layers, self.final_norm, self.head]

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
        """For each unit (each mixer of each schedule entry, in order) what it asks of the cache
        (None: it reads another's)."""
        return [None if e.cache_from is not None else m.cache_spec()
                for e in self.schedule for m in self.layer_mixers[e.layer]]

    # -- the forward pass of one step ---------------------------------------
    def forward(self, ctx, cache) -> torch.Tensor:
        """Runs the step's tokens through the schedule; returns float32 logits [n_want, vocab]."""
        x = self.embedding.forward(ctx)
        for i, e in enumerate(self.schedule):
            owner = i if e.cache_from is None else e.cache_from
            views = [cache.view(self._unit[owner, k]) for k in range(len(self.layer_mixers[e.layer]))]
            layer = self.layers[e.layer]
            if getattr(layer, "takes_next_norm", False):
                # the norm that reads the residual stream after this layer: the next layer's first
                nxt = self.layers[self.schedule[i + 1].layer] if i + 1 < len(self.schedule) else None
                first = getattr(nxt, "first_norm", None)
                layer.forward(x, ctx, views, e.cache_from is None, next_norm=first() if first else None)
            else:
                layer.forward(x, ctx, views, e.cache_from is None)
        if ctx.n_want == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=x.device)
        h = self.final_norm.forward(x, ctx.want_rows)
        return self.head.forward(h)
