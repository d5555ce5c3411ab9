"""What a model is made of, as data.

An architecture turns its typed configuration into a ``ModelSpec``: for every
layer which mixer, feed-forward, norm and position encoding it has and with which
sizes and constants, under which tensor names its weights lie, and in which order
the layers run.  The engine builds parts from this description alone; no part is
told which model it is in.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any


class ConfigError(ValueError):
    """A configuration that cannot be built."""


@dataclass(frozen=True)
class PartSpec:
    """One part: its registered kind, its parameters, and the prefix of its tensor names."""
    kind: str
    params: dict = field(default_factory=dict)
    prefix: str = ""

    def with_prefix(self, prefix: str) -> "PartSpec":
        return PartSpec(self.kind, self.params, prefix)


@dataclass(frozen=True)
class SubLayerSpec:
    """One sub-layer: a part that reads the residual stream and adds to it, with the norm on its input
    and, if the arrangement has one, a norm on its output.  ``role`` says what the part is to the
    engine: a "mixer" looks at other tokens and may keep a cache, a "feed_forward" does not."""
    role: str
    part: PartSpec
    norm: PartSpec | None = None
    post_norm: PartSpec | None = None


@dataclass(frozen=True)
class LayerSpec:
    """One layer: its sub-layers in the order in which they run (any number of mixers and
    feed-forwards, each with its norms), how they are arranged (``block``), and the position encoding
    that its mixers are handed."""
    block: str
    sublayers: tuple
    position: PartSpec | None = None

    @classmethod
    def mixer_then_feed_forward(cls, block: str, mixer: PartSpec, feed_forward: PartSpec, mixer_norm: PartSpec,
                                feed_forward_norm: PartSpec, position: PartSpec | None = None) -> "LayerSpec":
        """The common layer of two sub-layers, each with a norm on its input."""
        return cls(block, (SubLayerSpec("mixer", mixer, mixer_norm),
                           SubLayerSpec("feed_forward", feed_forward, feed_forward_norm)), position)


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  ``cache_from`` names an earlier entry of the schedule whose
    cache this run reads instead of keeping one of its own."""
    layer: int
    cache_from: int | None = None


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    layers: tuple
    schedule: tuple
    final_norm: PartSpec
    head: PartSpec
    stop_token_ids: tuple = ()

    def validate(self) -> None:
        if not self.layers:
            raise ConfigError("a model needs at least one layer")
        for i, layer in enumerate(self.layers):
            if not layer.sublayers:
                raise ConfigError(f"layer {i} has no sub-layer")
            for sub in layer.sublayers:
                if sub.role not in ("mixer", "feed_forward"):
                    raise ConfigError(f"layer {i}: a sub-layer is a 'mixer' or a 'feed_forward', not {sub.role!r}")
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < len(self.layers):
                raise ConfigError(f"schedule entry {i} names layer {e.layer}, there are {len(self.layers)}")
            if e.cache_from is not None:
                if not 0 <= e.cache_from < i:
                    raise ConfigError(f"schedule entry {i} reads the cache of entry {e.cache_from}, "
                                      "which does not run before it")
                if self.schedule[e.cache_from].cache_from is not None:
                    raise ConfigError(f"schedule entry {i} reads the cache of entry {e.cache_from}, "
                                      "which keeps none of its own")
