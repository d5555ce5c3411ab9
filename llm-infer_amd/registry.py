"""Registries: architecture name -> configuration class, and part kind -> part class.

``architectures`` in config.json chooses the configuration class, whose
``model_spec()`` describes the model as data; the kinds named there are looked up
in the part registries.  Tests and users add entries with the ``register_*``
functions; nothing else in the framework has to change for a new part.

The reference has no registry: it only prints ``architectures``
(tools/hf_info.cpp:20-26) and gates on ``general.architecture == "llama"``
(src/gguf.cpp:88).
"""
from __future__ import annotations

import json
import os

from .config.spec import ConfigError

ARCHITECTURES: dict = {}
MIXERS: dict = {}
FEED_FORWARDS: dict = {}
NORMS: dict = {}
POSITIONS: dict = {}
BLOCKS: dict = {}
EMBEDDINGS: dict = {}
HEADS: dict = {}

_TABLES = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS, "position": POSITIONS,
           "block": BLOCKS, "embedding": EMBEDDINGS, "head": HEADS}


def register_architecture(name: str, config_cls) -> None:
    ARCHITECTURES[name] = config_cls


def _register(table_name: str, kind: str):
    def deco(cls):
        _TABLES[table_name][kind] = cls
        return cls
    return deco


def register_mixer(kind): return _register("mixer", kind)
def register_feed_forward(kind): return _register("feed_forward", kind)
def register_norm(kind): return _register("norm", kind)
def register_position(kind): return _register("position", kind)
def register_block(kind): return _register("block", kind)
def register_embedding(kind): return _register("embedding", kind)
def register_head(kind): return _register("head", kind)


def lookup(table_name: str, kind: str):
    table = _TABLES[table_name]
    if kind not in table:
        raise ConfigError(f"unknown {table_name} kind {kind!r}; registered: {sorted(table)}")
    return table[kind]


def config_from_dict(raw: dict):
    archs = raw.get("architectures")
    if not archs:
        raise ConfigError("config.json names no architecture (key 'architectures'); known: "
                          + ", ".join(sorted(ARCHITECTURES)))
    name = archs[0]
    if name not in ARCHITECTURES:
        raise ConfigError(f"unknown architecture {name!r}; known: " + ", ".join(sorted(ARCHITECTURES)))
    return ARCHITECTURES[name].from_dict(raw)


def config_from_folder(folder: str):
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {folder}")
    with open(path) as f:
        return config_from_dict(json.load(f))
