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


def find_gguf(path: str):
    """The GGUF file that ``path`` names: the file itself, or the only ``*.gguf`` of a folder."""
    if os.path.isfile(path) and path.endswith(".gguf"):
        return path
    if os.path.isdir(path):
        found = sorted(f for f in os.listdir(path) if f.endswith(".gguf"))
        if len(found) == 1:
            return os.path.join(path, found[0])
        if len(found) > 1:
            raise ConfigError(f"{path} holds several GGUF files ({', '.join(found)}): name one")
    return None


def config_from_folder(folder: str):
    """The configuration of a model folder (config.json), or of a GGUF file or the folder that
    holds one (the reference's own model format: its metadata is the configuration)."""
    path = os.path.join(folder, "config.json")
    if os.path.isfile(path):
        with open(path) as f:
            return config_from_dict(json.load(f))
    gguf = find_gguf(folder)
    if gguf is None:
        raise ConfigError(f"no config.json in {folder}")
    from .weights.gguf_io import GGUFFile
    f = GGUFFile(gguf)
    arch = f.metadata.get("general.architecture")
    if arch is None:
        raise ConfigError("Missing required metadata: general.architecture")      # src/gguf.cpp:219-223
    for cls in ARCHITECTURES.values():
        if getattr(cls, "gguf_architecture", None) == arch and hasattr(cls, "from_gguf"):
            shapes = {}
            for n in f.names():
                try:
                    shapes[n] = f.info(n)[1]
                except ValueError:
                    shapes[n] = None                # a tensor type that is not read: the loader will say so
            return cls.from_gguf(f.metadata, shapes)
    known = sorted({getattr(c, "gguf_architecture", None) for c in ARCHITECTURES.values()} - {None})
    raise ConfigError(f"unknown GGUF architecture {arch!r}; known: " + ", ".join(known))
