"""Two kinds of registry, both plain dictionaries filled by decorators.

`ARCHITECTURES` maps the name in config.json's `architectures[0]` to the configuration class
that reads that architecture's keys and turns them into a `ModelSpec`.  The part registries map
a `PartSpec.kind` to the class that builds the part.  A new architecture registers a
configuration class; a new part registers itself; nothing else in the package changes.
"""
from __future__ import annotations

from typing import Any, Callable, Mapping

from .errors import invalid_config

ARCHITECTURES: dict[str, Any] = {}
MIXERS: dict[str, Any] = {}
FEED_FORWARDS: dict[str, Any] = {}
NORMS: dict[str, Any] = {}
POSITION_ENCODINGS: dict[str, Any] = {}
BLOCKS: dict[str, Any] = {}
EMBEDDINGS: dict[str, Any] = {}
HEADS: dict[str, Any] = {}

_TABLES = {"architecture": ARCHITECTURES, "mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS,
           "position_encoding": POSITION_ENCODINGS, "block": BLOCKS, "embedding": EMBEDDINGS, "head": HEADS}


def register(table: str, name: str) -> Callable:
    """`@register("mixer", "attention")` puts the decorated class into the mixers' table."""
    registry = _TABLES[table]

    def decorate(cls):
        registry[name] = cls
        return cls
    return decorate


def lookup(table: str, name: str):
    registry = _TABLES[table]
    if name not in registry:
        known = ", ".join(sorted(registry)) or "none"
        raise invalid_config(f"unsupported {table} '{name}' (registered: {known})")
    return registry[name]


def config_from_dict(raw: Mapping[str, Any]):
    """Chooses the configuration class by `architectures[0]`; without that key, by
    `model_type` == "llama" (the only key the reference checks, src/model_config.cpp:25-27)."""
    architectures = raw.get("architectures")
    if isinstance(architectures, list) and architectures and isinstance(architectures[0], str):
        name = architectures[0]
    elif raw.get("model_type") == "llama":
        name = "LlamaForCausalLM"
    else:
        raise invalid_config("config.json names no architecture ('architectures' or model_type 'llama')")
    return lookup("architecture", name).from_dict(raw)
