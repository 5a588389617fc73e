"""The registries: architecture name -> how to read its configuration and describe its model,
and part kind -> the class that implements it.

The reference chooses a C++ class and an enum by a preset name in each demo
(demo/llama.cpp:31-43, include/nanoinfer/base/base.h:36-41); it has no table keyed by the
``architectures`` entry of ``config.json``.  Here that entry is the only selector, everywhere.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List

from .config.spec import ModelSpec
from .weights.random_init import InitRule


@dataclass
class Architecture:
    """All an architecture has to say: how its ``config.json`` is read, how its model is described
    as parts, and (as data) how its random weights are drawn.  The typed configuration needs a
    ``to_dict()`` that gives back ``config.json`` keys, for the random-weights mode's folder."""

    name: str
    config_from_dict: Callable[[Dict[str, Any]], Any]   # config.json -> typed configuration
    build_spec: Callable[[Any], ModelSpec]               # typed configuration -> model as data
    init: InitRule = field(default_factory=InitRule)     # distribution of each tensor of the random-weights mode


ARCHITECTURES: Dict[str, Architecture] = {}

# one table per family of parts; a part class is looked up by the ``kind`` of its spec
PART_FAMILIES = ("embedding", "norm", "position", "mixer", "feed_forward", "block", "head")
PARTS: Dict[str, Dict[str, type]] = {family: {} for family in PART_FAMILIES}


class RegistryError(KeyError):
    def __str__(self) -> str:  # KeyError would quote the whole message
        return self.args[0] if self.args else ""


def register_architecture(arch: Architecture) -> Architecture:
    ARCHITECTURES[arch.name] = arch
    return arch


def get_architecture(name: str) -> Architecture:
    try:
        return ARCHITECTURES[name]
    except KeyError:
        raise RegistryError(f"architecture {name!r} is not registered; known: {sorted(ARCHITECTURES)}") from None


def register_part(family: str, kind: str):
    """Class decorator: ``@register_part("mixer", "attention")``."""
    if family not in PARTS:
        raise RegistryError(f"no part family {family!r}; families: {list(PART_FAMILIES)}")

    def deco(cls):
        PARTS[family][kind] = cls
        cls.family = family
        cls.kind = kind
        return cls

    return deco


def get_part(family: str, kind: str) -> type:
    try:
        return PARTS[family][kind]
    except KeyError:
        known: List[str] = sorted(PARTS.get(family, {}))
        raise RegistryError(f"no {family} part of kind {kind!r} is registered; known: {known}") from None


def architecture_of(config_json: Dict[str, Any]) -> Architecture:
    archs = config_json.get("architectures")
    if not archs:
        raise RegistryError(f"config.json names no architecture; known: {sorted(ARCHITECTURES)}")
    return get_architecture(str(archs[0]))
