"""Registries of the parts a layer is put together from.

A part is chosen by the `kind` of its spec: `mixer`, `feed_forward`, `norm`,
`position` (encoding) and `block` (their arrangement).  A new part is added by
registering a class under a new kind; the engine, cache and loader find it through
these tables and ask it for what it needs (see `parts.base`).
"""
from __future__ import annotations

from typing import Dict

_TABLES: Dict[str, Dict[str, type]] = {
    "mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "block": {},
}


def register(category: str, kind: str, cls: type, replace: bool = False) -> None:
    table = _TABLES[category]
    if kind in table and not replace:
        raise ValueError(f"{category} kind '{kind}' is already registered")
    table[kind] = cls


def unregister(category: str, kind: str) -> None:
    _TABLES[category].pop(kind, None)


def lookup(category: str, kind: str) -> type:
    try:
        return _TABLES[category][kind]
    except KeyError:
        raise KeyError(f"no {category} registered under kind '{kind}'; "
                       f"known: {sorted(_TABLES[category])}") from None


def register_mixer(kind, cls, replace=False):
    register("mixer", kind, cls, replace)


def register_feed_forward(kind, cls, replace=False):
    register("feed_forward", kind, cls, replace)


def register_norm(kind, cls, replace=False):
    register("norm", kind, cls, replace)


def register_position(kind, cls, replace=False):
    register("position", kind, cls, replace)


def register_block(kind, cls, replace=False):
    register("block", kind, cls, replace)
