"""Registries of the parts a block is made of.

Each family (norm, position, mixer, feed_forward, block, embedding, head) maps
a ``kind`` name to a class.  ``build_part(family, spec, ...)`` instantiates the
class named by ``spec.kind`` with ``spec.params`` and ``spec.tensors``.  A new
part is added with ``register_part(family, kind, cls)``; nothing else in the
framework needs to know of it.
"""
from __future__ import annotations

from typing import Any, Dict

FAMILIES = ("norm", "position", "mixer", "feed_forward", "block", "embedding", "head")
_PARTS: Dict[str, Dict[str, Any]] = {family: {} for family in FAMILIES}


def register_part(family: str, kind: str, cls, replace: bool = False) -> None:
    if family not in _PARTS:
        raise ValueError(f"unknown part family '{family}'; families: {', '.join(FAMILIES)}")
    if kind in _PARTS[family] and not replace:
        raise ValueError(f"{family} '{kind}' is already registered")
    _PARTS[family][kind] = cls


def unregister_part(family: str, kind: str) -> None:
    _PARTS[family].pop(kind, None)


def part_class(family: str, kind: str):
    try:
        return _PARTS[family][kind]
    except KeyError:
        raise ValueError(f"unknown {family} '{kind}'; registered: "
                         f"{', '.join(sorted(_PARTS[family]))}") from None


def build_part(family: str, spec, **extra):
    """Instantiate ``spec.kind`` of ``family``; ``spec.params`` become keyword
    arguments, ``spec.tensors`` the ``tensors`` argument (role -> file name)."""
    cls = part_class(family, spec.kind)
    return cls(tensors=dict(spec.tensors), **dict(spec.params), **extra)
