"""Registries: a part kind (a string in a ``PartSpec``) to the class that
builds it, one registry per category.  A new mixer, feed-forward, norm,
position encoding, block arrangement or part around the layers ("stream") is added by registering a class; the
model builder, the cache manager and the step function only see the
interfaces in ``parts.base``.
"""
from __future__ import annotations

from typing import Callable, Dict

CATEGORIES = ("mixer", "feed_forward", "norm", "position", "block", "stream")
_REGISTRY: Dict[str, Dict[str, Callable]] = {c: {} for c in CATEGORIES}


def register_part(category: str, kind: str, cls=None):
    """``register_part("mixer", "my_mixer", MyMixer)`` or as a decorator."""
    if category not in _REGISTRY:
        raise KeyError(f"unknown part category {category!r}; known: {', '.join(CATEGORIES)}")

    def _put(c):
        _REGISTRY[category][kind] = c
        return c
    return _put if cls is None else _put(cls)


def _register_own_parts() -> None:
    """The parts of this package register themselves when their modules load; whoever asks the registry first
    makes sure they have."""
    from . import attention, block, mlp, norm, rotary  # noqa: F401


def part_class(category: str, kind: str):
    if kind not in _REGISTRY.get(category, {}):
        _register_own_parts()
    try:
        return _REGISTRY[category][kind]
    except KeyError:
        known = ", ".join(sorted(_REGISTRY.get(category, {}))) or "(none)"
        raise KeyError(f"no {category} part of kind {kind!r} is registered; known: {known}") from None


def build_part(category: str, spec, **kw):
    """Instantiate ``spec`` (a PartSpec) of the given category."""
    return part_class(category, spec.kind)(**spec.params, **kw)
