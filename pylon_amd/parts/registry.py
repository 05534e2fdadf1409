"""Registries from a spec's ``kind`` to the class that implements it.

A model is put together by looking up each spec of a :class:`LayerSpec` here, so a new
mixer, feed-forward, norm, position encoding or block arrangement is added by
registering a class; no file of the framework has to change.  Two more families hold what
a model may do outside its layers: "stream" parts work on the embedded tokens before the
first layer, "logits" parts on the logits after the vocabulary head.
"""
from __future__ import annotations

from typing import Callable, Dict

_FAMILIES = ("mixer", "feed_forward", "norm", "position", "block", "stream", "logits")
_PARTS: Dict[str, Dict[str, Callable]] = {family: {} for family in _FAMILIES}


def register_part(family: str, kind: str, factory: Callable, *, replace: bool = False) -> Callable:
    """``factory(spec, dtype=..., device=...)`` builds the part for specs of ``kind``."""
    if family not in _PARTS:
        raise ValueError(f"unknown part family {family!r}; families: {', '.join(_FAMILIES)}")
    if kind in _PARTS[family] and not replace:
        raise ValueError(f"{family} kind {kind!r} is already registered")
    _PARTS[family][kind] = factory
    return factory


def unregister_part(family: str, kind: str) -> None:
    _PARTS[family].pop(kind, None)


def build_part(family: str, spec, **kwargs):
    kind = getattr(spec, "kind", None)
    try:
        factory = _PARTS[family][kind]
    except KeyError:
        known = ", ".join(sorted(_PARTS.get(family, {}))) or "none"
        raise ValueError(f"no {family} of kind {kind!r} is registered (known: {known})") from None
    return factory(spec, **kwargs)


def registered(family: str):
    return tuple(sorted(_PARTS[family]))
