"""One registry from an architecture's name to its model, and registries of
the parts a model is put together from.

An architecture is registered as (config reader, model builder): the reader
turns the raw config.json dictionary into a typed configuration, the builder
turns that configuration into a `ModelSpec` (parts and the order they run in).
The reference has no registry: it branches on `model_type` strings
(src/models/config.cpp:34-36).
"""
from __future__ import annotations

from typing import Any, Callable, Dict, Tuple

_ARCHITECTURES: Dict[str, Tuple[Callable[[dict], Any], Callable[[Any], Any]]] = {}
_PARTS: Dict[str, Dict[str, Callable[..., Any]]] = {
    "mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "block": {},
}


def register_architecture(name: str, read_config: Callable[[dict], Any],
                          build: Callable[[Any], Any]) -> None:
    """Make `architectures[0] == name` resolve to this reader and builder."""
    _ARCHITECTURES[name] = (read_config, build)


def architectures() -> Tuple[str, ...]:
    return tuple(sorted(_ARCHITECTURES))


def resolve_architecture(name: str) -> Tuple[Callable[[dict], Any], Callable[[Any], Any]]:
    if name not in _ARCHITECTURES:
        raise KeyError(f"architecture {name!r} is not registered; registered: "
                       f"{', '.join(architectures()) or '(none)'}")
    return _ARCHITECTURES[name]


def register_part(kind: str, name: str, factory: Callable[..., Any]) -> None:
    """Register a part factory under kind 'mixer', 'feed_forward', 'norm',
    'position' or 'block'."""
    if kind not in _PARTS:
        raise KeyError(f"unknown part kind {kind!r}; kinds: {', '.join(sorted(_PARTS))}")
    _PARTS[kind][name] = factory


def make_part(kind: str, name: str, **params: Any) -> Any:
    """Build a registered part from its parameters."""
    if kind not in _PARTS:
        raise KeyError(f"unknown part kind {kind!r}; kinds: {', '.join(sorted(_PARTS))}")
    if name not in _PARTS[kind]:
        raise KeyError(f"{kind} {name!r} is not registered; registered: "
                       f"{', '.join(sorted(_PARTS[kind])) or '(none)'}")
    return _PARTS[kind][name](**params)


def registered_parts(kind: str) -> Tuple[str, ...]:
    return tuple(sorted(_PARTS[kind]))
