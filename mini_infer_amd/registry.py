"""Registries: one from an architecture's name to its model, and one per kind of part.

The architecture registry follows the reference's `ModelRegistry`
(models/__init__.py:24-70): the key is `config.architectures[0]`, an unknown
key raises `ValueError` listing what is supported.  The part registries are
what lets one model hold different mixers and feed-forwards in different
layers: a layer's description names each part by `kind`, and the kind is
looked up here.
"""

from __future__ import annotations

import logging
from typing import Any, Callable, Generic, TypeVar

logger = logging.getLogger(__name__)

T = TypeVar("T")


class Registry(Generic[T]):
    def __init__(self, what: str) -> None:
        self.what = what
        self._entries: dict[str, T] = {}

    def register(self, name: str, entry: T) -> T:
        if not name:
            raise ValueError(f"a {self.what} needs a non-empty name")
        existing = self._entries.get(name)
        if existing is not None and existing is not entry:
            logger.warning("%s %r is being overwritten", self.what, name)
        self._entries[name] = entry
        return entry

    def lookup(self, name: str) -> T:
        if name not in self._entries:
            _load_builtins()
        if name not in self._entries:
            raise ValueError(
                f"no {self.what} named {name!r}; supported: {sorted(self._entries)}"
            )
        return self._entries[name]

    def unregister(self, name: str) -> None:
        self._entries.pop(name, None)

    def names(self) -> list[str]:
        return sorted(self._entries)

    def __contains__(self, name: str) -> bool:
        return name in self._entries


def _load_builtins() -> None:
    """Import the packages whose import registers the built-in parts and architecture."""
    import mini_infer_amd.models  # noqa: F401
    import mini_infer_amd.parts  # noqa: F401


# name in config.json's `architectures[0]` -> Architecture (models/architecture.py)
ARCHITECTURES: Registry[Any] = Registry("architecture")
# kind -> callable(description: dict, dtype, device, shared: dict | None) -> part
MIXERS: Registry[Callable[..., Any]] = Registry("mixer")
FEED_FORWARDS: Registry[Callable[..., Any]] = Registry("feed-forward")
NORMS: Registry[Callable[..., Any]] = Registry("norm")
POSITION_ENCODINGS: Registry[Callable[..., Any]] = Registry("position encoding")
BLOCKS: Registry[Callable[..., Any]] = Registry("block arrangement")
EMBEDDINGS: Registry[Callable[..., Any]] = Registry("embedding")
HEADS: Registry[Callable[..., Any]] = Registry("output head")


def _decorator(registry: Registry[Any], name: str) -> Callable[[T], T]:
    def wrap(entry: T) -> T:
        registry.register(name, entry)
        return entry

    return wrap


def register_architecture(name: str) -> Callable[[T], T]:
    return _decorator(ARCHITECTURES, name)


def register_mixer(kind: str) -> Callable[[T], T]:
    return _decorator(MIXERS, kind)


def register_feed_forward(kind: str) -> Callable[[T], T]:
    return _decorator(FEED_FORWARDS, kind)


def register_norm(kind: str) -> Callable[[T], T]:
    return _decorator(NORMS, kind)


def register_position_encoding(kind: str) -> Callable[[T], T]:
    return _decorator(POSITION_ENCODINGS, kind)


def register_block(kind: str) -> Callable[[T], T]:
    return _decorator(BLOCKS, kind)


def register_embedding(kind: str) -> Callable[[T], T]:
    return _decorator(EMBEDDINGS, kind)


def register_head(kind: str) -> Callable[[T], T]:
    return _decorator(HEADS, kind)
