"""Registries of part kinds.

Each registry maps a key to a factory ``factory(spec: PartSpec, **context)``.
A new mixer, feed-forward, norm, position encoding, block arrangement,
embedding or head is added by registering it; no file of the framework changes.
"""

from __future__ import annotations

from typing import Callable, Generic, TypeVar

from .spec import PartSpec

T = TypeVar("T")


class Registry(Generic[T]):
    def __init__(self, what: str):
        self.what = what
        self._factories: dict[str, Callable[..., T]] = {}

    def register(self, key: str, factory: Callable[..., T] | None = None, *, replace: bool = False):
        """Use as ``REG.register("key", factory)`` or as a decorator."""

        def add(f):
            if key in self._factories and not replace:
                raise KeyError(f"{self.what} {key!r} is already registered")
            self._factories[key] = f
            return f

        return add(factory) if factory is not None else add

    def unregister(self, key: str) -> None:
        self._factories.pop(key, None)

    def build(self, spec: PartSpec, **context) -> T:
        try:
            factory = self._factories[spec.kind]
        except KeyError:
            known = ", ".join(sorted(self._factories)) or "(none)"
            raise KeyError(f"unknown {self.what} {spec.kind!r}; registered: {known}") from None
        return factory(spec, **context)

    def names(self) -> list[str]:
        return sorted(self._factories)

    def __contains__(self, key: str) -> bool:
        return key in self._factories


MIXERS: Registry = Registry("mixer")
FEED_FORWARDS: Registry = Registry("feed-forward")
NORMS: Registry = Registry("norm")
POSITION_ENCODINGS: Registry = Registry("position encoding")
BLOCKS: Registry = Registry("block arrangement")
EMBEDDINGS: Registry = Registry("embedding")
HEADS: Registry = Registry("head")
