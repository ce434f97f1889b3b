"""Registries: an architecture's name (config.json "architectures") to what builds its model,
and a part's kind to the class that implements it.

The reference hard-wires its one model class (include/async_engine.h:40); here the model
class is looked up by name, and the same mechanism serves the parts of a layer, so that a
new mixer, feed-forward, norm, position encoding, block arrangement or whole architecture is
one ``register`` call and no change to existing files.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Generic, Iterable, TypeVar

T = TypeVar("T")


class RegistryError(KeyError):
    def __str__(self) -> str:  # KeyError would quote the message
        return self.args[0] if self.args else ""


class Registry(Generic[T]):
    def __init__(self, what: str):
        self.what = what
        self._items: Dict[str, T] = {}

    def register(self, name: str, item: T = None, *, replace: bool = False):
        """``register(name, item)`` or ``@register(name)`` above a class or function."""
        def put(obj: T) -> T:
            if name in self._items and not replace and self._items[name] is not obj:
                raise RegistryError(f"{self.what} '{name}' is already registered")
            self._items[name] = obj
            return obj
        if item is None:
            return put
        return put(item)

    def unregister(self, name: str) -> None:
        self._items.pop(name, None)

    def get(self, name: str) -> T:
        try:
            return self._items[name]
        except KeyError:
            known = ", ".join(sorted(self._items)) or "(none)"
            raise RegistryError(f"unknown {self.what} '{name}'; known: {known}") from None

    def names(self) -> Iterable[str]:
        return sorted(self._items)

    def __contains__(self, name: str) -> bool:
        return name in self._items


@dataclass(frozen=True)
class Architecture:
    """What the engine needs to know of an architecture.

    ``read_config`` turns the dict of config.json into the architecture's typed configuration;
    ``model_spec`` turns that configuration into a :class:`~lucciola_amd.config.specs.ModelSpec`.
    """

    name: str
    read_config: Callable[[Dict[str, Any]], Any]
    model_spec: Callable[[Any], Any]


ARCHITECTURES: Registry[Architecture] = Registry("architecture")
MIXERS: Registry[type] = Registry("mixer")
FEED_FORWARDS: Registry[type] = Registry("feed-forward")
NORMS: Registry[type] = Registry("norm")
POSITION_ENCODINGS: Registry[type] = Registry("position encoding")
BLOCKS: Registry[type] = Registry("block arrangement")
EMBEDDINGS: Registry[type] = Registry("embedding")
HEADS: Registry[type] = Registry("output head")

# the families a block's slots may name
FAMILIES = {"mixer": MIXERS, "feed_forward": FEED_FORWARDS, "norm": NORMS,
            "position": POSITION_ENCODINGS}


def architecture_for(config_dict: Dict[str, Any]) -> Architecture:
    names = config_dict.get("architectures")
    if not names or not isinstance(names, (list, tuple)):
        raise RegistryError("config.json: 'architectures' is missing or empty; known: "
                            + ", ".join(ARCHITECTURES.names()))
    return ARCHITECTURES.get(str(names[0]))
