"""Registries by name: the kinds of parts a model is put together from, and the architectures.

A part kind (a mixer, a feed-forward, a norm, a position encoding, a block arrangement) is a class
registered under a short name; an architecture is registered under the name that config.json
carries in ``architectures[0]`` and knows how to read its own config keys and to describe its
layers as data (see parts.spec).  Tests and users add kinds without touching the package:
``MIXERS.register("my_mixer", MyMixer)``.
"""
from dataclasses import dataclass
from typing import Callable


@dataclass(frozen=True)
class Architecture:
    """name: what config.json calls the model; config_class: has ``from_dict(raw)`` (validating)
    and ``to_dict()``; build_spec: config -> parts.base.ModelSpec."""
    name: str
    config_class: type
    build_spec: Callable


class Registry:
    def __init__(self, what):
        self.what = what
        self._items = {}

    def register(self, name, obj=None):
        """``register(name, obj)`` or ``@register(name)``."""
        if obj is None:
            def deco(o):
                self._items[name] = o
                return o
            return deco
        self._items[name] = obj
        return obj

    def get(self, name):
        try:
            return self._items[name]
        except KeyError:
            raise KeyError(f"unknown {self.what} {name!r}; registered: {sorted(self._items)}") from None

    def __contains__(self, name):
        return name in self._items

    def names(self):
        return sorted(self._items)


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITIONS = Registry("position encoding")
BLOCKS = Registry("block arrangement")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("output head")
ARCHITECTURES = Registry("architecture")
