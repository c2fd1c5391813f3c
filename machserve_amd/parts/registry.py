"""Registries from a spec's ``kind`` to the class that implements it, one per family of
parts.  ``build_*`` looks the kind up and constructs the part; an unknown kind is an error
that lists what is registered."""
from __future__ import annotations

from typing import Callable, Dict

from ..config.specs import ConfigError


class Registry:
    def __init__(self, family: str):
        self.family = family
        self._items: Dict[str, Callable] = {}

    def register(self, kind: str):
        def deco(cls):
            self._items[kind] = cls
            return cls
        return deco

    def get(self, kind: str):
        if kind not in self._items:
            raise ConfigError(f"no {self.family} of kind {kind!r}; registered: {sorted(self._items)}")
        return self._items[kind]

    def kinds(self):
        return sorted(self._items)

    def build(self, spec, *args, **kw):
        return self.get(spec.kind)(spec, *args, **kw)


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
BLOCKS = Registry("block arrangement")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("output head")

register_mixer = MIXERS.register
register_feed_forward = FEED_FORWARDS.register
register_norm = NORMS.register
register_position_encoding = POSITION_ENCODINGS.register
register_block = BLOCKS.register
register_embedding = EMBEDDINGS.register
register_head = HEADS.register
