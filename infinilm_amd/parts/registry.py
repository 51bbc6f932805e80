"""Registries of part kinds.  `register_*` are decorators; `build_*` make a part from a PartSpec.
Adding a mixer, feed-forward, norm, position encoding, arrangement, embedding or output head is one
decorated class."""
from __future__ import annotations

from typing import Callable, Dict

from ..config.spec import PartSpec
from .base import BuildContext

MIXERS: Dict[str, Callable] = {}
FEED_FORWARDS: Dict[str, Callable] = {}
NORMS: Dict[str, Callable] = {}
POSITION_ENCODINGS: Dict[str, Callable] = {}
ARRANGEMENTS: Dict[str, Callable] = {}
EMBEDDINGS: Dict[str, Callable] = {}
HEADS: Dict[str, Callable] = {}


def _register(table: Dict[str, Callable], what: str):
    def outer(kind: str):
        def deco(cls):
            table[kind] = cls
            return cls
        return deco
    return outer


register_mixer = _register(MIXERS, "mixer")
register_feed_forward = _register(FEED_FORWARDS, "feed-forward")
register_norm = _register(NORMS, "norm")
register_position_encoding = _register(POSITION_ENCODINGS, "position encoding")
register_arrangement = _register(ARRANGEMENTS, "arrangement")
register_embedding = _register(EMBEDDINGS, "embedding")
register_head = _register(HEADS, "output head")


def _build(table: Dict[str, Callable], what: str, spec: PartSpec, ctx: BuildContext):
    try:
        cls = table[spec.kind]
    except KeyError:
        raise KeyError(f"unknown {what} kind {spec.kind!r}; registered: {sorted(table)}") from None
    return cls(ctx=ctx, **spec.params)


def build_mixer(spec, ctx):
    return _build(MIXERS, "mixer", spec, ctx)


def build_feed_forward(spec, ctx):
    return _build(FEED_FORWARDS, "feed-forward", spec, ctx)


def build_norm(spec, ctx):
    return _build(NORMS, "norm", spec, ctx)


def build_position_encoding(spec, ctx):
    return _build(POSITION_ENCODINGS, "position encoding", spec, ctx)


def build_embedding(spec, ctx):
    return _build(EMBEDDINGS, "embedding", spec, ctx)


def build_head(spec, ctx):
    return _build(HEADS, "output head", spec, ctx)
