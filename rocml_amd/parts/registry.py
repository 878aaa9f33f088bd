"""Tables from a spec's ``kind`` to the builder of the part.

``register_*`` adds an entry; tests register toy parts this way without touching the
library's files.  A builder takes ``(spec, BuildContext)`` and returns the part.
"""
from __future__ import annotations

from typing import Any, Callable, Dict

from ..errors import ConfigError
from .base import BuildContext

_TABLES: Dict[str, Dict[str, Callable[[Any, BuildContext], Any]]] = {
    "mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "block": {}, "embedding": {}, "head": {},
}


def _register(table: str, kind: str, builder: Callable[[Any, BuildContext], Any]) -> None:
    _TABLES[table][kind] = builder


def register_mixer(kind, builder): _register("mixer", kind, builder)
def register_feed_forward(kind, builder): _register("feed_forward", kind, builder)
def register_norm(kind, builder): _register("norm", kind, builder)
def register_position(kind, builder): _register("position", kind, builder)
def register_block(kind, builder): _register("block", kind, builder)
def register_embedding(kind, builder): _register("embedding", kind, builder)
def register_head(kind, builder): _register("head", kind, builder)


def _build(table: str, kind: str, spec: Any, ctx: BuildContext) -> Any:
    builders = _TABLES[table]
    if kind not in builders:
        raise ConfigError(f"no {table.replace('_', '-')} of kind {kind!r} is registered; "
                          f"known: {', '.join(sorted(builders)) or 'none'}")
    return builders[kind](spec, ctx)


def build_mixer(spec, ctx): return _build("mixer", spec.kind, spec, ctx)
def build_feed_forward(spec, ctx): return _build("feed_forward", spec.kind, spec, ctx)
def build_norm(spec, ctx): return _build("norm", spec.kind, spec, ctx)
def build_position(spec, ctx): return _build("position", spec.kind, spec, ctx)
def build_block(spec, ctx): return _build("block", spec.arrangement, spec, ctx)
def build_embedding(spec, ctx): return _build("embedding", spec.kind, spec, ctx)
def build_head(spec, ctx): return _build("head", spec.kind, spec, ctx)
