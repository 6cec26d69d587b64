"""Registry of parts and of block arrangements.

``register_part(kind, cls)`` makes a class available to model plans under ``kind``;
``register_block(name, cls)`` does the same for an arrangement of parts in a layer.
Anything registered here (from inside the package or from user code) can be named
by a plan.
"""

from __future__ import annotations

from .base import (FeedForward, HostBatch, Mixer, Norm, Part, Partials, PositionEncoding, StepContext, matrix)

_PARTS: dict[str, type] = {}
_BLOCKS: dict[str, type] = {}


def register_part(kind: str, cls: type, replace: bool = False) -> None:
    if kind in _PARTS and not replace:
        raise ValueError(f"part kind {kind!r} is already registered")
    _PARTS[kind] = cls


def register_block(name: str, cls: type, replace: bool = False) -> None:
    if name in _BLOCKS and not replace:
        raise ValueError(f"block {name!r} is already registered")
    _BLOCKS[name] = cls


def part_class(kind: str) -> type:
    try:
        return _PARTS[kind]
    except KeyError:
        raise KeyError(f"no part registered as {kind!r}; known: {sorted(_PARTS)}") from None


def block_class(name: str) -> type:
    try:
        return _BLOCKS[name]
    except KeyError:
        raise KeyError(f"no block registered as {name!r}; known: {sorted(_BLOCKS)}") from None


def build_part(spec) -> Part:
    return part_class(spec.kind)(**spec.args)


from . import attention, block, embedding, mlp, norm, rope  # noqa: E402,F401  (register the built-in parts)

__all__ = ["FeedForward", "HostBatch", "Mixer", "Norm", "Part", "Partials", "PositionEncoding", "StepContext", "matrix",
           "register_part", "register_block", "part_class", "block_class", "build_part"]
