"""What a mixer asks of the cache.

The reference has one uniform key/value tensor for all layers
(engine/dryft_qwen3/cache.py:43-47). Here every cache line (one per writing run
of the schedule) states its need; lines with the same need form a group with
storage of its own.
"""

from __future__ import annotations

from dataclasses import dataclass

PAGE_TOKENS = 64  # a sequence's keys and values are stored in pages of this many positions


@dataclass(frozen=True)
class KVNeed:
    """Keys and values of every position, or of the last ``window`` positions."""

    num_kv_heads: int
    head_dim: int
    window: int | None = None


@dataclass(frozen=True)
class StateNeed:
    """State of fixed size per sequence, zero when a sequence starts."""

    shape: tuple[int, ...]
    dtype: str = "float32"


def pages_for(tokens: int) -> int:
    return (tokens + PAGE_TOKENS - 1) // PAGE_TOKENS
