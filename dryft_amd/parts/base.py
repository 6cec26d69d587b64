"""What a part is, and what it is told about a step.

A part (mixer, feed-forward, norm, position encoding, embedding, head) is built
from sizes and constants alone, names the tensors it needs by logical name, and
computes on packed rows. It never learns which model it is in: the model plan
maps logical tensor names to checkpoint names and wires the parts together.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

import torch

from ..weights.spec import MATRIX


@dataclass
class HostBatch:
    """The step as the host knows it (absent while a captured graph is replayed)."""

    slots: list[int]      # cache slot of each sequence, -1 for a sequence that sits out
    q_lens: list[int]     # rows each sequence occupies in this step
    starts: list[int]     # tokens each sequence had cached before the step


@dataclass
class StepContext:
    """Per-step facts shared by all parts. Index tensors are int32 on the device.

    Rows are the step's tokens, packed sequence after sequence. Row ``r`` belongs to
    sequence ``row_seq[r]`` in cache slot ``row_slot[r]`` (-1: takes no part) at
    position ``row_pos[r]``. ``cu_rows`` are prefix sums over sequences of rows;
    ``kv_len`` is each sequence's cached length after this step, ``seq_start`` before it.
    A part whose kernel walks the step in tiles of some number of rows asks ``tiles()``
    for the prefix sums of those.

    ``host`` is the step as the host knows it, or None while a captured step is replayed.
    A part must not let what it computes depend on whether ``host`` is there; it may only
    use it to do less (skip clearing rows that no sequence sitting out owns).
    """

    n_rows: int
    n_seqs: int
    dtype: torch.dtype
    device: torch.device
    row_seq: torch.Tensor
    row_slot: torch.Tensor
    row_pos: torch.Tensor
    cu_rows: torch.Tensor
    seq_slot: torch.Tensor
    q_len: torch.Tensor
    kv_len: torch.Tensor
    seq_start: torch.Tensor
    max_q_len: int                      # host bound on rows per sequence; 1 means a decoding step
    max_kv_len: int                     # host bound on any sequence's cached length after the step
    host: HostBatch | None = None
    positions: dict[str, Any] = field(default_factory=dict)   # name -> position encoding, tables ready
    _tiles: dict[int, tuple[torch.Tensor, int]] = field(default_factory=dict, repr=False)
    _kept: dict[Any, torch.Tensor] = field(default_factory=dict, repr=False)

    def tiles(self, rows_per_tile: int) -> tuple[torch.Tensor, int]:
        """For kernels that walk the step tile by tile: ``(tile_cu, bound)``. ``tile_cu`` (int32, device,
        ``n_seqs + 1`` entries) holds the prefix sums over the sequences of the tiles of ``rows_per_tile`` rows that
        their rows of this step fill (a sequence that sits out fills none); ``bound`` is what the host knows the
        total not to exceed (a grid size). Computed when first asked for, once per tile size and step."""
        from ..csrc import ops
        found = self._tiles.get(rows_per_tile)
        if found is None:
            tile_cu = torch.empty(self.n_seqs + 1, dtype=torch.int32, device=self.device)
            ops.tile_prefix(self.seq_slot, self.q_len, self.n_seqs, rows_per_tile, tile_cu)
            if self.host is not None:
                bound = sum(-(-q // rows_per_tile) for s, q in zip(self.host.slots, self.host.q_lens) if s >= 0)
            else:
                bound = self.n_seqs * -(-self.max_q_len // rows_per_tile)
            found = self._tiles[rows_per_tile] = (tile_cu, bound)
        return found

    def kept_zeros(self, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        """A tensor that starts as zeros and lives as long as the context, one per shape and dtype, shared by every
        part that asks: for an output of which a kernel writes only the rows of sequences that take part, while the
        other rows must hold something finite (zeros, or what an earlier step or layer left there) because products
        and norms downstream read whole rows. Cleared once, not once a layer. A part that hands such a tensor on must
        be done with it before the next part of the step asks for the same shape (the parts of a step run one after
        another on one stream, so a mixer's output that the same mixer's projection consumes qualifies)."""
        key = (tuple(shape), dtype)
        found = self._kept.get(key)
        if found is None:
            found = self._kept[key] = torch.zeros(shape, dtype=dtype, device=self.device)
        return found

    def forget_derived(self) -> None:
        """For a context that is used for more than one step: what ``tiles()`` has computed belongs to the step
        before."""
        self._tiles.clear()

    def some_sit_out(self) -> bool:
        """May the step hold sequences that sit out (slot -1)? Without the host's view: yes."""
        return self.host is None or any(s < 0 for s in self.host.slots)


@dataclass
class Partials:
    """A matrix product left as ``count`` float32 partial sums ``[count, rows, width]``."""

    data: torch.Tensor
    count: int

    def summed(self, dtype: torch.dtype) -> torch.Tensor:
        """The product itself, ``[rows, width]``: for a consumer that cannot add the partial sums on its way."""
        from ..csrc import ops
        out = torch.empty(self.data.shape[1:], dtype=dtype, device=self.data.device)
        return ops.sum_partials(self.data, out, self.count)


class Part:
    """Base of all parts. ``tensor_specs`` maps logical names to (shape, role, init)."""

    def tensor_specs(self) -> dict[str, tuple[tuple[int, ...], str, str]]:
        return {}

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        """Receives the tensors named by ``tensor_specs`` (on the device, in their held dtype)."""

    def kernel_modules(self, dtype: torch.dtype) -> tuple[str, ...]:
        """The kernel libraries this part will call, so they can be compiled together up front."""
        return ()

    # ---- what a step costs, for measurement (rooflines); nothing on the compute path reads these
    def reads_whole(self) -> bool:
        """Does a step read all of this part's tensors (a matrix product does; a row gather does not)?"""
        return True

    def flops(self, rows: int, spans: list[tuple[int, int]]) -> float:
        """Floating-point operations of one step of ``rows`` rows, whose sequences each bring ``q`` rows after
        ``start`` cached ones (``spans`` holds ``(start, q)``): by default two per row and matrix element."""
        if not self.reads_whole():
            return 0.0
        elements = sum(_numel(shape) for shape, role, _ in self.tensor_specs().values() if role == MATRIX)
        return 2.0 * rows * elements


class Norm(Part):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def add_forward(self, res: torch.Tensor, delta) -> tuple[torch.Tensor, torch.Tensor]:
        """``(res + delta, norm(res + delta))``; ``delta`` is a tensor like ``res`` or ``Partials``."""
        raise NotImplementedError


class Mixer(Part):
    """Mixes information across positions of a sequence; owns the cache line of each of its runs."""

    def cache_need(self):
        """What a run of this mixer keeps per sequence: a ``KVNeed``, a ``StateNeed``, None, or a dictionary from
        names of its own choosing to needs when it keeps several things (keys and values beside fixed-size state,
        two sets of keys with different windows)."""
        return None

    def forward(self, h: torch.Tensor, ctx: StepContext, line, writes_cache: bool):
        """``h`` is ``[rows, hidden]``; returns a tensor of the same shape or ``Partials``. ``line`` is the storage
        ``cache_need`` asked for: a ``KVLine``, a ``StateLine``, None, or a dictionary of those under the same names."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, ctx: StepContext):
        raise NotImplementedError


class PositionEncoding(Part):
    def prepare(self, n_positions: int, dtype: torch.dtype, device) -> None:
        """Build whatever tables are needed for positions ``0..n_positions-1``."""


def _numel(shape) -> int:
    n = 1
    for d in shape:
        n *= int(d)
    return n


def matrix(shape) -> tuple[tuple[int, ...], str, str]:
    return (tuple(shape), MATRIX, "normal")
