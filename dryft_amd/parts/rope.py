"""Rotary position encoding: the tables.

``inv_freq[i] = 1 / theta^(2i/dim)``, ``angle[p, i] = p * inv_freq[i]`` in float32,
``cos``/``sin`` of the angles, cast to the activation dtype (reference:
engine/dryft_qwen3/model.py:49-57). The reference stores ``cat(angle, angle)``; its two
halves are equal, so only ``[positions, dim/2]`` is kept here. The rotation itself
(pairs ``(j, j + dim/2)``, model.py:35-41) is applied by the attention part's fused kernel.
Tables are made once on the host with the float32 routines any plain implementation
would use, then uploaded.
"""

from __future__ import annotations

import torch

from . import register_part
from .base import PositionEncoding


class RotaryPositions(PositionEncoding):
    def __init__(self, dim: int, theta: float):
        if dim % 2:
            raise ValueError(f"rotary width must be even, got {dim}")
        self.dim, self.theta = int(dim), float(theta)
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None
        self.n_positions = 0

    def prepare(self, n_positions: int, dtype: torch.dtype, device) -> None:
        if self.cos is not None and n_positions <= self.n_positions and self.cos.dtype == dtype:
            return
        inv_freq = 1.0 / (self.theta ** (torch.arange(0, self.dim, 2, dtype=torch.int64).to(torch.float32) / self.dim))
        pos = torch.arange(n_positions, dtype=torch.float32)
        angle = pos[:, None] * inv_freq[None, :]
        self.cos = angle.cos().to(dtype).to(device).contiguous()
        self.sin = angle.sin().to(dtype).to(device).contiguous()
        self.n_positions = n_positions


register_part("rotary", RotaryPositions)
