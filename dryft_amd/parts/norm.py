"""RMSNorm: ``y = w * cast(x * rsqrt(mean(x^2) + eps))`` with float statistics.

Reference: engine/dryft_qwen3/model.py:28-32. The weight is a plain multiplier.
``add_forward`` is the reference's rotated pair "residual add, then the norm that
follows it" (model.py:144-148), done in one kernel.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from ..weights.spec import VECTOR
from . import register_part
from .base import Norm, Partials


class RMSNorm(Norm):
    def __init__(self, size: int, eps: float):
        self.size, self.eps = int(size), float(eps)
        self.weight: torch.Tensor | None = None

    def tensor_specs(self):
        return {"weight": ((self.size,), VECTOR, "ones")}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def kernel_modules(self, dtype):
        return ("norm",)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        y = torch.empty_like(x)
        ops.add_rmsnorm(x, None, self.weight, self.eps, None, y)
        return y

    def add_forward(self, res: torch.Tensor, delta):
        y = torch.empty_like(res)
        if isinstance(delta, Partials):
            ops.add_rmsnorm(res, delta.data, self.weight, self.eps, res, y, n_partials=delta.count)
        else:
            ops.add_rmsnorm(res, delta, self.weight, self.eps, res, y)
        return res, y                      # the residual stream is updated in place


register_part("rmsnorm", RMSNorm)
