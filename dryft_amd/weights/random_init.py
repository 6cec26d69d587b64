"""Seeded random weights, and writing them out as a model folder.

The reference has random weights only in its tooling, through a library's
initialiser (agent/verify.py:36-54). Here one generator seeded with ``seed``
draws the tensors in the order of the model's tensor list: matrices and
embeddings from N(0, std), norm weights 1.0 or 1 + N(0, norm_std).
"""

from __future__ import annotations

import json
import os
from typing import Any, Iterable

import torch
from safetensors.torch import save_file

from .spec import INT_TABLE, TensorSpec


def random_tensors(specs: Iterable[TensorSpec], seed: int, dtype: torch.dtype = torch.bfloat16,
                   std: float = 0.02, norm_std: float = 0.0,
                   device: torch.device | str = "cpu") -> dict[str, torch.Tensor]:
    """Tensors for every spec; values depend on ``seed``, ``device`` kind and order only.

    Values are drawn in float32 and then rounded to ``dtype``, so a bfloat16
    folder and its float32 reading hold the same numbers.
    """
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    out: dict[str, torch.Tensor] = {}
    for s in specs:
        if s.role == INT_TABLE:
            raise ValueError(f"{s.name}: integer tables have no random initialiser")
        if s.init == "ones":
            t = torch.ones(s.shape, dtype=torch.float32, device=device)
            if norm_std:
                t += norm_std * torch.randn(s.shape, generator=gen, dtype=torch.float32, device=device)
        else:
            t = std * torch.randn(s.shape, generator=gen, dtype=torch.float32, device=device)
        out[s.name] = t.to(dtype)
    return out


def write_model_dir(path: str, config: dict[str, Any], tensors: dict[str, torch.Tensor]) -> str:
    """Writes ``config.json`` and ``model.safetensors`` into ``path``."""
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config, f, indent=1)
    save_file({k: v.detach().cpu().contiguous() for k, v in tensors.items()},
              os.path.join(path, "model.safetensors"))
    return path
