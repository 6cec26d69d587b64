"""Reading a checkpoint by tensor name.

Shard discovery is the reference's (engine/dryft_qwen3/weights.py:52-61): the
files named by ``model.safetensors.index.json``, else every ``*.safetensors``
in the folder. Unlike the reference, which stops at the first bad tensor
(weights.py:73-75) and only warns about leftovers (weights.py:115-116), all
missing names, unexpected names and wrong shapes are gathered into one
``WeightError``; tensors are fetched one at a time rather than staged whole.

Storage rule: floating tensors are kept in bfloat16 when the compute dtype is
bfloat16 (weights.py:76-77); a vector the file stores in 32-bit stays 32-bit;
integer tables become int32. In the float32 mode every floating tensor is
widened to float32, which is exact.
"""

from __future__ import annotations

import glob
import json
import os
from typing import Iterable

import torch
from safetensors import safe_open

from .spec import INT_TABLE, MATRIX, TensorSpec, VECTOR


class WeightError(RuntimeError):
    """A checkpoint that does not fit the model; every finding is listed."""

    def __init__(self, where: str, missing: list[str], unexpected: list[str],
                 wrong_shape: list[tuple[str, tuple, tuple]], other: list[str] = ()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.other = list(other)
        lines = [f"checkpoint in {where} does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}):")
            lines += [f"    {n}" for n in self.missing]
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}):")
            lines += [f"    {n}" for n in self.unexpected]
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}):")
            lines += [f"    {n}: expected {tuple(e)}, file has {tuple(g)}" for n, e, g in self.wrong_shape]
        lines += [f"  {o}" for o in self.other]
        super().__init__("\n".join(lines))


def shard_files(model_dir: str) -> list[str]:
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.exists(index):
        with open(index, "r", encoding="utf-8") as f:
            weight_map = json.load(f)["weight_map"]
        return sorted({os.path.join(model_dir, v) for v in weight_map.values()})
    files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no .safetensors file in {model_dir}")
    return files


def stored_dtype_to_held(stored: torch.dtype, role: str, compute_dtype: torch.dtype) -> torch.dtype:
    """The dtype a tensor is held in, given how the file stores it."""
    if role == INT_TABLE:
        return torch.int32
    if compute_dtype == torch.float32:
        return torch.float32
    if role == VECTOR and stored in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


def load_tensors(model_dir: str, specs: Iterable[TensorSpec], compute_dtype: torch.dtype,
                 device: torch.device | str = "cpu", ignore: Iterable[str] = ()) -> dict[str, torch.Tensor]:
    """All tensors named by ``specs`` from the checkpoint in ``model_dir``.

    ``ignore`` names tensors that may be present without being used (a tied
    head's copy of the embedding); they are returned too when present.
    """
    specs = list(specs)
    by_name = {s.name: s for s in specs}
    ignore = set(ignore)
    where: dict[str, str] = {}
    handles = {}
    try:
        for path in shard_files(model_dir):
            h = safe_open(path, framework="pt", device="cpu")
            handles[path] = h
            for name in h.keys():
                where[name] = path
        missing = [s.name for s in specs if s.name not in where]
        unexpected = sorted(n for n in where if n not in by_name and n not in ignore)
        wrong = []
        other = []
        for s in specs:
            if s.name not in where:
                continue
            sl = handles[where[s.name]].get_slice(s.name)
            got = tuple(sl.get_shape())
            if got != tuple(s.shape):
                wrong.append((s.name, tuple(s.shape), got))
        if missing or unexpected or wrong:
            raise WeightError(model_dir, missing, unexpected, wrong, other)
        out: dict[str, torch.Tensor] = {}
        for name in list(by_name) + sorted(n for n in ignore if n in where):
            t = handles[where[name]].get_tensor(name)
            role = by_name[name].role if name in by_name else MATRIX
            if role == INT_TABLE:
                if t.is_floating_point():
                    raise WeightError(model_dir, [], [], [], [f"{name}: integer table stored as {t.dtype}"])
            elif not t.is_floating_point():
                raise WeightError(model_dir, [], [], [], [f"{name}: floating tensor stored as {t.dtype}"])
            held = stored_dtype_to_held(t.dtype, role, compute_dtype)
            out[name] = t.to(device=device, dtype=held).contiguous()
        return out
    finally:
        handles.clear()
