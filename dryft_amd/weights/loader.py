"""Reading a checkpoint by tensor name.

Which files hold the checkpoint is decided as in the reference
(engine/dryft_qwen3/weights.py:52-61): ``model.safetensors.index.json`` if there
is one, else every ``*.safetensors`` in the folder; here the index is also what
says in which shard a tensor lives, so no shard is opened for its names.
Unlike the reference, which stops at the first bad tensor (weights.py:73-75) and only warns about leftovers (weights.py:115-116), all
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


class ShardSet:
    """Where each tensor of a checkpoint lives, and the open files it has been read from so far.

    With an index file the map from tensor name to shard is taken from it as it stands, and a shard is
    opened only when one of its tensors is asked for; without one every ``*.safetensors`` file of the
    folder is opened once to learn its names.
    """

    INDEX = "model.safetensors.index.json"

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        self.where: dict[str, str] = {}
        self._open: dict[str, object] = {}
        index_path = os.path.join(model_dir, self.INDEX)
        if os.path.isfile(index_path):
            with open(index_path, "r", encoding="utf-8") as f:
                for tensor_name, file_name in json.load(f)["weight_map"].items():
                    self.where[tensor_name] = os.path.join(model_dir, file_name)
            return
        paths = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
        if not paths:
            raise FileNotFoundError(f"no .safetensors file in {model_dir}")
        for path in paths:
            for tensor_name in self._handle(path).keys():
                self.where[tensor_name] = path

    def _handle(self, path: str):
        h = self._open.get(path)
        if h is None:
            h = self._open[path] = safe_open(path, framework="pt", device="cpu")
        return h

    def files(self) -> list[str]:
        return sorted(set(self.where.values()))

    def shape(self, name: str) -> tuple[int, ...] | None:
        """The stored shape, or None when the shard the index names does not hold the tensor."""
        h = self._handle(self.where[name])
        if name not in h.keys():
            return None
        return tuple(h.get_slice(name).get_shape())

    def tensor(self, name: str) -> torch.Tensor:
        return self._handle(self.where[name]).get_tensor(name)

    def close(self) -> None:
        self._open.clear()


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
    shards = ShardSet(model_dir)
    try:
        where = shards.where
        missing = [s.name for s in specs if s.name not in where]
        unexpected = sorted(n for n in where if n not in by_name and n not in ignore)
        wrong = []
        for s in specs:
            if s.name in where:
                got = shards.shape(s.name)
                if got is None:                       # the index names a shard that does not hold it
                    missing.append(s.name)
                elif got != tuple(s.shape):
                    wrong.append((s.name, tuple(s.shape), got))
        if missing or unexpected or wrong:
            raise WeightError(model_dir, missing, unexpected, wrong)
        out: dict[str, torch.Tensor] = {}
        for name in list(by_name) + sorted(n for n in ignore if n in where):
            t = shards.tensor(name)
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
        shards.close()
