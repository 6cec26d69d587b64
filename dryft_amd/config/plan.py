"""The model plan: which parts make up each layer, and in which order layers run.

An architecture turns its typed configuration into a ``ModelPlan``. The plan is
plain data: every part is named by the key under which its class is registered
(``dryft_amd.parts``), carries its sizes and constants as arguments, and maps
its logical tensor names to names in the checkpoint. Layers may differ from
one another; the order of execution (``schedule``) may name a layer more than
once, and a run may read the cache that another run writes.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any


@dataclass(frozen=True)
class PartSpec:
    """One part: registry key, constructor arguments, logical → checkpoint names."""

    kind: str
    args: dict[str, Any] = field(default_factory=dict)
    tensors: dict[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: how the parts are arranged (``block``) and the parts themselves."""

    block: str
    parts: dict[str, PartSpec]


@dataclass(frozen=True)
class Run:
    """One entry of the schedule.

    ``layer`` indexes ``ModelPlan.layers``. ``cache_line`` names the storage the
    layer's mixer uses in this run; two runs with the same line share it, and
    only a run with ``writes_cache`` appends to it.
    """

    layer: int
    cache_line: int
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelPlan:
    vocab_size: int
    hidden_size: int
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    schedule: tuple[Run, ...]
    final_norm: PartSpec
    head: PartSpec
    positions: dict[str, PartSpec] = field(default_factory=dict)
    # Tensors a checkpoint may hold although the model reads them under another name: each maps to the name of
    # the tensor it has to equal when present (a tied head's copy of the embedding).
    optional_tensors: dict[str, str] = field(default_factory=dict)
    max_positions: int | None = None      # longest sequence the architecture allows; None: no bound of its own

    def validate(self) -> None:
        problems = []
        writers: dict[int, int] = {}
        for i, run in enumerate(self.schedule):
            if not 0 <= run.layer < len(self.layers):
                problems.append(f"schedule[{i}] names layer {run.layer}, plan has {len(self.layers)}")
            if run.writes_cache:
                if run.cache_line in writers:
                    problems.append(
                        f"schedule[{i}] and schedule[{writers[run.cache_line]}] both write cache line {run.cache_line}")
                writers[run.cache_line] = i
        for i, run in enumerate(self.schedule):
            if not run.writes_cache:
                w = writers.get(run.cache_line)
                if w is None or w > i:
                    problems.append(f"schedule[{i}] reads cache line {run.cache_line} before any run has written it")
        if problems:
            raise ValueError("invalid model plan:\n  " + "\n  ".join(problems))
