"""What a model expects of a checkpoint: one ``TensorSpec`` per tensor name."""

from __future__ import annotations

from dataclasses import dataclass

MATRIX = "matrix"        # a GEMM operand or embedding table: held in the compute dtype
VECTOR = "vector"        # norm weights and the like: bfloat16, or 32-bit if stored so
INT_TABLE = "int_table"  # integer lookup tables: int32


@dataclass(frozen=True)
class TensorSpec:
    name: str                      # name in the checkpoint
    shape: tuple[int, ...]
    role: str = MATRIX
    init: str = "normal"           # random-weights mode: "normal" or "ones"

    def __post_init__(self):
        if self.role not in (MATRIX, VECTOR, INT_TABLE):
            raise ValueError(f"{self.name}: unknown role {self.role!r}")
        if self.init not in ("normal", "ones"):
            raise ValueError(f"{self.name}: unknown init {self.init!r}")
