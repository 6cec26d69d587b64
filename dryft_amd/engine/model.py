"""A decoder assembled from a model plan.

The reference's model is two hand-written forward functions over one fixed layer
type (engine/dryft_qwen3/model.py:122-265). Here the model is whatever the plan says:
parts are built per layer from the registry, tensors are requested by the names the
plan gives, and layers run in the order of the schedule.
"""

from __future__ import annotations

import torch

from ..config.plan import ModelPlan
from ..parts import block_class, build_part
from ..parts.base import Partials, StepContext
from ..weights.spec import TensorSpec
from ..csrc import ops


class DecoderModel:
    def __init__(self, plan: ModelPlan, dtype: torch.dtype, device):
        plan.validate()
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"compute dtype must be float32 or bfloat16, got {dtype}")
        self.plan, self.dtype, self.device = plan, dtype, torch.device(device)
        self.embedding = build_part(plan.embedding)
        self.final_norm = build_part(plan.final_norm)
        self.head = build_part(plan.head)
        self.positions = {name: build_part(spec) for name, spec in plan.positions.items()}
        self.blocks = []
        self._bindings: list[tuple[object, dict[str, str]]] = []   # (part, logical -> checkpoint name)
        self._bindings.append((self.embedding, plan.embedding.tensors))
        for layer in plan.layers:
            cls = block_class(layer.block)
            missing = [r for r in cls.roles if r not in layer.parts]
            if missing:
                raise ValueError(f"block {layer.block!r} needs parts {missing}")
            parts = {role: build_part(layer.parts[role]) for role in cls.roles}
            self.blocks.append(cls(**parts))
            for role in cls.roles:
                self._bindings.append((parts[role], layer.parts[role].tensors))
        self._bindings.append((self.final_norm, plan.final_norm.tensors))
        self._bindings.append((self.head, plan.head.tensors))
        for name, part in self.positions.items():
            self._bindings.append((part, plan.positions[name].tensors))

    # ---- what the model wants from a checkpoint
    def tensor_specs(self) -> list[TensorSpec]:
        """Every checkpoint tensor the model reads, each once, in a fixed order."""
        specs: dict[str, TensorSpec] = {}
        for part, names in self._bindings:
            for logical, (shape, role, init) in part.tensor_specs().items():
                if logical not in names:
                    raise ValueError(f"{type(part).__name__}: the plan gives no checkpoint name for {logical!r}")
                spec = TensorSpec(names[logical], tuple(shape), role, init)
                seen = specs.get(spec.name)
                if seen is not None and (seen.shape != spec.shape or seen.role != spec.role):
                    raise ValueError(f"{spec.name}: requested as {seen.shape} and as {spec.shape}")
                specs[spec.name] = spec
        return list(specs.values())

    def optional_names(self) -> set[str]:
        """Tensors a checkpoint may hold without the model reading them (the plan lists them)."""
        return set(self.plan.optional_tensors)

    def load(self, tensors: dict[str, torch.Tensor]) -> None:
        """Hands every part its tensors. Parts whose plans name the same checkpoint tensor share it. ``tensors`` is
        emptied on the way: a tensor leaves it once the last part that reads it has loaded, so that a part which fuses
        several tensors into one of its own (and so no longer holds them) frees them there and then, and loading never
        holds much more than the weights themselves."""
        for extra, same_as in self.plan.optional_tensors.items():
            if extra in tensors and not torch.equal(tensors[extra], tensors[same_as]):
                # the reference's check of a tied head's copy (engine/dryft_qwen3/weights.py:86-87)
                raise ValueError(f"{extra} is present and differs from {same_as}, which the model reads in its place")
            tensors.pop(extra, None)
        readers: dict[str, int] = {}
        for part, names in self._bindings:
            for logical in part.tensor_specs():
                readers[names[logical]] = readers.get(names[logical], 0) + 1
        for part, names in self._bindings:
            wanted = [names[logical] for logical in part.tensor_specs()]
            part.load({logical: tensors[names[logical]] for logical in part.tensor_specs()})
            for name in wanted:
                readers[name] -= 1
                if readers[name] == 0:
                    tensors.pop(name, None)

    def kernel_modules(self) -> list[str]:
        mods = {"batch", "embed"}
        for part, _ in self._bindings:
            mods.update(part.kernel_modules(self.dtype))
        return sorted(mods)

    def weight_bytes(self) -> int:
        seen, total = set(), 0
        for part, _ in self._bindings:
            for v in vars(part).values():
                if isinstance(v, torch.Tensor) and v.data_ptr() not in seen:
                    seen.add(v.data_ptr())
                    total += v.numel() * v.element_size()
        return total

    def streamed_weight_bytes(self) -> int:
        """Bytes of the tensors that every step reads whole, each counted once (the decode roofline's weights)."""
        seen, total = set(), 0
        for part, _ in self._bindings:
            if not part.reads_whole():
                continue
            for v in vars(part).values():
                if isinstance(v, torch.Tensor) and v.data_ptr() not in seen:
                    seen.add(v.data_ptr())
                    total += v.numel() * v.element_size()
        return total

    def step_flops(self, spans: list[tuple[int, int]], logit_rows: int) -> float:
        """Floating-point operations of a step whose sequences bring ``q`` rows after ``start`` cached ones
        (``spans`` of ``(start, q)``) and whose logits are wanted at ``logit_rows`` rows."""
        rows = sum(q for _, q in spans)
        total = self.head.flops(logit_rows, spans)
        for run in self.plan.schedule:
            for part in self.blocks[run.layer].parts().values():
                total += part.flops(rows, spans)
        return total

    # ---- what the model wants from the cache
    def cache_needs(self) -> dict[int, object]:
        needs: dict[int, object] = {}
        for run in self.plan.schedule:
            if run.writes_cache:
                needs[run.cache_line] = self.blocks[run.layer].mixer.cache_need()
        return needs

    def prepare_positions(self, n_positions: int) -> None:
        for part in self.positions.values():
            part.prepare(n_positions, self.dtype, self.device)

    # ---- compute
    def forward(self, tokens: torch.Tensor, ctx: StepContext, cache, rows: torch.Tensor | None = None) -> torch.Tensor:
        """Hidden states after the final norm, ``[rows, hidden]``: of every row of the step, or of ``rows`` alone
        (int32 indices into the step's rows, on the device), which are picked before the final norm so that it runs
        over nothing else."""
        ctx.positions = self.positions
        x = self.embedding.forward(tokens)
        pending = None
        for run in self.plan.schedule:
            x, pending = self.blocks[run.layer].forward(x, pending, ctx, cache.line(run.cache_line), run.writes_cache)
        if rows is not None:
            if rows.numel() == 0:                              # nothing is wanted: the layers have run, that is all
                return x[:0]
            x, pending = _pick_rows(x, rows), _pick_rows(pending, rows)
        if pending is None:
            return self.final_norm.forward(x)
        _, h = self.final_norm.add_forward(x, pending)
        return h

    def logits(self, hidden: torch.Tensor, rows: torch.Tensor | None = None) -> torch.Tensor:
        """Float32 logits of hidden states that have been through the final norm (at ``rows`` of them; None: all)."""
        return self.head.forward(hidden if rows is None else _pick_rows(hidden, rows))


def _pick_rows(x, rows: torch.Tensor):
    """Rows ``rows`` of a tensor ``[n, width]`` or of partial sums ``[count, n, width]`` (a row gather is what the
    embedding kernel does)."""
    if x is None:
        return None
    if isinstance(x, Partials):
        parts = x.data[:x.count]
        picked = torch.empty((x.count, rows.numel(), parts.shape[2]), dtype=parts.dtype, device=parts.device)
        return Partials(ops.embed_rows(rows, parts, picked), x.count)
    picked = torch.empty((rows.numel(), x.shape[1]), dtype=x.dtype, device=x.device)
    return ops.embed_rows(rows, x, picked)
