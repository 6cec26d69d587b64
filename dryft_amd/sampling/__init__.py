"""Choosing tokens from logits.

The reference is greedy only: ``logits.argmax(-1)``, ties to the lowest index
(engine/dryft_qwen3/model.py:187, 262; AGENTS.md:174-175). Temperature sampling is this
library's addition: ``p = softmax(logits / T)`` in float32 and an inverse-CDF draw with
one uniform number per sequence and step. The uniforms come from a CPU generator seeded
with ``seed`` and are drawn as one vector per step in the order of the batch, whether or
not a sequence is still running, so a sequence's draws depend on nothing but the seed,
its place in the batch and the step.
"""

from __future__ import annotations

import torch

from ..csrc import ops


class Sampler:
    def __init__(self, temperature: float = 0.0, seed: int = 0):
        if temperature < 0:
            raise ValueError(f"temperature must be >= 0, got {temperature}")
        self.temperature = float(temperature)
        self._gen = torch.Generator(device="cpu")
        self._gen.manual_seed(int(seed))
        self._staged: torch.Tensor | None = None

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0

    def draw(self, n: int) -> torch.Tensor:
        """The step's uniform numbers in [0, 1), one per sequence of the batch (CPU, float32)."""
        return torch.rand(n, generator=self._gen, dtype=torch.float32)

    def state(self) -> torch.Tensor:
        """Where the stream of uniform numbers stands; ``restore`` goes back there."""
        return self._gen.get_state()

    def restore(self, state: torch.Tensor) -> None:
        self._gen.set_state(state)

    def choose(self, logits: torch.Tensor, uniforms: torch.Tensor | None = None,
               out: torch.Tensor | None = None) -> torch.Tensor:
        """Token ids (int32, on the device) for float32 logits ``[rows, vocab]`` on the device."""
        rows = logits.shape[0]
        if out is None:
            out = torch.empty(rows, dtype=torch.int32, device=logits.device)
        if self.greedy:
            return ops.argmax_rows(logits, out)
        if uniforms is None:
            uniforms = self.draw(rows)
        if uniforms.device != logits.device:
            # through pinned memory, so that the copy is queued behind the step instead of the host waiting for it;
            # the staging tensor is kept alive until the copy has surely run (the next draws replace it)
            self._staged = uniforms.pin_memory()
            uniforms = self._staged.to(logits.device, non_blocking=True)
        return ops.sample_rows(logits, self.temperature, uniforms, out)
