"""A decoding step captured once per batch size and replayed.

The reference captures one graph per (batch bucket, length bucket) after three warm
runs on a side stream and checks a replay against eager (engine/dryft_qwen3/graphs.py:108-135,
146-169). Here every quantity that changes from step to step (tokens, slots, positions,
lengths, page tables) is read from device memory, so one graph per batch size serves
every position and length; the engine keeps one more per range of context lengths
(powers of two), because how attention cuts a sequence's keys into runs is fixed when a
graph is captured and should fit the sequences it runs on. Warm runs and the capture
itself run with every row marked dead (slot -1), which launches the same kernels but
writes to no cache slot and advances no length.
"""

from __future__ import annotations

import numpy as np
import torch

from ..parts.base import StepContext
from .step import BatchBuffers, Stepper, make_context


class DecodeGraph:
    def __init__(self, stepper: Stepper, batch_size: int, max_kv_len: int | None = None, pool=None):
        """``max_kv_len``: the longest sequence the graph is meant for (default: the longest the cache holds). Parts
        size their launches by it (attention: into how many runs a sequence's keys are cut); a replay on longer
        sequences is still right, only sized for shorter ones. ``pool``: a graph memory pool to share with other
        captured steps (only one of them may run at a time; what each returns stays its own)."""
        self.pool = pool
        self.stepper, self.batch = stepper, int(batch_size)
        dev = stepper.device
        self.buf = BatchBuffers(self.batch, self.batch, dev)
        self.buf.q_len.fill_(1)
        self.max_kv_len = min(int(max_kv_len), stepper.cache.max_len) if max_kv_len else stepper.cache.max_len
        self.ctx: StepContext = make_context(self.buf, self.batch, self.batch, stepper.model.dtype, max_q_len=1,
                                             max_kv_len=self.max_kv_len, host=None)
        self.logits: torch.Tensor | None = None
        self.graph: torch.cuda.CUDAGraph | None = None
        # Host-side staging for tokens and slots. Steps may be launched one ahead of the host reading their
        # results, so a buffer must not be rewritten while an earlier step's copy may still be waiting: four
        # take turns, and a step is only launched once the step before the previous one has been waited for.
        self._stages = [torch.zeros(2 * self.batch, dtype=torch.int32).pin_memory() for _ in range(4)]
        self._turn = 0

    def _body(self) -> torch.Tensor:
        hidden = self.stepper.run(self.buf, self.ctx)
        return self.stepper.model.logits(hidden, None)

    def capture(self, warm_runs: int = 2) -> None:
        self.buf.seq_slot.fill_(-1)
        side = torch.cuda.Stream(device=self.stepper.device)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warm_runs):
                self._body()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, pool=self.pool):
            self.logits = self._body()
        self.graph = graph

    def replay(self, slots: list[int], tokens: list[int] | torch.Tensor) -> torch.Tensor:
        """Logits ``[batch, vocab]`` of one more token each; rows of dead sequences hold nothing of use.

        ``tokens`` are given by the host, or as an int32 tensor on the device (a previous step's choice).
        """
        n = self.batch
        stage = self._stages[self._turn]
        self._turn = (self._turn + 1) % len(self._stages)
        stage[n:] = torch.from_numpy(np.asarray(slots, dtype=np.int32))
        if isinstance(tokens, torch.Tensor):
            self.buf.tokens.copy_(tokens, non_blocking=True)
        else:
            stage[:n] = torch.from_numpy(np.asarray(tokens, dtype=np.int32))
            self.buf.tokens.copy_(stage[:n], non_blocking=True)
        self.buf.seq_slot.copy_(stage[n:], non_blocking=True)
        self.graph.replay()
        return self.logits
