"""Steps captured once and replayed: a decoding step per batch size, a prompts' step per number of rows.

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
        self._slots_there: list[int] | None = None          # the slots the device holds, when known

    def _body(self) -> torch.Tensor:
        hidden = self.stepper.run(self.buf, self.ctx)
        return self.stepper.model.logits(hidden, None)

    def capture(self, warm_runs: int = 2) -> None:
        self.buf.seq_slot.fill_(-1)
        self._slots_there = None
        self.graph, self.logits = capture_body(self._body, self.stepper.device, self.pool, warm_runs)

    @property
    def tokens(self) -> torch.Tensor:
        """Where the step reads its tokens (int32, on the device): whoever chooses a step's tokens may write them
        here for the next step and hand this very tensor to ``replay``, which then copies nothing."""
        return self.buf.tokens

    def replay(self, slots: list[int], tokens: list[int] | torch.Tensor) -> torch.Tensor:
        """Logits ``[batch, vocab]`` of one more token each; rows of dead sequences hold nothing of use.

        ``tokens`` are given by the host, or as an int32 tensor on the device (a previous step's choice).
        """
        n = self.batch
        stage = self._stages[self._turn]
        self._turn = (self._turn + 1) % len(self._stages)
        if isinstance(tokens, torch.Tensor):
            if tokens.data_ptr() != self.buf.tokens.data_ptr():
                self.buf.tokens.copy_(tokens, non_blocking=True)
        else:
            stage[:n] = torch.from_numpy(np.asarray(tokens, dtype=np.int32))
            self.buf.tokens.copy_(stage[:n], non_blocking=True)
        slots = list(slots)
        if slots != self._slots_there:                        # between two steps of a batch they rarely change
            stage[n:] = torch.from_numpy(np.asarray(slots, dtype=np.int32))
            self.buf.seq_slot.copy_(stage[n:], non_blocking=True)
            self._slots_there = slots
        self.graph.replay()
        return self.logits


def capture_body(body, device, pool, warm_runs: int):
    """Runs ``body`` a few times on a side stream, then once more under capture: ``(graph, what body returned)``."""
    side = torch.cuda.Stream(device=device)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(warm_runs):
            body()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, pool=pool):
        result = body()
    return graph, result


class PromptGraph:
    """The step in which sequences start, captured for ``n_seqs`` sequences and ``n_rows`` rows in all.

    A step of a few hundred rows is some three hundred kernel launches, which the host issues more slowly than the
    GPU runs them; captured, it is one launch (the reference warms its prompt path per shape for the same first-token
    time, engine/engine.py:114-124). Everything that varies (tokens, slots, rows per sequence, the rows whose logits
    are wanted) is read from device memory. A step with fewer sequences or rows is filled up with sequences that sit
    out (slot -1): they keep rows, which every kernel passes over. The logits come back at one row per sequence.
    """

    def __init__(self, stepper: Stepper, n_seqs: int, n_rows: int, pool=None):
        self.stepper, self.n_seqs, self.n_rows, self.pool = stepper, int(n_seqs), int(n_rows), pool
        dev = stepper.device
        # what a replay brings lies in one piece of device memory, so that one copy brings it:
        # tokens | seq_slot | q_len | the rows whose logits are wanted
        R, S = self.n_rows, self.n_seqs
        self._staged = torch.zeros(R + 3 * S, dtype=torch.int32, device=dev)
        self.buf = BatchBuffers(R, S, dev)
        self.buf.tokens, self.buf.seq_slot = self._staged[:R], self._staged[R:R + S]
        self.buf.q_len, self.want = self._staged[R + S:R + 2 * S], self._staged[R + 2 * S:]
        self.ctx: StepContext = make_context(self.buf, self.n_rows, self.n_seqs, stepper.model.dtype,
                                             max_q_len=self.n_rows, max_kv_len=stepper.cache.max_len, host=None)
        self.logits: torch.Tensor | None = None
        self.graph: torch.cuda.CUDAGraph | None = None
        self._stage = torch.zeros(R + 3 * S, dtype=torch.int32).pin_memory()
        self._copied = torch.cuda.Event()

    def _body(self) -> torch.Tensor:
        hidden = self.stepper.run(self.buf, self.ctx, rows=self.want)
        return self.stepper.model.logits(hidden, None)

    def capture(self, warm_runs: int = 2) -> None:
        self.buf.seq_slot.fill_(-1)                       # warm runs and capture: one dead sequence owns every row
        self.buf.q_len.zero_()
        self.buf.q_len[0] = self.n_rows
        self.graph, self.logits = capture_body(self._body, self.stepper.device, self.pool, warm_runs)

    def replay(self, slots: list[int], tokens_of: list[list[int]]) -> torch.Tensor:
        """Logits ``[n_seqs, vocab]`` at the last token each sequence brings (rows beyond ``len(slots)`` hold nothing
        of use). The caller has made room in the cache (``begin_step``) and records the step afterwards."""
        n, rows = len(slots), sum(len(t) for t in tokens_of)
        if n > self.n_seqs or rows > self.n_rows or (n == self.n_seqs and rows < self.n_rows):
            raise ValueError(f"a step of {n} sequences and {rows} rows does not fit a captured step of "
                             f"{self.n_seqs} and {self.n_rows} (the rows left over need a sequence of their own)")
        R, S = self.n_rows, self.n_seqs
        self._copied.synchronize()                        # the previous replay's copy has read the staging memory
        stage = self._stage.numpy()
        stage[:] = 0
        at = 0
        for i, toks in enumerate(tokens_of):
            stage[at:at + len(toks)] = toks
            at += len(toks)
            stage[R + i] = slots[i]
            stage[R + S + i] = len(toks)
            stage[R + 2 * S + i] = at - 1                 # the sequence's last row
        stage[R + n:R + S] = -1                           # the sequences that fill the step up sit out;
        if n < S:
            stage[R + S + n] = R - rows                   # the first of them owns the rows left over
        self._staged.copy_(self._stage, non_blocking=True)
        self._copied.record()
        self.graph.replay()
        return self.logits
