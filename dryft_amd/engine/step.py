"""The step function: one batch of sequences, the tokens it brings, logits where wanted.

The reference has two entry points, ``prefill`` for prompts of one length and
``decode_step`` for one token per row (engine/dryft_qwen3/model.py:122-128, 190-198), and
runs unequal prompts as one call per length (engine/engine.py:172-186). Here one function
serves both: the sequences of a step either all start (their prompts, of any lengths,
packed into one batch of rows) or all go on by one token; that is what the generation
loop and the replay program ask of it. The function itself takes any mixture: a sequence
may bring a further portion of its prompt, of any length, while others bring one token.
Only the tokens given are run; everything earlier comes from the cache. Tokens are always
given by the caller, never fed back from the model's own choice.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from ..cache.store import CacheStore
from ..csrc import ops
from ..parts.base import HostBatch, StepContext
from .model import DecoderModel


@dataclass
class SeqStep:
    """One sequence's share of a step."""

    slot: int                 # its cache slot; -1: the sequence sits this step out (its row is dead)
    tokens: list[int]         # its next tokens (a dead sequence still brings one placeholder)
    want: list[int]           # places among ``tokens`` whose logits are asked for


class BatchBuffers:
    """Device arrays that describe a step, at fixed addresses, sized for given capacities."""

    def __init__(self, max_rows: int, max_seqs: int, device):
        i32 = dict(dtype=torch.int32, device=device)
        self.max_rows, self.max_seqs = max_rows, max_seqs
        self.tokens = torch.zeros(max_rows, **i32)
        self.row_seq = torch.zeros(max_rows, **i32)
        self.row_slot = torch.full((max_rows,), -1, **i32)
        self.row_pos = torch.zeros(max_rows, **i32)
        self.seq_slot = torch.full((max_seqs,), -1, **i32)
        self.q_len = torch.zeros(max_seqs, **i32)
        self.cu_rows = torch.zeros(max_seqs + 1, **i32)
        self.kv_len = torch.zeros(max_seqs, **i32)
        self.seq_start = torch.zeros(max_seqs, **i32)


def stage_batch(cache: CacheStore, buf: BatchBuffers, slots: list[int], q_lens: list[int], tokens,
                dtype: torch.dtype) -> StepContext:
    """Host side of a step: room in the cache, the step's facts on the device, rows derived from them.

    ``slots[i] == -1`` marks a sequence that sits out; its ``q_lens[i]`` rows are dead. Advances the
    device's copy of the lengths; the caller records the same on the host with ``cache.end_step``
    once the model has run.
    """
    device = buf.tokens.device
    live = [(s, q) for s, q in zip(slots, q_lens) if s >= 0]
    live_slots, live_q = [s for s, _ in live], [q for _, q in live]
    if len(set(live_slots)) != len(live_slots):
        raise ValueError("a slot appears twice in one step")
    starts_live = cache.begin_step(live_slots, live_q)
    start_of = dict(zip(live_slots, starts_live))
    starts = [start_of.get(s, 0) for s in slots]
    n_rows, n_seqs = int(sum(q_lens)), len(slots)
    if n_rows > buf.max_rows or n_seqs > buf.max_seqs:
        raise ValueError(f"step of {n_rows} rows / {n_seqs} sequences exceeds the buffers ({buf.max_rows} / {buf.max_seqs})")
    # one staging array, one copy: tokens | seq_slot | q_len
    stage = torch.from_numpy(np.concatenate([np.asarray(tokens, dtype=np.int32), np.asarray(slots, dtype=np.int32),
                                             np.asarray(q_lens, dtype=np.int32)])).to(device)
    buf.tokens[:n_rows].copy_(stage[:n_rows])
    buf.seq_slot[:n_seqs].copy_(stage[n_rows:n_rows + n_seqs])
    buf.q_len[:n_seqs].copy_(stage[n_rows + n_seqs:])
    ctx = make_context(buf, n_rows, n_seqs, dtype, max_q_len=max(q_lens),
                       max_kv_len=max([st + q for st, q in zip(starts_live, live_q)], default=0),
                       host=HostBatch(list(slots), list(q_lens), starts))
    derive_rows(cache, buf, ctx)
    return ctx


def make_context(buf: BatchBuffers, n_rows: int, n_seqs: int, dtype: torch.dtype, *, max_q_len: int,
                 max_kv_len: int, host: HostBatch | None) -> StepContext:
    return StepContext(n_rows=n_rows, n_seqs=n_seqs, dtype=dtype, device=buf.tokens.device,
                       row_seq=buf.row_seq, row_slot=buf.row_slot, row_pos=buf.row_pos, cu_rows=buf.cu_rows,
                       seq_slot=buf.seq_slot, q_len=buf.q_len, kv_len=buf.kv_len,
                       seq_start=buf.seq_start, max_q_len=max_q_len, max_kv_len=max_kv_len,
                       host=host)


def derive_rows(cache: CacheStore, buf: BatchBuffers, ctx: StepContext) -> None:
    """Per-row facts from per-sequence facts, on the device; advances the device's lengths."""
    ops.prepare_batch(buf.seq_slot, buf.q_len, cache.lengths_dev, ctx.n_seqs, ctx.n_rows, buf.cu_rows,
                      buf.kv_len, buf.seq_start, buf.row_seq, buf.row_slot, buf.row_pos)


class Stepper:
    """Owns a model and its cache and runs steps on them."""

    def __init__(self, model: DecoderModel, cache: CacheStore):
        self.model, self.cache = model, cache
        self.device = model.device
        self.vocab = model.plan.vocab_size
        self._buffers: BatchBuffers | None = None
        ops.preload(model.kernel_modules())
        model.prepare_positions(cache.max_len)

    def _buffers_for(self, rows: int, seqs: int) -> BatchBuffers:
        b = self._buffers
        if b is None or b.max_rows < rows or b.max_seqs < seqs:
            b = BatchBuffers(max(rows, b.max_rows if b else 0, 64), max(seqs, b.max_seqs if b else 0, 8), self.device)
            self._buffers = b
        return b

    def step(self, seqs: list[SeqStep]) -> torch.Tensor:
        """Runs the step and returns float32 logits ``[sum(len(want)), vocab]`` in order."""
        if not seqs:
            return torch.empty((0, self.vocab), dtype=torch.float32, device=self.device)
        tokens: list[int] = []
        wanted: list[int] = []
        for s in seqs:
            if not s.tokens:
                raise ValueError("a sequence in a step must bring at least one token")
            for w in s.want:
                if not 0 <= w < len(s.tokens):
                    raise ValueError(f"wanted place {w} is outside the {len(s.tokens)} tokens given")
                if s.slot >= 0:
                    wanted.append(len(tokens) + w)
            tokens.extend(s.tokens)
        tok = np.asarray(tokens, dtype=np.int64)
        if tok.min() < 0 or tok.max() >= self.vocab:
            raise ValueError(f"token ids must lie in [0, {self.vocab}); got {int(tok.min())}..{int(tok.max())}")
        slots = [s.slot for s in seqs]
        q_lens = [len(s.tokens) for s in seqs]
        buf = self._buffers_for(len(tokens), len(seqs))
        ctx = stage_batch(self.cache, buf, slots, q_lens, tok, self.model.dtype)
        # the wanted rows are picked before the final norm; when every row is wanted in order, nothing is picked
        rows = None if wanted == list(range(ctx.n_rows)) else torch.tensor(wanted, dtype=torch.int32, device=self.device)
        hidden = self.model.forward(buf.tokens[:ctx.n_rows], ctx, self.cache, rows)
        self.cache.end_step([s for s in slots if s >= 0], [q for s, q in zip(slots, q_lens) if s >= 0])
        if not wanted:
            return torch.empty((0, self.vocab), dtype=torch.float32, device=self.device)
        return self.model.logits(hidden)

    def run(self, buf: BatchBuffers, ctx: StepContext, rows: torch.Tensor | None = None) -> torch.Tensor:
        """The device work of a step whose facts already sit in ``buf`` (what a captured graph holds); the hidden
        states after the final norm, of every row or of ``rows``."""
        ctx.forget_derived()
        derive_rows(self.cache, buf, ctx)
        return self.model.forward(buf.tokens[:ctx.n_rows], ctx, self.cache, rows)
