"""The Python entry point, in the manner of the reference's ``Engine``.

``Engine(model_path).generate(input_ids, max_new_tokens)`` yields one list of token ids
per step, one id per sequence (reference: engine/engine.py:28-29, 138-140). What differs:
any model folder whose ``config.json`` names a registered architecture is accepted rather
than one pinned checkpoint; prompts of unequal length run in one step; sampling may use
a temperature; stop tokens may end sequences early; capacities are constructor arguments
instead of a global settings object (engine/dryft_qwen3/config.py:161-196), and a request
beyond them is an error rather than a fallback to a freshly allocated cache
(engine/engine.py:153-165).
"""

from __future__ import annotations

import sys
import time
from collections import OrderedDict
from typing import Any, Iterator, Sequence

import torch

from ..cache.spec import PAGE_TOKENS, pages_for
from ..cache.store import CacheStore
from ..config.base import read_config_json
from ..models import resolve_architecture
from ..sampling import Sampler
from ..weights.loader import load_tensors
from ..weights.random_init import random_tensors
from . import generate as loop
from .graph import DecodeGraph, PromptGraph
from .model import DecoderModel
from .step import SeqStep, Stepper

DEFAULT_MAX_LEN = 8192
SHORTEST_GRAPH_CONTEXT = 256       # captured decoding steps come in context ranges of 256, 512, 1,024, ... tokens
PROMPT_GRAPH_ROWS = (16, 32, 64, 96, 128, 192, 256, 384, 512)   # captured prompts' steps come in these many rows
DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def log(*parts: object) -> None:
    """Diagnostics go to stderr, as the reference's do (engine/dryft_qwen3/config.py:228-230)."""
    print("[engine]", *parts, file=sys.stderr, flush=True)


def default_batch_buckets(max_batch: int) -> tuple[int, ...]:
    """Batch sizes that captured decoding steps come in: every size up to 8, then four to an octave (10, 12, 14, 16,
    20, 24, ...), the largest batch last. A step of another size runs in the next bucket with dead rows to fill it, at
    most a quarter more rows than it has."""
    sizes, n = [], 1
    while n < max_batch:
        sizes.append(n)
        n += max(1, 1 << max(0, n.bit_length() - 3))
    return tuple(sizes) + (int(max_batch),)


def pick_bucket(buckets: Sequence[int], need: int) -> int:
    """The smallest bucket that holds ``need`` (the reference's rule, engine/dryft_qwen3/config.py:203-207)."""
    for b in buckets:
        if b >= need:
            return b
    raise ValueError(f"{need} exceeds the largest bucket ({buckets[-1] if buckets else None})")


def require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("dryft_amd computes on an AMD GPU only (there is no CPU path); no GPU is visible")
    return device


class PendingStep:
    """A launched decoding step: where its chosen tokens will be, and when."""

    def __init__(self, n: int, chosen: torch.Tensor):
        self.n = n                                            # how many of the entries are the batch's own
        self.chosen = chosen                                  # on the device: where the captured step reads its tokens
        self.host = torch.empty(chosen.numel(), dtype=torch.int32).pin_memory()
        self.done = torch.cuda.Event()
        self.sampler_state = None


class Engine:
    def __init__(self, model_path: str | None = None, *, config: dict[str, Any] | None = None,
                 seed: int | None = None, norm_std: float = 0.0, dtype: str = "bfloat16", max_batch: int = 32,
                 max_len: int | None = None, max_tokens: int | None = None, use_graph: bool = True,
                 batch_buckets: Sequence[int] | None = None, max_graphs: int | None = None,
                 prompt_graph_rows: int = 256, device: str = "cuda:0", verbose: bool = False):
        """``batch_buckets``: the batch sizes captured decoding steps are made for (default: see
        ``default_batch_buckets``; the reference's are 1, 2, 4, ... 32, engine/dryft_qwen3/config.py:169); the largest
        must be ``max_batch``. ``max_graphs``: how many captured steps are kept at most, the one used longest ago going
        first (default: one per bucket and range of context lengths, so none ever goes). ``prompt_graph_rows``: the
        prompts of a batch that together have at most this many tokens run as a captured step too (0: never); such
        steps are bound by the host's launches otherwise."""
        t0 = time.time()
        self.device = require_gpu(device)
        torch.cuda.set_device(self.device)
        if dtype not in DTYPES:
            raise ValueError(f"dtype must be one of {sorted(DTYPES)}, got {dtype!r}")
        self.dtype = DTYPES[dtype]
        if (model_path is None) == (config is None):
            raise ValueError("give either model_path (a folder with config.json and safetensors) or config and seed")
        raw = read_config_json(model_path) if model_path is not None else config
        arch = resolve_architecture(raw)
        self.config = arch.config_class.from_dict(raw)
        self.model = DecoderModel(arch.plan(self.config), self.dtype, self.device)
        specs = self.model.tensor_specs()
        if model_path is not None:
            tensors = load_tensors(model_path, specs, self.dtype, self.device, ignore=self.model.optional_names())
        else:
            if seed is None:
                raise ValueError("random weights need a seed")
            tensors = random_tensors(specs, seed, self.dtype, norm_std=norm_std, device=self.device)
        self.model.load(tensors)
        del tensors
        # The longest sequence a slot holds: what is asked for, bounded by what the architecture allows (the reference
        # reads max_position_embeddings as that bound, engine/dryft_qwen3/config.py:154). Asking for more is an error.
        limit = self.model.plan.max_positions
        if max_len is None:
            max_len = min(DEFAULT_MAX_LEN, limit) if limit else DEFAULT_MAX_LEN
        if limit and max_len > limit:
            raise ValueError(f"max_len {max_len} exceeds the {limit} positions this model allows")
        self.max_batch, self.max_len = int(max_batch), int(max_len)
        per_seq = pages_for(self.max_len) * PAGE_TOKENS
        self.max_tokens = int(max_tokens) if max_tokens is not None else self.max_batch * per_seq
        self.cache = CacheStore(self.model.cache_needs(), max_tokens=self.max_tokens, n_slots=self.max_batch,
                                max_len=self.max_len, dtype=self.dtype, device=self.device)
        self.stepper = Stepper(self.model, self.cache)
        self.use_graph = bool(use_graph)
        buckets = sorted(set(int(b) for b in batch_buckets)) if batch_buckets is not None else \
            list(default_batch_buckets(self.max_batch))
        if not buckets or buckets[0] < 1 or buckets[-1] != self.max_batch:
            raise ValueError(f"batch_buckets must be positive and end at max_batch ({self.max_batch}), got {buckets}")
        self.batch_buckets = tuple(buckets)
        self.max_graphs = int(max_graphs) if max_graphs is not None else len(buckets) * len(self.context_ranges())
        if self.max_graphs < 1:
            raise ValueError("max_graphs must be at least 1")
        # (batch bucket, context range) -> captured step, least recently used first; one memory pool for all of them,
        # since only one runs at a time
        self._graphs: OrderedDict[tuple[int, int], DecodeGraph] = OrderedDict()
        self._graph_pool = None
        self.prompt_graph_rows = int(prompt_graph_rows) if self.use_graph else 0
        self._prompt_graphs: OrderedDict[tuple[int, int], PromptGraph] = OrderedDict()   # (sequences, rows) -> step
        self._sampler = Sampler()
        self._last_choice: torch.Tensor | None = None
        if verbose:
            log(f"{arch.name} ready in {time.time() - t0:.1f}s: weights {self.model.weight_bytes() / 2**30:.2f} GiB, "
                f"cache {self.cache.bytes() / 2**30:.2f} GiB for {self.max_tokens} tokens")

    # ------------------------------------------------------------------ the step function
    def step(self, seqs: list[SeqStep]) -> torch.Tensor:
        return self.stepper.step(seqs)

    def tune(self, row_counts: Sequence[int]) -> None:
        """Lets the vendor library choose its kernels for steps of these many rows (a prompt of 2,048 tokens is a
        step of 2,048 rows; 64 sequences decoding are a step of 64): one step of stand-in tokens for each count,
        a few seconds each, nothing kept in the cache; counts beyond the longest sequence are spread over several
        sequences. The choice holds for exactly these counts; any other keeps
        the library's default. Only the bfloat16 products of more than 64 rows, and some of 17 to 64, are the
        library's; everything else is untouched."""
        from ..parts.linear import library_tuning
        with library_tuning():
            for rows in row_counts:
                rows = int(rows)
                n_seqs = max(1, -(-rows // self.max_len))
                if rows <= 0 or n_seqs > self.max_batch or (pages_for(rows) + n_seqs) * PAGE_TOKENS > self.max_tokens:
                    raise ValueError(f"a step of {rows} rows does not fit this engine "
                                     f"({self.max_batch} sequences of {self.max_len}, {self.max_tokens} tokens)")
                lengths = [rows // n_seqs + (i < rows % n_seqs) for i in range(n_seqs)]
                slots = self.acquire(n_seqs)
                try:
                    self.stepper.step([SeqStep(s, [0] * n, [n - 1]) for s, n in zip(slots, lengths)])
                    torch.cuda.synchronize()
                finally:
                    self.release(slots)
        self._graphs.clear()            # graphs captured before would keep the kernels chosen then
        self._prompt_graphs.clear()

    # ------------------------------------------------------------------ StepBackend
    def acquire(self, n: int) -> list[int]:
        return self.cache.acquire(n)

    def release(self, slots: list[int]) -> None:
        self.cache.release(slots)

    def reserve(self, slots: list[int], lengths: list[int]) -> None:
        self.cache.reserve(slots, lengths)

    def start(self, slots: list[int], prompts: list[list[int]], step_index: int) -> list[int]:
        graph = self._prompt_graph_for(len(slots), sum(len(p) for p in prompts))
        if graph is None:
            logits = self.stepper.step([SeqStep(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)])
            return self._choose(logits, len(slots))
        vocab = self.stepper.vocab
        for p in prompts:
            if not p:
                raise ValueError("a sequence in a step must bring at least one token")
            if min(p) < 0 or max(p) >= vocab:
                raise ValueError(f"token ids must lie in [0, {vocab}); got {min(p)}..{max(p)}")
        q_lens = [len(p) for p in prompts]
        self.cache.begin_step(slots, q_lens)
        logits = graph.replay(slots, prompts)
        self.cache.end_step(slots, q_lens)
        return self._choose(logits[:len(slots)], len(slots))

    def _prompt_graph_for(self, n_seqs: int, rows: int) -> PromptGraph | None:
        """The captured step for ``n_seqs`` sequences that start with ``rows`` tokens in all, or None where such steps
        run launch by launch: one per number of rows in ``PROMPT_GRAPH_ROWS`` (up to ``prompt_graph_rows``; they keep
        to the row counts at which the matrix products change kernels) and per power-of-two number of sequences (at
        least one more than the batch has, so that the rows left over have a sequence to belong to), captured when
        first asked for; they share the decoding steps' memory pool and their cap."""
        n_rows = next((r for r in PROMPT_GRAPH_ROWS if r >= rows), None)
        if n_rows is None or n_rows > self.prompt_graph_rows:
            return None
        seqs = 2
        while seqs < n_seqs + 1:
            seqs *= 2
        key = (seqs, n_rows)
        g = self._prompt_graphs.get(key)
        if g is None:
            while len(self._prompt_graphs) >= self.max_graphs:
                self._prompt_graphs.popitem(last=False)
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            g = PromptGraph(self.stepper, seqs, n_rows, pool=self._graph_pool)
            g.capture()
            self._prompt_graphs[key] = g
        self._prompt_graphs.move_to_end(key)
        return g

    def advance(self, slots: list[int], tokens: list[int], step_index: int) -> list[int]:
        if self.use_graph:
            return self.advance_end(self.advance_begin(slots, tokens, step_index))
        return self._advance_eager(slots, tokens)

    @property
    def chains(self) -> bool:
        """Can a step be launched before the one before it has been read? (Captured graphs only.)"""
        return self.use_graph

    def advance_begin(self, slots: list[int], tokens: list[int] | None, step_index: int) -> "PendingStep":
        """Launches one more token each and returns without waiting. ``tokens`` None: every sequence goes on
        with the token the step launched before this one chose for it, handed over on the device."""
        n = len(slots)
        live = [s for s in slots if s >= 0]
        lengths = self.cache.slots.lengths
        graph = self._graph_for(n, max((int(lengths[s]) + 1 for s in live), default=1))
        width = graph.batch                                   # the bucket: rows beyond ``n`` are dead
        slots = list(slots) + [-1] * (width - n)
        self.cache.begin_step(live, [1] * len(live))
        if tokens is None:
            if self._last_choice is None or self._last_choice.numel() != width:
                raise RuntimeError("no previous step of this batch to take the tokens from")
            logits = graph.replay(slots, self._last_choice)
        else:
            logits = graph.replay(slots, list(tokens) + [0] * (width - n))
        self.cache.end_step(live, [1] * len(live))
        # the tokens are chosen straight into the place the next step reads them from; the copy for the host is
        # queued before that step, which is the next to write there
        pending = PendingStep(n, graph.tokens)
        pending.sampler_state = self._sampler.state()
        uniforms = None
        if not self._sampler.greedy:                          # the dead rows of the bucket draw nothing
            uniforms = torch.cat([self._sampler.draw(n), torch.zeros(width - n)]) if width > n else self._sampler.draw(n)
        self._sampler.choose(logits, uniforms, out=pending.chosen)
        pending.host.copy_(pending.chosen, non_blocking=True)
        pending.done.record()
        self._last_choice = pending.chosen
        return pending

    def advance_end(self, pending: "PendingStep") -> list[int]:
        """The tokens a launched step chose (waits for that step only)."""
        pending.done.synchronize()
        return pending.host[:pending.n].tolist()

    def advance_drop(self, pending: "PendingStep") -> None:
        """Forgets the step launched last: its random numbers count as not drawn."""
        self._sampler.restore(pending.sampler_state)
        self._last_choice = None

    def _advance_eager(self, slots: list[int], tokens: list[int]) -> list[int]:
        n = len(slots)
        # dead sequences keep their row so that rows and sequences stay aligned
        logits = self.stepper.step([SeqStep(s, [t], [0]) for s, t in zip(slots, tokens)])
        if len(logits) != n:
            full = torch.zeros((n, logits.shape[1]), dtype=logits.dtype, device=logits.device)
            idx = torch.tensor([i for i, s in enumerate(slots) if s >= 0], dtype=torch.long, device=logits.device)
            full[idx] = logits
            logits = full
        return self._choose(logits, n)

    def _choose(self, logits: torch.Tensor, n: int) -> list[int]:
        uniforms = None if self._sampler.greedy else self._sampler.draw(n)
        return self._sampler.choose(logits, uniforms).tolist()

    def context_ranges(self) -> list[int]:
        """The context lengths captured steps are sized for: 256, 512, 1,024, ... and the slot length last."""
        ranges, reach = [], SHORTEST_GRAPH_CONTEXT
        while reach < self.max_len:
            ranges.append(reach)
            reach *= 2
        return ranges + [self.max_len]

    def _graph_for(self, batch: int, context: int | None = None) -> DecodeGraph | None:
        """The captured step for ``batch`` sequences whose longest will hold ``context`` tokens after the step
        (default: as long as the cache allows): one graph per batch bucket and power-of-two range of contexts,
        captured when first asked for and kept until ``max_graphs`` others have been used since."""
        if not self.use_graph:
            return None
        bucket = pick_bucket(self.batch_buckets, batch)
        reach = self.max_len if context is None else next((r for r in self.context_ranges() if r >= context), self.max_len)
        key = (bucket, reach)
        g = self._graphs.get(key)
        if g is None:
            while len(self._graphs) >= self.max_graphs:
                self._graphs.popitem(last=False)
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            g = DecodeGraph(self.stepper, bucket, reach, pool=self._graph_pool)
            g.capture()
            self._graphs[key] = g
        self._graphs.move_to_end(key)
        return g

    def warm(self, batch_sizes: Sequence[int] | None = None, contexts: Sequence[int] | None = None,
             prompts: Sequence[tuple[int, int]] = ()) -> int:
        """Captures decoding steps before the first request needs them, as the reference does when it is built
        (engine/dryft_qwen3/graphs.py:39-59): for the buckets of ``batch_sizes`` (default: every bucket) and the ranges
        of the context lengths ``contexts`` (default: every range); and the prompts' steps for ``prompts``, pairs of
        (sequences, tokens in all). Returns how many captured decoding steps are held then."""
        if not self.use_graph:
            return 0
        for n_seqs, rows in prompts:
            self._prompt_graph_for(int(n_seqs), int(rows))
        buckets = sorted(set(pick_bucket(self.batch_buckets, int(b)) for b in batch_sizes)) \
            if batch_sizes is not None else list(self.batch_buckets)
        ranges = self.context_ranges()
        reaches = sorted(set(next((r for r in ranges if r >= int(c)), self.max_len) for c in contexts)) \
            if contexts is not None else ranges
        if len(buckets) * len(reaches) > self.max_graphs:
            raise ValueError(f"{len(buckets)} x {len(reaches)} captured steps asked for, max_graphs is {self.max_graphs}")
        for reach in reaches:
            for bucket in buckets:
                self._graph_for(bucket, reach)
        return len(self._graphs)

    def prepare(self, n: int, shortest_context: int, longest_context: int) -> None:
        """What the generation loop says before a batch's first step: ``n`` sequences will decode at contexts between
        these two. Captures what is missing now, so that no capture falls between two decoding steps."""
        if self.use_graph:
            ranges = self.context_ranges()
            lo = next((r for r in ranges if r >= shortest_context), self.max_len)
            hi = next((r for r in ranges if r >= longest_context), self.max_len)
            wanted = [r for r in ranges if lo <= r <= hi]
            for reach in wanted[-self.max_graphs:]:
                self._graph_for(n, reach)

    # ------------------------------------------------------------------ generation
    def generate(self, input_ids: Sequence[Sequence[int]], max_new_tokens: int, *, temperature: float = 0.0,
                 sample_seed: int = 0, stop_token_ids: Sequence[int] = ()) -> Iterator[list[int]]:
        """Yields one list of ``len(input_ids)`` token ids per step as the steps are computed; ``-1`` stands where
        a sequence has nothing in that step: it has ended, or, when there are more prompts than ``max_batch``, its
        batch is not the one running (batches run one after another, each yielding its own steps)."""
        prompts = [list(map(int, p)) for p in input_ids]
        if not prompts or max_new_tokens <= 0:
            return
        self._sampler = Sampler(temperature, sample_seed)
        yield from loop.generate_steps(self, prompts, max_new_tokens, stop_token_ids)

    def generate_all(self, input_ids: Sequence[Sequence[int]], max_new_tokens: int, *, temperature: float = 0.0,
                     sample_seed: int = 0, stop_token_ids: Sequence[int] = ()) -> list[list[int]]:
        """Per request the list of tokens generated for it (a stop token included)."""
        self._sampler = Sampler(temperature, sample_seed)
        return loop.generate_all(self, [list(map(int, p)) for p in input_ids], max_new_tokens, stop_token_ids)
