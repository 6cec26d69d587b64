"""The generation loop: batches of unequal prompts, stop tokens, sequences that end early.

Contract of the reference (engine/engine.py:138-143, 199-203): ``generate(input_ids,
max_new_tokens)`` yields ``max_new_tokens`` lists of one token per sequence; the first
comes from the prompts' step, every later one from a decoding step; an empty prompt is a
``ValueError`` (engine.py:176-177). The reference never stops early (engine.py:139-140).
Here ``stop_token_ids`` may end a sequence: it emits the stop token, and from then on its
place in every yielded list holds ``FILL``; the loop ends when every sequence has ended or
the limit is reached. With no stop tokens the behaviour is the reference's.

The loop only decides; all computing is behind ``backend`` (see ``StepBackend``), so the
decisions can be tested without a GPU.
"""

from __future__ import annotations

from typing import Iterator, Protocol, Sequence

FILL = -1   # what an ended sequence shows in later steps


class StepBackend(Protocol):
    max_batch: int
    max_len: int

    def acquire(self, n: int) -> list[int]: ...
    def release(self, slots: list[int]) -> None: ...
    def reserve(self, slots: list[int], lengths: list[int]) -> None: ...
    def start(self, slots: list[int], prompts: list[list[int]], step_index: int) -> list[int]:
        """Runs the prompts in one step; returns the chosen next token of every sequence."""
    def advance(self, slots: list[int], tokens: list[int], step_index: int) -> list[int]:
        """One more token each; ``slots[i] == -1`` marks a sequence that has ended."""

    # A backend whose ``chains`` is true can also launch a step without waiting for it:
    #   advance_begin(slots, tokens or None, step_index) -> handle    (None: the tokens the step launched
    #                                                                  before this one chose, kept on the device)
    #   advance_end(handle) -> list[int]
    #   advance_drop(handle)                                           (a launched step whose result nobody wants)
    # A backend may also have ``prepare(n, shortest_context, longest_context)``: told before a batch's first step how
    # many sequences will decode and between which context lengths, it can get ready what those steps need.


def check_request(prompts: Sequence[Sequence[int]], max_new_tokens: int, max_len: int) -> None:
    for i, p in enumerate(prompts):
        if len(p) == 0:
            raise ValueError("empty prompt")          # engine/engine.py:176-177
        if len(p) + max_new_tokens > max_len:
            raise ValueError(f"prompt {i}: {len(p)} tokens + {max_new_tokens} new exceed the longest "
                             f"sequence the cache allows ({max_len})")


def generate_batch(backend: StepBackend, prompts: list[list[int]], max_new_tokens: int,
                   stop_token_ids: Sequence[int] = ()) -> Iterator[list[int]]:
    """One batch that fits the backend: yields one list of ``len(prompts)`` tokens per step."""
    n = len(prompts)
    if n == 0 or max_new_tokens <= 0:
        return
    if n > backend.max_batch:
        raise ValueError(f"{n} sequences exceed the largest batch ({backend.max_batch})")
    check_request(prompts, max_new_tokens, backend.max_len)
    stops = set(int(t) for t in stop_token_ids)
    slots = backend.acquire(n)
    try:
        # a sequence needs room for its prompt and for every token that is fed back (all but the last)
        backend.reserve(slots, [len(p) + max_new_tokens - 1 for p in prompts])
        if max_new_tokens > 1 and hasattr(backend, "prepare"):
            # decoding steps will see contexts from the shortest prompt plus one to the longest sequence's end
            backend.prepare(n, min(len(p) for p in prompts) + 1, max(len(p) for p in prompts) + max_new_tokens - 1)
        running = [True] * n
        tokens = backend.start(slots, [list(p) for p in prompts], 0)
        if getattr(backend, "chains", False):
            yield from _chained_steps(backend, slots, running, tokens, max_new_tokens, stops)
            return
        for step in range(max_new_tokens):
            if step > 0:
                live_slots = [s if r else -1 for s, r in zip(slots, running)]
                tokens = backend.advance(live_slots, [t if r else 0 for t, r in zip(tokens, running)], step)
            out = [int(t) if r else FILL for t, r in zip(tokens, running)]
            for i in range(n):
                if running[i] and out[i] in stops:
                    running[i] = False
            yield out
            if not any(running):
                return
    finally:
        backend.release(slots)


def _chained_steps(backend, slots: list[int], running: list[bool], tokens: list[int], max_new_tokens: int,
                   stops: set[int]) -> Iterator[list[int]]:
    """The same steps with one launched ahead: step ``s + 1`` starts before the host has seen what step ``s``
    chose, on the tokens that step ``s`` left on the device. A sequence that step ``s`` ends therefore still runs
    in step ``s + 1`` (its place in the cache was reserved anyway); that token is dropped and it sits out from
    step ``s + 2`` on. What is yielded is exactly what the unchained loop yields.
    """
    n = len(slots)

    def decide(step_tokens: list[int]) -> list[int]:
        out = [int(t) if r else FILL for t, r in zip(step_tokens, running)]
        for i in range(n):
            if running[i] and out[i] in stops:
                running[i] = False
        return out

    out = decide(tokens)                                      # step 0: the prompts' step
    yield out
    if max_new_tokens == 1 or not any(running):
        return
    live = [s if r else -1 for s, r in zip(slots, running)]
    ahead = backend.advance_begin(live, [t if r else 0 for t, r in zip(tokens, running)], 1)
    try:
        for step in range(1, max_new_tokens):
            current, ahead = ahead, None
            if step + 1 < max_new_tokens:                     # launched on what is known now; see above
                live = [s if r else -1 for s, r in zip(slots, running)]
                ahead = backend.advance_begin(live, None, step + 1)
            out = decide(backend.advance_end(current))
            yield out
            if not any(running):
                return
    finally:
        if ahead is not None:                                 # launched, never read: it takes back what it drew
            backend.advance_drop(ahead)


def plan_batches(n_requests: int, max_batch: int) -> list[range]:
    """Requests in order, cut into batches of at most ``max_batch``, one after another."""
    return [range(i, min(n_requests, i + max_batch)) for i in range(0, n_requests, max_batch)]


def generate_steps(backend: StepBackend, prompts: list[list[int]], max_new_tokens: int,
                   stop_token_ids: Sequence[int] = ()) -> Iterator[list[int]]:
    """Any number of requests, step by step: every yielded list has one place per request; the places of requests
    whose batch is not the one running hold ``FILL``. With one batch this is ``generate_batch``."""
    n = len(prompts)
    for batch in plan_batches(n, backend.max_batch):
        idx = list(batch)
        for step in generate_batch(backend, [prompts[i] for i in idx], max_new_tokens, stop_token_ids):
            if len(idx) == n:
                yield step
                continue
            out = [FILL] * n
            for i, t in zip(idx, step):
                out[i] = t
            yield out


def generate_all(backend: StepBackend, prompts: list[list[int]], max_new_tokens: int,
                 stop_token_ids: Sequence[int] = ()) -> list[list[int]]:
    """Any number of requests: per request the tokens it generated (stop token included)."""
    results: list[list[int]] = [[] for _ in prompts]
    for step in generate_steps(backend, prompts, max_new_tokens, stop_token_ids):
        for i, t in enumerate(step):
            if t != FILL:
                results[i].append(t)
    return results
