"""The generation loop's decisions, driven by a scripted backend (no GPU)."""

import pytest

from dryft_amd.engine.generate import (FILL, check_request, generate_all, generate_batch, generate_steps,
                                       plan_batches)


class Scripted:
    """A backend whose 'model' continues each prompt by counting up from its last token."""

    def __init__(self, max_batch=4, max_len=64, fail_at=None):
        self.max_batch, self.max_len = max_batch, max_len
        self.free = list(range(max_batch))
        self.log = []
        self.fail_at = fail_at
        self.last = {}

    def acquire(self, n):
        assert n <= len(self.free)
        out = [self.free.pop(0) for _ in range(n)]
        self.log.append(("acquire", tuple(out)))
        return out

    def release(self, slots):
        assert not set(slots) & set(self.free), "released twice"
        self.free.extend(slots)
        self.log.append(("release", tuple(slots)))

    def reserve(self, slots, lengths):
        self.log.append(("reserve", tuple(lengths)))

    def start(self, slots, prompts, step_index):
        self.log.append(("start", tuple(len(p) for p in prompts)))
        for s, p in zip(slots, prompts):
            self.last[s] = p[-1]
        return self._next(slots)

    def advance(self, slots, tokens, step_index):
        if self.fail_at == step_index:
            raise RuntimeError("boom")
        self.log.append(("advance", tuple(slots), tuple(tokens)))
        for s, t in zip(slots, tokens):
            if s >= 0:
                assert t == self.last[s], "the loop must feed back the token it was given"
        return self._next(slots)

    def _next(self, slots):
        out = []
        for s in slots:
            if s >= 0:
                self.last[s] += 1
            out.append(self.last[s] if s >= 0 else 12345)      # a dead row's token is garbage and must be ignored
        return out


def test_yields_exactly_max_new_tokens_lists_without_stop_tokens():
    be = Scripted()
    steps = list(generate_batch(be, [[5], [10, 20], [7, 7, 7]], 4))
    assert steps == [[6, 21, 8], [7, 22, 9], [8, 23, 10], [9, 24, 11]]
    assert be.log[0] == ("acquire", (0, 1, 2)) and be.log[-1] == ("release", (0, 1, 2))
    assert ("reserve", (4, 5, 6)) in be.log                   # prompt + tokens that are fed back
    assert [e[0] for e in be.log].count("advance") == 3       # the first token comes from the prompts' step
    assert sorted(be.free) == [0, 1, 2, 3]


def test_stop_token_ends_one_sequence_and_the_rest_go_on():
    be = Scripted()
    steps = list(generate_batch(be, [[5], [20], [7]], 6, stop_token_ids=[22, 9]))
    assert steps == [[6, 21, 8], [7, 22, 9], [8, FILL, FILL], [9, FILL, FILL]]   # 9 stops the first one too
    advances = [e for e in be.log if e[0] == "advance"]
    assert advances[1][1] == (0, -1, -1)                       # ended sequences sit out with slot -1
    assert sorted(be.free) == [0, 1, 2, 3]


def test_loop_ends_when_every_sequence_has_ended():
    be = Scripted()
    steps = list(generate_batch(be, [[1], [1]], 50, stop_token_ids=[3]))
    assert steps == [[2, 2], [3, 3]]


def test_empty_requests_and_limits():
    be = Scripted(max_batch=2, max_len=10)
    assert list(generate_batch(be, [], 5)) == [] and list(generate_batch(be, [[1]], 0)) == []
    with pytest.raises(ValueError, match="empty prompt"):
        list(generate_batch(be, [[1], []], 3))
    with pytest.raises(ValueError, match="exceed the longest"):
        list(generate_batch(be, [[1] * 8], 3))
    check_request([[1] * 7], 3, 10)
    with pytest.raises(ValueError, match="largest batch"):
        list(generate_batch(be, [[1], [2], [3]], 2))
    assert be.log == [] and be.free == [0, 1]                  # nothing was taken for refused requests


def test_slots_are_released_when_a_step_fails_or_the_caller_stops_early():
    be = Scripted(fail_at=2)
    with pytest.raises(RuntimeError, match="boom"):
        list(generate_batch(be, [[1], [2]], 5))
    assert sorted(be.free) == [0, 1, 2, 3]
    be = Scripted()
    gen = generate_batch(be, [[1], [2]], 5)
    next(gen)
    gen.close()
    assert sorted(be.free) == [0, 1, 2, 3]


def test_batches_one_after_another():
    assert [list(r) for r in plan_batches(7, 3)] == [[0, 1, 2], [3, 4, 5], [6]]
    assert plan_batches(0, 3) == []
    be = Scripted(max_batch=3)
    prompts = [[10 * i] for i in range(7)]
    out = generate_all(be, prompts, 3, stop_token_ids=[32])
    assert out == [[1, 2, 3], [11, 12, 13], [21, 22, 23], [31, 32], [41, 42, 43], [51, 52, 53], [61, 62, 63]]
    acquires = [e for e in be.log if e[0] == "acquire"]
    assert [len(a[1]) for a in acquires] == [3, 3, 1]
    assert acquires[1][1] == acquires[0][1]                    # the second batch uses the first one's slots again


def test_more_requests_than_slots_are_yielded_step_by_step():
    """Batches run one after another and every step is handed out as it is computed: seven requests on three slots
    give the first batch's steps, then the second's, with FILL where a request's batch is not the one running."""
    be = Scripted(max_batch=3)
    prompts = [[10 * i] for i in range(7)]
    gen = generate_steps(be, prompts, 3, stop_token_ids=[32])
    first = next(gen)
    assert first == [1, 11, 21, FILL, FILL, FILL, FILL]
    assert [e[0] for e in be.log].count("acquire") == 1        # nothing of the second batch has run yet
    rest = list(gen)
    assert [first] + rest == [
        [1, 11, 21, FILL, FILL, FILL, FILL], [2, 12, 22, FILL, FILL, FILL, FILL], [3, 13, 23, FILL, FILL, FILL, FILL],
        [FILL, FILL, FILL, 31, 41, 51, FILL], [FILL, FILL, FILL, 32, 42, 52, FILL], [FILL, FILL, FILL, FILL, 43, 53, FILL],
        [FILL, FILL, FILL, FILL, FILL, FILL, 61], [FILL, FILL, FILL, FILL, FILL, FILL, 62],
        [FILL, FILL, FILL, FILL, FILL, FILL, 63]]
    assert sorted(be.free) == [0, 1, 2]
    # one batch: exactly what generate_batch yields
    assert list(generate_steps(Scripted(), prompts[:3], 3)) == list(generate_batch(Scripted(), prompts[:3], 3))


class Chained(Scripted):
    """The same model with steps that can be launched before the one before them has been read.

    A launched step keeps its result until it is asked for; ``tokens=None`` means "go on with what the
    step launched before this one chose", which the loop must only use when that is what it would have fed.
    """

    chains = True

    def __init__(self, **kw):
        super().__init__(**kw)
        self.drawn = 0                                          # stands for the sampler's stream of random numbers
        self.in_flight = 0
        self.previous = None

    def advance_begin(self, slots, tokens, step_index):
        if self.fail_at == step_index:
            raise RuntimeError("boom")
        assert self.in_flight <= 1, "more than one step ahead"
        if tokens is None:
            assert self.previous is not None
            tokens = self.previous
        self.log.append(("advance", tuple(slots), tuple(tokens)))
        for s, t in zip(slots, tokens):
            if s >= 0:
                assert t == self.last[s], "a chained step must go on with the token chosen before it"
        before = dict(self.last), self.drawn
        result = self._next(slots)
        self.drawn += 1
        self.previous = result
        self.in_flight += 1
        return {"result": result, "before": before}

    def advance_end(self, handle):
        self.in_flight -= 1
        return handle["result"]

    def advance_drop(self, handle):
        self.in_flight -= 1
        self.drawn = handle["before"][1]
        self.log.append(("drop",))


@pytest.mark.parametrize("stops", [(), (22, 9), (3,), (7,), (6, 21, 8)])
@pytest.mark.parametrize("limit", [1, 2, 3, 6])
def test_chained_loop_yields_what_the_plain_loop_yields(stops, limit):
    prompts = [[5], [20], [7]]
    plain = list(generate_batch(Scripted(), prompts, limit, stop_token_ids=stops))
    be = Chained()
    assert list(generate_batch(be, prompts, limit, stop_token_ids=stops)) == plain
    assert sorted(be.free) == [0, 1, 2, 3] and be.in_flight == 0
    # every random number drawn belongs to a step that was yielded: a step launched in vain gives its own back
    assert be.drawn == len(plain) - 1


def test_chained_loop_lets_an_ended_sequence_run_one_step_more_and_then_sit_out():
    be = Chained()
    steps = list(generate_batch(be, [[5], [20], [7]], 6, stop_token_ids=[22]))
    assert [s[1] for s in steps] == [21, 22, FILL, FILL, FILL, FILL]
    advances = [e for e in be.log if e[0] == "advance"]
    assert advances[1][1] == (0, 1, 2)                         # launched before 22 was seen
    assert advances[2][1] == (0, -1, 2)                        # from then on it sits out


def test_chained_loop_releases_and_drops_when_the_caller_stops_early_or_a_step_fails():
    be = Chained()
    gen = generate_batch(be, [[1], [2]], 5)
    next(gen)
    next(gen)
    gen.close()
    assert sorted(be.free) == [0, 1, 2, 3] and be.in_flight == 0 and ("drop",) in be.log
    be = Chained(fail_at=3)
    with pytest.raises(RuntimeError, match="boom"):
        list(generate_batch(be, [[1], [2]], 5))
    assert sorted(be.free) == [0, 1, 2, 3]


def test_chained_batches_one_after_another():
    be = Chained(max_batch=3)
    out = generate_all(be, [[10 * i] for i in range(7)], 3, stop_token_ids=[32])
    assert out == [[1, 2, 3], [11, 12, 13], [21, 22, 23], [31, 32], [41, 42, 43], [51, 52, 53], [61, 62, 63]]
