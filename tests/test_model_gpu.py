"""The engine against the plain implementation, in float32 and in bfloat16: whole requests, the last 32
tokens one by one, unequal batches whose slots are used again, long decoding, first tokens, generation
through the entry point, graph replay, and the trace program."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import (TINY, collect_positions, make_model_dir, max_live_tokens, random_tokens, read_model_dir,
                     trace_batches, trace_tail, trace_whole)
from plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
# Largest allowed |engine - plain| as a fraction of the largest |plain logit| of the request.
# float32: accumulated float rounding over a few layers (the oracle is float64).
# bfloat16: activations carry 8 significant bits (2^-9 relative per rounding) through 2-3 layers of
# about ten rounded tensors each. Models whose weights were sharpened on purpose amplify every rounding;
# for them the bound is what bfloat16 arithmetic itself does to the plain implementation on the same
# request (its error against the float64 run, times two), when that is larger.
TOL = {"float32": 1e-4, "bfloat16": 3e-2}
LENGTHS = [1, 5, 9, 17, 33, 64, 65, 70, 128, 129, 131, 200]     # 64-token cache pages: edges and one past them


class Case:
    """A tiny model folder, its plain logits and engines on it."""

    def __init__(self, name, tmp, sharp=False, raw=None, kw=None, lengths=LENGTHS, sharpness=4.0, plain_device="cpu"):
        """``plain_device``: where the plain implementation computes (the GPU's float64 library routines for layers of
        a real model's sizes, which would take minutes on the CPU)."""
        if raw is None:
            raw, kw = TINY[name]
        self.name = name
        self.dir = make_model_dir(os.path.join(tmp, name + ("_sharp" if sharp else "")), raw, **kw)
        if sharp:
            self._sharpen(sharpness)
        self.raw, self.weights = read_model_dir(self.dir)
        if plain_device != "cpu":
            self.weights = {k: v.to(plain_device) for k, v in self.weights.items()}
        self.vocab = raw["vocab_size"]
        self.requests = {f"r{n}": random_tokens(n, self.vocab, seed=1000 + n) for n in lengths}
        self._plain = {}
        self._engines = {}

    def _sharpen(self, factor):
        """Scale every q_norm weight so that attention is peaked and a lost or misplaced key shows."""
        from safetensors.torch import load_file, save_file
        path = os.path.join(self.dir, "model.safetensors")
        t = load_file(path)
        for k in t:
            if k.endswith("q_norm.weight"):
                t[k] = (t[k].float() * factor).to(t[k].dtype)
        save_file(t, path)

    def plain_logits(self, rid):
        rid = rid.split("#")[0]          # "r70#2" is request r70 replayed a second time
        if rid not in self._plain:
            self._plain[rid] = plain.forward(self.raw, self.weights, self.requests[rid], torch.float64).float().cpu()
        return self._plain[rid]

    def tolerance(self, rid, dtype):
        """Allowed error as a fraction of the request's largest plain logit."""
        if dtype == "float32":
            return TOL[dtype]
        rid = rid.split("#")[0]
        key = ("noise", rid)
        if key not in self._plain:
            ref = self.plain_logits(rid)
            low = plain.forward(self.raw, self.weights, self.requests[rid], torch.bfloat16).float().cpu()
            self._plain[key] = float((low - ref).abs().max()) / float(ref.abs().max())
        return max(TOL[dtype], 2.0 * self._plain[key])

    def engine(self, dtype, **kw):
        from dryft_amd import Engine
        key = (dtype, tuple(sorted(kw.items())))
        if key not in self._engines:
            args = dict(max_batch=8, max_len=512, use_graph=False)
            args.update(kw)
            self._engines[key] = Engine(self.dir, dtype=dtype, **args)
        return self._engines[key]


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    tmp = str(tmp_path_factory.mktemp("models"))
    out = {n: Case(n, tmp) for n in TINY}
    out["C_sharp"] = Case("C", tmp, sharp=True)
    out["A_sharp"] = Case("A", tmp, sharp=True)
    out["B_sharp"] = Case("B", tmp, sharp=True)
    return out


CASE_NAMES = ["A", "B", "C", "D", "E", "C_sharp", "A_sharp", "B_sharp"]


def replay(engine, records):
    from dryft_amd.engine.replay import Replayer
    r = Replayer(engine)
    outputs = {}
    for rec in records:
        logits = r.run_step(rec)
        if logits is not None and logits.shape[0]:
            outputs[rec["step"]] = logits.float().cpu()
    assert not r.slot_of, "every request of the trace must have ended"
    assert engine.cache.slots.free_count == engine.cache.n_slots, "a slot was lost"
    for g in engine.cache.kv_groups:
        assert g.table.pool.free_count == g.table.pool.n_pages, "a page was lost"
    return outputs


def check_against_plain(case, got, dtype, what):
    assert got, "nothing was compared"
    worst = 0.0
    for (rid, pos), row in got.items():
        ref = case.plain_logits(rid)
        scale = float(ref.abs().max())
        err = float((row - ref[pos]).abs().max()) / scale
        tol = case.tolerance(rid, dtype)
        assert np.isfinite(err), f"{what}: non-finite logits for {rid} at {pos}"
        assert err <= tol, f"{what}: {rid} position {pos}: error {err:.3g} of the logit scale > {tol:.3g}"
        worst = max(worst, err / tol)
    report = os.environ.get("DRYFT_TEST_REPORT")
    if report:
        with open(report, "a") as f:
            f.write(f"{what} {case.name} {case.dir[-6:]} {dtype}: worst error / tolerance = {worst:.3f}\n")
    return worst


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", CASE_NAMES)
def test_whole_requests(cases, name, dtype):
    case = cases[name]
    records = list(trace_whole(case.requests))
    got = collect_positions(records, replay(case.engine(dtype), records))
    assert len(got) == sum(LENGTHS)
    check_against_plain(case, got, dtype, "whole")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", CASE_NAMES)
def test_last_32_tokens_one_by_one(cases, name, dtype):
    case = cases[name]
    records = list(trace_tail(case.requests, 32))
    got = collect_positions(records, replay(case.engine(dtype), records))
    check_against_plain(case, got, dtype, "tail")


def unequal_batches(case):
    r = case.requests
    return [
        {"r5": (r["r5"], 3), "r70": (r["r70"], 40), "r17": (r["r17"], 9), "r1": (r["r1"], 0)},
        {"r131": (r["r131"], 66), "r9": (r["r9"], 8), "r33": (r["r33"], 2)},
        {"r200": (r["r200"], 150), "r70#2": (r["r70"], 6), "r5#2": (r["r5"], 4), "r17#2": (r["r17"], 16),
         "r33#2": (r["r33"], 32)},
        # prompts that end exactly at a page's edge, one token before and one after it, then cross further edges
        {"r129": (r["r129"], 65), "r128": (r["r128"], 64), "r65": (r["r65"], 2), "r64": (r["r64"], 1),
         "r131#2": (r["r131"], 3)},
    ]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", CASE_NAMES)
def test_unequal_batches_reuse_slots(cases, name, dtype):
    case = cases[name]
    engine = case.engine(dtype)
    records = list(trace_batches(unequal_batches(case)))
    got = collect_positions(records, replay(engine, records))
    check_against_plain(case, got, dtype, "batches")
    # the same trace again on the same engine: slots and pages now hold stale bytes of other requests
    again = collect_positions(records, replay(engine, records))
    for key in got:
        assert torch.equal(got[key], again[key]), f"second run differs at {key} (stale state)"


@pytest.mark.parametrize("dtype", DTYPES)
def test_alone_and_in_a_batch_agree(cases, dtype):
    """What else is in the batch changes a request's logits by rounding at most."""
    case = cases["C_sharp"]
    engine = case.engine(dtype)
    alone = list(trace_batches([{"r70": (case.requests["r70"], 40)}]))
    a = collect_positions(alone, replay(engine, alone))
    batch = list(trace_batches([unequal_batches(case)[0]]))
    b = collect_positions(batch, replay(engine, batch))
    tol = 1e-5 if dtype == "float32" else 2e-2
    for key, row in a.items():
        scale = float(row.abs().max())
        assert float((row - b[key]).abs().max()) <= tol * scale, f"{key} depends on the rest of the batch"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "C_sharp"])
def test_long_decoding_crosses_pages(cases, name, dtype):
    case = cases[name]
    toks = case.requests["r200"]
    records = list(trace_batches([{"r200": (toks, 197)}]))     # 3 tokens start, 197 follow one by one
    got = collect_positions(records, replay(case.engine(dtype), records))
    assert len(got) == 198
    check_against_plain(case, got, dtype, "long decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens(cases, name, dtype):
    """A sequence that starts with a single token, then grows one by one: positions 0, 1, 2, ..."""
    case = cases[name]
    toks = case.requests["r9"]
    records = [{"step": 0, "entries": [{"id": "r9", "tokens": toks[:1], "want": [0]}], "end": []}]
    for i in range(1, len(toks)):
        records.append({"step": i, "entries": [{"id": "r9", "tokens": [toks[i]], "want": [0]}],
                        "end": ["r9"] if i == len(toks) - 1 else []})
    got = collect_positions(records, replay(case.engine(dtype), records))
    check_against_plain(case, got, dtype, "first tokens")


def random_trace(case, seed, max_batch=8):
    """Batches drawn at random, one after another: one to ``max_batch`` requests each, lengths around the edges of
    the 64-token pages as often as anywhere, each request's last tokens (none to forty) fed one by one, logits wanted
    at random places of the prompts (nowhere, everywhere, a few) and at most decoding steps. Requests are added to
    ``case.requests`` under names that say seed, batch and place."""
    rng = np.random.default_rng(seed)
    edges = [1, 2, 63, 64, 65, 127, 128, 129, 191, 192, 193, 255, 256, 257]
    records, step = [], 0
    for b in range(4):
        batch = {}
        for i in range(int(rng.integers(1, max_batch + 1))):
            n = int(rng.choice(edges)) if rng.random() < 0.5 else int(rng.integers(1, 260))
            rid = f"s{seed}b{b}i{i}n{n}"
            case.requests[rid] = random_tokens(n, case.vocab, seed=7000 + 100 * seed + 10 * b + i)
            batch[rid] = (case.requests[rid], int(rng.integers(0, min(n, 41))))
        for rec in trace_batches([batch]):
            rec["step"] = step
            step += 1
            for e in rec["entries"]:
                n = len(e["tokens"])
                kind = rng.random()
                if n > 1:                                        # a prompt: nowhere, everywhere, or a few places
                    e["want"] = [] if kind < 0.2 else list(range(n)) if kind < 0.5 else \
                        sorted(set(int(x) for x in rng.integers(0, n, size=3)) | {n - 1})
                elif kind < 0.15:
                    e["want"] = []
            records.append(rec)
    return records


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,seed", [(n, 10 * i + k) for i, n in enumerate(["A_sharp", "B_sharp", "C_sharp", "D", "E", "B"])
                                       for k in range(3)])
def test_random_batches_against_plain(cases, name, seed, dtype):
    case = cases[name]
    records = random_trace(case, seed)
    got = collect_positions(records, replay(case.engine(dtype), records))
    check_against_plain(case, got, dtype, f"random batches, seed {seed}")


def portions_trace(case):
    """r200 arrives in portions of 63, 2, 63, 1 and 71 tokens: one starts in the middle of a page, one is two tokens
    long, one ends exactly at a page's edge, one is a single token. Beside it r131 starts with 127 tokens and then
    goes on one token a step, so every later step mixes a portion of a prompt with a decoding row; r17 joins the
    first step only. Logits are wanted everywhere."""
    long, short, tiny = case.requests["r200"], case.requests["r131"], case.requests["r17"]
    cuts = [0, 63, 65, 128, 129, 200]
    records = []
    for i in range(5):
        part = long[cuts[i]:cuts[i + 1]]
        entries = [{"id": "r200", "tokens": part, "want": list(range(len(part)))}]
        if i == 0:
            entries.append({"id": "r131", "tokens": short[:127], "want": list(range(127))})
            entries.append({"id": "r17", "tokens": tiny, "want": list(range(17))})
        else:
            entries.insert(0, {"id": "r131", "tokens": [short[126 + i]], "want": [0]})
        end = (["r17"] if i == 0 else []) + (["r200", "r131"] if i == 4 else [])
        records.append({"step": i, "entries": entries, "end": end})
    return records


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "C_sharp", "A_sharp", "B_sharp", "D", "E"])
def test_prompt_in_portions_beside_decoding_rows(cases, name, dtype):
    """How the tokens are cut into steps changes no logit: a prompt fed in portions, in steps that also hold
    sequences going on by one token, against the plain implementation of whole sequences."""
    case = cases[name]
    records = portions_trace(case)
    got = collect_positions(records, replay(case.engine(dtype), records))
    assert len(got) == 200 + 131 + 17
    check_against_plain(case, got, dtype, "portions")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B_sharp", "C"])
def test_sequences_that_sit_out_of_a_prompt_step(cases, name, dtype):
    """Sequences with slot -1 keep their rows in a step but take no part: prompts beside them come out as alone,
    no cache slot and no length changes for them, and what they leave in the residual stream is finite."""
    from dryft_amd.engine.step import SeqStep
    case = cases[name]
    engine = case.engine(dtype)
    a, b = case.requests["r70"], case.requests["r131"]
    filler = case.requests["r200"]
    slots = engine.acquire(2)
    try:
        steps = [SeqStep(-1, filler[:1], [0]), SeqStep(slots[0], a, list(range(len(a)))), SeqStep(-1, filler, []),
                 SeqStep(slots[1], b[:-1], list(range(len(b) - 1))), SeqStep(-1, filler[:65], [3])]
        first = engine.step(steps).float().cpu()
        assert first.shape[0] == len(a) + len(b) - 1 and torch.isfinite(first).all()
        last = engine.step([SeqStep(-1, [0], []), SeqStep(slots[1], b[-1:], [0])]).float().cpu()
        host = engine.cache.lengths_host()
        assert [int(host[s]) for s in slots] == [len(a), len(b)]
        assert int(engine.cache.lengths_dev.sum()) == len(a) + len(b)
    finally:
        engine.release(slots)
    got = {("r70", i): first[i] for i in range(len(a))}
    got.update({("r131", i): first[len(a) + i] for i in range(len(b) - 1)})
    got[("r131", len(b) - 1)] = last[0]
    check_against_plain(case, got, dtype, "sitting out")


@pytest.mark.parametrize("dtype", DTYPES)
def test_stale_cache_bytes_are_never_read(cases, dtype):
    """Fill every page with large finite garbage before a run: lengths and tables alone say what is valid."""
    case = cases["B"]
    engine = case.engine(dtype, max_batch=4, max_len=256)
    for g in engine.cache.kv_groups:
        g.k.fill_(3e4)
        g.v.fill_(-3e4)
    records = list(trace_batches([{"r70": (case.requests["r70"], 30), "r9": (case.requests["r9"], 3)}]))
    got = collect_positions(records, replay(engine, records))
    check_against_plain(case, got, dtype, "poisoned cache")


@pytest.mark.parametrize("dtype", DTYPES)
def test_device_lengths_follow_host(cases, dtype):
    case = cases["A"]
    engine = case.engine(dtype)
    from dryft_amd.engine.step import SeqStep
    slots = engine.acquire(3)
    engine.step([SeqStep(slots[0], [1, 2, 3], []), SeqStep(slots[1], [4], [0]), SeqStep(slots[2], list(range(70)), [])])
    engine.step([SeqStep(slots[0], [5], [0]), SeqStep(-1, [0], []), SeqStep(slots[2], [7], [])])
    host = engine.cache.lengths_host()
    assert [int(host[s]) for s in slots] == [4, 1, 71]
    assert engine.cache.lengths_dev.cpu().tolist() == [int(x) for x in host]
    engine.release(slots)
    assert not engine.cache.lengths_dev.any()


# ------------------------------------------------------------------------------------ generation
def plain_generation(case, prompt, n, temperature=0.0, uniforms=None):
    if temperature == 0.0:
        return plain.generate(case.raw, case.weights, prompt, n, dtype=torch.float64)
    choose = lambda logits, t: plain.sample_with_temperature(logits, temperature, float(uniforms[t]))
    return plain.generate(case.raw, case.weights, prompt, n, choose=choose, dtype=torch.float64)


def check_generation(case, prompts, ours, n, dtype, temperature=0.0, uniforms=None):
    """Tokens must equal the plain loop's unless the plain logits leave the choice open within rounding."""
    for b, prompt in enumerate(prompts):
        col = [step[b] for step in ours]
        u = None if uniforms is None else [float(uniforms[t][b]) for t in range(n)]
        want, logits = plain_generation(case, prompt, n, temperature, u)
        for t in range(n):
            if col[t] == want[t]:
                continue
            if temperature == 0.0:
                margin = float(logits[t].max() - logits[t][col[t]])
                slack = TOL[dtype] * float(logits[t].abs().max()) * 2
                assert margin <= slack, f"seq {b} step {t}: chose {col[t]}, plain {want[t]}, margin {margin}"
            else:
                assert plain.cdf_margin(logits[t], temperature, u[t]) < (1e-5 if dtype == "float32" else 2e-2), \
                    f"seq {b} step {t}: sampled {col[t]}, plain {want[t]}"
            break   # after a justified divergence the continuations differ


@pytest.mark.parametrize("use_graph", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_config_a(cases, dtype, use_graph):
    """Tiny A's workload: prompts of 5, 9 and 17 tokens, 8 greedy steps."""
    case = cases["A"]
    prompts = [random_tokens(n, case.vocab, seed=n) for n in (5, 9, 17)]
    engine = case.engine(dtype, use_graph=use_graph)
    ours = list(engine.generate(prompts, 8))
    assert len(ours) == 8 and all(len(s) == 3 and all(isinstance(t, int) for t in s) for s in ours)
    check_generation(case, prompts, ours, 8, dtype)
    assert list(engine.generate(prompts, 8)) == ours, "second run differs from the first"


@pytest.mark.parametrize("use_graph", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
def test_generation_config_b_greedy_and_temperature(cases, dtype, use_graph):
    """Tiny B's workload: prompts of 1, 6, 13 and 31 tokens, 12 steps, greedy and temperature 0.8."""
    case = cases["B"]
    prompts = [random_tokens(n, case.vocab, seed=50 + n) for n in (1, 6, 13, 31)]
    engine = case.engine(dtype, use_graph=use_graph)
    ours = list(engine.generate(prompts, 12))
    check_generation(case, prompts, ours, 12, dtype)
    sampled = list(engine.generate(prompts, 12, temperature=0.8, sample_seed=7))
    gen = torch.Generator().manual_seed(7)
    uniforms = [torch.rand(4, generator=gen, dtype=torch.float32) for _ in range(12)]
    check_generation(case, prompts, sampled, 12, dtype, 0.8, uniforms)
    assert sampled != ours
    assert list(engine.generate(prompts, 12, temperature=0.8, sample_seed=7)) == sampled


@pytest.mark.parametrize("dtype", DTYPES)
def test_small_batch_unchanged_after_a_big_one(cases, dtype):
    case = cases["B"]
    engine = case.engine(dtype, use_graph=True)
    small = [random_tokens(11, case.vocab, seed=3)]
    big = [random_tokens(n, case.vocab, seed=60 + n) for n in (40, 3, 19, 64, 65, 7, 100, 2)]
    a = list(engine.generate(small, 6))
    list(engine.generate(big, 9))
    assert list(engine.generate(small, 6)) == a, "state leaked from the larger batch"


def test_library_tuning_keeps_results_and_slots(cases):
    """`Engine.tune` runs stand-in steps of the given sizes while the vendor library times its candidate kernels:
    afterwards every slot is free again, nothing more is timed, and whole prompts (whose products go through
    the library) still match the plain implementation. A row count that does not fit is refused."""
    import torch.cuda.tunable as tunable
    from dryft_amd.engine.step import SeqStep
    case = cases["B"]
    engine = case.engine("bfloat16", max_batch=4, max_len=256, use_graph=True)
    was_enabled = tunable.is_enabled()
    try:
        engine.tune([70, 200, 300])                         # 300 rows: spread over two sequences
        assert engine.cache.slots.free_count == 4
        assert not tunable.tuning_is_enabled()
        with pytest.raises(ValueError):
            engine.tune([4 * 256 + 1])
        for rid in ("r70", "r200"):
            tokens = case.requests[rid]
            slots = engine.acquire(1)
            try:
                logits = engine.step([SeqStep(slots[0], tokens, list(range(len(tokens))))]).float().cpu()
            finally:
                engine.release(slots)
            ref = case.plain_logits(rid)
            err = float((logits - ref).abs().max()) / float(ref.abs().max())
            assert err <= case.tolerance(rid, "bfloat16"), f"{rid}: {err}"
    finally:
        tunable.tuning_enable(False)
        tunable.enable(was_enabled)
    assert engine.cache.slots.free_count == 4


@pytest.mark.parametrize("dtype", DTYPES)
def test_stop_tokens_and_more_requests_than_slots(cases, dtype):
    case = cases["A"]
    engine = case.engine(dtype, max_batch=3, max_len=128, use_graph=True)
    prompts = [random_tokens(n, case.vocab, seed=80 + n) for n in (4, 9, 2, 30, 7, 12, 5)]
    free_run = engine.generate_all(prompts, 10)
    assert [len(r) for r in free_run] == [10] * 7
    stop = free_run[1][3]
    stopped = engine.generate_all(prompts, 10, stop_token_ids=[stop])
    for full, cut in zip(free_run, stopped):
        want = full[: full.index(stop) + 1] if stop in full else full
        assert cut == want
    steps = list(engine.generate(prompts[:3], 10, stop_token_ids=[stop]))
    assert all(len(s) == 3 for s in steps)
    for b in range(3):
        col = [s[b] for s in steps]
        cut = stopped[b]
        assert col[: len(cut)] == cut and all(t == -1 for t in col[len(cut):])
    assert engine.cache.slots.free_count == 3


@pytest.mark.parametrize("dtype", DTYPES)
def test_steps_launched_ahead_change_nothing(cases, dtype):
    """With captured graphs the loop launches a step before it has read the one before. Stop tokens (seen one
    step late), sampling (random numbers drawn ahead, given back when a step is dropped) and batch after batch
    must give what the engine gives that finishes every step before it starts the next."""
    case = cases["B"]
    prompts = [random_tokens(n, case.vocab, seed=90 + n) for n in (3, 17, 8, 40, 5, 11, 26)]
    ahead = case.engine(dtype, max_batch=3, max_len=128, use_graph=True)
    plain_loop = case.engine(dtype, max_batch=3, max_len=128, use_graph=False)
    assert ahead.chains and not plain_loop.chains
    free_run = plain_loop.generate_all(prompts, 9, temperature=0.7, sample_seed=11)
    stops = [free_run[0][2], free_run[4][5], free_run[6][0]]
    for kw in (dict(), dict(temperature=0.7, sample_seed=11), dict(temperature=0.7, sample_seed=11, stop_token_ids=stops),
               dict(stop_token_ids=[plain_loop.generate_all(prompts, 9)[2][4]])):
        want = plain_loop.generate_all(prompts, 9, **kw)
        assert ahead.generate_all(prompts, 9, **kw) == want, f"differs with {kw}"
        assert list(ahead.generate(prompts[:3], 9, **kw)) == list(plain_loop.generate(prompts[:3], 9, **kw))
    early = ahead.generate(prompts[:3], 9)
    next(early), next(early)
    early.close()                                             # a step is in flight: it is dropped, slots come back
    assert ahead.cache.slots.free_count == 3
    assert ahead.generate_all(prompts, 9) == plain_loop.generate_all(prompts, 9)


def test_slots_longer_than_the_model_allows_are_refused(cases, tmp_path):
    """`max_position_embeddings` bounds the slot length (reference: config.py:154): asking for more is an error,
    asking for nothing gives at most that, and the replay program clamps its budget to it."""
    from dryft_amd import Engine
    case = cases["D"]                                            # allows 1,024 positions
    with pytest.raises(ValueError, match="1024 positions"):
        Engine(case.dir, dtype="float32", max_batch=2, max_len=1025)
    engine = Engine(case.dir, dtype="float32", max_batch=1)
    assert engine.max_len == 1024
    del engine
    record = {"step": 0, "entries": [{"id": "a", "tokens": case.requests["r9"], "want": [8]}], "end": ["a"]}
    out_dir = str(tmp_path / "out")
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", case.dir, "--dtype",
                           "float32", "--out", out_dir, "--max-tokens", "4096"], input=json.dumps(record) + "\n",
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = torch.from_numpy(np.fromfile(os.path.join(out_dir, "0.f32"), dtype="<f4").reshape(1, case.vocab))
    check_against_plain(case, {("r9", 8): got[0]}, "float32", "clamped budget")


@pytest.mark.parametrize("dtype", DTYPES)
def test_decoding_across_context_ranges(cases, dtype):
    """Captured steps come per range of context lengths (256, 512, ... tokens): a batch whose longest sequence
    grows from 250 to 262 tokens moves from one graph to the next, and the tokens stay the plain loop's."""
    case = cases["B"]
    engine = case.engine(dtype, max_batch=3, max_len=512, use_graph=True)
    prompts = [random_tokens(n, case.vocab, seed=400 + n) for n in (250, 3, 100)]
    ours = list(engine.generate(prompts, 12))
    check_generation(case, prompts, ours, 12, dtype)
    assert {key for key in engine._graphs if key[0] == 3} >= {(3, 256), (3, 512)}
    short = list(engine.generate([p[:40] for p in prompts], 5))          # back to the first range
    check_generation(case, [p[:40] for p in prompts], short, 5, dtype)
    assert list(engine.generate(prompts, 12)) == ours


@pytest.mark.parametrize("dtype", DTYPES)
def test_batch_buckets_bound_the_captured_steps(cases, dtype):
    """One engine generates at every batch size from 1 to 40 through captured steps that come in buckets of batch
    sizes, the rows beyond a batch dead: the tokens are those of an engine with a captured step per exact size, greedy
    and sampled; the number of captured steps stays within buckets x ranges; warmed beforehand, nothing is captured
    and no device memory is taken during generation; a cap on their number drops the one used longest ago."""
    from dryft_amd.engine.engine import default_batch_buckets, pick_bucket
    case = cases["B"]
    buckets = default_batch_buckets(40)
    assert buckets == (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16, 20, 24, 28, 32, 40)
    assert [pick_bucket(buckets, n) for n in (1, 8, 9, 17, 33, 40)] == [1, 8, 10, 20, 40, 40]
    bucketed = case.engine(dtype, max_batch=40, max_len=256, use_graph=True)
    exact = case.engine(dtype, max_batch=40, max_len=256, use_graph=True, batch_buckets=tuple(range(1, 41)))
    assert bucketed.batch_buckets == buckets and bucketed.context_ranges() == [256]
    assert bucketed.warm() == len(buckets) == len(bucketed._graphs)
    rng = np.random.default_rng(5)
    prompts = [random_tokens(int(rng.integers(1, 30)), case.vocab, seed=600 + i) for i in range(40)]
    how = {n: dict(temperature=0.8, sample_seed=n) if n % 3 == 0 else {} for n in range(1, 41)}
    want = {n: exact.generate_all(prompts[:n], 4, **how[n]) for n in range(1, 41)}
    for n in range(1, 41):
        assert bucketed.generate_all(prompts[:n], 4, **how[n]) == want[n], f"batch of {n}"
    # again: the prompts' captured steps exist now too, and nothing more may be captured or kept
    torch.cuda.synchronize()
    held, prompt_steps = torch.cuda.memory_allocated(), len(bucketed._prompt_graphs)
    for n in range(1, 41):
        assert bucketed.generate_all(prompts[:n], 4, **how[n]) == want[n], f"batch of {n}, second time"
    assert len(bucketed._prompt_graphs) == prompt_steps
    assert len(bucketed._graphs) == len(buckets), "a step was captured although every bucket was warm"
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == held, "generation kept device memory although every bucket was warm"
    assert len(exact._graphs) == 40
    check_generation(case, prompts[:9], [list(col) for col in zip(*bucketed.generate_all(prompts[:9], 4))], 4, dtype)
    # a cap: the captured step used longest ago goes, and comes back when asked for
    capped = case.engine(dtype, max_batch=40, max_len=256, use_graph=True, max_graphs=2)
    for n in (3, 9, 3, 17):
        assert capped.generate_all(prompts[:n], 3) == exact.generate_all(prompts[:n], 3)
    assert list(capped._graphs) == [(3, 256), (20, 256)]
    with pytest.raises(ValueError, match="max_graphs"):
        capped.warm()
    assert bucketed.cache.slots.free_count == exact.cache.slots.free_count == 40


@pytest.mark.parametrize("name", ["B", "C_sharp", "A_sharp"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_short_prompts_start_through_a_captured_step(cases, dtype, name):
    """Batches whose prompts have at most 256 tokens in all start in a captured step, filled up with sequences that
    sit out: the logits at each prompt's end against the plain implementation, on slots that are used again, batch
    shapes taking turns so that every captured step is replayed several times with other work in between; then
    generation, whose tokens are those of an engine that starts launch by launch."""
    case = cases[name]
    engine = case.engine(dtype, max_batch=9, max_len=512, use_graph=True)
    eager = case.engine(dtype, max_batch=9, max_len=512, use_graph=True, prompt_graph_rows=0)
    shapes = [[1], [5, 9, 17], [64], [70, 1, 33], [129, 65, 9, 17, 5, 1, 1, 1, 1], [200, 33], [17], [131, 70, 33, 17, 5],
              [9, 5], [200, 33, 17, 5, 1], [128, 128], [65, 17, 9]]
    assert engine._prompt_graph_for(3, 300) is None and eager._prompt_graph_for(1, 5) is None
    for turn in range(3):
        for lengths in shapes:
            names = [f"r{n}" for n in lengths]
            prompts = [case.requests[r] for r in names]
            graph = engine._prompt_graph_for(len(prompts), sum(lengths))
            assert graph.n_seqs > len(prompts) and sum(lengths) <= graph.n_rows <= max(32, 1.6 * sum(lengths))
            slots = engine.acquire(len(prompts))
            try:
                engine.cache.begin_step(slots, lengths)
                logits = graph.replay(slots, prompts)[:len(prompts)].float().cpu()
                engine.cache.end_step(slots, lengths)
                assert [int(engine.cache.lengths_host()[s]) for s in slots] == lengths
                assert engine.cache.lengths_dev[slots].tolist() == lengths
            finally:
                engine.release(slots)
            got = {(r, n - 1): logits[i] for i, (r, n) in enumerate(zip(names, lengths)) if names.index(r) == i}
            check_against_plain(case, got, dtype, f"captured prompts' step {lengths}")
    assert len(engine._prompt_graphs) <= 10
    for lengths in shapes + [[200, 131]]:                               # the last one has too many tokens: launch by launch
        prompts = [case.requests[f"r{n}"] for n in lengths]
        kw = dict(temperature=0.7, sample_seed=len(lengths)) if len(lengths) % 2 else {}
        ours = engine.generate_all(prompts, 5, **kw)
        assert ours == eager.generate_all(prompts, 5, **kw), lengths
    check_generation(case, [case.requests["r70"], case.requests["r9"]],
                     list(engine.generate([case.requests["r70"], case.requests["r9"]], 6)), 6, dtype)
    assert engine.cache.slots.free_count == 9


@pytest.mark.parametrize("name,n_seqs", [("A_sharp", 70), ("B", 130), ("C_sharp", 200)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_many_sequences_decode_through_the_graph(cases, dtype, name, n_seqs):
    """More sequences than the few-row products take (64): the decoding steps of 70 and 130 sequences, captured, give
    the plain loop's tokens, and the same with fewer requests than slots in the next batch."""
    case = cases[name]
    engine = case.engine(dtype, max_batch=n_seqs, max_len=128, use_graph=True)
    rng = np.random.default_rng(n_seqs)
    prompts = [random_tokens(int(rng.integers(1, 40)), case.vocab, seed=9000 + i) for i in range(n_seqs)]
    ours = list(engine.generate(prompts, 4))
    check_generation(case, prompts, ours, 4, dtype)
    fewer = prompts[: n_seqs - 3]
    check_generation(case, fewer, list(engine.generate(fewer, 3)), 3, dtype)
    assert engine.cache.slots.free_count == n_seqs


@pytest.mark.parametrize("dtype", DTYPES)
def test_graph_replay_equals_eager(cases, dtype):
    """A captured decoding step gives bit-identical logits to the same step run eagerly."""
    case = cases["B"]
    from dryft_amd.engine.graph import DecodeGraph
    from dryft_amd.engine.step import SeqStep
    engine = case.engine(dtype, max_batch=4, max_len=256)
    prompts = [random_tokens(n, case.vocab, seed=90 + n) for n in (70, 3, 129)]
    nxt = [random_tokens(5, case.vocab, seed=95 + i) for i in range(3)]
    graph = DecodeGraph(engine.stepper, 3)
    graph.capture()
    results = []
    for mode in ("eager", "graph", "graph", "eager"):
        slots = engine.acquire(3)
        engine.step([SeqStep(s, p, []) for s, p in zip(slots, prompts)])
        outs = []
        for t in range(5):
            live = [s if not (t >= 3 and i == 1) else -1 for i, s in enumerate(slots)]   # one ends early
            toks = [nxt[i][t] for i in range(3)]
            if mode == "eager":
                lg = engine.step([SeqStep(s, [tk], [0]) for s, tk in zip(live, toks)])
                keep = [i for i, s in enumerate(live) if s >= 0]
            else:
                held = [s for s in live if s >= 0]
                engine.cache.begin_step(held, [1] * len(held))
                lg = graph.replay(live, toks)
                engine.cache.end_step(held, [1] * len(held))
                keep = [i for i, s in enumerate(live) if s >= 0]
                lg = lg[keep]
            outs.append(lg.float().cpu().clone())
        engine.release(slots)
        results.append(outs)
    for other in results[1:]:
        for a, b in zip(results[0], other):
            assert torch.equal(a, b), "graph replay differs from eager"


# --------------------------------------------------------------------------------- the program
def test_layer_sizes_of_a_real_model_bfloat16_agrees_with_float32():
    """Two layers with Qwen3-4B's sizes (head size 128, four query heads to a kv head, widths 2560 / 9728, the
    151,936-token head), the sizes at which the matrix-core kernels take their fast paths: the bfloat16 engine
    against the float32 engine, which shares no matrix kernel with it. Prompts of unequal length in one step (one
    long enough for two heads per wave in the prompt attention, which starts at 4,096 positions of 32 heads),
    then decoding through captured graphs at 3 sequences, and 40 sequences for the products of 17 to 64 rows."""
    from dryft_amd import Engine
    from dryft_amd.engine.step import SeqStep
    from dryft_amd.models import load_preset
    raw = dict(load_preset("qwen3-4b"))
    raw["num_hidden_layers"] = 2
    vocab = raw["vocab_size"]
    engines = {dt: Engine(config=raw, seed=5, dtype=dt, max_batch=40, max_len=4608, max_tokens=40 * 320 + 3 * 4608)
               for dt in ("float32", "bfloat16")}
    prompts = [random_tokens(n, vocab, seed=7 + n) for n in (4200, 70, 300)]
    follow = [random_tokens(6, vocab, seed=50 + i) for i in range(3)]
    many = [random_tokens(100 + i, vocab, seed=200 + i) for i in range(40)]
    got = {}
    for dt, eng in engines.items():
        slots = eng.acquire(3)
        rows = [eng.step([SeqStep(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)]).float().cpu()]
        for t in range(6):                                      # given tokens, so both engines see the same ones
            rows.append(eng.step([SeqStep(s, [f[t]], [0]) for s, f in zip(slots, follow)]).float().cpu())
        eng.release(slots)
        slots = eng.acquire(40)
        rows.append(eng.step([SeqStep(s, p, [len(p) - 1]) for s, p in zip(slots, many)]).float().cpu())
        rows.append(eng.step([SeqStep(s, [p[0]], [0]) for s, p in zip(slots, many)]).float().cpu())
        eng.release(slots)
        got[dt] = torch.cat(rows)
        del eng
    ref, low = got["float32"], got["bfloat16"]
    assert torch.isfinite(ref).all() and torch.isfinite(low).all()
    err = float((low - ref).abs().max()) / float(ref.abs().max())
    assert err <= TOL["bfloat16"], err
    # and through the generation loop with captured graphs (random weights leave the greedy choice to differences
    # far below the tolerance above, so the tokens of the two precisions are not compared)
    out = engines["bfloat16"].generate_all([p[:200] for p in prompts], 5)
    assert [len(r) for r in out] == [5, 5, 5] and all(0 <= t < vocab for r in out for t in r)
    assert engines["bfloat16"].cache.slots.free_count == 40


def test_a_sequence_longer_than_65536_tokens():
    """One layer with Qwen3-4B's head geometry and one sequence of 66,001 tokens (positions and page counts past 16
    bits): the bfloat16 engine against the float32 engine, which shares no attention or matrix kernel with it, at the
    prompt's last positions and three decoded tokens; and the same prompt cut into two portions and two single
    tokens, which must give the same logits within rounding."""
    from dryft_amd import Engine
    from dryft_amd.engine.step import SeqStep
    from dryft_amd.models import load_preset
    raw = dict(load_preset("qwen3-4b"))
    raw.update(num_hidden_layers=1, vocab_size=4096)
    n = 66_001
    tokens = random_tokens(n + 3, 4096, seed=5)
    got = {}
    for dtype in ("bfloat16", "float32"):
        engine = Engine(config=raw, seed=3, dtype=dtype, max_batch=1, max_len=n + 64, max_tokens=n + 128)
        for mode in (("whole", "cut") if dtype == "bfloat16" else ("whole",)):
            slot = engine.acquire(1)[0]
            if mode == "whole":
                rows = [engine.step([SeqStep(slot, tokens[:n], [n - 2, n - 1])]).float().cpu()]
            else:
                engine.step([SeqStep(slot, tokens[:40_000], [])])
                engine.step([SeqStep(slot, tokens[40_000:n - 2], [])])
                rows = [engine.step([SeqStep(slot, [tokens[i]], [0])]).float().cpu() for i in (n - 2, n - 1)]
            rows += [engine.step([SeqStep(slot, [tokens[n + t]], [0])]).float().cpu() for t in range(3)]
            engine.release([slot])
            got[(dtype, mode)] = torch.cat(rows)
        del engine
    ref = got[("float32", "whole")]
    assert torch.isfinite(ref).all()
    for key in (("bfloat16", "whole"), ("bfloat16", "cut")):
        err = float((got[key] - ref).abs().max()) / float(ref.abs().max())
        assert err <= TOL["bfloat16"], (key, err)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_long_prompt_beside_a_short_one_against_plain(tmp_path, dtype):
    """One layer with Qwen3-4B's sizes, a prompt of 4,200 tokens beside one of 70 in one step: enough rows for the prompt
    attention to take 32 rows a wave by its own choice. Logits at 16 places of the long prompt (its first and last
    rows, both sides of page and tile edges) and at the short one's end, against the plain implementation in float64."""
    from dryft_amd.engine.step import SeqStep
    from dryft_amd.models import load_preset
    raw = dict(load_preset("qwen3-4b"))
    raw.update(num_hidden_layers=1, vocab_size=2048)
    case = Case("long", str(tmp_path), sharp=True, raw=raw, kw=dict(seed=31, norm_std=0.1, std=0.02),
                lengths=[4200, 70], sharpness=3.0, plain_device="cuda:0")
    engine = case.engine(dtype, max_batch=2, max_len=4224)
    places = [0, 1, 63, 64, 127, 128, 2047, 2048, 3000, 4095, 4096, 4159, 4160, 4197, 4198, 4199]
    slots = engine.acquire(2)
    try:
        logits = engine.step([SeqStep(slots[0], case.requests["r4200"], places),
                              SeqStep(slots[1], case.requests["r70"], [69])]).float().cpu()
    finally:
        engine.release(slots)
    got = {("r4200", p): logits[i] for i, p in enumerate(places)}
    got[("r70", 69)] = logits[len(places)]
    check_against_plain(case, got, dtype, "long prompt beside a short one")


REAL_LENGTHS = [78, 308, 1108] + list(range(20, 44))
# Presets whose layer sizes the tests run at, two layers each and a vocabulary of 2,048: four, eight, five and two
# query heads to a kv head at head size 128; widths 2560 to 5120; tied and untied heads.
REAL_SIZES = {"4b": "qwen3-4b", "8b": "qwen3-8b", "32b": "qwen3-32b", "14b": "qwen3-14b", "0.6b": "qwen3-0.6b"}


class RealCases:
    """Cases at real layer sizes, made when first asked for; the plain implementation computes on the GPU in float64."""

    def __init__(self, tmp):
        self.tmp, self.made = tmp, {}

    def get(self, size, sharp):
        from dryft_amd.models import load_preset
        if (size, sharp) not in self.made:
            raw = dict(load_preset(REAL_SIZES[size]))
            raw.update(num_hidden_layers=2, vocab_size=2048)
            self.made[(size, sharp)] = Case("real" + size, self.tmp, sharp=sharp, raw=raw, lengths=REAL_LENGTHS,
                                            kw=dict(seed=77, norm_std=0.1, std=0.02), sharpness=3.0,
                                            plain_device="cuda:0")
        return self.made[(size, sharp)]

    def drop(self, size, sharp):
        """Forgets a case with its engines and weights (the larger ones hold gigabytes of device memory)."""
        self.made.pop((size, sharp), None)
        torch.cuda.empty_cache()


@pytest.fixture(scope="module")
def real_cases(tmp_path_factory):
    return RealCases(str(tmp_path_factory.mktemp("real")))


REAL_RUNS = [("4b", False)] + [(size, True) for size in REAL_SIZES]


@pytest.mark.parametrize("size,sharp", REAL_RUNS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_real_layer_sizes_against_plain(real_cases, dtype, size, sharp):
    """The sizes at which the matrix-core kernels take their fast paths, against the plain implementation (not
    against the other precision of the engine): prompts of 70, 300 and 1,100 tokens in one step with logits
    everywhere, then 8 given tokens each through the captured decoding graph; then 24 short sequences, whose
    decoding steps take the products of 17 to 64 rows."""
    from dryft_amd.engine.step import SeqStep
    case = real_cases.get(size, sharp)
    engine = case.engine(dtype, max_batch=24, max_len=1280, max_tokens=3 * 1280 + 24 * 64, use_graph=True)
    names = ["r78", "r308", "r1108"]
    got = {}
    slots = engine.acquire(3)
    try:
        prompts = [case.requests[n][:-8] for n in names]
        logits = engine.step([SeqStep(s, p, list(range(len(p)))) for s, p in zip(slots, prompts)]).float().cpu()
        row = 0
        for n, p in zip(names, prompts):
            for i in range(len(p)):
                got[(n, i)] = logits[row + i]
            row += len(p)
        graph = engine._graph_for(3)
        for t in range(8):
            engine.cache.begin_step(slots, [1, 1, 1])
            lg = graph.replay(slots, [case.requests[n][len(case.requests[n]) - 8 + t] for n in names]).float().cpu()
            engine.cache.end_step(slots, [1, 1, 1])
            for b, n in enumerate(names):
                got[(n, len(case.requests[n]) - 8 + t)] = lg[b].clone()
    finally:
        engine.release(slots)
    assert len(got) == 78 + 308 + 1108
    check_against_plain(case, got, dtype, "real sizes")
    # 24 sequences: their prompts in one step, then two decoding steps of 24 rows, eager and through the graph
    many = [f"r{n}" for n in range(20, 44)]
    got = {}
    slots = engine.acquire(24)
    try:
        prompts = [case.requests[n][:-2] for n in many]
        logits = engine.step([SeqStep(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)]).float().cpu()
        for b, n in enumerate(many):
            got[(n, len(prompts[b]) - 1)] = logits[b]
        lg = engine.step([SeqStep(s, [case.requests[n][-2]], [0]) for s, n in zip(slots, many)]).float().cpu()
        for b, n in enumerate(many):
            got[(n, len(case.requests[n]) - 2)] = lg[b]
        graph = engine._graph_for(24)
        engine.cache.begin_step(slots, [1] * 24)
        lg = graph.replay(slots, [case.requests[n][-1] for n in many]).float().cpu()
        engine.cache.end_step(slots, [1] * 24)
        for b, n in enumerate(many):
            got[(n, len(case.requests[n]) - 1)] = lg[b].clone()
    finally:
        engine.release(slots)
    check_against_plain(case, got, dtype, "real sizes, 24 sequences")


@pytest.mark.parametrize("size,seed,max_batch", [("4b", 2000, 40), ("4b", 2001, 8)] +
                         [(size, 2002, 40) for size in REAL_SIZES if size != "4b"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_random_batches_at_real_layer_sizes(real_cases, dtype, size, seed, max_batch):
    """Batches drawn at random (up to 40 requests, so that the decoding steps take every product for 1 to 64 rows),
    at the sizes at which the matrix-core kernels take their fast paths, with sharpened attention."""
    case = real_cases.get(size, True)
    records = random_trace(case, seed, max_batch=max_batch)
    engine = case.engine(dtype, max_batch=40, max_len=512, max_tokens=40 * 320)
    got = collect_positions(records, replay(engine, records))
    check_against_plain(case, got, dtype, f"random batches at real sizes, seed {seed}")


# --------------------------------------------------------------------------------- the command line
def run_cli(*argv, timeout=600):
    proc = subprocess.run([sys.executable, "-m", "dryft_amd", *argv], capture_output=True, text=True, timeout=timeout,
                          cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-3000:]
    return proc.stdout


@pytest.mark.parametrize("dtype", DTYPES)
def test_command_line_generate(cases, dtype):
    """`python -m dryft_amd generate` prints what the entry point generates, and what the plain greedy loop does."""
    case = cases["B"]
    prompts = [random_tokens(n, case.vocab, seed=300 + n) for n in (4, 17, 9)]
    text = ";".join(",".join(map(str, p)) for p in prompts)
    out = run_cli("generate", "--model", case.dir, "--dtype", dtype, "--prompt-ids", text, "--max-new-tokens", "7",
                  "--max-len", "64")
    printed = [[int(t) for t in line.split(",")] for line in out.strip().splitlines()]
    assert printed == case.engine(dtype, max_batch=3, max_len=64, use_graph=True).generate_all(prompts, 7)
    check_generation(case, prompts, [[col[t] for col in printed] for t in range(7)], 7, dtype)
    # one JSON list per step with --stream, stop tokens and a temperature with its seed
    stop = printed[1][3]
    out = run_cli("generate", "--model", case.dir, "--dtype", dtype, "--prompt-ids", text, "--max-new-tokens", "7",
                  "--max-len", "64", "--stream", "--stop-ids", str(stop), "--temperature", "0.7", "--sample-seed", "5")
    steps = [json.loads(line) for line in out.strip().splitlines()]
    want = list(case.engine(dtype, max_batch=3, max_len=64, use_graph=True).generate(
        prompts, 7, temperature=0.7, sample_seed=5, stop_token_ids=[stop]))
    assert steps == want


def test_command_line_bench_and_profile():
    """`bench` prints one JSON line per workload with the reference's quantities (agent/bench.py:61-81); `profile`
    prints a per-kernel table in which this library's kernels appear by name."""
    out = run_cli("bench", "--tiny", "--workload", "t,2,16,4", "--workload", "u,1,5,3", "--samples", "1")
    lines = [json.loads(line) for line in out.strip().splitlines()]
    assert [(r["workload"], r["batch"], r["in"], r["out"]) for r in lines] == [("t", 2, 16, 4), ("u", 1, 5, 3)]
    for r in lines:
        assert r["tok_s"] > 0 and r["total_ms"] >= r["ttft_ms"] > 0 and r["tpot_ms"] > 0
    out = run_cli("profile", "--tiny", "--batch", "2", "--prompt-len", "16", "--steps", "2")
    assert "2 decoding steps of 2 sequences" in out and "kernels a step" in out and "GB/s" in out
    table = out.splitlines()
    assert any("attn_split_kernel" in row for row in table) and any("add_rmsnorm" in row for row in table)
    out = run_cli("profile", "--tiny", "--batch", "2", "--prompt-len", "70", "--prefill")
    assert "one step of 2 prompts of 70 tokens" in out and any("attn_causal_kernel" in row for row in out.splitlines())
    out = run_cli("attention", "--shapes", "2x200,1x70", "--modes", "0,1,5", "--heads", "8", "--kv-heads", "2")
    rows = out.strip().splitlines()
    assert len(rows) == 2 and rows[0].startswith("2 x 200:") and rows[0].count("PFLOP/s") == 3


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_run_program(cases, dtype, tmp_path):
    case = cases["B"]
    records = list(trace_batches(unequal_batches(case)))
    out_dir = str(tmp_path / "out")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", case.dir, "--dtype", dtype, "--out",
           out_dir, "--max-tokens", str(max_live_tokens(records))]
    feed = "".join(json.dumps(r) + "\n" for r in records)
    proc = subprocess.run(cmd, input=feed, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split("\n")[:-1] == [f"done {r['step']}" for r in records]
    outputs = {}
    for r in records:
        n_want = sum(len(e["want"]) for e in r["entries"])
        path = os.path.join(out_dir, f"{r['step']}.f32")
        if n_want:
            outputs[r["step"]] = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(n_want, case.vocab))
        else:
            assert not os.path.exists(path)
    check_against_plain(case, collect_positions(records, outputs), dtype, "trace_run")
