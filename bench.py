"""Decode and prefill throughput of the Qwen3 engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--preset qwen3-4b] [--batch 8] [--layers L]
                    [--prompt-len 2048] [--slot-len 4096]

The workload is the one named for the reference's headline metric: Qwen3-4B layer sizes with
random weights in bfloat16, prompts of 2,048 uniform random token ids in 4,096-token cache
slots, greedy decoding. A step is one decode step of the whole batch through the generation
machinery (graph replay, token choice, token hand-back). One JSON line is printed:
decoded tokens per second at the main batch size, the prefill rate of one 2,048-token prompt
with its fraction of the bf16 matrix-core peak, the decode step's fraction of the HBM
roofline (with the bytes, the time and the peak it is made of), and as further points the
decode rates at batch 1 and 64 and the rate of eight 2,048-token prompts prefilled in one
step. Timing protocol after the reference's harness
(agent/bench.py:96-126): untimed warm-up, synchronise on both sides of the timed region.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X: 8 TB/s
PEAK_FLOPS = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}
PROMPT, SLOT = 2048, 4096


def decode_bytes(engine, batch: int, context: float) -> float:
    """What a decode step has to read: every weight it uses once, and the cache of the live requests."""
    return engine.model.streamed_weight_bytes() + batch * engine.cache.bytes_read(context)


def prefill_flops(engine, tokens: int) -> float:
    """One prompt of `tokens` tokens whose logits are wanted at its last position."""
    return engine.model.step_flops([(0, tokens)], 1)


def main() -> int:
    global PROMPT, SLOT
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--preset", default="qwen3-4b")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the preset has")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and batch 64 points")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--phase", default="all", choices=["all", "decode", "prefill"],
                    help="measure only one phase (for profiling); the JSON line then lacks the other")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-tune", action="store_true",
                    help="keep the vendor library's default kernels for the prompt's matrix products")
    ap.add_argument("--prompt-len", type=int, default=PROMPT, help="tokens of every prompt (the context decoding starts at)")
    ap.add_argument("--slot-len", type=int, default=None, help="tokens a cache slot holds (default: twice the prompt)")
    args = ap.parse_args()
    PROMPT = args.prompt_len
    SLOT = args.slot_len or max(SLOT, 2 * PROMPT)
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (asked for {args.gpus}); this library has no multi-GPU path")
        return 2

    import numpy as np
    import torch

    from dataclasses import asdict

    from dryft_amd import Engine
    from dryft_amd.models import load_preset

    raw = dict(load_preset(args.preset))
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    # the cache holds what the largest batch needs at the end of its run, no more (long contexts at small batches)
    engine = Engine(config=raw, seed=args.seed, dtype=args.dtype, max_batch=max_batch, max_len=SLOT,
                    max_tokens=max_batch * (PROMPT + 2 * (args.steps + args.warmup) + 192), use_graph=not args.no_graph,
                    verbose=True)
    cfg = engine.config
    vocab = engine.model.plan.vocab_size
    if not args.no_tune and args.dtype == "bfloat16":
        t0 = time.perf_counter()
        rows = sorted({PROMPT, args.batch, args.batch * PROMPT} | (set() if args.no_points else {64}))
        engine.tune(rows)                                               # outside every timed region
        print(f"[bench] vendor library tuned for steps of {rows} rows in {time.perf_counter() - t0:.1f}s",
              file=sys.stderr, flush=True)
    rng = np.random.default_rng(args.seed)

    def prompts(b):
        return [[int(t) for t in rng.integers(0, vocab, size=PROMPT)] for _ in range(b)]

    def sync():
        torch.cuda.synchronize()

    def decode_rate(batch: int, steps: int, warmup: int):
        """(tokens/s, ms per step, mean context) for `steps` decode steps after a 2,048-token prefill."""
        stream = engine.generate(prompts(batch), warmup + steps + 1)      # the library's own generation loop
        try:
            next(stream)                                                  # the prompts' step
            for _ in range(warmup):
                next(stream)
            sync()
            t0 = time.perf_counter()
            for _ in range(steps):
                next(stream)
            sync()
            dt = time.perf_counter() - t0
        finally:
            stream.close()
        context = PROMPT + warmup + (steps + 1) / 2.0
        return batch * steps / dt, dt / steps * 1e3, context

    def prefill_rate(n_prompts: int = 1, repeats: int = 3):
        """(tokens/s, ms) of `n_prompts` prompts prefilled in one step: the best of `repeats` runs."""
        best = None
        for _ in range(repeats + 1):                       # the first run warms libraries up
            slots = engine.acquire(n_prompts)
            p = prompts(n_prompts)
            sync()
            t0 = time.perf_counter()
            engine.start(slots, p, 0)
            sync()
            dt = time.perf_counter() - t0
            engine.release(slots)
            best = dt if best is None else min(best, dt)
        return n_prompts * PROMPT / best, best * 1e3

    tok_s = ms_step = achieved = need = pf_tok_s = pf_ms = pf_frac = pf_flops = 0.0
    peak = PEAK_FLOPS["bf16" if args.dtype == "bfloat16" else "fp32"]
    if args.phase in ("all", "decode"):
        tok_s, ms_step, context = decode_rate(args.batch, args.steps, args.warmup)
        need = decode_bytes(engine, args.batch, context)
        achieved = need / (ms_step * 1e-3) / 1e9
    if args.phase in ("all", "prefill"):
        pf_tok_s, pf_ms = prefill_rate()
        pf_flops = prefill_flops(engine, PROMPT)
        pf_frac = pf_flops / (pf_ms * 1e-3) / peak
    points, points_frac = {}, {}
    if not args.no_points and args.phase == "all":
        for b in (1, 64):
            rate, ms, ctx = decode_rate(b, max(16, args.steps // 2), max(4, args.warmup // 2))
            points[f"decode_b{b}"] = round(rate, 1)
            # the same roofline as the main batch: bytes the step has to read / its time / the HBM peak
            points_frac[f"decode_b{b}"] = round(decode_bytes(engine, b, ctx) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
        # eight prompts in one step: tokens a second, and the step's flops / time / peak
        if 8 * (PROMPT + 64) <= engine.max_tokens:
            rate, ms = prefill_rate(8, repeats=2)
            points["prefill_b8"] = round(rate, 1)
            points_frac["prefill_b8"] = round(engine.model.step_flops([(0, PROMPT)] * 8, 8) / (ms * 1e-3) / peak, 4)
    line = {
        "metric": f"decode tok/s ({args.preset} layer sizes, {PROMPT:,}-token prompts, {SLOT:,}-token slots)",
        "value": round(tok_s, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights, uniform random token ids)",
        # every size of the typed configuration under its config.json name (the layers are those that ran), flat
        "config": {
            "model": args.preset, "global_batch": args.batch, "seq_len": SLOT, "prompt_len": PROMPT,
            "parallelism": "none", "layers_of_model": full_layers, "graph": not args.no_graph,
            "library_tuned": not args.no_tune,
            **{k: v for k, v in asdict(cfg).items() if isinstance(v, (bool, int, float, str))},
        },
        "prefill": {"value": round(pf_tok_s, 1), "tokens": PROMPT, "ms": round(pf_ms, 3), "frac": round(pf_frac, 4),
                    "tflop": round(pf_flops / 1e12, 3), "peak_tflops": peak / 1e12},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "gbytes": round(need / 1e9, 4),
                     "ms": round(ms_step, 4)},
        "points": points,
        "points_frac": points_frac,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
