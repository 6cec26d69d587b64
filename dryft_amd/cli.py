"""Command line: token ids in, token ids out (the library has no tokenizer, like the reference:
AGENTS.md:120). Option names follow the reference's tools where it has them: ``--model`` with the
``DRYFT_MODEL_PATH`` environment variable as its default, ``--tiny`` for a random tiny model,
``--seed``, ``--samples`` and ``--workload name,b,in,out`` (agent/verify.py:181-190,
agent/bench.py:180-192).

    python -m dryft_amd generate --model DIR --prompt-ids "1,2,3;4,5" --max-new-tokens 8
    python -m dryft_amd generate --preset tiny-b --weight-seed 0 --random-prompts 3,5,9 --temperature 0.8
    python -m dryft_amd make-model --preset tiny-a --weight-seed 1 --out DIR
    python -m dryft_amd bench --preset qwen3-4b --workload b8,8,2048,64
    python -m dryft_amd profile --preset qwen3-4b --batch 8 --prompt-len 2048 --steps 8
    python -m dryft_amd attention --shapes 1x2048,8x2048 --modes 1,3,5,7
    python -m dryft_amd replay --model DIR --dtype float32 --out DIR --max-tokens 4096 < steps.jsonl
    python -m dryft_amd build [names...]
"""

from __future__ import annotations

import argparse
import json
import os
import random
import statistics
import sys
import time


def _add_model_options(ap: argparse.ArgumentParser) -> None:
    ap.add_argument("--model", default=os.environ.get("DRYFT_MODEL_PATH"),
                    help="folder with config.json and safetensors (default: $DRYFT_MODEL_PATH)")
    ap.add_argument("--preset", help="a named config with random weights instead of --model")
    ap.add_argument("--tiny", action="store_true", help="same as --preset tiny-a")
    ap.add_argument("--weight-seed", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32", "bfloat16", "float32"])
    ap.add_argument("--max-len", type=int, default=None,
                    help="longest sequence a cache slot can hold (default: what the command needs, or 8,192 where it "
                         "cannot know, bounded by what the model allows)")
    ap.add_argument("--max-batch", type=int, default=None, help="cache slots (default: the number of prompts)")
    ap.add_argument("--no-graph", action="store_true", help="run decoding steps without graph capture")


def _engine(args, max_batch: int, max_tokens: int | None = None):
    from . import Engine
    from .models import load_preset

    kw = dict(dtype=args.dtype, max_batch=args.max_batch or max_batch, max_len=args.max_len, max_tokens=max_tokens,
              use_graph=not args.no_graph, verbose=True)
    preset = "tiny-a" if args.tiny else args.preset
    if preset:
        return Engine(config=load_preset(preset), seed=args.weight_seed, **kw)
    if not args.model:
        raise SystemExit("need --model DIR (or DRYFT_MODEL_PATH), --preset NAME or --tiny")
    return Engine(args.model, **kw)


def _prompts(args, vocab: int) -> list[list[int]]:
    if args.prompt_ids:
        return [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt_ids.split(";")]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            return [[int(t) for t in p] for p in json.load(f)]
    if args.random_prompts:
        rng = random.Random(args.prompt_seed)
        return [[rng.randrange(vocab) for _ in range(int(n))] for n in args.random_prompts.split(",")]
    raise SystemExit("need --prompt-ids, --prompt-file or --random-prompts")


def cmd_generate(args) -> int:
    n = len(args.prompt_ids.split(";")) if args.prompt_ids else (len(args.random_prompts.split(",")) if args.random_prompts else 8)
    engine = _engine(args, max(1, n))
    prompts = _prompts(args, engine.model.plan.vocab_size)
    stops = [int(t) for t in args.stop_ids.split(",")] if args.stop_ids else []
    columns: list[list[int]] = [[] for _ in prompts]
    for step in engine.generate(prompts, args.max_new_tokens, temperature=args.temperature,
                                sample_seed=args.sample_seed, stop_token_ids=stops):
        for col, t in zip(columns, step):
            if t >= 0:
                col.append(t)
        if args.stream:
            print(json.dumps(step), flush=True)
    if not args.stream:
        for col in columns:
            print(",".join(map(str, col)))
    return 0


def cmd_make_model(args) -> int:
    import torch

    from .engine.model import DecoderModel
    from .models import resolve_architecture
    from .models import load_preset
    from .weights import random_tensors, write_model_dir

    if args.config:
        with open(args.config) as f:
            raw = json.load(f)
    else:
        raw = load_preset("tiny-a" if args.tiny else args.preset)
    arch = resolve_architecture(raw)
    model = DecoderModel(arch.plan(arch.config_class.from_dict(raw)), torch.float32, "cpu")
    dtype = torch.bfloat16 if args.dtype in ("bf16", "bfloat16") else torch.float32
    tensors = random_tensors(model.tensor_specs(), args.weight_seed, dtype, std=args.std, norm_std=args.norm_std)
    print(write_model_dir(args.out, raw, tensors))
    return 0


def cmd_build(args) -> int:
    """Compile the kernel libraries for gfx950 (all of them, or the named ones) without running anything."""
    from .csrc import build

    names = args.names or list(build.MODULES)
    for name, path in sorted(build.build(names, force=args.force).items()):
        print(f"{name}: {path}")
    return 0


def cmd_bench(args) -> int:
    """Per workload: one untimed warm-up call, then ``--samples`` timed calls with fresh random prompts
    (agent/bench.py:96-126); reports median tokens/s, time to first token and time per output token."""
    import torch

    workloads = [w.split(",") for w in (args.workload or ["b1,1,512,32", "b4,4,2048,32", "b16,16,512,128"])]
    workloads = [(n, int(b), int(i), int(o)) for n, b, i, o in workloads]
    args.max_len = max(args.max_len or 0, max(i + o for _, _, i, o in workloads))
    # the cache holds the largest workload, not the largest batch times the longest sequence
    engine = _engine(args, max(b for _, b, _, _ in workloads), max(b * (-(-(i + o) // 64) * 64) for _, b, i, o in workloads))
    if args.tune:
        engine.tune(sorted({b for _, b, _, _ in workloads} | {b * inp for _, b, inp, _ in workloads}))
    rng = random.Random(args.seed)
    vocab = engine.model.plan.vocab_size
    for name, b, inp, out in workloads:
        totals, firsts = [], []
        for sample in range(args.samples + 1):
            ids = [[rng.randrange(vocab) for _ in range(inp)] for _ in range(b)]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            first = None
            for _ in engine.generate(ids, out, temperature=args.temperature, sample_seed=args.seed + sample):
                if first is None:
                    first = time.perf_counter() - t0
            torch.cuda.synchronize()
            if sample:
                totals.append(time.perf_counter() - t0)
                firsts.append(first)
        med, ttft = statistics.median(totals), statistics.median(firsts)
        tpot = (med - ttft) / (out - 1) if out > 1 else 0.0
        print(json.dumps({"workload": name, "batch": b, "in": inp, "out": out, "tok_s": round(b * out / med, 1),
                          "total_ms": round(med * 1e3, 2), "ttft_ms": round(ttft * 1e3, 2),
                          "tpot_ms": round(tpot * 1e3, 3), "spread": round((max(totals) - min(totals)) / med, 3)}))
    return 0


def cmd_profile(args) -> int:
    """Where the time of decoding steps or of one prompt step goes, from ``torch.profiler``'s averages per kernel
    name: share, running share, microseconds and calls per step, and for decoding the bandwidth the step's bytes
    imply (what agent/profiler.py:58-89 reports).
    Decoding steps run without graph capture so that every kernel is visible by name (profiler.py:47-48)."""
    import torch
    from torch.profiler import ProfilerActivity, profile

    from .engine.step import SeqStep

    args.no_graph = True
    args.max_len = max(args.max_len or 0, args.prompt_len + args.steps + 8)
    engine = _engine(args, args.batch)
    rng = random.Random(args.seed)
    vocab = engine.model.plan.vocab_size
    prompts = [[rng.randrange(vocab) for _ in range(args.prompt_len)] for _ in range(args.batch)]
    slots = engine.acquire(args.batch)
    try:
        engine.reserve(slots, [args.prompt_len + args.steps + 4] * args.batch)
        if args.prefill:
            engine.step([SeqStep(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)])       # warm-up, then again
            engine.release(slots)
            slots = engine.acquire(args.batch)
            engine.reserve(slots, [args.prompt_len + args.steps + 4] * args.batch)
            torch.cuda.synchronize()
            with profile(activities=[ProfilerActivity.CPU, ProfilerActivity.CUDA]) as prof:
                engine.step([SeqStep(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)])
                torch.cuda.synchronize()
            steps, what = 1, f"one step of {args.batch} prompts of {args.prompt_len} tokens"
        else:
            tokens = engine.start(slots, prompts, 0)
            for i in range(2):
                tokens = engine.advance(slots, tokens, 1 + i)
            torch.cuda.synchronize()
            with profile(activities=[ProfilerActivity.CPU, ProfilerActivity.CUDA]) as prof:
                for i in range(args.steps):
                    tokens = engine.advance(slots, tokens, 3 + i)
                torch.cuda.synchronize()
            steps, what = args.steps, f"{args.steps} decoding steps of {args.batch} sequences at {args.prompt_len} tokens"
    finally:
        engine.release(slots)
    # the profiler's own per-name averages, device kernels only, longest first, with the share that has run up so far
    kernels = [(float(avg.self_device_time_total), int(avg.count), str(avg.key)) for avg in prof.key_averages()
               if "cuda" in str(avg.device_type).lower() and avg.self_device_time_total > 0]
    kernels.sort(reverse=True)
    total = sum(us for us, _, _ in kernels)
    launches = sum(n for _, n, _ in kernels)
    print(f"{what}")
    print(f"  {total / steps:.1f} us in {launches / steps:.0f} kernels a step")
    so_far = 0.0
    for us, n, name in kernels[: args.rows]:
        so_far += us
        print(f"  {us / total:6.1%} (to here {so_far / total:6.1%})  {us / steps:9.1f} us  x{n / steps:<6.1f} {name[:90]}")
    if not args.prefill and total > 0:
        weights = engine.model.streamed_weight_bytes()
        cache = args.batch * engine.cache.bytes_read(args.prompt_len + 2 + args.steps / 2)
        print(f"  the weights once and the cache of the live sequences in that time: "
              f"{(weights + cache) / (total / steps * 1e-6) / 1e9:.0f} GB/s")
    return 0


def cmd_kernel_table(args) -> int:
    """Reduces a ``rocprofv3 --kernel-trace`` recording of this library at work (its ``*_results.db``) to one table:
    the kernels of a step, how often each runs in it and for how long. Steps are told apart by the kernel that
    opens every step (``prepare_batch``); ``--kind decode`` keeps the steps that hold no prompt attention,
    ``--kind prompt`` those that do, and the last ``--steps`` of them are averaged."""
    import re
    import sqlite3
    import statistics

    cur = sqlite3.connect(args.database).cursor()
    tables = [r[0] for r in cur.execute("select name from sqlite_master where type='table'")]
    dispatches = next(t for t in tables if t.startswith("rocpd_kernel_dispatch"))
    symbols = next(t for t in tables if t.startswith("rocpd_info_kernel_symbol"))
    launches = cur.execute(f"select d.start, d.end, s.kernel_name from {dispatches} d join {symbols} s "
                           f"on d.kernel_id = s.id order by d.start").fetchall()
    opens = [i for i, (_, _, name) in enumerate(launches) if "prepare_batch" in name]
    steps = []
    for a, b in zip(opens[:-1], opens[1:]):
        step = launches[a:b]
        has_prompt = any("attn_causal" in name for _, _, name in step)
        if len(step) >= args.min_kernels and has_prompt == (args.kind == "prompt"):
            steps.append(step)
    steps = steps[-args.steps:]
    if not steps:
        print("no step of that kind in the recording", file=sys.stderr)
        return 1

    def plain_name(name: str) -> str:
        name = re.sub(r"\.kd$", "", re.sub(r"^_Z\d+", "", name))
        m = re.match(r"([a-z_0-9]+kernel)(I.*?E)?Ev", name)
        return (m.group(1) + (" <" + m.group(2)[1:-1] + ">" if m.group(2) else "")) if m else name[:64]

    per_kernel: dict[str, list[float]] = {}
    for step in steps:
        for start, end, name in step:
            entry = per_kernel.setdefault(plain_name(name), [0, 0.0])
            entry[0] += 1
            entry[1] += (end - start) / 1e3
    n = len(steps)
    busy = statistics.median(sum(e - s for s, e, _ in step) / 1e3 for step in steps)
    span = statistics.median((step[-1][1] - step[0][0]) / 1e3 for step in steps)
    print(f"{args.kind} steps averaged: {n}; kernels in a step: {len(steps[-1])}; "
          f"median time inside kernels {busy:.0f} us, median first start to last end {span:.0f} us")
    print(f"{'kernel':70s} {'in a step':>9s} {'us a step':>10s} {'us each':>8s} {'of the step':>11s}")
    for name, (count, us) in sorted(per_kernel.items(), key=lambda kv: -kv[1][1]):
        print(f"{name:70s} {count / n:9.1f} {us / n:10.1f} {us / count:8.2f} {us / n / busy:11.1%}")
    return 0


def cmd_attention(args) -> int:
    """Times the bfloat16 prompt-attention kernel alone: for each ``BxL`` (B sequences of L new positions each, nothing
    cached before them) and each way of running it (``ops.attn_causal_bf16``'s ``mode``), the best of four timings
    of about two milliseconds of calls each, the ways taking turns. PFLOP/s count the causal half of both products."""
    import torch

    from .cache.spec import PAGE_TOKENS, pages_for
    from .csrc import ops
    from .engine.engine import require_gpu

    dev = require_gpu("cuda:0")
    heads, kv, dim = args.heads, args.kv_heads, args.head_dim
    modes = [int(m) for m in args.modes.split(",")]
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    rand = lambda *shape: torch.randn(*shape, device=dev, generator=gen).to(torch.bfloat16)
    ints = lambda values: torch.tensor(values, dtype=torch.int32, device=dev)
    for shape in args.shapes.split(","):
        n_seqs, length = (int(x) for x in shape.lower().split("x"))
        pages = pages_for(length)
        k, v = rand(n_seqs * pages, kv, PAGE_TOKENS, dim), rand(n_seqs * pages, kv, dim, PAGE_TOKENS)
        q = rand(n_seqs * length, heads, dim)
        out = torch.empty_like(q)
        table = torch.arange(n_seqs * pages, dtype=torch.int32, device=dev).view(n_seqs, pages)
        seq_slot, seq_start = ints(list(range(n_seqs))), ints([0] * n_seqs)
        cu_rows = ints([length * i for i in range(n_seqs + 1)])
        tile_cu = ints([(-(-length // ops.ATTN_ROW_TILE)) * i for i in range(n_seqs + 1)])
        flops = 2.0 * n_seqs * length * length * heads * dim
        calls = max(3, int(2e-3 * 0.8e15 / flops))
        best = {m: float("inf") for m in modes}
        for _ in range(4):
            for m in modes:
                run = lambda: ops.attn_causal_bf16(q, k, v, table, seq_slot, cu_rows, tile_cu, seq_start, n_seqs,
                                                   n_seqs * (-(-length // ops.ATTN_ROW_TILE)), out, heads, kv, dim, dim ** -0.5, 0, m)
                run()
                torch.cuda.synchronize()
                begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                begin.record()
                for _ in range(calls):
                    run()
                end.record()
                torch.cuda.synchronize()
                best[m] = min(best[m], begin.elapsed_time(end) / calls * 1e-3)
        print(f"{n_seqs} x {length}: " + "  ".join(f"mode {m}: {best[m] * 1e6:8.1f} us {flops / best[m] / 1e15:5.3f} PFLOP/s"
                                                  for m in modes), flush=True)
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="dryft_amd", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="command", required=True)

    g = sub.add_parser("generate", help="generate token ids for given prompts")
    _add_model_options(g)
    g.add_argument("--prompt-ids", help='prompts as "1,2,3;4,5"')
    g.add_argument("--prompt-file", help="JSON file with a list of token-id lists")
    g.add_argument("--random-prompts", help="lengths of random prompts, e.g. 5,9,17")
    g.add_argument("--prompt-seed", type=int, default=0)
    g.add_argument("--max-new-tokens", type=int, default=16)
    g.add_argument("--temperature", type=float, default=0.0, help="0 = greedy")
    g.add_argument("--sample-seed", type=int, default=0)
    g.add_argument("--stop-ids", help="token ids that end a sequence, e.g. 151645,151643")
    g.add_argument("--stream", action="store_true", help="print one JSON list per step instead of one line per sequence")
    g.set_defaults(fn=cmd_generate)

    m = sub.add_parser("make-model", help="write a model folder with seeded random weights")
    m.add_argument("--preset", default="tiny-a")
    m.add_argument("--tiny", action="store_true")
    m.add_argument("--config", help="a config.json to use instead of a preset")
    m.add_argument("--weight-seed", type=int, default=0)
    m.add_argument("--std", type=float, default=0.02)
    m.add_argument("--norm-std", type=float, default=0.0)
    m.add_argument("--dtype", default="bf16", choices=["bf16", "fp32", "bfloat16", "float32"])
    m.add_argument("--out", required=True)
    m.set_defaults(fn=cmd_make_model)

    b = sub.add_parser("bench", help="time whole generate calls on given workloads")
    _add_model_options(b)
    b.add_argument("--samples", type=int, default=5)
    b.add_argument("--tune", action="store_true",
                   help="first let the vendor library choose its kernels for the workloads' step sizes")
    b.add_argument("--seed", type=int, default=0)
    b.add_argument("--temperature", type=float, default=0.0, help="0 = greedy")
    b.add_argument("--workload", action="append", help="name,batch,in,out (may repeat)")
    b.set_defaults(fn=cmd_bench)

    pr = sub.add_parser("profile", help="per-kernel table of decoding steps or of one prompt step")
    _add_model_options(pr)
    pr.add_argument("--batch", type=int, default=8)
    pr.add_argument("--prompt-len", type=int, default=2048)
    pr.add_argument("--steps", type=int, default=8)
    pr.add_argument("--prefill", action="store_true", help="profile the prompts' step instead of decoding steps")
    pr.add_argument("--rows", type=int, default=20, help="kernels to list")
    pr.add_argument("--seed", type=int, default=0)
    pr.set_defaults(fn=cmd_profile)

    kt = sub.add_parser("kernel-table", help="per-step kernel table from a rocprofv3 --kernel-trace recording (no GPU)")
    kt.add_argument("database", help="the recording's *_results.db")
    kt.add_argument("--kind", choices=["decode", "prompt"], default="decode")
    kt.add_argument("--steps", type=int, default=32, help="average over the last so many steps of that kind")
    kt.add_argument("--min-kernels", type=int, default=50, help="ignore stretches with fewer launches (warm-up odds and ends)")
    kt.set_defaults(fn=cmd_kernel_table)

    at = sub.add_parser("attention", help="time the prompt-attention kernel alone, in each way of running it")
    at.add_argument("--shapes", default="1x2048,1x4096,8x2048", help="BxL,...: B sequences of L positions each")
    at.add_argument("--modes", default="0", help="ways of running the kernel (ops.attn_causal_bf16's mode), e.g. 1,3,5,7")
    at.add_argument("--heads", type=int, default=32)
    at.add_argument("--kv-heads", type=int, default=8)
    at.add_argument("--head-dim", type=int, default=128)
    at.add_argument("--seed", type=int, default=0)
    at.set_defaults(fn=cmd_attention)

    bd = sub.add_parser("build", help="compile the HIP kernel libraries (needs hipcc, no GPU)")
    bd.add_argument("names", nargs="*", help="libraries to build (default: all)")
    bd.add_argument("--force", action="store_true", help="also rebuild what is up to date")
    bd.set_defaults(fn=cmd_build)

    r = sub.add_parser("replay", help="trace replay (same as bin/trace_run)", add_help=False)
    r.set_defaults(fn=None)

    if argv is None:
        argv = sys.argv[1:]
    if argv and argv[0] == "replay":
        from .engine.replay import main as replay_main
        return replay_main(argv[1:])
    args = ap.parse_args(argv)
    return args.fn(args)


if __name__ == "__main__":
    sys.exit(main())
