"""Trace replay: feed given token ids through a model step by step and write logits.

It samples nothing and has no forward pass, cache or loader of its own: it builds an
``Engine`` and calls its step function. The reference has no such program; its nearest
relatives are the teacher-forced margin check (agent/verify.py:100-109) and the graph
validation that restores inputs and replays (engine/dryft_qwen3/graphs.py:146-169).

Input, one JSON object per line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
The requests of a step either all start or all go on by one token. For a step in which
logits are wanted, ``<out>/<step>.f32`` receives them as little-endian float32
``[wanted, vocab]`` in the order of the entries and of ``want``. After each step a line
``done <step>`` is printed and flushed.
"""

from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time, each request rounded up to a whole cache page")
    return ap


class Replayer:
    """Keeps the request-id -> cache-slot map and drives ``Engine.step``."""

    def __init__(self, engine):
        self.engine = engine
        self.slot_of: dict[str, int] = {}

    def run_step(self, record: dict):
        from .step import SeqStep

        seqs = []
        for e in record.get("entries", []):
            rid = str(e["id"])
            if rid not in self.slot_of:
                self.slot_of[rid] = self.engine.acquire(1)[0]
            seqs.append(SeqStep(self.slot_of[rid], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
        logits = self.engine.step(seqs) if seqs else None
        ended = [str(r) for r in record.get("end", [])]
        slots = [self.slot_of.pop(r) for r in ended if r in self.slot_of]
        if slots:
            self.engine.release(slots)
        return logits


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    from ..cache.spec import PAGE_TOKENS, pages_for
    from ..config.base import read_config_json
    from ..models import resolve_architecture
    from .engine import Engine

    os.makedirs(args.out, exist_ok=True)
    # the budget in whole pages; one request may take all of it, up to what the model allows
    pages = max(1, pages_for(args.max_tokens))
    raw = read_config_json(args.model)
    arch = resolve_architecture(raw)
    limit = arch.plan(arch.config_class.from_dict(raw)).max_positions
    max_len = min(pages * PAGE_TOKENS, limit) if limit else pages * PAGE_TOKENS
    engine = Engine(args.model, dtype=args.dtype, max_batch=min(pages, 4096), max_len=max_len,
                    max_tokens=pages * PAGE_TOKENS, use_graph=False)
    replayer = Replayer(engine)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        logits = replayer.run_step(record)
        if logits is not None and logits.shape[0] > 0:
            arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            tmp = os.path.join(args.out, f".{record['step']}.f32.tmp")
            arr.tofile(tmp)
            os.replace(tmp, os.path.join(args.out, f"{record['step']}.f32"))
        print(f"done {record['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
