"""Shared by the tests: the two tiny configurations, model folders, paged-cache builders."""

from __future__ import annotations

import json
import os

import numpy as np
import torch
from safetensors import safe_open

# Two tiny Qwen3 configurations that differ in every size and option.
TINY_A = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": 2, "hidden_size": 64,
    "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 128, "vocab_size": 256,
    "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 4096,
    "hidden_act": "silu", "attention_bias": False,
}
TINY_B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": 3, "hidden_size": 96,
    "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 32, "intermediate_size": 224, "vocab_size": 384,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 4096,
    "hidden_act": "silu", "attention_bias": False,
}
# a third one with a wider head and more heads per group, sizes that are no power of two
TINY_C = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": 2, "hidden_size": 80,
    "num_attention_heads": 6, "num_key_value_heads": 3, "head_dim": 48, "intermediate_size": 136, "vocab_size": 331,
    "rope_theta": 50000.0, "rms_norm_eps": 3e-6, "tie_word_embeddings": False, "max_position_embeddings": 2048,
    "hidden_act": "silu", "attention_bias": False,
}
# a fourth one whose widths are not multiples of 8 (no 16-byte rows) and whose vocabulary is a prime: it takes
# the plain kernels where the vector and matrix-core kernels refuse the sizes; one kv head per query head
TINY_D = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": 2, "hidden_size": 100,
    "num_attention_heads": 5, "num_key_value_heads": 5, "head_dim": 16, "intermediate_size": 108, "vocab_size": 257,
    "rope_theta": 20000.0, "rms_norm_eps": 2e-6, "tie_word_embeddings": True, "max_position_embeddings": 1024,
    "hidden_act": "silu", "attention_bias": False,
}
# a fifth one whose head size (40) is no multiple of 16: the matrix-core attention kernels do not take it, so
# bfloat16 runs on the plain attention kernel like float32; three query heads on one kv head
TINY_E = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": 2, "hidden_size": 72,
    "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 40, "intermediate_size": 104, "vocab_size": 300,
    "rope_theta": 30000.0, "rms_norm_eps": 4e-6, "tie_word_embeddings": False, "max_position_embeddings": 512,
    "hidden_act": "silu", "attention_bias": False,
}
TINY = {"D": (TINY_D, dict(seed=44, norm_std=0.1, std=0.04)), "A": (TINY_A, dict(seed=11, norm_std=0.0, std=0.02)), "B": (TINY_B, dict(seed=22, norm_std=0.1, std=0.02)),
        "C": (TINY_C, dict(seed=33, norm_std=0.1, std=0.05)), "E": (TINY_E, dict(seed=55, norm_std=0.1, std=0.05))}


def make_model_dir(path: str, raw_config: dict, seed: int, norm_std: float = 0.0, std: float = 0.02,
                   dtype=torch.bfloat16, scale: float = 1.0) -> str:
    """A model folder with seeded random weights, written through the library's random-weights mode."""
    from dryft_amd.engine.model import DecoderModel
    from dryft_amd.models import resolve_architecture
    from dryft_amd.weights import random_tensors, write_model_dir

    arch = resolve_architecture(raw_config)
    cfg = arch.config_class.from_dict(raw_config)
    model = DecoderModel(arch.plan(cfg), torch.float32, "cpu")
    tensors = random_tensors(model.tensor_specs(), seed, dtype, std=std * scale, norm_std=norm_std)
    return write_model_dir(path, raw_config, tensors)


def read_model_dir(path: str):
    """(raw config, tensors by name as float32), read with the safetensors library directly."""
    with open(os.path.join(path, "config.json")) as f:
        raw = json.load(f)
    tensors = {}
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name).to(torch.float32)
    return raw, tensors


def random_tokens(n: int, vocab: int, seed: int) -> list[int]:
    rng = np.random.default_rng(seed)
    return [int(t) for t in rng.integers(0, vocab, size=n)]


def value_columns() -> torch.Tensor:
    """Column of a page of values that holds each of its 64 positions: within a block of 32, position
    ``16a + 4g + i`` sits in column ``8g + 4a + i`` (the order in which attention's second product takes them)."""
    pos = torch.arange(64)
    o = pos % 32
    return (pos // 32) * 32 + 8 * ((o // 4) % 4) + 4 * (o // 16) + o % 4


def build_pages(k: torch.Tensor, v: torch.Tensor, lengths, n_pages: int, n_slots: int, seed: int = 0,
                poison: float | None = None):
    """Scatter dense keys/values ``[B, L, nKV, D]`` into shuffled pages.

    Returns (k_pages [P,nKV,64,D], v_pages [P,nKV,D,64] viewed as [P,nKV,64,D] storage, page_table
    [n_slots, max_pages], slots). Sequence b lives in slot ``slots[b]``. Page bytes that no length
    covers are filled with ``poison`` (finite garbage) when given.
    """
    B, L, n_kv, D = k.shape
    max_pages = (L + 63) // 64
    rng = np.random.default_rng(seed)
    order = rng.permutation(n_pages)
    slots = [int(s) for s in rng.permutation(n_slots)[:B]]
    fill = 0.0 if poison is None else poison
    k_pages = torch.full((n_pages, n_kv, 64, D), fill, dtype=k.dtype)
    v_pages_t = torch.full((n_pages, n_kv, D, 64), fill, dtype=v.dtype)
    table = torch.full((n_slots, max_pages), -1, dtype=torch.int32)
    cols = value_columns()
    nxt = 0
    for b in range(B):
        n = int(lengths[b])
        for pg in range((n + 63) // 64):
            page = int(order[nxt]); nxt += 1
            table[slots[b], pg] = page
            lo, hi = pg * 64, min(n, pg * 64 + 64)
            k_pages[page, :, : hi - lo] = k[b, lo:hi].transpose(0, 1)
            v_pages_t[page][:, :, cols[: hi - lo]] = v[b, lo:hi].permute(1, 2, 0)
    return k_pages, v_pages_t.reshape(n_pages, n_kv, 64, D), table, slots


def bf16_tolerance(ref: torch.Tensor, ulps: float = 2.0, floor: float = 0.0) -> float:
    """'One bf16 ulp of slack relative to the largest output' times ``ulps`` (kernels/rmsnorm.py:108)."""
    return ulps * 2.0 ** -8 * float(ref.abs().max()) + floor


# ------------------------------------------------------------------------------------------ traces
def trace_whole(requests: dict[str, list[int]]):
    """Each request alone, all tokens in one step, logits everywhere. Yields step records."""
    step = 0
    for rid, toks in requests.items():
        yield {"step": step, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
        step += 1


def trace_tail(requests: dict[str, list[int]], tail: int = 32):
    """Each request alone: all but the last ``tail`` tokens in one step, then one token per step."""
    step = 0
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        yield {"step": step, "entries": [{"id": rid, "tokens": toks[:head], "want": [head - 1]}],
               "end": [rid] if head == len(toks) else []}
        step += 1
        for i in range(head, len(toks)):
            yield {"step": step, "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}],
                   "end": [rid] if i == len(toks) - 1 else []}
            step += 1


def trace_batches(batches: list[dict[str, tuple[list[int], int]]]):
    """Batches one after another. Each batch maps id -> (tokens, k): the first len-k tokens start together
    in one step, then every live request goes on by one token per step; shorter requests end earlier."""
    step = 0
    for batch in batches:
        fed = {rid: max(1, len(toks) - k) for rid, (toks, k) in batch.items()}
        entries = [{"id": rid, "tokens": toks[:fed[rid]], "want": [fed[rid] - 1]} for rid, (toks, k) in batch.items()]
        end = [rid for rid, (toks, k) in batch.items() if fed[rid] == len(toks)]
        yield {"step": step, "entries": entries, "end": end}
        step += 1
        live = [rid for rid in batch if rid not in end]
        while live:
            entries, end = [], []
            for rid in live:
                toks = batch[rid][0]
                entries.append({"id": rid, "tokens": [toks[fed[rid]]], "want": [0]})
                fed[rid] += 1
                if fed[rid] == len(toks):
                    end.append(rid)
            yield {"step": step, "entries": entries, "end": end}
            step += 1
            live = [rid for rid in live if rid not in end]


def collect_positions(records, outputs):
    """Match the rows of each step's output to (request id, position). ``outputs[step]`` is [wanted, vocab].
    Returns {(id, position): logits row}."""
    seen: dict[str, int] = {}
    got = {}
    for rec in records:
        row = 0
        for e in rec["entries"]:
            base = seen.get(e["id"], 0)
            for w in e["want"]:
                got[(e["id"], base + w)] = outputs[rec["step"]][row]
                row += 1
            seen[e["id"]] = base + len(e["tokens"])
        for rid in rec["end"]:
            seen.pop(rid, None)
    return got


def max_live_tokens(records) -> int:
    """The --max-tokens a trace needs: most tokens held at once, each request rounded up to 64."""
    held: dict[str, int] = {}
    peak = 0
    for rec in records:
        for e in rec["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // 64) * 64 for n in held.values()))
        for rid in rec["end"]:
            held.pop(rid, None)
    return peak
