"""Typed configuration of the Qwen3 dense decoder.

Field names are the ``config.json`` key names. The keys read and the options
refused follow the reference (engine/dryft_qwen3/config.py:137-155): read are
the sizes, ``rms_norm_eps``, ``rope_theta``, ``tie_word_embeddings`` and
``max_position_embeddings`` (optional here: it only bounds lengths); ``hidden_act`` must be ``silu``, ``attention_bias``
false, ``rope_scaling`` null, ``use_sliding_window`` false, and the q heads a
multiple of the kv heads. ``head_dim`` falls back to ``hidden_size //
num_attention_heads`` (config.py:142). Unlike the reference no checkpoint is
pinned: every size comes from the file.
"""

from __future__ import annotations

from dataclasses import asdict, dataclass
from typing import Any

from ..limits import MAX_HEAD_DIM
from .base import KeyReader


@dataclass(frozen=True)
class Qwen3Config:
    num_hidden_layers: int
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    max_position_embeddings: int | None = None      # only bounds lengths; absent: no bound from the model

    architecture = "Qwen3ForCausalLM"

    # ---- derived widths (config.py:87-101 of the reference)
    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def group(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "Qwen3Config":
        r = KeyReader(raw)
        hidden = r.integer("hidden_size")
        heads = r.integer("num_attention_heads")
        kv_heads = r.integer("num_key_value_heads", default=heads if heads else 1)
        if raw.get("head_dim"):
            head_dim = r.integer("head_dim")
        else:                                        # absent, null or 0: config.py:142 of the reference
            head_dim = hidden // heads if heads else 0
        cfg = cls(
            num_hidden_layers=r.integer("num_hidden_layers"),
            hidden_size=hidden,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=r.integer("intermediate_size"),
            vocab_size=r.integer("vocab_size"),
            rms_norm_eps=r.number("rms_norm_eps"),
            rope_theta=r.number("rope_theta"),
            tie_word_embeddings=r.boolean("tie_word_embeddings", default=False),
            max_position_embeddings=(r.integer("max_position_embeddings")
                                     if raw.get("max_position_embeddings") is not None else None),
        )
        r.require("hidden_act", lambda v: v == "silu", "silu", "only 'silu' is supported")
        r.require("attention_bias", lambda v: v is False, False, "projection biases are not supported")
        r.require("rope_scaling", lambda v: v is None, None, "scaled rotary positions are not supported")
        r.require("use_sliding_window", lambda v: not v, False, "sliding-window attention is not supported")
        if heads and kv_heads:
            r.check(heads % kv_heads == 0,
                    f"num_attention_heads ({heads}) is not a multiple of num_key_value_heads ({kv_heads})")
        if cfg.head_dim:
            r.check(cfg.head_dim % 2 == 0, f"head_dim: must be even for rotary pairs, got {cfg.head_dim}")
            r.check(cfg.head_dim <= MAX_HEAD_DIM,
                    f"head_dim: the attention kernels take at most {MAX_HEAD_DIM}, got {cfg.head_dim}")
        r.finish("unsupported or malformed Qwen3 config.json")
        return cfg

    def to_dict(self) -> dict[str, Any]:
        """The ``config.json`` content that reads back as this configuration."""
        d = {k: v for k, v in asdict(self).items() if v is not None}
        d.update(architectures=[self.architecture], model_type="qwen3", hidden_act="silu",
                 attention_bias=False, rope_scaling=None, use_sliding_window=False,
                 torch_dtype="bfloat16")
        return d
