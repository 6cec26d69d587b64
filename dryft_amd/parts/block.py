"""Arrangement of parts in a layer.

``PreNormBlock``: ``x = x + mixer(norm(x))``; ``x = x + ffn(norm(x))`` (reference:
engine/dryft_qwen3/model.py:151-184). Each residual sum is folded into the norm that
follows it, so a block receives the previous block's not-yet-added output as
``pending`` and hands its own feed-forward output on in the same way.
"""

from __future__ import annotations

from . import register_block
from .base import FeedForward, Mixer, Norm


class PreNormBlock:
    roles = ("mixer_norm", "mixer", "ffn_norm", "ffn")

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, ffn: FeedForward):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def parts(self):
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "ffn_norm": self.ffn_norm, "ffn": self.ffn}

    def forward(self, x, pending, ctx, line, writes_cache: bool):
        if pending is None:
            h = self.mixer_norm.forward(x)
        else:
            x, h = self.mixer_norm.add_forward(x, pending)
        mixed = self.mixer.forward(h, ctx, line, writes_cache)
        x, h = self.ffn_norm.add_forward(x, mixed)
        return x, self.ffn.forward(h, ctx)


register_block("prenorm", PreNormBlock)
