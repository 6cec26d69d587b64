"""Token embedding and output head.

Embedding: a row gather without scaling (reference: engine/dryft_qwen3/model.py:132).
Head: ``logits = h @ W.T`` as float32. A tied head is a plan that gives the head the
embedding's tensor name (weights.py:47-49): both parts then hold the same tensor. The reference keeps bfloat16 logits (model.py:186, 261); here the
float accumulators are stored directly.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from . import register_part
from .base import Part, matrix
from .linear import linear


class TokenEmbedding(Part):
    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab, self.hidden = int(vocab_size), int(hidden_size)
        self.weight: torch.Tensor | None = None

    def tensor_specs(self):
        return {"weight": matrix((self.vocab, self.hidden))}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def kernel_modules(self, dtype):
        return ("embed",)

    def reads_whole(self) -> bool:
        return False                      # a step gathers its rows' entries only

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        out = torch.empty((tokens.numel(), self.hidden), dtype=self.weight.dtype, device=self.weight.device)
        return ops.embed_rows(tokens, self.weight, out)


class LMHead(Part):
    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab, self.hidden = int(vocab_size), int(hidden_size)
        self.weight: torch.Tensor | None = None

    def tensor_specs(self):
        return {"weight": matrix((self.vocab, self.hidden))}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def kernel_modules(self, dtype):
        return ("gemm",)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return linear(h, self.weight, out_dtype=torch.float32)


register_part("token_embedding", TokenEmbedding)
register_part("lm_head", LMHead)
