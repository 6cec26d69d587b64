"""SwiGLU feed-forward: ``down( silu(gate(h)) * up(h) )``, dense, no bias.

Reference: engine/dryft_qwen3/model.py:44-46, 180. Gate and up are fused into one
product by stacking their rows (weights.py:98-100).
"""

from __future__ import annotations

import torch

from ..csrc import ops
from . import register_part
from .base import FeedForward, matrix
from .linear import STREAM_ROWS, few_rows_ok, linear, panel_swiglu_ok, tall_swiglu_ok


class SwiGLU(FeedForward):
    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden, self.inter = int(hidden_size), int(intermediate_size)
        self.w_gate_up: torch.Tensor | None = None
        self.w_down: torch.Tensor | None = None

    def tensor_specs(self):
        return {"gate_proj": matrix((self.inter, self.hidden)), "up_proj": matrix((self.inter, self.hidden)),
                "down_proj": matrix((self.hidden, self.inter))}

    def load(self, tensors):
        self.w_gate_up = torch.cat([tensors["gate_proj"], tensors["up_proj"]], dim=0).contiguous()
        self.w_down = tensors["down_proj"]

    def kernel_modules(self, dtype):
        return ("gemm", "activation")

    def forward(self, h, ctx):
        act = torch.empty((h.shape[0], self.inter), dtype=h.dtype, device=h.device)
        if h.dtype == torch.bfloat16 and panel_swiglu_ok(h, self.w_gate_up):
            ops.gemm_panel_swiglu_bf16(h, self.w_gate_up, act)        # product and activation in one kernel
        elif h.dtype == torch.bfloat16 and tall_swiglu_ok(h, self.w_gate_up):
            ops.gemm_tall_swiglu_bf16(h, self.w_gate_up, act)         # the same at 65 to 256 rows
        elif h.dtype == torch.bfloat16 and h.shape[0] <= STREAM_ROWS and few_rows_ok(h, self.w_gate_up):
            ops.gemm_stream_swiglu_bf16(h, self.w_gate_up, act)       # the same for any K that is a multiple of 8
        else:
            ops.silu_mul(linear(h, self.w_gate_up), act)
        return linear(act, self.w_down, allow_partials=True)


register_part("swiglu", SwiGLU)
