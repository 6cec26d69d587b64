"""Grouped-query attention over the paged cache.

Per row: ``q, k, v`` from one fused projection (reference: engine/dryft_qwen3/weights.py:93-96);
optional RMSNorm over each q and k head (one weight per head width, before the rotation,
model.py:165-166); optional rotary positions; append k and v to the cache line (model.py:170-171);
causal scores ``(q . k) / sqrt(head_dim)`` against every cached key of the sequence up to the row's
own position (or the last ``window`` of them), query head ``h`` reading kv head ``h // group``
(model.py:172-177, 254-257); output projection (model.py:179). No biases.

The part knows nothing of the model around it: sizes and constants are constructor arguments, the
position encoding is looked up by name in the step context, and its storage is the cache line it
is handed.
"""

from __future__ import annotations

import math

import torch

from ..cache.spec import KVNeed
from ..cache.store import KVLine
from ..csrc import ops
from ..limits import MATRIX_CORE_HEAD_STEP, MAX_HEAD_DIM
from ..weights.spec import VECTOR
from . import register_part
from .base import Mixer, Partials, StepContext, matrix
from .linear import linear

_RESIDENT_WORKGROUPS = 512     # of the split kernel: two per compute unit (its registers allow no more)
_MAX_SPLITS = 32
_QKV_PARTIAL_ROWS = 256         # decoding steps of up to so many rows take the projection as partial sums over K
_PROMPT_PARTIAL_ROWS = 256      # and so do prompt steps of at most so many rows


class GQAAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 qk_norm_eps: float | None = None, positions: str | None = None, rotary_dim: int | None = None,
                 window: int | None = None, scale: float | None = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads cannot share {num_kv_heads} kv heads evenly")
        if not 0 < head_dim <= MAX_HEAD_DIM:
            raise ValueError(f"head_dim must lie in 1..{MAX_HEAD_DIM}, got {head_dim}")
        self.hidden, self.n_heads, self.n_kv, self.head_dim = int(hidden_size), int(num_heads), int(num_kv_heads), int(head_dim)
        self.qk_norm_eps = qk_norm_eps
        self.positions = positions
        self.rotary_dim = int(rotary_dim if rotary_dim is not None else head_dim) if positions else 0
        if self.rotary_dim % 2 or self.rotary_dim > head_dim:
            raise ValueError(f"the rotated width must be even and at most head_dim ({head_dim}), got {self.rotary_dim}")
        self.window = int(window) if window else None
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)   # model.py:65
        self.q_dim, self.kv_dim = self.n_heads * self.head_dim, self.n_kv * self.head_dim
        self.w_qkv = self.w_o = self.q_norm = self.k_norm = None

    def tensor_specs(self):
        specs = {"q_proj": matrix((self.q_dim, self.hidden)), "k_proj": matrix((self.kv_dim, self.hidden)),
                 "v_proj": matrix((self.kv_dim, self.hidden)), "o_proj": matrix((self.hidden, self.q_dim))}
        if self.qk_norm_eps is not None:
            specs["q_norm"] = ((self.head_dim,), VECTOR, "ones")
            specs["k_norm"] = ((self.head_dim,), VECTOR, "ones")
        return specs

    def load(self, tensors):
        self.w_qkv = torch.cat([tensors["q_proj"], tensors["k_proj"], tensors["v_proj"]], dim=0).contiguous()
        self.w_o = tensors["o_proj"]
        if self.qk_norm_eps is not None:
            self.q_norm, self.k_norm = tensors["q_norm"], tensors["k_norm"]
            if self.q_norm.dtype != self.k_norm.dtype:          # one kernel argument says how both are stored
                self.q_norm, self.k_norm = self.q_norm.float(), self.k_norm.float()

    def cache_need(self):
        return KVNeed(self.n_kv, self.head_dim, self.window)

    def kernel_modules(self, dtype):
        return ("gemm", "rope_kv", "attn_rows") + (("attn_mfma",) if dtype == torch.bfloat16 else ())

    def forward(self, h: torch.Tensor, ctx: StepContext, line: KVLine, writes_cache: bool):
        rows = h.shape[0]
        # bfloat16 on the matrix cores where they take the head size; float32 and the other head sizes on the plain kernel
        matrix_cores = h.dtype == torch.bfloat16 and self.head_dim % MATRIX_CORE_HEAD_STEP == 0
        decoding = matrix_cores and ctx.max_q_len == 1
        fused_decoding = decoding and self.n_heads // self.n_kv <= 16
        # The kernel that norms, rotates, appends and attends in one adds up partial sums of the projection on its way
        # in, so K may be split over workgroups. Measured on Qwen3-4B's sizes, a decoding step with the split against
        # without: 2.980 against 3.008 ms at 8 sequences, 4.63 against 4.74 at 32, 6.75 against 6.86 at 64, 8.92 against
        # 9.04 at 96 and, since the product whose waves own rows of x, 5.89 against 5.97 at 192.
        cos = sin = None
        if self.positions:
            table = ctx.positions[self.positions]
            cos, sin = table.cos, table.sin
            if ctx.max_kv_len > table.n_positions:
                raise ValueError(f"position tables cover {table.n_positions} positions, the step reaches {ctx.max_kv_len}")
        # So does the kernel that takes a short prompt's keys and values to the cache (and its queries out): up to 256
        # rows the split product is ahead of the vendor library's (Qwen3-4B's q/k/v: 11.7 against 15.2 us at 64 rows,
        # 17.9 against 31.0 at 256).
        prompt_parts = matrix_cores and not decoding and writes_cache and cos is not None and \
            rows <= _PROMPT_PARTIAL_ROWS and \
            ops.rows_to_cache_takes(rows, self.head_dim, self.rotary_dim, True)
        if prompt_parts:
            qkv = linear(h, self.w_qkv, allow_partials=True)
        else:
            qkv = linear(h, self.w_qkv, allow_partials=fused_decoding, partial_rows=_QKV_PARTIAL_ROWS)
        window = self.window or 0
        # The tiled prompt kernels never visit the rows of sequences that sit out, and the projection after them reads
        # every row: where the step may hold such sequences the output lives in a tensor that started as zeros, so
        # that those rows hold zeros or an earlier layer's or step's output, never what memory happened to hold.
        if ctx.max_q_len > 1 and ctx.some_sit_out():
            out = ctx.kept_zeros((rows, self.n_heads, self.head_dim), h.dtype)
        else:
            out = torch.empty((rows, self.n_heads, self.head_dim), dtype=h.dtype, device=h.device)
        if decoding:
            splits = self.decode_splits(ctx.n_seqs, ctx.max_kv_len)
            part_o = torch.empty((ctx.n_seqs, self.n_heads, splits, self.head_dim), dtype=torch.float32, device=h.device)
            part_ml = torch.empty((ctx.n_seqs, self.n_heads, splits, 2), dtype=torch.float32, device=h.device)
        if fused_decoding:
            # one token per sequence: norm, rotation, append and attention in one kernel
            parts = qkv.count if isinstance(qkv, Partials) else 0
            ops.attn_decode_fused_bf16(qkv.data if parts else qkv, self.q_norm, self.k_norm, self.qk_norm_eps or 0.0, cos, sin, self.rotary_dim,
                                       writes_cache, line.k, line.v, line.page_table, ctx.seq_slot, ctx.cu_rows,
                                       ctx.kv_len, ctx.n_seqs, part_o, part_ml, splits, out, self.n_heads, self.n_kv,
                                       self.head_dim, self.scale, window, qkv_parts=parts)
            return linear(out.view(rows, self.q_dim), self.w_o, allow_partials=True)
        if prompt_parts and isinstance(qkv, Partials):
            q = torch.empty((rows, self.n_heads, self.head_dim), dtype=h.dtype, device=h.device)
            ops.rows_to_cache_from_partials(qkv.data, self.q_norm, self.k_norm, self.qk_norm_eps or 0.0, cos, sin,
                                            self.rotary_dim, ctx.row_slot, ctx.row_pos, q, line.k, line.v,
                                            line.page_table, self.n_heads, self.n_kv, self.head_dim)
            tile_cu, max_tiles = ctx.tiles(ops.ATTN_ROW_TILE)
            ops.attn_causal_bf16(q, line.k, line.v, line.page_table, ctx.seq_slot, ctx.cu_rows, tile_cu,
                                 ctx.seq_start, ctx.n_seqs, max_tiles, out, self.n_heads, self.n_kv,
                                 self.head_dim, self.scale, window)
            return linear(out.view(rows, self.q_dim), self.w_o, allow_partials=True)
        if matrix_cores and not decoding and cos is not None and \
                ops.attn_causal_takes_projection(self.head_dim, self.rotary_dim):
            # the prompt kernel norms and rotates the queries on their way in: only keys and values go to the cache here
            if writes_cache:
                ops.qk_norm_rope_kv(qkv, self.q_norm, self.k_norm, self.qk_norm_eps or 0.0, cos, sin, self.rotary_dim,
                                    ctx.row_slot, ctx.row_pos, None, line.k, line.v, line.page_table, True,
                                    self.n_heads, self.n_kv, self.head_dim)
            tile_cu, max_tiles = ctx.tiles(ops.ATTN_ROW_TILE)
            ops.attn_causal_projected_bf16(qkv, self.q_norm, self.qk_norm_eps or 0.0, cos, sin, line.k, line.v,
                                           line.page_table, ctx.seq_slot, ctx.cu_rows, tile_cu, ctx.seq_start,
                                           ctx.n_seqs, max_tiles, out, self.n_heads, self.n_kv, self.head_dim,
                                           self.scale, window)
            return linear(out.view(rows, self.q_dim), self.w_o, allow_partials=True)
        q = torch.empty((rows, self.n_heads, self.head_dim), dtype=h.dtype, device=h.device)
        ops.qk_norm_rope_kv(qkv, self.q_norm, self.k_norm, self.qk_norm_eps or 0.0, cos, sin, self.rotary_dim,
                            ctx.row_slot, ctx.row_pos, q, line.k, line.v, line.page_table, writes_cache,
                            self.n_heads, self.n_kv, self.head_dim)
        if decoding:
            ops.attn_split_bf16(q, line.k, line.v, line.page_table, ctx.seq_slot, ctx.cu_rows, ctx.kv_len,
                                ctx.n_seqs, part_o, part_ml, splits, out, self.n_heads, self.n_kv, self.head_dim,
                                self.scale, window)
        elif matrix_cores:
            tile_cu, max_tiles = ctx.tiles(ops.ATTN_ROW_TILE)
            ops.attn_causal_bf16(q, line.k, line.v, line.page_table, ctx.seq_slot, ctx.cu_rows, tile_cu,
                                 ctx.seq_start, ctx.n_seqs, max_tiles, out, self.n_heads, self.n_kv,
                                 self.head_dim, self.scale, window)
        else:
            ops.attn_rows(q, line.k, line.v, line.page_table, ctx.row_slot, ctx.row_pos, out, self.n_heads, self.n_kv,
                          self.head_dim, self.scale, window)
        return linear(out.view(rows, self.q_dim), self.w_o, allow_partials=True)

    def flops(self, rows, spans):
        """The projections, and both attention products over the keys each row sees."""
        seen = 0
        for start, q in spans:
            first, last = start + 1, start + q                  # keys that the span's first and last row see
            if self.window:
                full = max(0, min(last, self.window) - first + 1)          # rows that still see every key
                seen += (2 * first + full - 1) * full // 2 + (q - full) * self.window
            else:
                seen += (first + last) * q // 2
        return super().flops(rows, spans) + 4.0 * self.q_dim * seen

    def decode_splits(self, n_seqs: int, max_kv_len: int) -> int:
        """How many ways each sequence's keys are split: as many as run at the same time, and no more.

        Workgroups beyond what the chip holds at once start when the first ones end, which costs more than
        the longer walk of fewer, larger splits.
        """
        blocks = self.n_kv * ((self.n_heads // self.n_kv + 15) // 16)
        want = _RESIDENT_WORKGROUPS // (n_seqs * blocks)
        span = self.window if self.window else max_kv_len
        pages = max(1, (span + 63) // 64)
        return max(1, min(want, _MAX_SPLITS, pages))


register_part("gqa_attention", GQAAttention)
