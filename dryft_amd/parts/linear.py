"""``y = x @ W.T`` for weights in checkpoint layout ``[out, in]`` (no bias).

The reference hands every projection to a vendor library (F.linear,
engine/dryft_qwen3/model.py:153, 179-180, 237, 258-261). Here:

* float32: this library's own kernel, plain multiply-adds, so the 32-bit path has no
  reduced-precision matrix mode anywhere;
* bfloat16, at most 16 rows (decoding at small batch) and the output head up to 64 rows:
  this library's weight-streaming matrix-core kernels (up to 16 rows the one that stages
  whole cache lines through LDS), which can leave their result as float32 partial sums
  over K for the consumer to add;
* bfloat16, 17 to 64 rows into a product whose consumer adds partial sums (the projections
  back to the hidden width): this library's shared-activation kernel with K split across
  workgroups;
* bfloat16, otherwise (prompts, decoding at large batch): the vendor library through
  ``torch.mm``, as in the reference; sizes it or the skinny kernel cannot take go to the
  plain kernel.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import Partials

SKINNY_ROWS = 64          # the most rows the skinny kernel takes
SKINNY_BEST = 16          # up to here it beats the vendor library on every projection shape measured
STREAM_ROWS = 16          # the most rows the line-staging variant takes
_TARGET_WORKGROUPS = 320   # a little more than one per compute unit
_BLOCKS_PER_WAVE = 10      # 64-value blocks of K a wave should walk at most


def skinny_plan(m: int, n: int, k: int) -> tuple[int, int]:
    """(weight tiles per wave, splits of K across workgroups) for the skinny kernel."""
    tiles = (n + 15) // 16
    m_tiles = (m + 15) // 16
    ntw = 1
    if m_tiles >= 2 and tiles >= 1024:
        ntw = 2
    if m_tiles >= 3 and tiles >= 4096:
        ntw = 4
    workgroups = (tiles + ntw - 1) // ntw
    k_blocks = (k + 63) // 64
    want = max((_TARGET_WORKGROUPS + workgroups - 1) // workgroups,        # enough workgroups to fill the chip
               (k_blocks + 4 * _BLOCKS_PER_WAVE - 1) // (4 * _BLOCKS_PER_WAVE))  # and no wave with a long walk over K
    splits = max(1, min(want, k_blocks // 8, 16))
    return ntw, splits


_STREAM_BLOCKS_PER_WAVE = 5     # measured on the projection shapes of 4B to 32B models inside captured graphs:
_STREAM_WORKGROUPS = 1536       # short walks over K, as long as the launch stays under about six workgroups a unit


def stream_plan(n: int, k: int, may_split: bool) -> tuple[int, int, int]:
    """(splits of K across workgroups, blocks per group, groups in flight) for the line-staging kernel.

    Splitting pays only where the consumer adds the partial sums up on its way (a pass of their own
    costs more than the split gains).
    """
    tiles = (n + 15) // 16
    k_blocks = (k + 63) // 64
    want = (k_blocks + 4 * _STREAM_BLOCKS_PER_WAVE - 1) // (4 * _STREAM_BLOCKS_PER_WAVE)
    splits = max(1, min(want, _STREAM_WORKGROUPS // tiles, k_blocks // 8, 16)) if may_split else 1
    return (splits, 1, 2) if splits > 1 else (1, 2, 2)


WIDE_ROWS = 64                  # the most rows the shared-activation kernel takes
_WIDE_BLOCKS = 8                # blocks of K a workgroup of it should walk


def wide_splits(n: int, k: int) -> int:
    """Splits of K for the shared-activation kernel where the consumer adds the partial sums."""
    tiles = (n + 63) // 64
    k_blocks = (k + 63) // 64
    return max(1, min((k_blocks + _WIDE_BLOCKS - 1) // _WIDE_BLOCKS, 1024 // tiles, k_blocks // 4, 16))


def skinny_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    return x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0


def linear(x: torch.Tensor, w: torch.Tensor, *, out_dtype: torch.dtype | None = None, allow_partials: bool = False):
    """Returns ``[rows, out]`` in ``out_dtype`` (default: the dtype of ``x``), or ``Partials``."""
    m, k = x.shape
    n = w.shape[0]
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.float32:
        return ops.gemm_tiled(x, w, torch.empty((m, n), dtype=torch.float32, device=x.device))
    library_ok = k % 8 == 0 and n % 8 == 0 and x.is_contiguous()
    if m <= SKINNY_ROWS and skinny_ok(x, w) and (m <= SKINNY_BEST or out_dtype == torch.float32 or not library_ok):
        stream = m <= STREAM_ROWS
        if stream:
            splits, group, depth = stream_plan(n, k, allow_partials)
        else:
            ntw, splits = skinny_plan(m, n, k)
        if splits > 1:
            partials = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
            if stream:
                ops.gemm_stream_bf16(x, w, None, partials, group, splits, depth)
            else:
                ops.gemm_skinny_bf16(x, w, None, partials, ntw, splits)
            if allow_partials:
                return Partials(partials, splits)
            return ops.sum_partials(partials, torch.empty((m, n), dtype=out_dtype, device=x.device), splits)
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
        if stream:
            ops.gemm_stream_bf16(x, w, out, None, group, 1, depth)
        else:
            ops.gemm_skinny_bf16(x, w, out, None, ntw, 1)
        return out
    if allow_partials and m <= WIDE_ROWS and skinny_ok(x, w):
        # 17 to 64 rows into a narrow output (the projections back to the hidden width): the vendor library has
        # too few tiles to fill the chip, this kernel splits K and leaves the sum to the consumer
        splits = wide_splits(n, k)
        if splits > 1:
            partials = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
            ops.gemm_wide_bf16(x, w, None, partials, 2, splits)
            return Partials(partials, splits)
    if out_dtype == torch.float32:
        out = torch.empty((m, n), dtype=torch.float32, device=x.device)
        if skinny_ok(x, w):
            ntw, _ = skinny_plan(SKINNY_ROWS, n, k)
            for m0 in range(0, m, SKINNY_ROWS):
                ops.gemm_skinny_bf16(x[m0:m0 + SKINNY_ROWS], w, out[m0:m0 + SKINNY_ROWS], None, ntw, 1)
            return out
        return ops.gemm_tiled(x, w, out)
    if library_ok:
        return torch.mm(x, w.t())
    return ops.gemm_tiled(x, w, torch.empty((m, n), dtype=x.dtype, device=x.device))


def linear_modules(dtype: torch.dtype) -> tuple[str, ...]:
    return ("gemm",)
