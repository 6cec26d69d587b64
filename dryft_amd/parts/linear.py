"""``y = x @ W.T`` for weights in checkpoint layout ``[out, in]`` (no bias).

The reference hands every projection to a vendor library (F.linear,
engine/dryft_qwen3/model.py:153, 179-180, 237, 258-261). Here:

* float32: this library's own kernels, so the 32-bit path has no reduced-precision matrix
  mode anywhere: plain multiply-adds that read every weight once for at most 16 rows, the
  matrix cores' full-precision instruction (``v_mfma_f32_16x16x4_f32``) in blocks of
  128 x 128 for more, and a plain tiled kernel for sizes those do not take;
* bfloat16, at most 16 rows (decoding at small batch): this library's weight-streaming
  matrix-core kernel, which stages whole cache lines through LDS and can leave its result
  as float32 partial sums over K for the consumer to add;
* bfloat16, at most 64 rows, the fused gate/up product with its activation: this library's kernel that brings
  its operands straight into LDS (``panel_swiglu_ok``; K a multiple of 128, else the two kernels below);
* bfloat16, 33 to 64 rows, where the consumer adds partial sums (q/k/v of decoding steps, the projections back to
  the hidden width) and K is a multiple of 64: this library's kernel that splits K and brings its operands straight
  into LDS (``small_mid_plan``);
* bfloat16, 17 to 64 rows otherwise: this library's shared-activation kernel where the consumer adds
  partial sums (the projections back to the hidden width, which give the vendor library too
  few tiles to fill the chip), where the result is wanted in float32 (the output head) and
  for sizes the vendor library does not take;
* bfloat16, 65 to 256 rows (short prompts, decoding at large batch) where the consumer adds partial sums and K is a
  multiple of 64: this library's kernel whose waves each own rows of x, operands straight into LDS (``tall_plan``);
  the fused gate/up product of as many rows goes to its other form (``tall_swiglu_ok``);
* bfloat16, otherwise (prompts, decoding at large batch): the vendor library through
  ``torch.mm``, as in the reference; float32 results of many rows and output sizes the
  library does not take are this library's block kernel (128 x 128 or 256 x 256 outputs
  per workgroup, about 0.6 of the library's speed), and what no matrix-core kernel takes goes
  to the plain kernel.
"""

from __future__ import annotations

import contextlib
import functools
import os
import tempfile

import torch

from ..csrc import ops
from .base import Partials

STREAM_ROWS = 16                # the most rows the line-staging kernel takes; up to here it beats the vendor library
WIDE_ROWS = 64                  # the most rows the shared-activation kernel takes
_SMALL_MID_BYTES = 48 << 20     # the largest matrix that goes there
SMALL_MID_ROWS = 32             # above so many rows (and up to WIDE_ROWS) split products go to the direct-to-LDS kernel
_STREAM_BLOCKS_PER_WAVE = 5     # measured on the projection shapes of 4B to 32B models inside captured graphs:
_STREAM_WORKGROUPS = 1536       # short walks over K, as long as the launch stays under about six workgroups a unit
_COMPUTE_UNITS = 256            # of the MI355X


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


def wide_plan(n: int, k: int, may_split: bool) -> tuple[int, int, int]:
    """(splits of K across workgroups, blocks per group, groups in flight) for the shared-activation kernel.

    Its workgroups are bound by their own compute unit (LDS and barriers), not by memory, so where the
    consumer adds partial sums the split of K is chosen to give every compute unit one workgroup; measured
    on the o and down shapes of 4B, 8B and 32B models at 24 and 64 rows.
    """
    tiles = (n + 63) // 64
    k_blocks = (k + 63) // 64
    splits = max(1, min(_COMPUTE_UNITS // tiles, k_blocks // 4, 16)) if may_split else 1
    return (splits, 1, 3) if splits > 1 else (1, 2, 1)


def tall_plan(m: int, n: int, k: int) -> tuple[int, int]:
    return _tall_plan(128 if m <= 128 else 256, n, k)


@functools.lru_cache(maxsize=None)
def _tall_plan(loaded: int, n: int, k: int) -> tuple[int, int]:
    """(tiles of 16 outputs a workgroup, splits of K across workgroups) for the product of 65 to 256 rows whose waves
    each own rows of x: the pair with the lowest modelled time. The model, fitted (to 4 % in the mean) to in-graph
    times on rotating cold weights of the q/k/v, o and down shapes of Qwen3-0.6B, 4B, 8B and 14B at 128 and 256 rows,
    every tile count with four to five split counts each, in us (the rows counted as the 128 or 256 the kernel loads):
    3.2 + rounds * (11.1 * MB of x a workgroup takes in + 22.5 * MB of W it takes in) + 0.23 * MB of partial sums
    + 0.074 * MB of W, rounds being how often the workgroups fill the 256 compute units. (A workgroup takes in all
    rows of x, 128 or 256 of them, over its run of K: that is what the time goes to, and why a split pays also where
    the outputs alone would fill the chip.) Its choice is within 5 % of the best measured pair for each of those
    shapes. The choice itself counts 0.42 us a MB of partial sums: the kernel that adds them up on its way in takes
    0.19 us a MB more to read them (the norm after o and down at 256 rows: 6.9 us with eight parts, 21 MB; the
    cache writer after q/k/v 12.0 us with four parts, 7.8 without). Against the kernel it replaces here (64 outputs a workgroup, every wave reading all rows of x from LDS),
    at 256 rows: Qwen3-4B's down 22.5 against 26.8, Qwen3-8B's 34.7 against 59.8, Qwen3-14B's 55.3 against 96.2."""
    groups = k // ops.TALL_GROUP
    best, best_cost = (4, 1), float("inf")
    for tiles in (4, 5, 6, 7, 8):
        blocks = -(-n // (16 * tiles))
        seen = set()
        for want in range(1, min(groups, 32) + 1):
            splits = ops.gemm_mid_splits(k, want)
            if splits in seen:
                continue
            seen.add(splits)
            per = -(-groups // splits)
            rounds = -(-(blocks * splits) // _COMPUTE_UNITS)
            cost = 3.2 + rounds * (11.1 * loaded + 22.5 * 16 * tiles) * per * 128e-6 + 0.42e-6 * splits * loaded * n * 4 + \
                0.074e-6 * n * k * 2
            if cost < best_cost:
                best, best_cost = (tiles, splits), cost
    return best


def small_mid_plan(n: int, k: int) -> int:
    """Splits of K across workgroups for the kernel that brings its operands straight into LDS, at 33 to 64 rows (64
    outputs a workgroup): as many as give every compute unit one workgroup; 1 where the product stays with the
    shared-activation kernel or the vendor library. Measured alone in a captured graph at 64 rows, us, against the
    better of those two: Qwen3-4B's q/k/v 11.7 (13.7), o 8.1 (10.2), down 14.3 (15.6); Qwen3-8B's 16.0 (17.8), 9.9 (11.6),
    23.3 (25.5); and a decoding step of 64 sequences with it 6.28 against 6.50 ms (Qwen3-4B), 7.58 against 7.71
    (Qwen3-8B). On larger matrices the same kernel is ahead alone (Qwen3-14B's q/k/v 20.5 against 25.0) and behind in
    the step (11.27 against 11.18 ms; Qwen3-32B 21.9 against 21.5), so matrices beyond 48 MiB stay where they were."""
    if n * k * 2 > _SMALL_MID_BYTES:
        return 1
    blocks = (n + 63) // 64
    return ops.gemm_mid_splits(k, max(1, min(16, _COMPUTE_UNITS // blocks)))


def few_rows_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Can the few-row kernels read these operands? (16-byte pieces of rows.)"""
    return x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0


def panel_swiglu_ok(x: torch.Tensor, w_gate_up: torch.Tensor) -> bool:
    """Does the fused gate/up product with its activation go to the kernel that brings its operands straight into
    LDS? Up to 64 rows, K a multiple of its group. In-graph times on rotating cold weights, us, against the
    line-staging kernel (up to 16 rows) or the vendor library plus the activation kernel (more): Qwen3-4B's sizes
    20.3 against 21.5 at 8 rows, 20.3 against 22.4 at 16, 21.2 against 26.8 at 24, 24.9 against 30.7 at 64;
    Qwen3-8B's 36.7 against 37.8, 36.8 against 38.0, 37.6 against 52.1, 39.9 against 52.7; Qwen3-32B's 96.9 against
    98.4, 95.0 against 103.8, 97.6 against 100.9, 107.8 against 110.4."""
    m, k = x.shape
    return m <= WIDE_ROWS and k % ops.PANEL_GROUP == 0 and few_rows_ok(x, w_gate_up) and within_direct_reach(x, w_gate_up)


_TALL_SMALL_BYTES = 128 << 20   # matrices from here on go to the kernel whose waves own rows of x already at 33 to 64 rows.
# Whole decoding steps, ms, against the shared-activation kernel or the vendor library there: Qwen3-14B (down, 178 MB) 10.99
# against 11.19 at 64 sequences, the same at 48. With every matrix beyond 48 MiB sent there Qwen3-14B gains more (10.89; 9.97
# against 10.09 at 48), Qwen3-32B a little (20.35 against 20.63; 19.01 against 19.10), and Qwen3-8B (q/k/v 50 MB, down 100 MB)
# loses (7.60 against 7.54 at 64), though each of its products alone is faster: so only the large ones.
_TALL_SWIGLU_BYTES = 256 << 20  # gate/up matrices up to here go to the kernel whose waves own rows of x at 65 to 256 rows


def tall_swiglu_ok(x: torch.Tensor, w_gate_up: torch.Tensor) -> bool:
    """Does the fused gate/up product with its activation go, at 65 to 256 rows, to the kernel whose waves each own
    rows of x? In-graph times on rotating cold weights, us, against the vendor library plus the activation kernel:
    Qwen3-4B's sizes 30.0 against 35.6 at 128 rows, 36.3 against 51.0 at 256; Qwen3-8B's 46.8 against 55.5 and 57.9
    against 66.1; Qwen3-14B's (356 MB) 102 against 100 and 129 against 111, so matrices beyond 256 MiB stay with the
    library."""
    m, k = x.shape
    return WIDE_ROWS < m <= ops.TALL_ROWS and k % ops.TALL_GROUP == 0 and few_rows_ok(x, w_gate_up) and \
        within_direct_reach(x, w_gate_up) and w_gate_up.numel() * w_gate_up.element_size() <= _TALL_SWIGLU_BYTES


def within_direct_reach(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Do both operands lie within what the kernels that bring them straight into LDS can address (32-bit byte
    offsets from the operand's start)? Larger ones go to the kernels that hold 64-bit addresses."""
    return w.numel() * w.element_size() < ops.DIRECT_REACH and \
        x.shape[0] * x.stride(0) * x.element_size() < ops.DIRECT_REACH


def linear(x: torch.Tensor, w: torch.Tensor, *, out_dtype: torch.dtype | None = None, allow_partials: bool = False,
           partial_rows: int | None = None):
    """Returns ``[rows, out]`` in ``out_dtype`` (default: the dtype of ``x``), or, where the caller allows it and a
    split of K pays, ``Partials`` (``partial_rows``: only for steps of at most so many rows)."""
    m, k = x.shape
    if partial_rows is not None and m > partial_rows:
        allow_partials = False
    n = w.shape[0]
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.float32:
        out = torch.empty((m, n), dtype=torch.float32, device=x.device)
        if k % 4 == 0 and w.data_ptr() % 16 == 0:
            if m <= STREAM_ROWS:
                return ops.gemm_rows_f32(x, w, out)
            if x.stride(0) % 4 == 0 and x.data_ptr() % 16 == 0:
                return ops.gemm_block_f32(x, w, out, shape=0)
        return ops.gemm_tiled(x, w, out)
    few_ok = few_rows_ok(x, w)
    library_ok = k % 8 == 0 and n % 8 == 0 and x.is_contiguous() and out_dtype == x.dtype
    if m <= STREAM_ROWS and few_ok:
        splits, group, depth = stream_plan(n, k, allow_partials)
        if splits > 1:
            partials = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
            ops.gemm_stream_bf16(x, w, None, partials, group, splits, depth)
            return Partials(partials, splits)
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
        ops.gemm_stream_bf16(x, w, out, None, group, 1, depth)
        return out
    if SMALL_MID_ROWS < m <= WIDE_ROWS and allow_partials and few_ok and k % ops.MID_GROUP == 0 and \
            within_direct_reach(x, w):
        splits = small_mid_plan(n, k)
        if splits > 1:
            partials = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
            ops.gemm_mid_bf16(x, w, partials, splits)
            return Partials(partials, splits)
        if n * k * 2 >= _TALL_SMALL_BYTES:
            tiles, splits = tall_plan(m, n, k)
            partials = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
            ops.gemm_tall_bf16(x, w, partials, splits, tiles)
            return Partials(partials, splits)
    if m <= WIDE_ROWS and few_ok:
        splits, group, depth = wide_plan(n, k, allow_partials)
        if splits > 1:
            partials = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
            ops.gemm_wide_bf16(x, w, None, partials, group, splits, depth)
            return Partials(partials, splits)
        if not library_ok:
            out = torch.empty((m, n), dtype=out_dtype, device=x.device)
            ops.gemm_wide_bf16(x, w, out, None, group, 1, depth)
            return out
    if m <= ops.TALL_ROWS and allow_partials and few_ok and k % ops.TALL_GROUP == 0 and within_direct_reach(x, w):
        tiles, splits = tall_plan(m, n, k)
        partials = torch.empty((splits, m, n), dtype=torch.float32, device=x.device)
        ops.gemm_tall_bf16(x, w, partials, splits, tiles)
        return Partials(partials, splits)
    if library_ok:
        return torch.mm(x, w.t())
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    if few_ok:
        return ops.gemm_block_bf16(x, w, out)
    return ops.gemm_tiled(x, w, out)


@contextlib.contextmanager
def library_tuning():
    """While open, the vendor library times its candidate kernels for every product shape it meets for the
    first time and keeps the fastest; afterwards those shapes use what was kept and nothing more is timed.

    The reference plans the same kind of choice, measured on the real GPU before the timed region
    (AGENTS.md:567). It is torch's TunableOp; what it finds is written to a file in the temporary folder
    when the process ends, never to the working directory. Not to be open while a graph is captured.
    """
    import torch.cuda.tunable as tunable
    if not tunable.is_enabled():
        tunable.set_filename(os.path.join(tempfile.gettempdir(), f"dryft_amd-products-{os.getpid()}.csv"))
        tunable.enable(True)
    tunable.tuning_enable(True)
    try:
        yield
    finally:
        tunable.tuning_enable(False)
