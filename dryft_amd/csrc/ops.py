"""Python faces of the HIP kernels: argument checks, then one ctypes call each.

Every function checks on the host that the operands have the dtypes, shapes and
strides its kernel assumes, and raises rather than launch a kernel that would read
outside its operands. Kernels run on torch's current stream, so they can be
recorded into a graph like any other work on it. There is no CPU path: tensors
must live on the GPU, and a missing library is compiled or the call fails.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p

import torch

from . import build

_P, _I, _L, _F = c_void_p, c_int, c_int64, c_float
_SIGNATURES = {
    "batch": {"dryft_prepare_batch": [_P, _P, _P, _I, _I, _P, _P, _P, _P, _P, _P, _P],
              "dryft_tile_prefix": [_P, _P, _I, _I, _P, _P]},
    "embed": {"dryft_embed_rows": [_P, _P, _P, _I, _I, _I, _I, _I, _P]},
    "norm": {"dryft_add_rmsnorm": [_P, _P, _I, _I, _L, _P, _I, _P, _P, _I, _I, _F, _I, _P],
             "dryft_add_rows": [_P, _P, _P, _L, _I, _P]},
    "activation": {"dryft_silu_mul": [_P, _P, _I, _I, _L, _I, _P]},
    "rope_kv": {"dryft_qk_norm_rope_kv": [_P, _L, _P, _P, _I, _I, _F, _P, _P, _I, _P, _P, _P, _P, _P, _P, _I, _I,
                                          _I, _I, _I, _I, _I, _P],
                "dryft_rows_to_cache_takes": [_I, _I, _I, _I],
                "dryft_rows_to_cache_parts": [_P, _I, _L, _P, _P, _I, _I, _F, _P, _P, _I, _P, _P, _P, _P, _P, _P, _I, _I,
                                              _I, _I, _I, _P]},
    "attn_rows": {"dryft_attn_rows": [_P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _F, _I, _I, _P]},
    "attn_mfma": {"dryft_attn_causal_bf16": [_P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _P, _I, _I, _I, _F, _I, _I, _P],
                  "dryft_attn_causal_takes_projection": [_I, _I],
                  "dryft_attn_causal_projected_bf16": [_P, _L, _P, _I, _I, _F, _P, _P, _P, _P, _P, _I, _P, _P, _P, _P, _I,
                                                       _I, _P, _I, _I, _I, _F, _I, _I, _P],
                  "dryft_attn_split_bf16": [_P, _P, _P, _P, _I, _P, _P, _P, _I, _P, _P, _I, _P, _I, _I, _I, _F, _I,
                                            _P],
                  "dryft_attn_decode_fused_bf16": [_P, _L, _I, _L, _P, _P, _I, _I, _F, _P, _P, _I, _I, _P, _P, _P, _I, _P, _P,
                                                   _P, _I, _P, _P, _I, _P, _I, _I, _I, _F, _I, _P]},
    "gemm": {"dryft_gemm_tiled": [_P, _L, _P, _P, _I, _I, _I, _I, _I, _P],
             "dryft_gemm_stream_bf16": [_P, _L, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P],
             "dryft_gemm_stream_swiglu_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _I, _P],
             "dryft_gemm_wide_bf16": [_P, _L, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P],
             "dryft_gemm_panel_swiglu_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _P],
             "dryft_gemm_panel_waves": [_I],
             "dryft_gemm_tall_swiglu_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _P],
             "dryft_gemm_tall_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _I, _P],
             "dryft_gemm_tall_tiles": [_I],
             "dryft_gemm_mid_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _P],
             "dryft_gemm_block_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _I, _I, _P],
             "dryft_gemm_block_f32": [_P, _L, _P, _P, _I, _I, _I, _I, _P],
             "dryft_gemm_rows_f32": [_P, _L, _P, _P, _I, _I, _I, _P],
             "dryft_gemm_wide_swiglu_bf16": [_P, _L, _P, _P, _I, _I, _I, _I, _I, _P],
             "dryft_sum_partials": [_P, _P, _L, _I, _I, _P]},
    "sampling": {"dryft_argmax_rows": [_P, _I, _I, _L, _P, _I, _P, _P, _P],
                 "dryft_sample_rows": [_P, _I, _I, _L, _F, _P, _P, _I, _P, _P, _P]},
}
_functions: dict[str, object] = {}


class KernelError(RuntimeError):
    pass


def _fn(module: str, name: str):
    f = _functions.get(name)
    if f is None:
        lib = build.load(module)
        f = getattr(lib, name)
        f.argtypes = _SIGNATURES[module][name]
        f.restype = c_int
        _functions[name] = f
    return f


def preload(modules) -> None:
    build.ensure(list(modules))


# the current stream's handle without building a stream object per launch (hundreds of launches a step)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _check(rc: int, what: str) -> None:
    if rc == -1:
        raise KernelError(f"{what}: the kernel refuses these sizes")
    if rc != 0:
        raise KernelError(f"{what}: launch failed with HIP error {rc}")


def _gpu(t: torch.Tensor, name: str, dtype=None) -> None:
    if not (isinstance(t, torch.Tensor) and t.is_cuda):
        raise KernelError(f"{name}: must be a GPU tensor (there is no CPU path)")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, got {t.dtype}")


def _float_flag(t: torch.Tensor, name: str) -> int:
    if t.dtype not in (torch.float32, torch.bfloat16):
        raise KernelError(f"{name}: expected float32 or bfloat16, got {t.dtype}")
    return 1 if t.dtype == torch.float32 else 0


def _ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


# ------------------------------------------------------------------------------------------- batch
def prepare_batch(seq_slot, q_len, lengths, n_seqs: int, n_rows: int, cu_rows, kv_len, seq_start,
                  row_seq, row_slot, row_pos) -> None:
    for name, t, n in (("seq_slot", seq_slot, n_seqs), ("q_len", q_len, n_seqs), ("cu_rows", cu_rows, n_seqs + 1),
                       ("kv_len", kv_len, n_seqs), ("seq_start", seq_start, n_seqs),
                       ("row_seq", row_seq, n_rows), ("row_slot", row_slot, n_rows), ("row_pos", row_pos, n_rows),
                       ("lengths", lengths, 1)):
        _gpu(t, name, torch.int32)
        if not (t.is_contiguous() and t.numel() >= n):
            raise KernelError(f"{name}: needs {n} contiguous entries, has {t.numel()}")
    _check(_fn("batch", "dryft_prepare_batch")(
        _ptr(seq_slot), _ptr(q_len), _ptr(lengths), n_seqs, n_rows, _ptr(cu_rows), _ptr(kv_len),
        _ptr(seq_start), _ptr(row_seq), _ptr(row_slot), _ptr(row_pos), _stream()), "prepare_batch")


def tile_prefix(seq_slot, q_len, n_seqs: int, tile_rows: int, tile_cu) -> None:
    """``tile_cu[s]``: how many tiles of ``tile_rows`` rows the sequences before ``s`` fill with their rows of this
    step (a sequence that sits out, slot -1, fills none); ``tile_cu[n_seqs]``: the step's tiles."""
    for name, t, n in (("seq_slot", seq_slot, n_seqs), ("q_len", q_len, n_seqs), ("tile_cu", tile_cu, n_seqs + 1)):
        _gpu(t, name, torch.int32)
        if not (t.is_contiguous() and t.numel() >= n):
            raise KernelError(f"{name}: needs {n} contiguous entries, has {t.numel()}")
    if tile_rows <= 0:
        raise KernelError(f"tile_prefix: tiles of {tile_rows} rows")
    _check(_fn("batch", "dryft_tile_prefix")(_ptr(seq_slot), _ptr(q_len), n_seqs, int(tile_rows), _ptr(tile_cu),
                                             _stream()), "tile_prefix")


# ------------------------------------------------------------------------------------------- embed
def embed_rows(tokens: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out[r] = table[tokens[r]]`` for a table ``[vocab, hidden]``; for several tables ``[tables, vocab, hidden]`` the same
    rows of each, ``out[t, r] = table[t, tokens[r]]``."""
    _gpu(tokens, "tokens", torch.int32)
    _gpu(table, "table")
    _gpu(out, "out", table.dtype)
    n = tokens.numel()
    tables = table.shape[0] if table.dim() == 3 else 1
    vocab, hidden = table.shape[-2:]
    if not (table.dim() in (2, 3) and table.is_contiguous() and out.is_contiguous() and tokens.is_contiguous()):
        raise KernelError("embed_rows: contiguous operands, the table [vocab, hidden] or [tables, vocab, hidden]")
    want = (n, hidden) if table.dim() == 2 else (tables, n, hidden)
    if not (out.shape == want):
        raise KernelError(f"embed_rows: out is {tuple(out.shape)}, expected {want}")
    _check(_fn("embed", "dryft_embed_rows")(_ptr(tokens), _ptr(table), _ptr(out), n, hidden, vocab, tables,
                                            _float_flag(table, "table"), _stream()), "embed_rows")
    return out


# -------------------------------------------------------------------------------------------- norm
def add_rmsnorm(res: torch.Tensor, delta, weight: torch.Tensor, eps: float, res_out, y: torch.Tensor,
                n_partials: int = 1) -> None:
    """``res_out = res + delta`` (when ``delta`` is given) and ``y = rmsnorm(res_out) * weight``.

    ``delta`` is ``[rows, width]`` in the dtype of ``res``, or ``[n_partials, rows, width]`` float32
    partial sums. Without ``delta`` nothing is added and ``res_out`` is ignored.
    """
    _gpu(res, "res")
    rows, width = res.shape
    is_f32 = _float_flag(res, "res")
    _gpu(weight, "weight")
    w_f32 = _float_flag(weight, "weight")
    if not (weight.shape == (width,) and weight.is_contiguous()):
        raise KernelError(f"add_rmsnorm: weight must be [{width}]")
    _gpu(y, "y", res.dtype)
    if not (res.is_contiguous() and y.is_contiguous() and y.shape == res.shape):
        raise KernelError("add_rmsnorm: res and y contiguous, same shape")
    kind, stride = 0, 0
    if delta is not None:
        _gpu(delta, "delta")
        _gpu(res_out, "res_out", res.dtype)
        if not (res_out.shape == res.shape and res_out.is_contiguous()):
            raise KernelError("add_rmsnorm: res_out like res")
        if not (delta.is_contiguous()):
            raise KernelError("add_rmsnorm: delta contiguous")
        if delta.dim() == 3:
            if not (delta.dtype == torch.float32 and delta.shape[1:] == res.shape and delta.shape[0] >= n_partials):
                raise KernelError("add_rmsnorm: partial sums must be float32 [n, rows, width]")
            kind, stride = 2, rows * width
        else:
            if not (delta.dtype == res.dtype and delta.shape == res.shape):
                raise KernelError("add_rmsnorm: delta like res")
            kind, n_partials, stride = 1, 1, rows * width
    else:
        n_partials = 0
    _check(_fn("norm", "dryft_add_rmsnorm")(_ptr(res), _ptr(delta), kind, n_partials, stride, _ptr(weight), w_f32,
                                            _ptr(res_out), _ptr(y), rows, width, float(eps), is_f32, _stream()),
           "add_rmsnorm")


def add_rows(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _gpu(a, "a")
    _gpu(b, "b", a.dtype)
    _gpu(out, "out", a.dtype)
    if not (a.shape == b.shape == out.shape and a.is_contiguous() and b.is_contiguous() and out.is_contiguous()):
        raise KernelError("add_rows: contiguous operands of one shape")
    _check(_fn("norm", "dryft_add_rows")(_ptr(a), _ptr(b), _ptr(out), a.numel(), _float_flag(a, "a"), _stream()),
           "add_rows")
    return out


# -------------------------------------------------------------------------------------- activation
def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _gpu(gate_up, "gate_up")
    _gpu(out, "out", gate_up.dtype)
    rows, two_i = gate_up.shape
    if not (two_i % 2 == 0 and out.shape == (rows, two_i // 2)):
        raise KernelError("silu_mul: out must be [rows, width / 2]")
    if not (gate_up.stride(1) == 1 and out.is_contiguous()):
        raise KernelError("silu_mul: unit stride along the width")
    _check(_fn("activation", "dryft_silu_mul")(_ptr(gate_up), _ptr(out), rows, two_i // 2, gate_up.stride(0),
                                               _float_flag(gate_up, "gate_up"), _stream()), "silu_mul")
    return out


# ----------------------------------------------------------------------------------------- rope_kv
def qk_norm_rope_kv(qkv: torch.Tensor, q_weight, k_weight, eps: float, cos, sin, rot: int, row_slot, row_pos,
                    q_out, k_pages, v_pages, page_table, write_kv: bool, n_heads: int, n_kv: int,
                    head_dim: int) -> None:
    """Per-head norm and rotation of a step's query and key heads, and the append of keys and values to the cache.
    ``q_out`` None: only keys and values are handled (the attention kernel takes the queries from ``qkv`` itself)."""
    _gpu(qkv, "qkv")
    is_f32 = _float_flag(qkv, "qkv")
    rows = qkv.shape[0]
    need_cols = (n_heads + (2 * n_kv if write_kv else 0)) * head_dim
    if not (qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= need_cols):
        raise KernelError(f"qk_norm_rope_kv: qkv needs {need_cols} columns, has {tuple(qkv.shape)}")
    has_norm = q_weight is not None
    w_f32 = 0
    if has_norm:
        for name, w in (("q_weight", q_weight), ("k_weight", k_weight)):
            _gpu(w, name)
            if not (w.shape == (head_dim,) and w.is_contiguous()):
                raise KernelError(f"{name}: must be [{head_dim}]")
        if not (q_weight.dtype == k_weight.dtype):
            raise KernelError("q_weight and k_weight must share a dtype")
        w_f32 = _float_flag(q_weight, "q_weight")
    if rot:
        if not (rot % 2 == 0 and rot <= head_dim):
            raise KernelError(f"rotary width {rot} must be even and at most {head_dim}")
        for name, t in (("cos", cos), ("sin", sin)):
            _gpu(t, name, qkv.dtype)
            if not (t.dim() == 2 and t.shape[1] == rot // 2 and t.is_contiguous()):
                raise KernelError(f"{name}: must be [positions, {rot // 2}]")
    for name, t in (("row_slot", row_slot), ("row_pos", row_pos)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= rows and t.is_contiguous()):
            raise KernelError(f"{name}: needs {rows} entries")
    if q_out is not None:
        _gpu(q_out, "q_out", qkv.dtype)
        if not (q_out.is_contiguous() and q_out.numel() == rows * n_heads * head_dim):
            raise KernelError("q_out: must be [rows, heads, head_dim]")
    else:
        if not (write_kv):
            raise KernelError("qk_norm_rope_kv: nothing to do without q_out and without a cache to write")
    max_pages = 0
    if write_kv:
        _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, qkv.dtype)
        max_pages = page_table.shape[1]
    _check(_fn("rope_kv", "dryft_qk_norm_rope_kv")(
        _ptr(qkv), qkv.stride(0), _ptr(q_weight), _ptr(k_weight), w_f32, int(has_norm), float(eps), _ptr(cos),
        _ptr(sin), int(rot), _ptr(row_slot), _ptr(row_pos), _ptr(q_out), _ptr(k_pages), _ptr(v_pages),
        _ptr(page_table), max_pages, int(write_kv), rows, n_heads, n_kv, head_dim, is_f32, _stream()),
        "qk_norm_rope_kv")


def rows_to_cache_takes(n_rows: int, head_dim: int, rot: int, write_kv: bool) -> bool:
    """Can ``rows_to_cache_from_partials`` take a step of so many rows, heads of this size rotated over ``rot``
    features?"""
    return bool(_fn("rope_kv", "dryft_rows_to_cache_takes")(int(n_rows), int(head_dim), int(rot), int(write_kv)))


def rows_to_cache_from_partials(parts: torch.Tensor, q_weight, k_weight, eps: float, cos, sin, rot: int, row_slot,
                                row_pos, q_out, k_pages, v_pages, page_table, n_heads: int, n_kv: int,
                                head_dim: int) -> None:
    """``qk_norm_rope_kv`` for a bfloat16 step whose projection was left as float partial sums ``parts`` [count, rows,
    columns]: each value is the sum of its parts rounded to bfloat16, then normed, rotated and written as there (queries
    to ``q_out``, or nowhere if it is None; keys and values to the cache)."""
    _gpu(parts, "parts", torch.float32)
    if not (parts.dim() == 3 and parts.is_contiguous()):
        raise KernelError("rows_to_cache_from_partials: parts must be [count, rows, columns], contiguous")
    count, rows, cols = parts.shape
    if not (cols >= (n_heads + 2 * n_kv) * head_dim and cols % 8 == 0):
        raise KernelError(f"rows_to_cache_from_partials: parts need {(n_heads + 2 * n_kv) * head_dim} columns, a multiple "
                          f"of 8; have {cols}")
    if not rows_to_cache_takes(rows, head_dim, rot, True):
        raise KernelError(f"rows_to_cache_from_partials: takes a full rotation and head sizes 32, 64, 128, 256; got head "
                          f"size {head_dim}, rotation over {rot}")
    has_norm = q_weight is not None
    w_f32 = 0
    if has_norm:
        for name, w in (("q_weight", q_weight), ("k_weight", k_weight)):
            _gpu(w, name)
            if not (w.shape == (head_dim,) and w.is_contiguous()):
                raise KernelError(f"{name}: must be [{head_dim}]")
        if not (q_weight.dtype == k_weight.dtype):
            raise KernelError("q_weight and k_weight must share a dtype")
        w_f32 = _float_flag(q_weight, "q_weight")
    for name, t in (("cos", cos), ("sin", sin)):
        _gpu(t, name, torch.bfloat16)
        if not (t.dim() == 2 and t.shape[1] == rot // 2 and t.is_contiguous()):
            raise KernelError(f"{name}: must be [positions, {rot // 2}]")
    for name, t in (("row_slot", row_slot), ("row_pos", row_pos)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= rows and t.is_contiguous()):
            raise KernelError(f"{name}: needs {rows} entries")
    if q_out is not None:
        _gpu(q_out, "q_out", torch.bfloat16)
        if not (q_out.is_contiguous() and q_out.numel() == rows * n_heads * head_dim):
            raise KernelError("q_out: must be [rows, heads, head_dim]")
    _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, torch.bfloat16)
    _check(_fn("rope_kv", "dryft_rows_to_cache_parts")(
        _ptr(parts), int(count), cols, _ptr(q_weight), _ptr(k_weight), w_f32, int(has_norm), float(eps), _ptr(cos),
        _ptr(sin), int(rot), _ptr(row_slot), _ptr(row_pos), _ptr(q_out), _ptr(k_pages), _ptr(v_pages),
        _ptr(page_table), page_table.shape[1], rows, n_heads, n_kv, head_dim, _stream()), "rows_to_cache_parts")


def _check_pages(k_pages, v_pages, page_table, n_kv: int, head_dim: int, dtype) -> None:
    for name, t in (("k_pages", k_pages), ("v_pages", v_pages)):
        _gpu(t, name, dtype)
        if not (t.dim() == 4 and t.shape[1] == n_kv and t.shape[2] * t.shape[3] == 64 * head_dim and t.is_contiguous()):
            raise KernelError(f"{name}: must be contiguous [pages, {n_kv}, 64, {head_dim}], got {tuple(t.shape)}")
    _gpu(page_table, "page_table", torch.int32)
    if not (page_table.dim() == 2 and page_table.is_contiguous()):
        raise KernelError("page_table: must be contiguous [slots, pages]")


# --------------------------------------------------------------------------------------- attention
def attn_rows(q, k_pages, v_pages, page_table, row_slot, row_pos, out, n_heads: int, n_kv: int, head_dim: int,
              scale: float, window: int) -> None:
    _gpu(q, "q")
    is_f32 = _float_flag(q, "q")
    rows = q.numel() // (n_heads * head_dim)
    if not (q.is_contiguous() and q.numel() == rows * n_heads * head_dim):
        raise KernelError("attn_rows: q must be [rows, heads, head_dim]")
    _gpu(out, "out", q.dtype)
    if not (out.is_contiguous() and out.numel() == q.numel()):
        raise KernelError("attn_rows: out like q")
    _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, q.dtype)
    for name, t in (("row_slot", row_slot), ("row_pos", row_pos)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= rows):
            raise KernelError(f"{name}: needs {rows} entries")
    if not (n_heads <= 65535):
        raise KernelError("attn_rows: too many heads")
    _check(_fn("attn_rows", "dryft_attn_rows")(
        _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(page_table), page_table.shape[1], _ptr(row_slot), _ptr(row_pos),
        _ptr(out), rows, n_heads, n_kv, head_dim, float(scale), int(window), is_f32, _stream()), "attn_rows")


ATTN_ROW_TILE = 64      # rows of a sequence that one workgroup of the prompt-attention kernels takes (``tile_cu``)


def attn_causal_bf16(q, k_pages, v_pages, page_table, seq_slot, cu_rows, tile_cu, seq_start, n_seqs: int,
                     max_tiles: int, out, n_heads: int, n_kv: int, head_dim: int, scale: float, window: int,
                     mode: int = 0) -> None:
    """Causal attention of steps with many rows per sequence. ``mode``: 0 lets the library choose how much a wave
    takes; 1 = one head and 16 rows, 2 = two heads of a kv group, 3 = one head and 32 rows. At head size 128, 1 and
    3 bring the pages straight into LDS; 5 and 7 are 1 and 3 with the pages staged through registers, as at every
    other head size."""
    _gpu(q, "q", torch.bfloat16)
    _gpu(out, "out", torch.bfloat16)
    if not (q.is_contiguous() and out.is_contiguous() and out.numel() == q.numel()):
        raise KernelError("attn_causal: q and out contiguous")
    _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, torch.bfloat16)
    for name, t, n in (("seq_slot", seq_slot, n_seqs), ("cu_rows", cu_rows, n_seqs + 1),
                       ("tile_cu", tile_cu, n_seqs + 1), ("seq_start", seq_start, n_seqs)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= n):
            raise KernelError(f"{name}: needs {n} entries")
    if not (n_heads <= 65535):
        raise KernelError("attn_causal: too many heads")
    _check(_fn("attn_mfma", "dryft_attn_causal_bf16")(
        _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(page_table), page_table.shape[1], _ptr(seq_slot), _ptr(cu_rows),
        _ptr(tile_cu), _ptr(seq_start), n_seqs, max_tiles, _ptr(out), n_heads, n_kv, head_dim, float(scale),
        int(window), int(mode), _stream()), "attn_causal_bf16")


def attn_causal_takes_projection(head_dim: int, rot: int) -> bool:
    """Can ``attn_causal_projected_bf16`` run heads of this size, rotated over ``rot`` features?"""
    return bool(_fn("attn_mfma", "dryft_attn_causal_takes_projection")(int(head_dim), int(rot)))


def attn_causal_projected_bf16(qkv, q_weight, eps: float, cos, sin, k_pages, v_pages, page_table, seq_slot, cu_rows,
                               tile_cu, seq_start, n_seqs: int, max_tiles: int, out, n_heads: int, n_kv: int,
                               head_dim: int, scale: float, window: int, mode: int = 0) -> None:
    """``attn_causal_bf16`` with the queries taken from the fused projection ``qkv`` [rows, >= n_heads * head_dim]
    (query heads first): their per-head norm (``q_weight`` or None) and rotation happen inside the kernel, so they
    are neither written out nor read back. Keys and values must be in the cache already."""
    _gpu(qkv, "qkv", torch.bfloat16)
    _gpu(out, "out", torch.bfloat16)
    rows = qkv.shape[0]
    if not (qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= n_heads * head_dim and qkv.stride(0) % 8 == 0):
        raise KernelError(
            "attn_causal_projected: qkv must be [rows, >= heads * head_dim] with rows 16 bytes apart or a multiple"
        )
    if not (out.is_contiguous() and out.numel() == rows * n_heads * head_dim):
        raise KernelError("attn_causal_projected: out [rows, heads, head_dim]")
    if not (attn_causal_takes_projection(head_dim, 2 * cos.shape[1] if cos is not None else 0)):
        raise KernelError("attn_causal_projected: the kernel refuses these sizes")
    w_f32 = 0
    if q_weight is not None:
        _gpu(q_weight, "q_weight")
        if not (q_weight.shape == (head_dim,) and q_weight.is_contiguous()):
            raise KernelError(f"q_weight: must be [{head_dim}]")
        w_f32 = _float_flag(q_weight, "q_weight")
    for name, t in (("cos", cos), ("sin", sin)):
        _gpu(t, name, torch.bfloat16)
        if not (t.dim() == 2 and t.shape[1] == head_dim // 2 and t.is_contiguous()):
            raise KernelError(f"{name}: must be [positions, {head_dim // 2}]")
    _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, torch.bfloat16)
    for name, t, n in (("seq_slot", seq_slot, n_seqs), ("cu_rows", cu_rows, n_seqs + 1),
                       ("tile_cu", tile_cu, n_seqs + 1), ("seq_start", seq_start, n_seqs)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= n):
            raise KernelError(f"{name}: needs {n} entries")
    if not (n_heads <= 65535):
        raise KernelError("attn_causal: too many heads")
    _check(_fn("attn_mfma", "dryft_attn_causal_projected_bf16")(
        _ptr(qkv), qkv.stride(0), _ptr(q_weight), w_f32, int(q_weight is not None), float(eps), _ptr(cos), _ptr(sin),
        _ptr(k_pages), _ptr(v_pages), _ptr(page_table), page_table.shape[1], _ptr(seq_slot), _ptr(cu_rows), _ptr(tile_cu),
        _ptr(seq_start), n_seqs, max_tiles, _ptr(out), n_heads, n_kv, head_dim, float(scale), int(window), int(mode),
        _stream()), "attn_causal_projected_bf16")


def attn_split_bf16(q, k_pages, v_pages, page_table, seq_slot, cu_rows, kv_len, n_seqs: int, part_o, part_ml,
                    n_splits: int, out, n_heads: int, n_kv: int, head_dim: int, scale: float, window: int) -> None:
    _gpu(q, "q", torch.bfloat16)
    _gpu(out, "out", torch.bfloat16)
    if not (q.is_contiguous() and out.is_contiguous() and out.numel() == q.numel()):
        raise KernelError("attn_split: q and out contiguous")
    _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, torch.bfloat16)
    for name, t, n in (("seq_slot", seq_slot, n_seqs), ("cu_rows", cu_rows, n_seqs + 1), ("kv_len", kv_len, n_seqs)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= n):
            raise KernelError(f"{name}: needs {n} entries")
    _gpu(part_o, "part_o", torch.float32)
    _gpu(part_ml, "part_ml", torch.float32)
    entries = n_seqs * n_heads * n_splits
    if part_o.numel() < entries * head_dim or part_ml.numel() < entries * 2:
        raise KernelError("attn_split: partial buffers too small")
    if not (n_splits <= 65535 and n_kv * ((n_heads // n_kv + 15) // 16) <= 65535):
        raise KernelError("attn_split: grid too large")
    _check(_fn("attn_mfma", "dryft_attn_split_bf16")(
        _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(page_table), page_table.shape[1], _ptr(seq_slot), _ptr(cu_rows),
        _ptr(kv_len), n_seqs, _ptr(part_o), _ptr(part_ml), n_splits, _ptr(out), n_heads, n_kv, head_dim, float(scale),
        int(window), _stream()), "attn_split_bf16")


def attn_decode_fused_bf16(qkv, q_weight, k_weight, eps: float, cos, sin, rot: int, write_kv: bool, k_pages, v_pages,
                           page_table, seq_slot, cu_rows, kv_len, n_seqs: int, part_o, part_ml, n_splits: int, out,
                           n_heads: int, n_kv: int, head_dim: int, scale: float, window: int, qkv_parts: int = 0) -> None:
    """One row per sequence: q/k norm, rotation, append to the cache and attention in one kernel (plus the combine).

    ``qkv`` is the fused projection's output ``[n_seqs rows, (heads + 2 kv heads) * head_dim]``; row ``i`` belongs to
    sequence ``i`` (``cu_rows[i] == i``). It may also be that product left as float32 partial sums over K,
    ``[parts, rows, width]`` (``qkv_parts`` of them): the kernel adds them up in order and rounds the sum to bfloat16
    as the product would have.
    """
    _gpu(out, "out", torch.bfloat16)
    need_cols = (n_heads + 2 * n_kv) * head_dim
    if qkv_parts:
        _gpu(qkv, "qkv", torch.float32)
        if not (qkv.dim() == 3 and qkv.is_contiguous() and qkv.shape[0] >= qkv_parts and qkv.shape[1] >= n_seqs
                and qkv.shape[2] >= need_cols):
            raise KernelError(f"attn_decode_fused: partial sums must be [>= {qkv_parts}, rows >= {n_seqs}, >= {need_cols}]")
        row_stride, part_stride = qkv.stride(1), qkv.stride(0)
    else:
        _gpu(qkv, "qkv", torch.bfloat16)
        if not (qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= need_cols and qkv.shape[0] >= n_seqs):
            raise KernelError(f"attn_decode_fused: qkv must be [rows >= {n_seqs}, >= {need_cols}]")
        row_stride, part_stride = qkv.stride(0), 0
    if not (out.is_contiguous() and out.numel() >= n_seqs * n_heads * head_dim):
        raise KernelError("attn_decode_fused: out too small")
    if not (n_heads // n_kv <= 16):
        raise KernelError("attn_decode_fused: at most 16 query heads per kv head")
    _check_pages(k_pages, v_pages, page_table, n_kv, head_dim, torch.bfloat16)
    has_norm = q_weight is not None
    w_f32 = 0
    if has_norm:
        for name, w in (("q_weight", q_weight), ("k_weight", k_weight)):
            _gpu(w, name)
            if not (w.shape == (head_dim,) and w.is_contiguous()):
                raise KernelError(f"{name}: must be [{head_dim}]")
        if not (q_weight.dtype == k_weight.dtype):
            raise KernelError("q_weight and k_weight must share a dtype")
        w_f32 = _float_flag(q_weight, "q_weight")
    if rot:
        if not (rot % 2 == 0 and rot <= head_dim):
            raise KernelError(f"rotary width {rot} must be even and at most {head_dim}")
        for name, t in (("cos", cos), ("sin", sin)):
            _gpu(t, name, torch.bfloat16)
            if not (t.dim() == 2 and t.shape[1] == rot // 2 and t.is_contiguous()):
                raise KernelError(f"{name}: must be [positions, {rot // 2}]")
    for name, t, n in (("seq_slot", seq_slot, n_seqs), ("cu_rows", cu_rows, n_seqs + 1), ("kv_len", kv_len, n_seqs)):
        _gpu(t, name, torch.int32)
        if not (t.numel() >= n):
            raise KernelError(f"{name}: needs {n} entries")
    _gpu(part_o, "part_o", torch.float32)
    _gpu(part_ml, "part_ml", torch.float32)
    entries = n_seqs * n_heads * n_splits
    if part_o.numel() < entries * head_dim or part_ml.numel() < entries * 2:
        raise KernelError("attn_decode_fused: partial buffers too small")
    _check(_fn("attn_mfma", "dryft_attn_decode_fused_bf16")(
        _ptr(qkv), row_stride, int(qkv_parts), part_stride, _ptr(q_weight), _ptr(k_weight), w_f32, int(has_norm),
        float(eps), _ptr(cos), _ptr(sin),
        int(rot), int(write_kv), _ptr(k_pages), _ptr(v_pages), _ptr(page_table), page_table.shape[1], _ptr(seq_slot),
        _ptr(cu_rows), _ptr(kv_len), n_seqs, _ptr(part_o), _ptr(part_ml), n_splits, _ptr(out), n_heads, n_kv, head_dim,
        float(scale), int(window), _stream()), "attn_decode_fused_bf16")


# -------------------------------------------------------------------------------------------- gemm
def gemm_tiled(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out = x @ w.T`` with float accumulation by plain multiply-adds (any sizes)."""
    _gpu(x, "x")
    _gpu(w, "w", x.dtype)
    is_f32 = _float_flag(x, "x")
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_tiled: x [M,K] row-major, w [N,K] contiguous")
    _gpu(out, "out")
    out_f32 = 1 if out.dtype == torch.float32 else 0
    if not (out.shape == (m, n) and out.is_contiguous() and (out.dtype == x.dtype or out_f32)):
        raise KernelError(f"gemm_tiled: out must be [{m},{n}] in the input dtype or float32")
    for m0 in range(0, m, 65535 * 64):                      # the row tiles ride on grid.y
        m1 = min(m, m0 + 65535 * 64)
        _check(_fn("gemm", "dryft_gemm_tiled")(_ptr(x[m0:m1]), x.stride(0), _ptr(w), _ptr(out[m0:m1]), m1 - m0, n, k,
                                               is_f32, out_f32, _stream()), "gemm_tiled")
    return out


def gemm_stream_bf16(x, w, out, partials=None, group_blocks: int = 2, splits: int = 1, depth: int = 2) -> None:
    """``x [M<=16, K] @ w[N, K].T`` by the kernel that reads whole cache lines and stages operands in LDS.

    ``group_blocks`` (1 or 2) is how many 64-value blocks of K a wave loads at a time and ``depth``
    (1 or 2) how many such groups it keeps in flight; with ``splits > 1`` the result is left as
    ``partials[splits, M, N]``.
    """
    _gpu(x, "x", torch.bfloat16)
    _gpu(w, "w", torch.bfloat16)
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_stream: x [M,K] row-major, w [N,K] contiguous")
    if not (m <= 16 and k % 8 == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_stream: needs M <= 16 and K % 8 == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        raise KernelError("gemm_stream: operands must be 16-byte aligned")
    if not (group_blocks in (1, 2) and depth in (1, 2) and 1 <= splits <= 64):
        raise KernelError("gemm_stream: group_blocks and depth in 1, 2 and splits in 1..64")
    out_f32 = 0
    if splits > 1:
        _gpu(partials, "partials", torch.float32)
        if not (partials.numel() >= splits * m * n and partials.is_contiguous()):
            raise KernelError("gemm_stream: partials too small")
    else:
        _gpu(out, "out")
        out_f32 = 1 if out.dtype == torch.float32 else 0
        if not (out.shape == (m, n) and out.is_contiguous() and out.dtype in (torch.float32, torch.bfloat16)):
            raise KernelError(f"gemm_stream: out must be contiguous [{m},{n}]")
    _check(_fn("gemm", "dryft_gemm_stream_bf16")(_ptr(x), x.stride(0), _ptr(w), _ptr(out), _ptr(partials), m, n, k,
                                                 int(group_blocks), int(depth), int(splits), out_f32, _stream()), "gemm_stream_bf16")


def gemm_stream_swiglu_bf16(x, w_gate_up, out, group_blocks: int = 2, depth: int = 1) -> torch.Tensor:
    """``silu(x @ Wg.T) * (x @ Wu.T)`` for ``w_gate_up = [Wg; Wu]``, at most 16 rows, in one kernel."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(w_gate_up, "w_gate_up", torch.bfloat16)
    _gpu(out, "out", torch.bfloat16)
    m, k = x.shape
    two_n = w_gate_up.shape[0]
    if not (two_n % 2 == 0 and w_gate_up.shape == (two_n, k) and w_gate_up.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_stream_swiglu: x [M,K] row-major, w [2N,K] contiguous")
    if not (m <= 16 and k % 8 == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_stream_swiglu: needs M <= 16 and K % 8 == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w_gate_up.data_ptr() % 16 == 0):
        raise KernelError("gemm_stream_swiglu: operands must be 16-byte aligned")
    if not (out.shape == (m, two_n // 2) and out.is_contiguous()):
        raise KernelError(f"gemm_stream_swiglu: out must be [{m},{two_n // 2}]")
    if not (group_blocks in (1, 2) and depth in (1, 2)):
        raise KernelError("gemm_stream_swiglu: group_blocks and depth in 1, 2")
    _check(_fn("gemm", "dryft_gemm_stream_swiglu_bf16")(_ptr(x), x.stride(0), _ptr(w_gate_up), _ptr(out), m, two_n // 2, k,
                                                        int(group_blocks), int(depth), _stream()), "gemm_stream_swiglu_bf16")
    return out


def gemm_wide_bf16(x, w, out, partials=None, group_blocks: int = 2, splits: int = 1, depth: int = 2) -> None:
    """``x [M<=64, K] @ w[N, K].T`` by the kernel whose workgroups share the rows of ``x`` in LDS.

    ``group_blocks`` (1 or 2) is how many 64-value blocks of K are staged at a time and ``depth`` (1 to 3)
    how many such groups a wave has in flight; with ``splits > 1`` the result is left as
    ``partials[splits, M, N]``.
    """
    _gpu(x, "x", torch.bfloat16)
    _gpu(w, "w", torch.bfloat16)
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_wide: x [M,K] row-major, w [N,K] contiguous")
    if not (m <= 64 and k % 8 == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_wide: needs M <= 64 and K % 8 == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        raise KernelError("gemm_wide: operands must be 16-byte aligned")
    if not (group_blocks in (1, 2) and depth in (1, 2, 3) and 1 <= splits <= 64):
        raise KernelError("gemm_wide: group_blocks in 1, 2, depth in 1..3 and splits in 1..64")
    out_f32 = 0
    if splits > 1:
        _gpu(partials, "partials", torch.float32)
        if not (partials.numel() >= splits * m * n and partials.is_contiguous()):
            raise KernelError("gemm_wide: partials too small")
    else:
        _gpu(out, "out")
        out_f32 = 1 if out.dtype == torch.float32 else 0
        if not (out.shape == (m, n) and out.is_contiguous() and out.dtype in (torch.float32, torch.bfloat16)):
            raise KernelError(f"gemm_wide: out must be contiguous [{m},{n}]")
    _check(_fn("gemm", "dryft_gemm_wide_bf16")(_ptr(x), x.stride(0), _ptr(w), _ptr(out), _ptr(partials), m, n, k,
                                               int(group_blocks), int(depth), int(splits), out_f32, _stream()), "gemm_wide_bf16")


PANEL_GROUP = 128     # values of K the panel kernel moves at a time; K must be a multiple of it
DIRECT_REACH = 1 << 32    # bytes: the kernels that bring operands straight into LDS address them by 32-bit offsets


def gemm_panel_waves(n_outputs: int) -> int:
    """Waves per workgroup (8 outputs each) that the panel kernel chooses for this many outputs."""
    return int(_fn("gemm", "dryft_gemm_panel_waves")(int(n_outputs)))


def gemm_panel_swiglu_bf16(x, w_gate_up, out, waves: int = 0) -> torch.Tensor:
    """``silu(x @ Wg.T) * (x @ Wu.T)`` for ``w_gate_up = [Wg; Wu]``, at most 64 rows, by the kernel whose operands go
    from memory straight into LDS. K must be a multiple of 128. ``waves`` (4 to 8, 8 outputs each) per workgroup;
    0 lets the library choose."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(w_gate_up, "w_gate_up", torch.bfloat16)
    _gpu(out, "out", torch.bfloat16)
    m, k = x.shape
    two_n = w_gate_up.shape[0]
    if not (two_n % 2 == 0 and w_gate_up.shape == (two_n, k) and w_gate_up.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_panel_swiglu: x [M,K] row-major, w [2N,K] contiguous")
    if not (m <= 64 and k % PANEL_GROUP == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_panel_swiglu: needs M <= 64 and K % {PANEL_GROUP} == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w_gate_up.data_ptr() % 16 == 0):
        raise KernelError("gemm_panel_swiglu: operands must be 16-byte aligned")
    if not (out.shape == (m, two_n // 2) and out.is_contiguous()):
        raise KernelError(f"gemm_panel_swiglu: out must be [{m},{two_n // 2}]")
    if not (waves == 0 or 4 <= waves <= 8):
        raise KernelError("gemm_panel_swiglu: waves 4 to 8, or 0")
    _check(_fn("gemm", "dryft_gemm_panel_swiglu_bf16")(_ptr(x), x.stride(0), _ptr(w_gate_up), _ptr(out), m, two_n // 2, k,
                                                       int(waves), _stream()), "gemm_panel_swiglu_bf16")
    return out


TALL_ROWS = 256     # the most rows gemm_tall_swiglu takes
TALL_GROUP = 64     # values of K it moves at a time; K must be a multiple of it


def gemm_tall_swiglu_bf16(x, w_gate_up, out, tiles: int = 0) -> torch.Tensor:
    """``silu(x @ Wg.T) * (x @ Wu.T)`` for ``w_gate_up = [Wg; Wu]``, at most 256 rows, by the kernel whose waves each own
    rows of x and multiply them with all of the workgroup's rows of W (operands straight into LDS). K must be a multiple
    of 64. ``tiles`` (4 to 8, 8 outputs each) per workgroup; 0 lets the library choose."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(w_gate_up, "w_gate_up", torch.bfloat16)
    _gpu(out, "out", torch.bfloat16)
    m, k = x.shape
    two_n = w_gate_up.shape[0]
    if not (two_n % 2 == 0 and w_gate_up.shape == (two_n, k) and w_gate_up.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_tall_swiglu: x [M,K] row-major, w [2N,K] contiguous")
    if not (m <= TALL_ROWS and k % TALL_GROUP == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_tall_swiglu: needs M <= {TALL_ROWS} and K % {TALL_GROUP} == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w_gate_up.data_ptr() % 16 == 0):
        raise KernelError("gemm_tall_swiglu: operands must be 16-byte aligned")
    if not (out.shape == (m, two_n // 2) and out.is_contiguous()):
        raise KernelError(f"gemm_tall_swiglu: out must be [{m},{two_n // 2}]")
    if not (tiles == 0 or 4 <= tiles <= 8):
        raise KernelError("gemm_tall_swiglu: tiles 4 to 8, or 0")
    _check(_fn("gemm", "dryft_gemm_tall_swiglu_bf16")(_ptr(x), x.stride(0), _ptr(w_gate_up), _ptr(out), m, two_n // 2, k,
                                                      int(tiles), _stream()), "gemm_tall_swiglu_bf16")
    return out


def gemm_tall_bf16(x, w, partials, splits: int, tiles: int) -> torch.Tensor:
    """Float partial sums ``partials[s] = x @ w.T`` over the s-th run of K, at most 256 rows, by the kernel whose waves
    each own rows of x (see ``gemm_tall_swiglu_bf16``); a workgroup owns ``16 * tiles`` outputs (tiles 4 to 8). K must
    be a multiple of 64 and ``splits`` a count ``gemm_mid_splits`` gives."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(w, "w", torch.bfloat16)
    _gpu(partials, "partials", torch.float32)
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_tall: x [M,K] row-major, w [N,K] contiguous")
    if not (m <= TALL_ROWS and k % TALL_GROUP == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_tall: needs M <= {TALL_ROWS} and K % {TALL_GROUP} == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and partials.data_ptr() % 16 == 0):
        raise KernelError("gemm_tall: operands must be 16-byte aligned")
    if not (partials.shape == (splits, m, n) and partials.is_contiguous()):
        raise KernelError(f"gemm_tall: partials must be [{splits},{m},{n}]")
    if not 4 <= tiles <= 8:
        raise KernelError("gemm_tall: tiles 4 to 8")
    if gemm_mid_splits(k, splits) != splits:
        raise KernelError(f"gemm_tall: {splits} runs of K={k} would leave one empty")
    _check(_fn("gemm", "dryft_gemm_tall_bf16")(_ptr(x), x.stride(0), _ptr(w), _ptr(partials), m, n, k, int(splits),
                                               int(tiles), _stream()), "gemm_tall_bf16")
    return partials


MID_ROWS = 256      # the most rows gemm_mid takes
MID_GROUP = 64      # values of K it walks at a time; K must be a multiple, and the splits are runs of such groups


def gemm_mid_splits(k: int, splits: int) -> int:
    """The number of splits closest below ``splits`` that cuts ``k`` into runs of groups none of which is empty."""
    groups = k // MID_GROUP
    splits = max(1, min(splits, groups))
    while splits > 1 and -(-groups // -(-groups // splits)) != splits:
        splits -= 1
    return splits


def gemm_mid_bf16(x, w, partials, splits: int) -> torch.Tensor:
    """Float partial sums ``partials[splits, M, N]`` of ``x @ w.T`` over ``splits`` runs of K, for 1 to 256 rows, by the
    kernel whose operands go from memory straight into LDS. K must be a multiple of 64 and ``splits`` one that
    ``gemm_mid_splits`` returns."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(w, "w", torch.bfloat16)
    _gpu(partials, "partials", torch.float32)
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_mid: x [M,K] row-major, w [N,K] contiguous")
    if not (m <= MID_ROWS and k % MID_GROUP == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_mid: needs M <= {MID_ROWS} and K % {MID_GROUP} == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and partials.data_ptr() % 16 == 0):
        raise KernelError("gemm_mid: operands must be 16-byte aligned")
    if not (splits >= 1 and gemm_mid_splits(k, splits) == splits):
        raise KernelError(f"gemm_mid: {splits} splits would leave a run of K = {k} empty")
    if not (partials.shape == (splits, m, n) and partials.is_contiguous()):
        raise KernelError(f"gemm_mid: partials must be [{splits},{m},{n}]")
    _check(_fn("gemm", "dryft_gemm_mid_bf16")(_ptr(x), x.stride(0), _ptr(w), _ptr(partials), m, n, k, int(splits),
                                              _stream()), "gemm_mid_bf16")
    return partials


def gemm_wide_swiglu_bf16(x, w_gate_up, out, group_blocks: int = 2, depth: int = 1) -> torch.Tensor:
    """``silu(x @ Wg.T) * (x @ Wu.T)`` for ``w_gate_up = [Wg; Wu]``, at most 64 rows, in one kernel."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(w_gate_up, "w_gate_up", torch.bfloat16)
    _gpu(out, "out", torch.bfloat16)
    m, k = x.shape
    two_n = w_gate_up.shape[0]
    if not (two_n % 2 == 0 and w_gate_up.shape == (two_n, k) and w_gate_up.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_wide_swiglu: x [M,K] row-major, w [2N,K] contiguous")
    if not (m <= 64 and k % 8 == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_wide_swiglu: needs M <= 64 and K % 8 == 0, got M={m} K={k}")
    if not (x.data_ptr() % 16 == 0 and w_gate_up.data_ptr() % 16 == 0):
        raise KernelError("gemm_wide_swiglu: operands must be 16-byte aligned")
    if not (out.shape == (m, two_n // 2) and out.is_contiguous()):
        raise KernelError(f"gemm_wide_swiglu: out must be [{m},{two_n // 2}]")
    if not (group_blocks in (1, 2) and depth in (1, 2, 3)):
        raise KernelError("gemm_wide_swiglu: group_blocks in 1, 2 and depth in 1..3")
    _check(_fn("gemm", "dryft_gemm_wide_swiglu_bf16")(_ptr(x), x.stride(0), _ptr(w_gate_up), _ptr(out), m, two_n // 2, k,
                                                      int(group_blocks), int(depth), _stream()), "gemm_wide_swiglu_bf16")
    return out


def gemm_block_bf16(x, w, out, swiglu: bool = False, shape: int | None = None) -> torch.Tensor:
    """``x [M, K] @ w[N, K].T`` for any number of rows, by the kernel that owns blocks of 128 rows by 128 outputs;
    ``out`` bfloat16 or float32. With ``swiglu``, ``w = [Wg; Wu]`` of ``2N`` rows and
    ``out = silu(x @ Wg.T) * (x @ Wu.T)`` in bfloat16. ``shape``: 0 = blocks of 128 x 128, 1 = 256 x 256; by default
    the large blocks where there are enough of them to give every compute unit one."""
    _gpu(x, "x", torch.bfloat16)
    _gpu(w, "w", torch.bfloat16)
    _gpu(out, "out")
    m, k = x.shape
    n = w.shape[0] // 2 if swiglu else w.shape[0]
    if not (w.dim() == 2 and w.shape[1] == k and w.is_contiguous() and x.stride(1) == 1) or (swiglu and w.shape[0] % 2):
        raise KernelError("gemm_block: x [M,K] row-major, w [N,K] (or [2N,K]) contiguous")
    if not (k % 8 == 0 and x.stride(0) % 8 == 0):
        raise KernelError(f"gemm_block: needs K % 8 == 0, got K={k}")
    if not (x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        raise KernelError("gemm_block: operands must be 16-byte aligned")
    out_dtypes = (torch.bfloat16,) if swiglu else (torch.float32, torch.bfloat16)
    if not (out.shape == (m, n) and out.is_contiguous() and out.dtype in out_dtypes):
        raise KernelError(f"gemm_block: out must be contiguous [{m},{n}]")
    if shape is None:
        shape = 1 if -(-m // 256) * -(-(2 * n if swiglu else n) // 256) >= 256 else 0
    if not (shape in (0, 1)):
        raise KernelError("gemm_block: shape 0 or 1")
    _check(_fn("gemm", "dryft_gemm_block_bf16")(_ptr(x), x.stride(0), _ptr(w), _ptr(out), m, n, k, 1 if swiglu else 0,
                                                1 if out.dtype == torch.float32 else 0, int(shape), _stream()), "gemm_block_bf16")
    return out


def gemm_block_f32(x, w, out, shape: int | None = None) -> torch.Tensor:
    """``x [M, K] @ w[N, K].T`` on float32 values with the matrix cores' full-precision instruction
    (``v_mfma_f32_16x16x4_f32``); ``K`` a multiple of 4, operands 16-byte aligned."""
    _gpu(x, "x", torch.float32)
    _gpu(w, "w", torch.float32)
    _gpu(out, "out", torch.float32)
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_block_f32: x [M,K] row-major, w [N,K] contiguous")
    if not (k % 4 == 0 and x.stride(0) % 4 == 0):
        raise KernelError(f"gemm_block_f32: needs K % 4 == 0, got K={k}")
    if not (x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0):
        raise KernelError("gemm_block_f32: operands must be 16-byte aligned")
    if not (out.shape == (m, n) and out.is_contiguous()):
        raise KernelError(f"gemm_block_f32: out must be contiguous [{m},{n}]")
    if shape is None:
        shape = 1 if -(-m // 256) * -(-n // 256) >= 256 else 0
    if not (shape in (0, 1)):
        raise KernelError("gemm_block_f32: shape 0 or 1")
    _check(_fn("gemm", "dryft_gemm_block_f32")(_ptr(x), x.stride(0), _ptr(w), _ptr(out), m, n, k, int(shape), _stream()),
           "gemm_block_f32")
    return out


def gemm_rows_f32(x, w, out) -> torch.Tensor:
    """``x [M<=16, K] @ w[N, K].T`` on float32 values by plain multiply-adds, every weight read once; ``K`` a
    multiple of 4 and ``w`` 16-byte aligned."""
    _gpu(x, "x", torch.float32)
    _gpu(w, "w", torch.float32)
    _gpu(out, "out", torch.float32)
    m, k = x.shape
    n = w.shape[0]
    if not (w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1):
        raise KernelError("gemm_rows_f32: x [M,K] row-major, w [N,K] contiguous")
    if not (m <= 16 and k % 4 == 0 and w.data_ptr() % 16 == 0):
        raise KernelError(f"gemm_rows_f32: needs M <= 16, K % 4 == 0, aligned w; got M={m} K={k}")
    if not (out.shape == (m, n) and out.is_contiguous()):
        raise KernelError(f"gemm_rows_f32: out must be contiguous [{m},{n}]")
    _check(_fn("gemm", "dryft_gemm_rows_f32")(_ptr(x), x.stride(0), _ptr(w), _ptr(out), m, n, k, _stream()), "gemm_rows_f32")
    return out


def sum_partials(partials: torch.Tensor, out: torch.Tensor, splits: int) -> torch.Tensor:
    _gpu(partials, "partials", torch.float32)
    _gpu(out, "out")
    if not (out.is_contiguous() and partials.is_contiguous() and partials.numel() >= splits * out.numel()):
        raise KernelError("sum_partials: partials must hold splits * out.numel() values")
    if not (out.dtype in (torch.float32, torch.bfloat16)):
        raise KernelError("sum_partials: out must be float32 or bfloat16")
    _check(_fn("gemm", "dryft_sum_partials")(_ptr(partials), _ptr(out), out.numel(), splits,
                                             1 if out.dtype == torch.float32 else 0, _stream()), "sum_partials")
    return out


# ---------------------------------------------------------------------------------------- sampling
def argmax_rows(logits: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _gpu(logits, "logits", torch.float32)
    _gpu(out, "out", torch.int32)
    rows, vocab = logits.shape
    if not (logits.stride(1) == 1 and out.numel() >= rows and out.is_contiguous()):
        raise KernelError("argmax_rows: bad operands")
    chunks = 1 if vocab < 8192 else min(64, vocab // 2048)
    scratch_v = scratch_i = None
    if chunks > 1:
        scratch_v = torch.empty(rows * chunks, dtype=torch.float32, device=logits.device)
        scratch_i = torch.empty(rows * chunks, dtype=torch.int32, device=logits.device)
    _check(_fn("sampling", "dryft_argmax_rows")(_ptr(logits), rows, vocab, logits.stride(0), _ptr(out), chunks,
                                                _ptr(scratch_v), _ptr(scratch_i), _stream()), "argmax_rows")
    return out


def sample_rows(logits: torch.Tensor, temperature: float, uniforms: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    _gpu(logits, "logits", torch.float32)
    _gpu(uniforms, "uniforms", torch.float32)
    _gpu(out, "out", torch.int32)
    rows, vocab = logits.shape
    if not (temperature > 0):
        raise KernelError("sample_rows: temperature must be positive (use argmax_rows for greedy)")
    if not (logits.stride(1) == 1 and out.numel() >= rows and uniforms.numel() >= rows):
        raise KernelError("sample_rows: bad operands")
    chunks = 1 if vocab < 8192 else min(64, vocab // 2048)
    chunk_max = chunk_sum = None
    if chunks > 1:
        chunk_max = torch.empty(rows * chunks, dtype=torch.float32, device=logits.device)
        chunk_sum = torch.empty(rows * chunks, dtype=torch.float32, device=logits.device)
    _check(_fn("sampling", "dryft_sample_rows")(_ptr(logits), rows, vocab, logits.stride(0), float(temperature),
                                                _ptr(uniforms), _ptr(out), chunks, _ptr(chunk_max), _ptr(chunk_sum),
                                                _stream()), "sample_rows")
    return out
