"""Each HIP kernel alone against a plain float32 reference of the same operation, at sizes other
than the engine's tiny models use. Shapes and tolerances follow the reference's kernel self-tests
(kernels/rmsnorm.py:106-132, rope_qknorm.py:172-227, attn_decode.py:180-226, silu_mul.py:53-63)."""

import math

import numpy as np
import pytest
import torch

from helpers import bf16_tolerance, build_pages, value_columns

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def ops():
    from dryft_amd.csrc import ops as o
    return o


def close(got, want, dtype, ulps=2.0, floor=0.0, what=""):
    got, want = got.float().cpu(), want.float().cpu()
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    tol = bf16_tolerance(want, ulps, floor) if dtype == torch.bfloat16 else 2e-5 * float(want.abs().max()) + 1e-6
    diff = float((got - want).abs().max())
    assert diff <= tol, f"{what}: max diff {diff} > {tol}"


# ------------------------------------------------------------------------------------------- embed
@pytest.mark.parametrize("dtype", DTYPES)
def test_embed_rows(dtype):
    torch.manual_seed(0)
    table = torch.randn(331, 100).to(dtype)
    tokens = torch.tensor([0, 330, 5, 5, 17, 200, 1], dtype=torch.int32)
    out = torch.empty(7, 100, dtype=dtype, device=DEV)
    ops().embed_rows(tokens.to(DEV), table.to(DEV), out)
    assert torch.equal(out.cpu(), table[tokens.long()])
    # the same rows of each of several tables (the wanted rows of a product left as partial sums)
    tables = torch.randn(5, 331, 100).to(dtype)
    outs = torch.full((5, 7, 100), float("nan"), dtype=dtype, device=DEV)
    ops().embed_rows(tokens.to(DEV), tables.to(DEV), outs)
    assert torch.equal(outs.cpu(), tables[:, tokens.long()])
    with pytest.raises(Exception, match="expected"):
        ops().embed_rows(tokens.to(DEV), tables.to(DEV), out)


# -------------------------------------------------------------------------------------------- norm
def rmsnorm_ref(x, w, eps, dtype):
    xf = x.float()
    n = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(dtype).float()
    return (n * w.float()).to(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,width", [(1, 2560), (7, 2560), (33, 128), (1000, 128), (5, 100), (3, 9), (2, 5120)])
def test_rmsnorm_and_add(dtype, rows, width):
    torch.manual_seed(rows * 1000 + width)
    res = (3 * torch.randn(rows, width)).to(dtype)
    x = (3 * torch.randn(rows, width)).to(dtype)
    w = (1 + 0.1 * torch.randn(width)).to(dtype)
    eps = 1e-6
    o = ops()
    y = torch.empty(rows, width, dtype=dtype, device=DEV)
    o.add_rmsnorm(res.to(DEV), None, w.to(DEV), eps, None, y)
    close(y, rmsnorm_ref(res, w, eps, dtype), dtype, what="rmsnorm")
    # weights stored in 32-bit are taken as they are
    o.add_rmsnorm(res.to(DEV), None, w.float().to(DEV), eps, None, y)
    close(y, rmsnorm_ref(res, w, eps, dtype), dtype, what="rmsnorm with float32 weight")
    # residual add: the sum is rounded once and must be bit-equal to the library's add
    res_d, y2 = res.to(DEV).clone(), torch.empty(rows, width, dtype=dtype, device=DEV)
    o.add_rmsnorm(res_d, x.to(DEV), w.to(DEV), eps, res_d, y2)
    want_res = (res.float() + x.float()).to(dtype)
    assert torch.equal(res_d.cpu(), want_res), "residual sum differs"
    close(y2, rmsnorm_ref(want_res, w, eps, dtype), dtype, what="add_rmsnorm")
    # partial sums in float32 are added in order
    parts = torch.randn(3, rows, width)
    res_d = res.to(DEV).clone()
    o.add_rmsnorm(res_d, parts.to(DEV), w.to(DEV), eps, res_d, y2, n_partials=3)
    want_res = (res.float() + ((parts[0] + parts[1]) + parts[2])).to(dtype)
    close(res_d, want_res, dtype, ulps=1.0, what="residual + partials")
    close(y2, rmsnorm_ref(res_d.cpu(), w, eps, dtype), dtype, what="norm after partials")


@pytest.mark.parametrize("dtype", DTYPES)
def test_add_rows(dtype):
    torch.manual_seed(1)
    a, b = torch.randn(37, 96).to(dtype), torch.randn(37, 96).to(dtype)
    out = torch.empty(37, 96, dtype=dtype, device=DEV)
    ops().add_rows(a.to(DEV), b.to(DEV), out)
    assert torch.equal(out.cpu(), (a.float() + b.float()).to(dtype))


# -------------------------------------------------------------------------------------- activation
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,inter", [(1, 9728), (7, 9728), (3, 2048), (5, 224), (2, 37)])
def test_silu_mul(dtype, rows, inter):
    torch.manual_seed(rows + inter)
    gu = (3 * torch.randn(rows, 2 * inter)).to(dtype)
    g, u = gu[:, :inter].float(), gu[:, inter:].float()
    want = (torch.nn.functional.silu(g).to(dtype).float() * u).to(dtype)
    out = torch.empty(rows, inter, dtype=dtype, device=DEV)
    ops().silu_mul(gu.to(DEV), out)
    close(out, want, dtype, what="silu_mul")


# ----------------------------------------------------------------------------------------- rope_kv
def rope_ref(x, cos, sin, dtype):
    """x [rows, heads, D] float; cos/sin [rows, D/2] (already in dtype); rounding as the bf16 path does."""
    half = x.shape[-1] // 2
    c, s = cos.float()[:, None, :], sin.float()[:, None, :]
    x1, x2 = x[..., :half], x[..., half:]
    r = lambda t: t.to(dtype).float()
    return torch.cat((r(r(x1 * c) - r(x2 * s)), r(r(x2 * c) + r(x1 * s))), dim=-1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_heads,n_kv,D,theta", [(32, 8, 128, 5e6), (6, 3, 48, 1e4), (4, 2, 16, 1e6), (5, 1, 256, 1e5),
                                                  (9, 3, 64, 1e4), (70, 2, 32, 1e4)])
@pytest.mark.parametrize("rows", [23, 150])                 # few rows, and enough for the kernels of long steps
def test_qk_norm_rope_kv(dtype, n_heads, n_kv, D, theta, rows):
    torch.manual_seed(D)
    n_slots, max_pages, n_pages = 7, 6, 42
    L = max_pages * 64
    eps = 1e-6
    qkv = (2 * torch.randn(rows, (n_heads + 2 * n_kv) * D)).to(dtype)
    wq = (1 + 0.1 * torch.randn(D)).to(dtype)
    wk = (1 + 0.1 * torch.randn(D)).to(dtype)
    inv = 1.0 / (theta ** (torch.arange(0, D, 2).float() / D))
    ang = torch.arange(L).float()[:, None] * inv[None]
    cos, sin = ang.cos().to(dtype), ang.sin().to(dtype)
    rng = np.random.default_rng(D)
    # rows spread over slots at distinct (slot, position) places; one row is dead
    places = rng.permutation(n_slots * L)[:rows]
    row_slot = torch.tensor(places // L, dtype=torch.int32)
    row_pos = torch.tensor(places % L, dtype=torch.int32)
    row_slot[5] = -1
    table = torch.tensor(rng.permutation(n_pages).reshape(n_slots, max_pages), dtype=torch.int32)
    k_pages = torch.zeros(n_pages, n_kv, 64, D, dtype=dtype, device=DEV)
    v_pages = torch.zeros(n_pages, n_kv, D, 64, dtype=dtype, device=DEV)
    q_out = torch.full((rows, n_heads, D), 7.0, dtype=dtype, device=DEV)
    ops().qk_norm_rope_kv(qkv.to(DEV), wq.to(DEV), wk.to(DEV), eps, cos.to(DEV), sin.to(DEV), D, row_slot.to(DEV),
                          row_pos.to(DEV), q_out, k_pages, v_pages, table.to(DEV), True, n_heads, n_kv, D)
    q = qkv[:, : n_heads * D].view(rows, n_heads, D)
    k = qkv[:, n_heads * D: (n_heads + n_kv) * D].view(rows, n_kv, D)
    v = qkv[:, (n_heads + n_kv) * D:].view(rows, n_kv, D)

    def norm(x, w):
        xf = x.float()
        n = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(dtype).float()
        return (n * w.float()).to(dtype).float()

    pos = row_pos.long()
    q_want = rope_ref(norm(q, wq), cos[pos], sin[pos], dtype)
    k_want = rope_ref(norm(k, wk), cos[pos], sin[pos], dtype)
    live = row_slot >= 0
    close(q_out[live.to(DEV)], q_want[live], dtype, what="q")
    assert not q_out[5].any(), "a dead row's q must be zero"
    kp, vp = k_pages.cpu(), v_pages.cpu()
    for r in range(rows):
        if not live[r]:
            continue
        page = int(table[row_slot[r], row_pos[r] // 64])
        at = int(row_pos[r]) % 64
        close(kp[page, :, at], k_want[r], dtype, what=f"k row {r}")
        col = int(value_columns()[at])                        # values sit in the column the second product wants
        assert torch.equal(vp[page, :, :, col], v[r]), f"v row {r} must be copied unchanged"
        kp[page, :, at] = 0
        vp[page, :, :, col] = 0
    assert not kp.any() and not vp.any(), "the kernel wrote outside the rows' places"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_kv,D", [(2, 128), (3, 48), (1, 16)])
def test_values_of_many_rows_land_in_their_columns(dtype, n_kv, D):
    """A step of many rows writes values tile by tile: whole aligned blocks of 32 positions with vector
    stores, everything else one by one. Three sequences: from position 0, from the middle of a block, dead."""
    torch.manual_seed(D)
    n_heads, n_slots, max_pages, n_pages = n_kv, 4, 4, 16
    spans = [(2, 0, 150), (0, 37, 50), (-1, 0, 9), (3, 64, 70)]            # (slot, first position, rows)
    row_slot = torch.tensor([s for s, _, n in spans for _ in range(n)], dtype=torch.int32)
    row_pos = torch.tensor([p0 + i for _, p0, n in spans for i in range(n)], dtype=torch.int32)
    rows = len(row_slot)
    qkv = torch.randn(rows, (n_heads + 2 * n_kv) * D).to(dtype)
    w = torch.ones(D).to(dtype)
    cos, sin = torch.ones(max_pages * 64, D // 2).to(dtype), torch.zeros(max_pages * 64, D // 2).to(dtype)
    table = torch.tensor(np.random.default_rng(1).permutation(n_pages).reshape(n_slots, max_pages), dtype=torch.int32)
    k_pages = torch.zeros(n_pages, n_kv, 64, D, dtype=dtype, device=DEV)
    v_pages = torch.zeros(n_pages, n_kv, D, 64, dtype=dtype, device=DEV)
    q_out = torch.empty(rows, n_heads, D, dtype=dtype, device=DEV)
    ops().qk_norm_rope_kv(qkv.to(DEV), w.to(DEV), w.to(DEV), 1e-6, cos.to(DEV), sin.to(DEV), D, row_slot.to(DEV),
                          row_pos.to(DEV), q_out, k_pages, v_pages, table.to(DEV), True, n_heads, n_kv, D)
    v = qkv[:, (n_heads + n_kv) * D:].view(rows, n_kv, D)
    vp, cols = v_pages.cpu(), value_columns()
    for r in range(rows):
        if row_slot[r] < 0:
            continue
        page, col = int(table[row_slot[r], row_pos[r] // 64]), int(cols[int(row_pos[r]) % 64])
        assert torch.equal(vp[page, :, :, col], v[r]), f"v row {r}"
        vp[page, :, :, col] = 0
    assert not vp.any(), "values were written outside the rows' places"


@pytest.mark.parametrize("dtype", DTYPES)
def test_rope_partial_width_and_no_norm(dtype):
    """Rotation over the first `rot` lanes only, no q/k norm, and a run that writes no cache."""
    torch.manual_seed(3)
    rows, n_heads, n_kv, D, rot = 9, 4, 2, 64, 32
    qkv = torch.randn(rows, (n_heads + 2 * n_kv) * D).to(dtype)
    ang = torch.arange(128).float()[:, None] * (1.0 / (1e4 ** (torch.arange(0, rot, 2).float() / rot)))[None]
    cos, sin = ang.cos().to(dtype), ang.sin().to(dtype)
    row_slot = torch.zeros(rows, dtype=torch.int32)
    row_pos = torch.arange(10, 10 + rows, dtype=torch.int32)
    q_out = torch.empty(rows, n_heads, D, dtype=dtype, device=DEV)
    ops().qk_norm_rope_kv(qkv.to(DEV), None, None, 0.0, cos.to(DEV), sin.to(DEV), rot, row_slot.to(DEV),
                          row_pos.to(DEV), q_out, None, None, None, False, n_heads, n_kv, D)
    q = qkv[:, : n_heads * D].view(rows, n_heads, D).float()
    want = q.clone()
    want[..., :rot] = rope_ref(q[..., :rot], cos[row_pos.long()], sin[row_pos.long()], dtype)
    close(q_out, want, dtype, what="partial rotary")


# --------------------------------------------------------------------------------------- attention
def attention_ref(q, k, v, lengths, q_pos, scale, window=None):
    """q [B, Tq, nH, D] at positions q_pos [B, Tq]; k, v [B, L, nKV, D] float32; float64 softmax."""
    B, Tq, n_heads, D = q.shape
    group = n_heads // k.shape[2]
    out = torch.zeros(B, Tq, n_heads, D, dtype=torch.float64)
    for b in range(B):
        kk = k[b].double().repeat_interleave(group, dim=1)
        vv = v[b].double().repeat_interleave(group, dim=1)
        for t in range(Tq):
            p = int(q_pos[b, t])
            if p < 0:
                continue
            lo = 0 if window is None else max(0, p - window + 1)
            s = torch.einsum("hd,jhd->hj", q[b, t].double(), kk[lo: p + 1]) * scale
            out[b, t] = torch.einsum("hj,jhd->hd", torch.softmax(s, -1), vv[lo: p + 1])
    return out.float()


CASES = [  # n_heads, n_kv, D, lengths (cached tokens incl. the rows'), q rows per sequence
    (32, 8, 128, [1, 513, 300, 64], 1),
    (32, 8, 128, [700], 1),
    (8, 2, 32, [5, 130, 31, 64, 65, 1], 1),
    (6, 3, 48, [100, 129], 1),
    (4, 2, 16, [17, 9, 200], 1),
    (20, 1, 64, [77, 140], 1),          # 20 heads on one kv head: two blocks of 16 rows
    (32, 8, 128, [150, 64, 209], 70),   # prompts continuing after cached tokens
    (8, 2, 32, [31, 13, 6, 1], 31),
    (6, 3, 48, [129, 90], 64),
    (4, 2, 16, [300], 300),
    # head size 128 with eight, five and two query heads to a kv head (the architecture allows any whole number)
    (64, 8, 128, [1, 513, 300, 64], 1),
    (40, 8, 128, [257, 64, 1, 130], 1),
    (16, 8, 128, [700, 65], 1),
    (64, 8, 128, [150, 64, 209], 70),
    (40, 8, 128, [150, 64, 209], 70),
    (16, 8, 128, [150, 64, 209], 70),
]


def run_attention_case(kind, dtype, n_heads, n_kv, D, lengths, tq, window=None, seed=0, misaligned=False, dead=(),
                       drop_pages_behind_window=False):
    """``dead``: sequences that sit the step out (slot -1). They keep their rows, which every kernel leaves at
    zero (the tiled prompt kernel by never visiting them), and have no tiles. ``drop_pages_behind_window``: pages
    that no row of the step can see any more are gone from the page table (-1), as in a windowed cache."""
    torch.manual_seed(seed + D + len(lengths))
    B, L = len(lengths), max(lengths)
    n_slots, n_pages = B + 2, sum((n + 63) // 64 for n in lengths) + 3
    k = torch.randn(B, L, n_kv, D).to(dtype)
    v = torch.randn(B, L, n_kv, D).to(dtype)
    q_lens = [min(tq, n) for n in lengths]
    q_pos = torch.full((B, max(q_lens)), -1, dtype=torch.long)
    for b, (n, ql) in enumerate(zip(lengths, q_lens)):
        q_pos[b, :ql] = torch.arange(n - ql, n)
    q = torch.randn(B, max(q_lens), n_heads, D).to(dtype)
    # make one far key stand out for the last row of each sequence, so a lost key shows
    for b, n in enumerate(lengths):
        far = 0 if window is None else max(0, n - window)
        k[b, far, :, :] = (4.0 * q[b, q_lens[b] - 1].float().view(n_kv, -1, D).mean(1)).to(dtype)
    scale = 1.0 / math.sqrt(D)
    for b in dead:
        q_pos[b] = -1                                            # the reference leaves these rows at zero
    want = attention_ref(q.float(), k.float(), v.float(), lengths, q_pos, scale, window)
    k_pages, v_pages, table, slots = build_pages(k, v, lengths, n_pages, n_slots, seed=seed, poison=1e4)
    if drop_pages_behind_window:
        for b, (n, ql) in enumerate(zip(lengths, q_lens)):
            table[slots[b], : max(0, n - ql - window + 1) // 64] = -1
    slots = [-1 if b in dead else s for b, s in enumerate(slots)]
    rows = sum(q_lens)
    q_packed = torch.cat([q[b, :ql] for b, ql in enumerate(q_lens)]).contiguous()
    want_packed = torch.cat([want[b, :ql] for b, ql in enumerate(q_lens)])
    row_slot = torch.tensor([slots[b] for b, ql in enumerate(q_lens) for _ in range(ql)], dtype=torch.int32)
    row_pos = torch.tensor([int(p) for b, ql in enumerate(q_lens) for p in q_pos[b, :ql]], dtype=torch.int32)
    cu = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    tiles = np.concatenate([[0], np.cumsum([0 if b in dead else (ql + 63) // 64 for b, ql in enumerate(q_lens)])]).astype(np.int32)
    d = lambda t: t.to(DEV)
    out = torch.zeros(rows, n_heads, D, dtype=dtype, device=DEV)
    o = ops()
    w = window or 0
    if kind == "rows":
        kp, vp = d(k_pages), d(v_pages)
        if misaligned:                                       # pages that start one value past a 16-byte boundary
            def shifted(t):
                view = torch.empty(t.numel() + 1, dtype=t.dtype, device=DEV)[1:].view(t.shape)
                view.copy_(t)
                return view
            kp, vp = shifted(kp), shifted(vp)
        o.attn_rows(d(q_packed), kp, vp, d(table), d(row_slot), d(row_pos), out, n_heads, n_kv, D, scale, w)
    elif str(kind).startswith("causal"):                     # "causal2": with the kernel's mode 2
        o.attn_causal_bf16(d(q_packed), d(k_pages), d(v_pages), d(table), d(torch.tensor(slots, dtype=torch.int32)),
                           d(torch.from_numpy(cu)), d(torch.from_numpy(tiles)),
                           d(torch.tensor([n - ql for n, ql in zip(lengths, q_lens)], dtype=torch.int32)), B,
                           int(tiles[-1]) + 1, out, n_heads, n_kv, D, scale, w, int(str(kind)[6:] or 0))
    else:
        splits = kind
        part_o = torch.empty(B * n_heads * splits * D, dtype=torch.float32, device=DEV)
        part_ml = torch.empty(B * n_heads * splits * 2, dtype=torch.float32, device=DEV)
        o.attn_split_bf16(d(q_packed), d(k_pages), d(v_pages), d(table), d(torch.tensor(slots, dtype=torch.int32)),
                          d(torch.from_numpy(cu)), d(torch.tensor(lengths, dtype=torch.int32)), B, part_o, part_ml,
                          splits, out, n_heads, n_kv, D, scale, w)
    close(out, want_packed, dtype, ulps=4.0, floor=1e-3, what=f"attention {kind} {n_heads}/{n_kv}/{D} {lengths} tq={tq}")
    for b in dead:
        assert not out[int(cu[b]):int(cu[b + 1])].any(), f"rows of sequence {b}, which sits out, were written"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", CASES)
def test_attn_rows(dtype, case):
    run_attention_case("rows", dtype, *case)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attn_rows_takes_pages_at_any_address(dtype):
    """Pages that are not 16-byte aligned go value by value instead of eight a load."""
    run_attention_case("rows", dtype, 6, 3, 48, [200, 70, 130], 33, misaligned=True)
    run_attention_case("rows", dtype, 8, 2, 32, [200, 70, 130], 200, window=70, misaligned=True)


CAUSAL_CASES = CASES + [      # many rows: several tiles per sequence, sequences that end inside a tile
    (8, 2, 64, [300, 129, 70, 500], 500),
    (32, 8, 128, [260], 260),
    (32, 8, 128, [700, 330], 290),      # rows that continue after 410 and 40 cached tokens
    (9, 3, 32, [200, 150, 1, 65], 200),   # three heads to a kv head: no pairs of heads
    (64, 8, 128, [260, 70], 260),
    (40, 8, 128, [330, 129], 200),
    (16, 8, 128, [700, 330], 290),
]


# chosen by the kernel; 16 rows; two heads; 32 rows a wave; 16 and 32 rows with the pages staged through registers
# also at head size 128, where 1 and 3 bring them straight into LDS
CAUSAL_MODES = [0, 1, 2, 3, 5, 7]


@pytest.mark.parametrize("mode", CAUSAL_MODES)
@pytest.mark.parametrize("case", CAUSAL_CASES)
def test_attn_causal_bf16(case, mode):
    if mode == 2 and (case[0] // case[1]) % 2:
        pytest.skip("two heads per wave need an even number of heads per kv head")
    run_attention_case(f"causal{mode}", torch.bfloat16, *case)


# Sequences that sit out, of one row and of several hundred, before and between the ones that take part. The
# second case has enough rows (33 tiles of 64 heads) for the kernel to choose 32 rows a wave by itself.
DEAD_CASES = [((8, 2, 32, [1, 200, 330, 150, 70], 330), (0, 2)),
              ((64, 16, 32, [1, 1000, 300, 1030, 64], 1030), (0, 2)),
              ((32, 8, 128, [300, 260, 1, 129], 300), (0, 2, 3))]


@pytest.mark.parametrize("mode", CAUSAL_MODES)
@pytest.mark.parametrize("case,dead", DEAD_CASES)
def test_attn_causal_bf16_with_sequences_that_sit_out(case, dead, mode):
    run_attention_case(f"causal{mode}", torch.bfloat16, *case, dead=dead)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attn_rows_with_sequences_that_sit_out(dtype):
    run_attention_case("rows", dtype, *DEAD_CASES[0][0], dead=DEAD_CASES[0][1])


@pytest.mark.parametrize("splits", [1, 2, 5, 32])
@pytest.mark.parametrize("case", [c for c in CASES if c[4] == 1])
def test_attn_split_bf16(case, splits):
    run_attention_case(splits, torch.bfloat16, *case)


# The reference's own lengths for its split-KV kernel (kernels/attn_decode.py:204-215) at Qwen3-4B's heads: a
# split here walks up to 128 pages, four waves taking them in turn.
LONG_DECODE = [(32, 8, 128, [2047], 1), (32, 8, 128, [8191, 4096], 1), (32, 8, 128, list(range(3, 3 + 16 * 31, 31)), 1),
               (64, 8, 128, [2047, 4100], 1), (40, 8, 128, [8191, 2049], 1), (16, 8, 128, [2047, 4096], 1)]


@pytest.mark.parametrize("splits", [1, 8, 32])
@pytest.mark.parametrize("case", LONG_DECODE)
def test_attn_split_bf16_long_sequences(case, splits):
    run_attention_case(splits, torch.bfloat16, *case)
    if splits == 8:
        run_attention_case(splits, torch.bfloat16, *case, dead=(0,) if len(case[3]) > 1 else ())


@pytest.mark.parametrize("kind", ["causal0", "causal1", "causal7", 16])
def test_attention_past_65536_positions(kind):
    """One sequence of 66,001 positions (positions, row numbers and page counts past 16 bits) against float64
    arithmetic at sampled rows: the first, both sides of a page's edge, 65,535 and 65,536, and the last. The key that
    stands out for each sampled row lies at a third of its distance, far from where a wrapped index would look. With
    this many rows the kernel's own choice (mode 0) is 32 rows a wave."""
    torch.manual_seed(9)
    n, n_heads, n_kv, D = 66_001, 8, 2, 128
    group = n_heads // n_kv
    sampled = [0, 63, 64, 40_000, 65_535, 65_536, 65_999, 66_000]
    k = torch.randn(1, n, n_kv, D).to(torch.bfloat16)
    v = torch.randn(1, n, n_kv, D).to(torch.bfloat16)
    decoding = not str(kind).startswith("causal")
    rows = [n - 1] if decoding else list(range(n))
    q = torch.randn(len(rows), n_heads, D).to(torch.bfloat16)
    for r in ([n - 1] if decoding else sampled):
        k[0, r // 3] = (3.0 * q[0 if decoding else r].float().view(n_kv, group, D).mean(1)).to(torch.bfloat16)
    scale = D ** -0.5
    k_pages, v_pages, table, slots = build_pages(k, v, [n], (n + 63) // 64 + 2, 3, seed=4, poison=1e4)
    d = lambda t: t.to(DEV)
    out = torch.zeros(len(rows), n_heads, D, dtype=torch.bfloat16, device=DEV)
    o = ops()
    seq_slot = d(torch.tensor(slots, dtype=torch.int32))
    if decoding:
        splits = kind
        part_o = torch.empty(n_heads * splits * D, dtype=torch.float32, device=DEV)
        part_ml = torch.empty(n_heads * splits * 2, dtype=torch.float32, device=DEV)
        o.attn_split_bf16(d(q), d(k_pages), d(v_pages), d(table), seq_slot, d(torch.tensor([0, 1], dtype=torch.int32)),
                          d(torch.tensor([n], dtype=torch.int32)), 1, part_o, part_ml, splits, out, n_heads, n_kv, D,
                          scale, 0)
    else:
        tiles = (n + 63) // 64
        o.attn_causal_bf16(d(q), d(k_pages), d(v_pages), d(table), seq_slot, d(torch.tensor([0, n], dtype=torch.int32)),
                           d(torch.tensor([0, tiles], dtype=torch.int32)), d(torch.tensor([0], dtype=torch.int32)), 1,
                           tiles, out, n_heads, n_kv, D, scale, 0, int(kind[6:]))
    kk, vv = k[0].double().repeat_interleave(group, dim=1), v[0].double().repeat_interleave(group, dim=1)
    for r in ([n - 1] if decoding else sampled):
        i = 0 if decoding else r
        s = torch.einsum("hd,jhd->hj", q[i].double(), kk[: r + 1]) * scale
        want = torch.einsum("hj,jhd->hd", torch.softmax(s, -1), vv[: r + 1]).float()
        close(out[i], want, torch.bfloat16, ulps=4.0, floor=1e-3, what=f"{kind}: row {r} of {n}")


@pytest.mark.parametrize("n_heads,n_kv,D,splits,window", [(32, 8, 128, 3, 0), (6, 3, 48, 1, 0), (4, 2, 16, 2, 0),
                                                          (16, 1, 64, 4, 0), (8, 2, 32, 2, 50),
                                                          (64, 8, 128, 3, 0), (40, 8, 128, 2, 0), (16, 8, 128, 4, 0),
                                                          (10, 2, 128, 1, 70)])
def test_attn_decode_fused_equals_the_two_kernels(n_heads, n_kv, D, splits, window):
    """Norm + rotation + append + attention in one kernel gives what the separate kernels give, bit for bit,
    in the output and in the cache."""
    torch.manual_seed(n_heads + D)
    o = ops()
    lengths = [1, 64, 65, 200, 130]                  # cached tokens after the step (the new one included)
    B, n_slots, max_pages = len(lengths), 7, 4
    n_pages = n_slots * max_pages
    rng = np.random.default_rng(D)
    table = torch.tensor(rng.permutation(n_pages).reshape(n_slots, max_pages), dtype=torch.int32, device=DEV)
    slots = [int(x) for x in rng.permutation(n_slots)[:B]]
    slots[2] = -1                                    # one sequence sits out
    seq_slot = torch.tensor(slots, dtype=torch.int32, device=DEV)
    cu = torch.arange(B + 1, dtype=torch.int32, device=DEV)
    kv_len = torch.tensor(lengths, dtype=torch.int32, device=DEV)
    row_pos = torch.tensor([n - 1 for n in lengths], dtype=torch.int32, device=DEV)
    qkv = (2 * torch.randn(B, (n_heads + 2 * n_kv) * D)).to(torch.bfloat16).to(DEV)
    wq = (1 + 0.1 * torch.randn(D)).to(torch.bfloat16).to(DEV)
    wk = (1 + 0.1 * torch.randn(D)).to(torch.bfloat16).to(DEV)
    ang = torch.arange(256).float()[:, None] * (1.0 / (1e4 ** (torch.arange(0, D, 2).float() / D)))[None]
    cos, sin = ang.cos().to(torch.bfloat16).to(DEV), ang.sin().to(torch.bfloat16).to(DEV)
    k0 = torch.randn(n_pages, n_kv, 64, D).to(torch.bfloat16).to(DEV)
    v0 = torch.randn(n_pages, n_kv, D, 64).to(torch.bfloat16).to(DEV)
    scale = D ** -0.5
    po = torch.empty(B * n_heads * splits * D, dtype=torch.float32, device=DEV)
    pml = torch.empty(B * n_heads * splits * 2, dtype=torch.float32, device=DEV)
    # the two kernels
    k1, v1 = k0.clone(), v0.clone()
    q = torch.empty(B, n_heads, D, dtype=torch.bfloat16, device=DEV)
    out1 = torch.zeros(B, n_heads, D, dtype=torch.bfloat16, device=DEV)
    o.qk_norm_rope_kv(qkv, wq, wk, 1e-6, cos, sin, D, seq_slot, row_pos, q, k1, v1, table, True, n_heads, n_kv, D)
    o.attn_split_bf16(q, k1, v1, table, seq_slot, cu, kv_len, B, po, pml, splits, out1, n_heads, n_kv, D, scale, window)
    # the one kernel
    k2, v2 = k0.clone(), v0.clone()
    out2 = torch.zeros(B, n_heads, D, dtype=torch.bfloat16, device=DEV)
    o.attn_decode_fused_bf16(qkv, wq, wk, 1e-6, cos, sin, D, True, k2, v2, table, seq_slot, cu, kv_len, B, po, pml,
                             splits, out2, n_heads, n_kv, D, scale, window)
    assert torch.equal(k1, k2) and torch.equal(v1, v2), "the cache differs"
    assert not torch.equal(k1, k0), "nothing was appended"
    assert torch.equal(out1, out2), "the output differs"
    # a run that only reads the cache leaves it alone
    k3, v3 = k1.clone(), v1.clone()
    out3 = torch.zeros_like(out2)
    o.attn_decode_fused_bf16(qkv, wq, wk, 1e-6, cos, sin, D, False, k3, v3, table, seq_slot, cu, kv_len, B, po, pml,
                             splits, out3, n_heads, n_kv, D, scale, window)
    assert torch.equal(k3, k1) and torch.equal(v3, v1) and torch.equal(out3, out2)
    # the projection handed over as float partial sums over K: the kernel adds them up in order and rounds, so it
    # gives what it gives for the rounded sum, bit for bit
    parts = torch.randn(3, B, qkv.shape[1], device=DEV)
    summed = ((parts[0] + parts[1]) + parts[2]).to(torch.bfloat16)
    k4, v4, k5, v5 = k0.clone(), v0.clone(), k0.clone(), v0.clone()
    out4, out5 = torch.zeros_like(out2), torch.zeros_like(out2)
    o.attn_decode_fused_bf16(summed, wq, wk, 1e-6, cos, sin, D, True, k4, v4, table, seq_slot, cu, kv_len, B, po, pml,
                             splits, out4, n_heads, n_kv, D, scale, window)
    o.attn_decode_fused_bf16(parts, wq, wk, 1e-6, cos, sin, D, True, k5, v5, table, seq_slot, cu, kv_len, B, po, pml,
                             splits, out5, n_heads, n_kv, D, scale, window, qkv_parts=3)
    assert torch.equal(k4, k5) and torch.equal(v4, v5) and torch.equal(out4, out5), "partial sums of the projection"
    assert not torch.equal(out4, out2)


@pytest.mark.parametrize("heads", [(8, 2), (16, 2), (10, 2), (4, 2), (3, 3)])       # 4, 8, 5, 2 and 1 to a kv head
@pytest.mark.parametrize("mode,few_rows,w_f32,window", [(1, False, False, 0), (3, False, True, 0), (0, True, False, 0),
                                                      (1, False, False, 100)])
def test_prompt_attention_that_takes_the_queries_from_the_projection(mode, few_rows, w_f32, window, heads):
    """At head size 128 the prompt kernel norms and rotates the queries itself. It gives what the stand-alone
    kernel plus the prompt kernel give (the sum of squares is added up in another order, so a value may land on the
    neighbouring bfloat16 now and then), and the cache gets the same keys and values whether or not the queries are
    written out. Sequences continue cached tokens, one sits out, one has a single row."""
    torch.manual_seed(7 + mode)
    o = ops()
    (n_heads, n_kv), D = heads, 128
    assert o.attn_causal_takes_projection(D, D) and not o.attn_causal_takes_projection(64, 64)
    assert not o.attn_causal_takes_projection(D, 64)
    q_lens = [3, 1, 5, 2] if few_rows else [150, 1, 70, 260]        # few rows: the append goes through the other kernels
    starts = [40, 0, 100, 9]
    B, n_slots, max_pages = len(q_lens), 6, 6
    n_pages = n_slots * max_pages
    rng = np.random.default_rng(mode)
    table = torch.tensor(rng.permutation(n_pages).reshape(n_slots, max_pages), dtype=torch.int32, device=DEV)
    slots = [int(x) for x in rng.permutation(n_slots)[:B]]
    slots[2] = -1                                                 # this sequence sits out
    rows = sum(q_lens)
    cu = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    tiles = np.concatenate([[0], np.cumsum([0 if s < 0 else (n + 63) // 64 for s, n in zip(slots, q_lens)])]).astype(np.int32)
    row_slot = torch.tensor([slots[b] for b, n in enumerate(q_lens) for _ in range(n)], dtype=torch.int32, device=DEV)
    row_pos = torch.tensor([starts[b] + i for b, n in enumerate(q_lens) for i in range(n)], dtype=torch.int32, device=DEV)
    seq_slot = torch.tensor(slots, dtype=torch.int32, device=DEV)
    cu_d, tiles_d = torch.from_numpy(cu).to(DEV), torch.from_numpy(tiles).to(DEV)
    seq_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
    qkv = (2 * torch.randn(rows, (n_heads + 2 * n_kv) * D)).to(torch.bfloat16).to(DEV)
    wdt = torch.float32 if w_f32 else torch.bfloat16
    wq, wk = (1 + 0.1 * torch.randn(D)).to(wdt).to(DEV), (1 + 0.1 * torch.randn(D)).to(wdt).to(DEV)
    ang = torch.arange(512).float()[:, None] * (1.0 / (1e4 ** (torch.arange(0, D, 2).float() / D)))[None]
    cos, sin = ang.cos().to(torch.bfloat16).to(DEV), ang.sin().to(torch.bfloat16).to(DEV)
    k0 = torch.randn(n_pages, n_kv, 64, D).to(torch.bfloat16).to(DEV)
    v0 = torch.randn(n_pages, n_kv, D, 64).to(torch.bfloat16).to(DEV)
    scale = D ** -0.5
    k1, v1 = k0.clone(), v0.clone()
    q = torch.empty(rows, n_heads, D, dtype=torch.bfloat16, device=DEV)
    out1 = torch.zeros(rows, n_heads, D, dtype=torch.bfloat16, device=DEV)
    o.qk_norm_rope_kv(qkv, wq, wk, 1e-6, cos, sin, D, row_slot, row_pos, q, k1, v1, table, True, n_heads, n_kv, D)
    o.attn_causal_bf16(q, k1, v1, table, seq_slot, cu_d, tiles_d, seq_start, B, int(tiles[-1]), out1, n_heads, n_kv, D,
                       scale, window, mode)
    k2, v2 = k0.clone(), v0.clone()
    out2 = torch.zeros_like(out1)
    o.qk_norm_rope_kv(qkv, wq, wk, 1e-6, cos, sin, D, row_slot, row_pos, None, k2, v2, table, True, n_heads, n_kv, D)
    o.attn_causal_projected_bf16(qkv, wq, 1e-6, cos, sin, k2, v2, table, seq_slot, cu_d, tiles_d, seq_start, B,
                                 int(tiles[-1]), out2, n_heads, n_kv, D, scale, window, mode)
    assert torch.equal(k1, k2) and torch.equal(v1, v2), "the cache differs"
    assert not torch.equal(k1, k0), "nothing was appended"
    dead = slice(int(cu[2]), int(cu[3]))
    assert not out2[dead].any(), "rows of the sequence that sits out were written"
    assert out1.abs().max() > 0.1
    close(out2, out1.float().cpu(), torch.bfloat16, ulps=2.0, floor=1e-3, what=f"queries from the projection, mode {mode}")
    assert (out1 != out2).float().mean() < 0.02, "more than a rounding here and there"
    # without the norm
    o.qk_norm_rope_kv(qkv, None, None, 0.0, cos, sin, D, row_slot, row_pos, q, k1, v1, table, True, n_heads, n_kv, D)
    o.attn_causal_bf16(q, k1, v1, table, seq_slot, cu_d, tiles_d, seq_start, B, int(tiles[-1]), out1, n_heads, n_kv, D,
                       scale, window, mode)
    o.attn_causal_projected_bf16(qkv, None, 0.0, cos, sin, k1, v1, table, seq_slot, cu_d, tiles_d, seq_start, B,
                                 int(tiles[-1]), out2, n_heads, n_kv, D, scale, window, mode)
    assert torch.equal(out1, out2), "without a norm nothing is summed: bit for bit"


@pytest.mark.parametrize("kind", ["rows", "causal1", "causal2", "causal3", "causal5", "causal7", 3])
def test_attention_window(kind):
    tq = 1 if kind == 3 else 90
    run_attention_case(kind, torch.bfloat16, 8, 2, 32, [200, 70, 130], tq, window=70)
    if kind == "rows":
        run_attention_case(kind, torch.float32, 8, 2, 32, [200, 70, 130], tq, window=70)
    # head size 128, windows shorter and longer than a page, rows that continue cached tokens, and the pages that
    # no row sees any more taken out of the table
    for window, drop in ((70, False), (70, True), (40, True), (200, True)):
        run_attention_case(kind, torch.bfloat16, 8, 2, 128, [700, 330, 129], 1 if kind == 3 else 150, window=window,
                           drop_pages_behind_window=drop)


# -------------------------------------------------------------------------------------------- gemm
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(1, 256, 64), (5, 384, 96), (37, 331, 80), (64, 224, 96), (130, 100, 36), (3, 17, 5)])
def test_gemm_tiled(dtype, m, n, k):
    torch.manual_seed(m * n + k)
    x, w = torch.randn(m, k).to(dtype), torch.randn(n, k).to(dtype)
    want = x.double() @ w.double().T
    out = torch.empty(m, n, dtype=dtype, device=DEV)
    ops().gemm_tiled(x.to(DEV), w.to(DEV), out)
    close(out, want, dtype, what="gemm_tiled")
    if dtype == torch.bfloat16:
        out32 = torch.empty(m, n, dtype=torch.float32, device=DEV)
        ops().gemm_tiled(x.to(DEV), w.to(DEV), out32)
        close(out32, want, torch.float32, what="gemm_tiled float32 out")


@pytest.mark.parametrize("m", [1, 2, 3, 8, 11, 16])
@pytest.mark.parametrize("n,k", [(2560, 2560), (384, 96), (331, 80), (256, 9728), (48, 136), (17, 8), (100, 1000)])
@pytest.mark.parametrize("group,depth,splits", [(2, 2, 1), (2, 1, 1), (1, 2, 1), (1, 1, 3), (2, 2, 4), (2, 1, 16)])
def test_gemm_stream(m, n, k, group, depth, splits):
    torch.manual_seed(m + n + k)
    x, w = torch.randn(m, k).to(torch.bfloat16), (torch.randn(n, k) / math.sqrt(k)).to(torch.bfloat16)
    want = x.double() @ w.double().T
    o = ops()
    if splits == 1:
        out = torch.empty(m, n, dtype=torch.float32, device=DEV)
        o.gemm_stream_bf16(x.to(DEV), w.to(DEV), out, None, group, 1, depth)
        close(out, want, torch.float32, what="stream float32 out")
        outb = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
        o.gemm_stream_bf16(x.to(DEV), w.to(DEV), outb, None, group, 1, depth)
        close(outb, want, torch.bfloat16, ulps=1.0, what="stream bfloat16 out")
    else:
        parts = torch.full((splits, m, n), float("nan"), dtype=torch.float32, device=DEV)
        o.gemm_stream_bf16(x.to(DEV), w.to(DEV), None, parts, group, splits, depth)
        out = o.sum_partials(parts, torch.empty(m, n, dtype=torch.float32, device=DEV), splits)
        close(out, want, torch.float32, what="stream split-K")


def test_gemm_stream_strided_rows():
    """Activation rows that are a slice of a wider matrix (row stride larger than K)."""
    torch.manual_seed(3)
    wide = torch.randn(5, 3 * 96).to(torch.bfloat16).to(DEV)
    x = wide[:, 96:192]
    w = (torch.randn(200, 96) / 10).to(torch.bfloat16).to(DEV)
    out = torch.empty(5, 200, dtype=torch.float32, device=DEV)
    ops().gemm_stream_bf16(x, w, out, None, 2, 1)
    close(out, x.double().cpu() @ w.double().cpu().T, torch.float32, what="stream strided x")


@pytest.mark.parametrize("m", [1, 5, 8, 16])
@pytest.mark.parametrize("inter,k", [(9728, 2560), (224, 96), (136, 80), (37 * 8, 72)])
@pytest.mark.parametrize("group,depth", [(1, 1), (2, 1), (2, 2), (1, 2)])
def test_gemm_stream_swiglu(m, inter, k, group, depth):
    torch.manual_seed(m + inter)
    x = torch.randn(m, k).to(torch.bfloat16)
    w = (torch.randn(2 * inter, k) * 2 / math.sqrt(k)).to(torch.bfloat16)
    gu = (x.double() @ w.double().T).to(torch.bfloat16).float()            # the unfused path rounds the product first
    want = (torch.nn.functional.silu(gu[:, :inter]).to(torch.bfloat16).float() * gu[:, inter:]).to(torch.bfloat16)
    out = torch.empty(m, inter, dtype=torch.bfloat16, device=DEV)
    ops().gemm_stream_swiglu_bf16(x.to(DEV), w.to(DEV), out, group, depth)
    close(out, want, torch.bfloat16, what="stream swiglu")


@pytest.mark.parametrize("m", [1, 16, 17, 31, 33, 48, 64])
@pytest.mark.parametrize("n,k", [(2560, 2560), (384, 96), (331, 80), (256, 9728), (48, 136), (17, 8), (100, 1000)])
@pytest.mark.parametrize("group,splits", [(2, 1), (1, 1), (2, 3), (1, 4), (2, 16)])
def test_gemm_wide(m, n, k, group, splits):
    torch.manual_seed(m + n + k)
    x, w = torch.randn(m, k).to(torch.bfloat16), (torch.randn(n, k) / math.sqrt(k)).to(torch.bfloat16)
    want = x.double() @ w.double().T
    o = ops()
    depth = 1 + (m + n + splits) % 3                          # groups in flight: every depth meets every shape class
    if splits == 1:
        out = torch.empty(m, n, dtype=torch.float32, device=DEV)
        o.gemm_wide_bf16(x.to(DEV), w.to(DEV), out, None, group, 1, depth)
        close(out, want, torch.float32, what="wide float32 out")
        outb = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
        o.gemm_wide_bf16(x.to(DEV), w.to(DEV), outb, None, group, 1, 1 + depth % 3)
        close(outb, want, torch.bfloat16, ulps=1.0, what="wide bfloat16 out")
    else:
        parts = torch.full((splits, m, n), float("nan"), dtype=torch.float32, device=DEV)
        o.gemm_wide_bf16(x.to(DEV), w.to(DEV), None, parts, group, splits, depth)
        out = o.sum_partials(parts, torch.empty(m, n, dtype=torch.float32, device=DEV), splits)
        close(out, want, torch.float32, what="wide split-K")


@pytest.mark.parametrize("m", [5, 17, 40, 64])
@pytest.mark.parametrize("inter,k", [(9728, 2560), (224, 96), (136, 80), (37 * 8, 72), (40, 64)])
@pytest.mark.parametrize("group", [1, 2])
def test_gemm_wide_swiglu(m, inter, k, group):
    torch.manual_seed(m + inter)
    x = torch.randn(m, k).to(torch.bfloat16)
    w = (torch.randn(2 * inter, k) * 2 / math.sqrt(k)).to(torch.bfloat16)
    gu = (x.double() @ w.double().T).to(torch.bfloat16).float()            # the unfused path rounds the product first
    want = (torch.nn.functional.silu(gu[:, :inter]).to(torch.bfloat16).float() * gu[:, inter:]).to(torch.bfloat16)
    out = torch.empty(m, inter, dtype=torch.bfloat16, device=DEV)
    ops().gemm_wide_swiglu_bf16(x.to(DEV), w.to(DEV), out, group, 1 + (m + inter) % 3)
    close(out, want, torch.bfloat16, what="wide swiglu")


@pytest.mark.parametrize("m", [5, 17, 33, 48, 64])
@pytest.mark.parametrize("inter,k", [(9728, 2560), (224, 128), (136, 384), (37 * 8, 640), (47, 128), (49, 256)])
def test_gemm_panel_swiglu(m, inter, k):
    """Operands straight into LDS: row counts with one to four tiles of 16, output counts that are no multiple of
    the 48 a workgroup owns, one group of K and many; a row of x strided wider than K."""
    torch.manual_seed(m + inter)
    x = torch.randn(m, k).to(torch.bfloat16)
    w = (torch.randn(2 * inter, k) * 2 / math.sqrt(k)).to(torch.bfloat16)
    gu = (x.double() @ w.double().T).to(torch.bfloat16).float()            # the unfused path rounds the product first
    want = (torch.nn.functional.silu(gu[:, :inter]).to(torch.bfloat16).float() * gu[:, inter:]).to(torch.bfloat16)
    out = torch.full((m, inter), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops().gemm_panel_swiglu_bf16(x.to(DEV), w.to(DEV), out)
    close(out, want, torch.bfloat16, what="panel swiglu")
    wide = torch.zeros(m, k + 8, dtype=torch.bfloat16, device=DEV)
    wide[:, :k] = x.to(DEV)
    out2 = torch.full((m, inter), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops().gemm_panel_swiglu_bf16(wide[:, :k], w.to(DEV), out2)
    assert torch.equal(out, out2)
    with pytest.raises(Exception, match="K % 128"):
        ops().gemm_panel_swiglu_bf16(x.to(DEV)[:, :64].contiguous(), w.to(DEV)[:, :64].contiguous(), out)


@pytest.mark.parametrize("m", [1, 65, 100, 128, 129, 200, 256])
@pytest.mark.parametrize("inter,k,tiles", [(9728, 2560, 0), (224, 128, 4), (136, 384, 5), (37 * 8, 640, 6), (47, 64, 7),
                                           (49, 256, 8), (700, 192, 0)])
def test_gemm_tall_swiglu(m, inter, k, tiles):
    """The gate/up product with its activation for up to 256 rows: row counts on both sides of one tile of 16 a wave
    and of two, output counts that are no multiple of 8 or of what a workgroup owns, every count of tiles a workgroup,
    one group of K and many; a row of x strided wider than K."""
    torch.manual_seed(m + inter)
    x = torch.randn(m, k).to(torch.bfloat16)
    w = (torch.randn(2 * inter, k) * 2 / math.sqrt(k)).to(torch.bfloat16)
    gu = (x.double() @ w.double().T).to(torch.bfloat16).float()            # the unfused path rounds the product first
    want = (torch.nn.functional.silu(gu[:, :inter]).to(torch.bfloat16).float() * gu[:, inter:]).to(torch.bfloat16)
    out = torch.full((m, inter), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops().gemm_tall_swiglu_bf16(x.to(DEV), w.to(DEV), out, tiles)
    close(out, want, torch.bfloat16, what="tall swiglu")
    wide = torch.zeros(m, k + 8, dtype=torch.bfloat16, device=DEV)
    wide[:, :k] = x.to(DEV)
    out2 = torch.full((m, inter), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops().gemm_tall_swiglu_bf16(wide[:, :k], w.to(DEV), out2, tiles)
    assert torch.equal(out, out2)


@pytest.mark.parametrize("n_heads,n_kv,head_dim,rows,count", [(8, 2, 128, 200, 4), (3, 1, 64, 64, 1), (4, 4, 32, 130, 3),
                                                                  (2, 1, 256, 97, 2), (8, 2, 128, 5, 2), (4, 2, 64, 33, 6)])
def test_rows_to_cache_from_partial_sums(n_heads, n_kv, head_dim, rows, count):
    """A projection left as float partial sums goes to the cache and to the queries exactly as its rounded sum does:
    the parts are made so that their sums are exact in float32 whatever the order."""
    torch.manual_seed(rows + count)
    o = ops()
    cols = (n_heads + 2 * n_kv) * head_dim
    parts = (torch.randint(-64, 65, (count, rows, cols)).float() / 16).to(DEV)
    whole = parts.sum(0).to(torch.bfloat16)
    n_slots, max_pages = 3, 4
    n_pages = n_slots * max_pages
    table = torch.randperm(n_pages, dtype=torch.int32).view(n_slots, max_pages).to(DEV)
    row_slot = torch.tensor([0] * 70 + [-1] * 5 + [2] * (rows - 75) if rows > 75 else [1] * rows, dtype=torch.int32, device=DEV)
    row_pos = torch.cat([torch.arange(70), torch.zeros(5), torch.arange(3, 3 + rows - 75)]).int().to(DEV) if rows > 75 \
        else torch.arange(5, 5 + rows, dtype=torch.int32, device=DEV)
    cos = torch.randn(256, head_dim // 2, device=DEV).to(torch.bfloat16)
    sin = torch.randn(256, head_dim // 2, device=DEV).to(torch.bfloat16)
    qw, kw = (1 + 0.1 * torch.randn(head_dim, device=DEV)).to(torch.bfloat16), (1 + 0.1 * torch.randn(head_dim, device=DEV)).to(torch.bfloat16)
    got, want = [], []
    for source, into in ((parts, got), (whole, want)):
        k = torch.zeros(n_pages, n_kv, 64, head_dim, dtype=torch.bfloat16, device=DEV)
        v = torch.zeros(n_pages, n_kv, head_dim, 64, dtype=torch.bfloat16, device=DEV)
        q = torch.full((rows, n_heads, head_dim), float("nan"), dtype=torch.bfloat16, device=DEV)
        if source is parts:
            assert o.rows_to_cache_takes(rows, head_dim, head_dim, True)
            o.rows_to_cache_from_partials(parts, qw, kw, 1e-6, cos, sin, head_dim, row_slot, row_pos, q, k, v, table,
                                          n_heads, n_kv, head_dim)
        else:
            o.qk_norm_rope_kv(whole, qw, kw, 1e-6, cos, sin, head_dim, row_slot, row_pos, q, k, v, table, True, n_heads,
                              n_kv, head_dim)
        into.extend([q, k, v])
    for a, b, what in zip(got, want, ("q", "k", "v")):
        assert torch.equal(a, b), what
    assert got[1].any() and got[2].any()
    assert not o.rows_to_cache_takes(rows, 48, 48, True) and not o.rows_to_cache_takes(rows, head_dim, head_dim // 2, True)
    with pytest.raises(Exception, match="a full rotation"):
        o.rows_to_cache_from_partials(parts, qw, kw, 1e-6, cos[:, :head_dim // 4].contiguous(), sin[:, :head_dim // 4].contiguous(),
                                      head_dim // 2, row_slot, row_pos, None, got[1], got[2], table, n_heads, n_kv, head_dim)


@pytest.mark.parametrize("m", [1, 65, 128, 129, 200, 256])
@pytest.mark.parametrize("n,k,splits,tiles", [(2560, 4096, 6, 5), (77, 64, 1, 4), (100, 192, 3, 6), (136, 640, 4, 7),
                                              (64, 1024, 16, 8), (130, 9728, 6, 4), (1000, 1280, 2, 5)])
def test_gemm_tall(m, n, k, splits, tiles):
    """Float partial sums over runs of K by the kernel whose waves own rows of x: row counts on both sides of one tile
    of 16 a wave and of two, output counts that are no multiple of 4 or of what a workgroup owns, every count of tiles,
    runs of one group (shorter than the rings are deep) and of many, of unequal length; every run against the product
    over itself; a row of x strided wider than K."""
    torch.manual_seed(m + n + k)
    o = ops()
    assert o.gemm_mid_splits(k, splits) == splits
    x, w = torch.randn(m, k).to(torch.bfloat16), (torch.randn(n, k) / math.sqrt(k)).to(torch.bfloat16)
    parts = torch.full((splits, m, n), float("nan"), dtype=torch.float32, device=DEV)
    o.gemm_tall_bf16(x.to(DEV), w.to(DEV), parts, splits, tiles)
    groups = k // 64
    per = -(-groups // splits)
    for s in range(splits):
        a, b = 64 * per * s, min(k, 64 * per * (s + 1))
        close(parts[s], x[:, a:b].double() @ w[:, a:b].double().T, torch.float32, what=f"tall, run {s}")
    close(parts.sum(0), x.double() @ w.double().T, torch.float32, what="tall, sum")
    wide = torch.zeros(m, k + 8, dtype=torch.bfloat16, device=DEV)
    wide[:, :k] = x.to(DEV)
    parts2 = torch.full((splits, m, n), float("nan"), dtype=torch.float32, device=DEV)
    o.gemm_tall_bf16(wide[:, :k], w.to(DEV), parts2, splits, tiles)
    assert torch.equal(parts, parts2)


def test_gemm_tall_at_random_sizes():
    """Forty shapes drawn with a fixed seed: any row count up to 256, output counts from 1, K of 1 to 40 groups,
    every tile count, any split that leaves no run empty; both forms of the kernel."""
    import random
    rng = random.Random(7)
    o = ops()
    for case in range(40):
        m, n, groups, tiles = rng.randint(1, 256), rng.randint(1, 700), rng.randint(1, 40), rng.randint(4, 8)
        k = 64 * groups
        splits = o.gemm_mid_splits(k, rng.randint(1, min(groups, 12)))
        torch.manual_seed(case)
        x, w = torch.randn(m, k).to(torch.bfloat16), (torch.randn(n, k) / math.sqrt(k)).to(torch.bfloat16)
        parts = torch.full((splits, m, n), float("nan"), dtype=torch.float32, device=DEV)
        o.gemm_tall_bf16(x.to(DEV), w.to(DEV), parts, splits, tiles)
        close(parts.sum(0), x.double() @ w.double().T, torch.float32, what=f"tall, case {case}: {m}x{n}x{k}, {tiles} tiles, {splits} runs")
        inter = max(1, n // 2)
        w2 = (torch.randn(2 * inter, k) * 2 / math.sqrt(k)).to(torch.bfloat16)
        gu = (x.double() @ w2.double().T).to(torch.bfloat16).float()
        want = (torch.nn.functional.silu(gu[:, :inter]).to(torch.bfloat16).float() * gu[:, inter:]).to(torch.bfloat16)
        out = torch.full((m, inter), float("nan"), dtype=torch.bfloat16, device=DEV)
        o.gemm_tall_swiglu_bf16(x.to(DEV), w2.to(DEV), out, tiles)
        close(out, want, torch.bfloat16, what=f"tall swiglu, case {case}: {m}x{inter}x{k}, {tiles} tiles")


def test_gemm_tall_refuses():
    o = ops()
    w = torch.zeros(64, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(Exception, match="M <= 256"):
        o.gemm_tall_bf16(torch.zeros(257, 128, dtype=torch.bfloat16, device=DEV), w,
                         torch.empty(1, 257, 64, dtype=torch.float32, device=DEV), 1, 4)
    with pytest.raises(Exception, match="leave one empty"):
        o.gemm_tall_bf16(torch.zeros(80, 256, dtype=torch.bfloat16, device=DEV), torch.zeros(64, 256, dtype=torch.bfloat16, device=DEV),
                         torch.empty(3, 80, 64, dtype=torch.float32, device=DEV), 3, 4)
    with pytest.raises(Exception, match="tiles 4 to 8"):
        o.gemm_tall_bf16(torch.zeros(80, 128, dtype=torch.bfloat16, device=DEV), w,
                         torch.empty(1, 80, 64, dtype=torch.float32, device=DEV), 1, 3)


def test_gemm_tall_swiglu_refuses():
    o = ops()
    w = torch.zeros(64, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(Exception, match="M <= 256"):
        o.gemm_tall_swiglu_bf16(torch.zeros(257, 128, dtype=torch.bfloat16, device=DEV), w,
                                torch.empty(257, 32, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(Exception, match="K % 64"):
        o.gemm_tall_swiglu_bf16(torch.zeros(80, 96, dtype=torch.bfloat16, device=DEV), w[:, :96].contiguous(),
                                torch.empty(80, 32, dtype=torch.bfloat16, device=DEV))


@pytest.mark.parametrize("m", [1, 17, 32, 33, 48, 49, 64, 65, 96, 97, 128, 129, 192, 193, 256])
@pytest.mark.parametrize("n,k,splits", [(2560, 4096, 6), (77, 64, 1), (100, 192, 3), (136, 640, 4), (64, 1024, 16),
                                         (130, 9728, 6)])
def test_gemm_mid(m, n, k, splits):
    """Float partial sums over runs of K, operands straight into LDS: row counts around the kernel's three tile
    counts, output counts that are no multiple of 4 or of the 64 a workgroup owns, one group of K and many, runs of
    unequal length; every split against the product over its own run; a row of x strided wider than K."""
    torch.manual_seed(m + n + k)
    o = ops()
    assert o.gemm_mid_splits(k, splits) == splits
    x, w = torch.randn(m, k).to(torch.bfloat16), (torch.randn(n, k) / math.sqrt(k)).to(torch.bfloat16)
    parts = torch.full((splits, m, n), float("nan"), dtype=torch.float32, device=DEV)
    o.gemm_mid_bf16(x.to(DEV), w.to(DEV), parts, splits)
    groups = k // 64
    per = -(-groups // splits)
    for s in range(splits):
        a, b = 64 * per * s, min(k, 64 * per * (s + 1))
        close(parts[s], x[:, a:b].double() @ w[:, a:b].double().T, torch.float32, what=f"mid, split {s}")
    close(parts.sum(0), x.double() @ w.double().T, torch.float32, what="mid, sum")
    wide = torch.zeros(m, k + 8, dtype=torch.bfloat16, device=DEV)
    wide[:, :k] = x.to(DEV)
    parts2 = torch.full((splits, m, n), float("nan"), dtype=torch.float32, device=DEV)
    o.gemm_mid_bf16(wide[:, :k], w.to(DEV), parts2, splits)
    assert torch.equal(parts, parts2)


def test_gemm_mid_refuses():
    o = ops()
    x, w = torch.zeros(257, 128, dtype=torch.bfloat16, device=DEV), torch.zeros(64, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(Exception, match="M <= 256"):
        o.gemm_mid_bf16(x, w, torch.empty(1, 257, 64, device=DEV), 1)
    with pytest.raises(Exception, match="K % 64"):
        o.gemm_mid_bf16(x[:100, :96].contiguous(), w[:, :96].contiguous(), torch.empty(1, 100, 64, device=DEV), 1)
    assert o.gemm_mid_splits(5 * 64, 4) == 3                  # four runs of two groups would leave the last one empty
    with pytest.raises(Exception, match="empty"):
        o.gemm_mid_bf16(x[:100, :64].contiguous().repeat(1, 5), w[:, :64].contiguous().repeat(1, 5),
                        torch.empty(4, 100, 64, device=DEV), 4)
    with pytest.raises(Exception, match="partials must be"):
        o.gemm_mid_bf16(x[:100], w, torch.empty(1, 100, 64, device=DEV), 2)


@pytest.mark.parametrize("m,n,k", [(130, 331, 72), (1, 17, 8), (257, 128, 64), (300, 100, 1000), (128, 129, 136),
                                   (513, 2560, 2560), (64, 64, 9728)])
@pytest.mark.parametrize("shape", [0, 1])
def test_gemm_block(m, n, k, shape):
    torch.manual_seed(m + n + k)
    x, w = torch.randn(m, k).to(torch.bfloat16), (torch.randn(n, k) / math.sqrt(k)).to(torch.bfloat16)
    want = x.double() @ w.double().T
    o = ops()
    out = o.gemm_block_bf16(x.to(DEV), w.to(DEV), torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV), shape=shape)
    close(out, want, torch.float32, what="block float32 out")
    outb = o.gemm_block_bf16(x.to(DEV), w.to(DEV), torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV), shape=shape)
    close(outb, want, torch.bfloat16, ulps=1.0, what="block bfloat16 out")
    wide = torch.randn(m, k + 24).to(torch.bfloat16).to(DEV)               # rows that are not contiguous
    got = o.gemm_block_bf16(wide[:, :k], w.to(DEV), torch.empty(m, n, dtype=torch.float32, device=DEV))
    close(got, wide[:, :k].cpu().double() @ w.double().T, torch.float32, what="block strided rows")


@pytest.mark.parametrize("m,inter,k", [(200, 224, 96), (129, 40, 64), (70, 37 * 8, 72), (300, 9728, 256)])
@pytest.mark.parametrize("shape", [0, 1])
def test_gemm_block_swiglu(m, inter, k, shape):
    torch.manual_seed(m + inter)
    x = torch.randn(m, k).to(torch.bfloat16)
    w = (torch.randn(2 * inter, k) * 2 / math.sqrt(k)).to(torch.bfloat16)
    gu = (x.double() @ w.double().T).to(torch.bfloat16).float()            # the unfused path rounds the product first
    want = (torch.nn.functional.silu(gu[:, :inter]).to(torch.bfloat16).float() * gu[:, inter:]).to(torch.bfloat16)
    out = ops().gemm_block_bf16(x.to(DEV), w.to(DEV), torch.empty(m, inter, dtype=torch.bfloat16, device=DEV), swiglu=True,
                                shape=shape)
    close(out, want, torch.bfloat16, what="block swiglu")


@pytest.mark.parametrize("m,n,k", [(130, 331, 72), (1, 17, 4), (257, 128, 64), (300, 100, 1000), (128, 129, 136),
                                   (513, 700, 2560)])
@pytest.mark.parametrize("shape", [0, 1])
def test_gemm_block_f32(m, n, k, shape):
    torch.manual_seed(m + n + k)
    x, w = torch.randn(m, k), torch.randn(n, k) / math.sqrt(k)
    out = ops().gemm_block_f32(x.to(DEV), w.to(DEV), torch.full((m, n), float("nan"), device=DEV), shape=shape)
    close(out, x.double() @ w.double().T, torch.float32, what="block float32")
    wide = torch.randn(m, k + 12).to(DEV)                                  # rows that are not contiguous
    got = ops().gemm_block_f32(wide[:, :k], w.to(DEV), torch.empty(m, n, device=DEV), shape=shape)
    close(got, wide[:, :k].cpu().double() @ w.double().T, torch.float32, what="block float32 strided rows")


@pytest.mark.parametrize("m", [1, 2, 3, 5, 8, 11, 16])
@pytest.mark.parametrize("n,k", [(17, 4), (331, 72), (100, 1000), (129, 260), (64, 2560), (2560, 256)])
def test_gemm_rows_f32(m, n, k):
    torch.manual_seed(m + n + k)
    x, w = torch.randn(m, k), torch.randn(n, k) / math.sqrt(k)
    out = ops().gemm_rows_f32(x.to(DEV), w.to(DEV), torch.full((m, n), float("nan"), device=DEV))
    close(out, x.double() @ w.double().T, torch.float32, what="rows float32")
    wide = torch.randn(m, k + 3).to(DEV)                                   # rows of a wider matrix, not even aligned
    got = ops().gemm_rows_f32(wide[:, :k], w.to(DEV), torch.empty(m, n, device=DEV))
    close(got, wide[:, :k].cpu().double() @ w.double().T, torch.float32, what="rows float32 strided rows")


def test_linear_dispatch_matches_everywhere():
    """The same product through every route the linear helper can take."""
    from dryft_amd.parts.linear import linear
    from dryft_amd.parts.base import Partials
    torch.manual_seed(5)
    for n, k in ((384, 96), (100, 2560), (331, 72)):           # 331 outputs: no size the vendor library takes
        w = (torch.randn(n, k) / math.sqrt(k)).to(torch.bfloat16).to(DEV)
        for m in (1, 7, 16, 17, 32, 33, 40, 64, 65, 130, 256, 257, 300):
            x = torch.randn(m, k).to(torch.bfloat16).to(DEV)
            want = x.double().cpu() @ w.double().cpu().T
            close(linear(x, w), want, torch.bfloat16, ulps=1.0, what=f"linear m={m}")
            close(linear(x, w, out_dtype=torch.float32), want, torch.float32, what=f"linear m={m} float32 out")
            got = linear(x, w, allow_partials=True)
            if isinstance(got, Partials):
                assert got.count > 1 and (m <= 64 or (m <= 256 and k % 64 == 0))
                got = got.data[: got.count].sum(0)
            close(got, want, torch.bfloat16, ulps=1.0, what=f"linear partials m={m}")
            close(linear(x.float(), w.float()), want, torch.float32, what=f"linear float32 m={m}")
        strided = torch.randn(5, 3 * k).to(torch.bfloat16).to(DEV)[:, k:2 * k]     # rows of a wider matrix
        close(linear(strided, w), strided.double().cpu() @ w.double().cpu().T, torch.bfloat16, ulps=1.0, what="strided rows")


# ---------------------------------------------------------------------------------------- sampling
def test_argmax_rows_ties_to_lowest_index():
    torch.manual_seed(0)
    logits = torch.randn(5, 151936)
    logits[0, 777] = logits[0, 150000] = 50.0
    logits[1, 151935] = 60.0
    logits[2, 0] = 60.0
    logits[3, :] = 1.0
    out = torch.empty(5, dtype=torch.int32, device=DEV)
    ops().argmax_rows(logits.to(DEV), out)
    assert out.tolist() == [777, 151935, 0, 0, int(torch.argmax(logits[4]))]


@pytest.mark.parametrize("vocab", [331, 9001, 151936])        # one workgroup a row; few stretches; many
def test_sample_rows_follows_inverse_cdf(vocab):
    torch.manual_seed(1)
    rows, temperature = 64, 0.8
    logits = 3 * torch.randn(rows, vocab)
    u = torch.rand(rows)
    u[0], u[1] = 0.0, 0.999999
    logits[2, vocab - vocab // 3:] = -float("inf")            # whole stretches without weight at the end,
    logits[3, :vocab // 2] = -float("inf")                    # and at the start
    u[2], u[3] = 0.9999999, 0.0
    logits[4, :] = -30.0                                      # one token holds nearly everything, far into the row
    logits[4, (2 * vocab) // 3 + 5] = 40.0
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    ops().sample_rows(logits.to(DEV), temperature, u.to(DEV), out)
    p = torch.softmax(logits.double() / temperature, -1)
    cdf = torch.cumsum(p, -1)
    # The kernel adds float32 terms (exp within a few units in the last place) in its own order, so its running
    # sums stand within a few 1e-7 of the exact ones, relative to a total of 1: a token is right if it answers
    # the inverse-CDF question for some draw within 2e-6 of the given one. (Where the draw falls among tail
    # tokens of probability 1e-8, several neighbours are right.)
    tol = 2e-6
    exact = 0
    for r, tok in enumerate(out.tolist()):
        want = min(int(torch.searchsorted(cdf[r], u[r].double(), right=True)), vocab - 1)
        exact += tok == want
        assert float(p[r, tok]) > 0, f"row {r}: token {tok} has no weight"
        assert float(cdf[r, tok]) > float(u[r]) - tol, f"row {r}: got {tok}, want {want}"
        assert tok == 0 or float(cdf[r, tok - 1]) <= float(u[r]) + tol, f"row {r}: got {tok}, want {want}"
    assert exact >= rows - 4


# ------------------------------------------------------------------------------------------- batch
def test_prepare_batch():
    o = ops()
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    lengths = i32([0, 10, 64, 7, 0, 3])
    seq_slot, q_len = i32([3, -1, 1, 5]), i32([70, 1, 1, 130])
    n_seqs, n_rows = 4, 202
    z = lambda n: torch.full((n,), -7, dtype=torch.int32, device=DEV)
    cu, tiles, kv, start, rseq, rslot, rpos = z(5), z(5), z(4), z(4), z(n_rows), z(n_rows), z(n_rows)
    o.prepare_batch(seq_slot, q_len, lengths, n_seqs, n_rows, cu, kv, start, rseq, rslot, rpos)
    assert cu.tolist() == [0, 70, 71, 72, 202]
    o.tile_prefix(seq_slot, q_len, n_seqs, 64, tiles)
    assert tiles.tolist() == [0, 2, 2, 3, 6]
    o.tile_prefix(seq_slot, q_len, n_seqs, 16, tiles)
    assert tiles.tolist() == [0, 5, 5, 6, 15]
    assert kv.tolist() == [77, 0, 11, 133]
    assert start.tolist() == [7, 0, 10, 3]
    assert lengths.tolist() == [0, 11, 64, 77, 0, 133]
    assert rseq.tolist() == [0] * 70 + [1] + [2] + [3] * 130
    assert rslot.tolist() == [3] * 70 + [-1] + [1] + [5] * 130
    assert rpos.tolist() == list(range(7, 77)) + [0] + [10] + list(range(3, 133))


@pytest.mark.parametrize("n_seqs", [1, 64, 255, 256, 257, 1000])
def test_prepare_batch_many_sequences(n_seqs):
    """More sequences than the kernel has threads: every thread sums a run of them; against plain prefix sums."""
    o = ops()
    rng = np.random.default_rng(n_seqs)
    q = rng.integers(1, 200, size=n_seqs)
    q[rng.random(n_seqs) < 0.5] = 1
    slots = rng.permutation(n_seqs + 5)[:n_seqs]
    slots[rng.random(n_seqs) < 0.2] = -1
    past = rng.integers(0, 500, size=n_seqs + 5)
    i32 = lambda x: torch.tensor(np.asarray(x), dtype=torch.int32, device=DEV)
    lengths, seq_slot, q_len = i32(past), i32(slots), i32(q)
    n_rows = int(q.sum())
    z = lambda n: torch.full((n,), -7, dtype=torch.int32, device=DEV)
    cu, tiles, kv, start = z(n_seqs + 1), z(n_seqs + 1), z(n_seqs), z(n_seqs)
    rseq, rslot, rpos = z(n_rows), z(n_rows), z(n_rows)
    o.prepare_batch(seq_slot, q_len, lengths, n_seqs, n_rows, cu, kv, start, rseq, rslot, rpos)
    live = slots >= 0
    want_start = np.where(live, past[np.maximum(slots, 0)], 0)
    assert cu.tolist() == [0] + np.cumsum(q).tolist()
    for tile_rows in (64, 48):
        o.tile_prefix(seq_slot, q_len, n_seqs, tile_rows, tiles)
        assert tiles.tolist() == [0] + np.cumsum(np.where(live, (q + tile_rows - 1) // tile_rows, 0)).tolist()
    assert start.tolist() == want_start.tolist()
    assert kv.tolist() == (want_start + np.where(live, q, 0)).tolist()
    new_len = past.copy()
    new_len[slots[live]] += q[live]
    assert lengths.tolist() == new_len.tolist()
    seq_of_row = np.repeat(np.arange(n_seqs), q)
    assert rseq.tolist() == seq_of_row.tolist()
    assert rslot.tolist() == slots[seq_of_row].tolist()
    within = np.arange(n_rows) - np.repeat(np.cumsum(q) - q, q)
    assert rpos.tolist() == np.where(live[seq_of_row], want_start[seq_of_row] + within, 0).tolist()


@pytest.mark.parametrize("D", list(range(16, 257, 16)))
def test_attention_kernels_take_every_head_size_in_steps_of_16(D):
    """Every head size a configuration may have in steps of 16, up to 256, through the three bfloat16 matrix-core
    kernels and the plain one: a prompt that continues cached tokens, and one row per sequence with and without
    splits. Three query heads to a kv head, lengths that end inside a page."""
    for kind, tq in (("causal1", 70), ("causal0", 200), ("rows", 33), (1, 1), (3, 1)):
        run_attention_case(kind, torch.bfloat16, 6, 2, D, [200, 70, 131], tq)
    if D <= 128:
        run_attention_case("causal3", torch.bfloat16, 6, 2, D, [200, 70, 131], 200)
        run_attention_case("causal2", torch.bfloat16, 8, 2, D, [200, 70, 131], 200)
    else:                                           # 32 rows or two heads a wave hold head sizes up to 128 only
        for mode in (2, 3):
            with pytest.raises(Exception, match="refuses these sizes"):
                run_attention_case(f"causal{mode}", torch.bfloat16, 8, 2, D, [200, 70, 131], 200)


@pytest.mark.parametrize("D", [8, 24, 40, 72, 100, 250])
def test_plain_attention_takes_head_sizes_the_matrix_cores_do_not(D):
    for dtype in DTYPES:
        run_attention_case("rows", dtype, 6, 2, D, [200, 70, 131], 33)
    with pytest.raises(Exception, match="refuses these sizes"):
        run_attention_case("causal0", torch.bfloat16, 6, 2, D, [200, 70, 131], 70)
    with pytest.raises(Exception, match="refuses these sizes"):
        run_attention_case(2, torch.bfloat16, 6, 2, D, [200, 70, 131], 1)
