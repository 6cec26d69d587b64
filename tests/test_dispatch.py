"""Which matrix-product kernel a shape goes to, decided on the host: checked here with tensors that have shapes but
no storage."""

import torch


def fake(rows, cols, dtype=torch.bfloat16):
    return torch.empty((rows, cols), dtype=dtype, device="meta")


def test_operands_beyond_32_bit_offsets_stay_away_from_the_direct_to_lds_kernels():
    """The kernels that bring their operands straight into LDS address them by 32-bit byte offsets and refuse more;
    the dispatch must not send them such operands (every step of up to 64 or 256 rows would fail)."""
    from dryft_amd.csrc import ops
    from dryft_amd.parts.linear import panel_swiglu_ok, within_direct_reach
    x = fake(8, 16384)
    assert panel_swiglu_ok(x, fake(2 * 25600, 16384))                  # 1.7 GB: within reach
    big = fake(2 * 70000, 16384)                                       # 4.6 GB of weights
    assert big.numel() * 2 >= ops.DIRECT_REACH
    assert not panel_swiglu_ok(x, big) and not within_direct_reach(x, big)
    assert within_direct_reach(fake(256, 16384), fake(5120, 16384))
    wide_rows = torch.empty((200, 16), dtype=torch.bfloat16, device="meta").as_strided((200, 16), (1 << 24, 1))
    assert not within_direct_reach(wide_rows, fake(64, 16))            # rows 32 MB apart: the activations are out of reach


def test_plans_split_k_only_where_partial_sums_are_taken():
    from dryft_amd.parts.linear import small_mid_plan, stream_plan, tall_plan, wide_plan
    # 33 to 64 rows: one workgroup of 64 outputs a compute unit, and no run of K left empty
    assert small_mid_plan(6144, 2560) == 2 and small_mid_plan(2560, 4096) == 6 and small_mid_plan(2560, 9728) == 6
    assert small_mid_plan(5120, 25600) == 1 and small_mid_plan(64, 64) == 1          # beyond 48 MiB; one group of K
    assert stream_plan(6144, 2560, may_split=False)[0] == 1
    assert stream_plan(2560, 9728, may_split=True)[0] > 1
    assert wide_plan(6144, 2560, may_split=False)[0] == 1
    assert wide_plan(2560, 4096, may_split=True)[0] > 1
    # 65 to 256 rows: a split that leaves no run of K empty, tile counts the kernel has, about one workgroup a
    # compute unit where the shape allows it; a single group of K cannot be split
    from dryft_amd.csrc import ops
    for n, k in ((6144, 2560), (2560, 9728), (5120, 17408), (1024, 2048), (80, 64), (100, 192)):
        for m in (65, 128, 129, 256):
            tiles, splits = tall_plan(m, n, k)
            assert 4 <= tiles <= 8 and ops.gemm_mid_splits(k, splits) == splits
    assert tall_plan(256, 80, 64) == (4, 1)
    tiles, splits = tall_plan(256, 2560, 9728)
    assert 200 <= -(-2560 // (16 * tiles)) * splits <= 256


def test_gate_up_kernel_by_rows_and_size():
    from dryft_amd.parts.linear import panel_swiglu_ok, tall_swiglu_ok
    fake = lambda rows, cols: torch.empty((rows, cols), dtype=torch.bfloat16, device="meta")
    w = fake(2 * 9728, 2560)
    assert panel_swiglu_ok(fake(64, 2560), w) and not tall_swiglu_ok(fake(64, 2560), w)
    assert tall_swiglu_ok(fake(65, 2560), w) and tall_swiglu_ok(fake(256, 2560), w) and not tall_swiglu_ok(fake(257, 2560), w)
    assert not tall_swiglu_ok(fake(128, 5120), fake(2 * 17408, 5120))           # beyond 256 MiB: the vendor library
    assert not tall_swiglu_ok(fake(128, 2592), fake(512, 2592))                 # K no multiple of 64


def test_every_entry_point_is_called_with_as_many_arguments_as_it_declares():
    """The table of ctypes signatures against the ``extern "C"`` declarations in the HIP sources: every entry point the
    Python side calls exists in its library's source and takes as many arguments as the table lists."""
    import os
    import re

    from dryft_amd.csrc import ops
    folder = os.path.dirname(os.path.abspath(ops.__file__))
    for module, functions in ops._SIGNATURES.items():
        with open(os.path.join(folder, module + ".hip")) as f:
            text = f.read()
        declared = {m.group(1): m.group(2) for m in re.finditer(r"DRYFT_API\s+\w+\s+(\w+)\s*\(([^)]*)\)", text)}
        for name, signature in functions.items():
            assert name in declared, f"{module}.hip declares no {name}"
            count = len([a for a in declared[name].split(",") if a.strip()])
            assert count == len(signature), f"{name}: declared with {count} arguments, called with {len(signature)}"
