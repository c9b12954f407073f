"""The host-side choices of the attention kernels' shapes: pure functions of
the step's sizes, checked for their invariants (what a kernel's launch
assumes) and for the measured cases their docstrings name."""

import pytest

from nnis_amd.kernels.ops import PREFILL_CLASS_LENGTH, decode_plan, prefill_plan_class, prefill_tile_items


@pytest.mark.parametrize("batch", [1, 2, 8, 33, 64, 256])
@pytest.mark.parametrize("kv_heads", [1, 3, 8, 32])
@pytest.mark.parametrize("longest", [1, 63, 64, 65, 600, 1100, 2048, 8191])
@pytest.mark.parametrize("width", [0, 576, 2048, 4096])
def test_decode_plan_invariants(batch, kv_heads, longest, width):
    splits, waves = decode_plan(batch, kv_heads, longest, max_waves=4, width=width)
    pages = (longest + 63) // 64
    for n in (splits, waves):
        assert n >= 1 and n & (n - 1) == 0  # powers of two
    assert waves <= 4 and waves <= max(1, pages)  # no wave without a page
    assert splits <= 8
    if pages <= 8:
        assert splits == 1  # short sequences are never cut into runs
    if splits > 1:
        assert batch * kv_heads * waves * splits <= 2048  # runs only while the chip has room for their blocks
    assert decode_plan(batch, kv_heads, longest, max_waves=1, width=width)[1] == 1


def test_decode_plan_measured_cases():
    assert decode_plan(8, 3, 2048, width=576) == (8, 4)      # a narrow model: a page or two a wave
    assert decode_plan(64, 3, 2048, width=576) == (1, 4)     # no room for runs
    assert decode_plan(16, 32, 2048, width=2048) == (1, 4)
    assert decode_plan(64, 32, 2048, width=2048) == (1, 2)   # four and more blocks a compute unit: two waves a block
    assert decode_plan(8, 3, 64, width=576) == (1, 1)


def test_prefill_plan_class_and_work_lists():
    assert [prefill_plan_class(n) for n in (1, 127, 128, 511, 512, 1023, 1024, 1279, 1280, 5000)] == [0, 0, 1, 1, 2, 2, 3, 3, 4, 4]
    for plan_class, least in enumerate(PREFILL_CLASS_LENGTH):
        assert prefill_plan_class(least) == plan_class
    # every row of every sequence lies in exactly one tile; longest tiles (by the keys they read) first
    counts, first = [37, 5, 70, 1], [0, 100, 3, 64]
    for rows in (16, 32, 64):
        seqs, row0s = prefill_tile_items(counts, first, rows)
        seen = sorted((s, r) for s, r in zip(seqs, row0s))
        assert seen == sorted((s, r) for s, n in enumerate(counts) for r in range(0, n, rows))
        ends = [first[s] + min(r + rows, counts[s]) for s, r in zip(seqs, row0s)]
        assert ends == sorted(ends, reverse=True)


def test_prefill_plan_by_class_and_size():
    from nnis_amd.engine.graph import prompt_rows as prefill_rows
    from nnis_amd.kernels import ops

    def prefill_plan(longest, rows, *sizes):
        return ops.prefill_plan(longest, prefill_rows(rows), *sizes)  # (the engine plans for a step's rows rounded up)

    assert [prefill_rows(n) for n in (1, 64, 65, 1024, 1025, 2048, 2049, 4000)] == [64, 64, 128, 1024, 1152, 2048, 2304, 4096]
    for n in (1, 64, 100, 1000, 1100, 2000, 3000):
        assert prefill_rows(prefill_rows(n)) == prefill_rows(n)  # a step replayed from a graph's rows plans as the step launched
    assert prefill_plan(100, 100, 9) == (1, 0)
    assert prefill_plan(300, 300, 9) == (2, 1)
    assert prefill_plan(700, 700, 9) == (4, 2)
    assert prefill_plan(1024, 1024, 32) == (4, 2) and prefill_plan(1024, 1024, 9) == (8, 0)
    assert prefill_plan(1024, 1900, 32) == (4, 2) and prefill_plan(1024, 2000, 33, 64, 11) == (8, 0)  # items enough: the widest tiles
    assert prefill_plan(600, 4000, 36, 64, 12) == (4, 0)
    assert prefill_plan(2048, 2048, 9) == (8, 0) and prefill_plan(1300, 1300, 32) == (4, 0)
    assert prefill_plan(2048, 2048, 16) == (8, 0)  # few items of four columns: 8 waves deal an item's keys
    # items for twice the chip's waves: one wave an item (64 rows x heads an item up to 64 channels, 32 up to 128)
    assert prefill_plan(8192, 8192, 32) == (1, 0) and prefill_plan(8192, 8192, 9, 64, 3) == (8, 0)
    # half of that: one wave an item of two columns, where two divide the group
    assert prefill_plan(4096, 4096, 32) == (1, 2) and prefill_plan(2048, 2048, 64, 64, 8) == (1, 2) and prefill_plan(4096, 4096, 36, 64, 12) == (8, 0)
    assert prefill_plan(2048, 2048, 32) == (4, 0)
    assert prefill_plan(4096, 4096, 32, 128) == (1, 0) and prefill_plan(2048, 2048, 32, 128) == (8, 0) and prefill_plan(2048, 2048, 16, 128) == (8, 0)
    assert prefill_plan(600, 34000, 32) == (1, 0) and prefill_plan(1024, 1024, 32, 256) == (1, 0) and prefill_plan(1024, 1024, 32, 128) == (4, 2)
    # a group of 3 heads: items of three columns (no two-column plans), one wave an item from twice the chip's waves of them
    assert prefill_plan(8192, 8192, 24, 64, 8) == (1, 0) and prefill_plan(1216, 1216, 24, 64, 8) == (4, 0)
    assert prefill_plan(3072, 3072, 32, 64, 32) == (4, 0)
