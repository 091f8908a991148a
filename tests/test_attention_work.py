"""The host side of the block attention kernel: work items dealt to blocks."""
from types import SimpleNamespace

import pytest


def _batch(entries):
    cu = [0]
    for _, n in entries:
        cu.append(cu[-1] + n)
    return SimpleNamespace(host_cu_tokens=cu, host_start_pos=[p for p, _ in entries])


def _slices(P, n, G, c0, cols, window):
    ncols = n * G
    first, last = P + c0 // G, P + (min(c0 + cols, ncols) - 1) // G
    lo = max(0, first - window + 1) if window > 0 else 0
    return last // 32 - lo // 32 + 1


@pytest.mark.parametrize("window", [0, 300])
@pytest.mark.parametrize("bins", [1, 3, 32, 500])
def test_every_item_once_and_even_loads(bins, window):
    from tffinfer_amd.kernels.ops import _attention_block_work
    entries = [(0, 2048), (333, 200), (5, 1), (1000, 130), (0, 37)]
    G, cols = 4, 128
    batch = _batch(entries)
    items, starts, blocks, groups = _attention_block_work(batch, G, 8, window, "cpu", cols, bins=bins)
    assert groups in (1, 2)
    items, starts = items.tolist(), starts.tolist()
    want = sorted((r, c0) for r, (P, n) in enumerate(entries) for c0 in range(0, n * G, cols))
    assert sorted(map(tuple, items)) == want                      # no item lost, none twice
    assert blocks == len(starts) - 1 == min(bins, len(want))
    assert starts[0] == 0 and starts[-1] == len(items) and all(a < b for a, b in zip(starts, starts[1:]))
    loads = []
    for b in range(blocks):
        loads.append(sum(_slices(*entries[r], G, c0, cols, window) for r, c0 in items[starts[b]:starts[b + 1]]))
    biggest = max(_slices(*entries[r], G, c0, cols, window) for r, c0 in want)
    # longest-first dealing: no block carries more than the mean plus one item
    assert max(loads) <= sum(loads) / blocks + biggest
    if blocks == len(want):
        assert loads == sorted(loads, reverse=True)              # one item each, the longest first


def test_entry_filters():
    from tffinfer_amd.kernels.ops import _attention_block_work, _attention_work, _entries
    batch = _batch([(900, 1), (0, 300), (40, 1), (333, 150)])
    assert _entries(batch, "single") == [0, 2] and _entries(batch, "multi") == [1, 3]
    items, starts, blocks, _ = _attention_block_work(batch, 4, 2, 0, "cpu", 128, bins=64, which="multi")
    assert {r for r, _ in items.tolist()} == {1, 3}
    single = _attention_work(batch, 20, 16, "cpu", "single").tolist()     # 20 heads to a kv head: two tiles
    assert single == [[0, 0], [0, 16], [2, 0], [2, 16]]


def test_key_groups_and_blocks_follow_the_amount_of_work():
    """Little work: one block a CU, two groups of waves in it that share an item's slices; plenty:
    two blocks of one group a CU; large heads always one group, one block a CU."""
    from tffinfer_amd.kernels.ops import _attention_block_work
    short, long_ = _batch([(0, 2048)]), _batch([(0, 8192)])
    _, _, blocks, groups = _attention_block_work(short, 4, 8, 0, "cpu", num_cus=256)
    assert (blocks, groups) == (32, 2)
    _, _, blocks, groups = _attention_block_work(long_, 4, 8, 0, "cpu", num_cus=256)
    assert (blocks, groups) == (64, 1)
    _, _, blocks, groups = _attention_block_work(long_, 4, 8, 0, "cpu", num_cus=256, head_dim=256)
    assert (blocks, groups) == (32, 1)
    _, _, blocks, groups = _attention_block_work(long_, 4, 8, 0, "cpu", num_cus=256, key_groups=2)
    assert (blocks, groups) == (32, 2)
    # a portion of 2,048 tokens late in a long context is plenty of work as well
    _, _, blocks, groups = _attention_block_work(_batch([(6144, 2048)]), 4, 8, 0, "cpu", num_cus=256)
    assert (blocks, groups) == (64, 1)


def test_staged_tables_keep_shape_and_type_on_the_host():
    """The staging module's host form (what the work lists' tests above go through): every
    column comes back as a tensor of its own shape and element type, a copy of the array."""
    import numpy as np
    import torch
    from tffinfer_amd.kernels import staging
    a = np.arange(12, dtype=np.int32).reshape(-1, 2)
    b = np.asarray([0.5, 1.5, -2.0], dtype=np.float32)
    c = np.zeros((0, 2), dtype=np.int32)
    ta, tb, tc = staging.send("cpu", [a, b, c])
    assert ta.dtype == torch.int32 and tuple(ta.shape) == (6, 2) and ta.tolist() == a.tolist()
    assert tb.dtype == torch.float32 and tb.tolist() == b.tolist() and tuple(tc.shape) == (0, 2)
    a[0, 0] = 99
    assert ta[0, 0] == 0
