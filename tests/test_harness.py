"""The restated caller side (tests/harness.py) against the closed forms the reference states for it:
core/python/crit_plugins/device.py:586-633 (StepBatch) and inference/attention-state/code/device_attention.py:123-152
(Windows.launches), 428-440 (the step's split), 847-863 (launch width), 1077-1105 (_windows_of)."""
import math

import pytest
import torch

from tests import harness


def test_a_step_batch_packs_its_rows_tokens_in_order():
    rows = [("a", 10, 1), ("b", 0, 5), ("c", 7, 2)]
    batch = harness.StepBatch.build(rows)
    assert (batch.rows, batch.tokens) == (3, 8)
    assert batch.starts == [0, 1, 6, 8] and batch.positions == [10, 0, 1, 2, 3, 4, 7, 8]
    assert batch.starts_t.dtype == torch.int32 and batch.positions_t.dtype == torch.int64 and batch.rows_t.dtype == torch.int64
    assert batch.rows_t.tolist() == [0, 1, 1, 1, 1, 1, 2, 2]
    # row(r): (sequence, first token, count, first position)
    assert [batch.row(r) for r in range(3)] == [("a", 0, 1, 10), ("b", 1, 5, 0), ("c", 6, 2, 7)]
    for bad in ([("a", 0, 0)], [("a", -1, 1)]):
        with pytest.raises(ValueError):
            harness.StepBatch.build(bad)


def _pool(page=16, window=16, lengths=(5, 16, 17, 300, 1000), dump=999):
    tables, at = {}, 0
    for s, n in enumerate(lengths):
        held = math.ceil(n / page)
        tables[s] = list(range(at + 100, at + 100 + held))
        at += held
    pages = (torch.zeros(1, page, 2, 8), torch.zeros(1, page, 2, 8))
    return harness.PoolView("bf16", page, dump, window, tables, pages)


def test_window_rows_tables_are_cut_at_their_positions_and_padded_with_the_dump_page_in_sixteens():
    pool = _pool()
    # (sequence, first token, count, first position)
    rows = [(0, 0, 1, 4), (1, 1, 3, 13), (3, 4, 2, 250), (2, 6, 1, 16), (4, 7, 5, 995)]
    meta = harness.windows_of(pool, rows, "cpu")
    assert meta.tables.dtype == torch.int32 and meta.tables.shape == (5, 64)      # ceil(1000 / 16) = 63 -> 64
    for i, (s, _, count, position) in enumerate(rows):
        held = math.ceil((position + count) / pool.page)
        assert meta.tables[i, :held].tolist() == pool.table(s)[:held]
        assert meta.tables[i, held:].eq(pool.dump).all()
    assert meta.rows.tolist() == [0, 1, 2, 3, 4] and meta.rows.dtype == torch.int32
    assert meta.starts.tolist() == [0, 1, 4, 6, 7] and meta.counts.tolist() == [1, 3, 2, 1, 5]
    assert meta.firsts.tolist() == [4, 13, 250, 16, 995] and meta.firsts.dtype == torch.int64
    assert meta.offsets.tolist() == [0, 1, 4, 6, 7] and (meta.bounds, meta.total) == ([1, 3, 2, 1, 5], 12)
    assert meta.columns == 8      # the widest row's next power of two
    for widest, columns in ((1, 1), (2, 2), (3, 4), (16, 16), (17, 32), (33, 64)):
        assert harness.windows_of(pool, [(4, 0, widest, 0)], "cpu").columns == columns
    # short rows only: one width of sixteen pages
    assert harness.windows_of(pool, rows[:2], "cpu").tables.shape == (2, 16)


def test_launches_cut_the_rows_where_the_partials_run_out():
    pool = _pool()
    counts = [1, 3, 2, 1, 5, 4]
    rows = [(4, sum(counts[:i]), c, 100 + i) for i, c in enumerate(counts)]
    meta = harness.windows_of(pool, rows, "cpu")
    assert meta.launches(None) == [(slice(0, 6), 16)]
    assert meta.launches(16) == [(slice(0, 6), 16)]
    for capacity in (5, 6, 7, 9, 15):
        cuts = meta.launches(capacity)
        assert [c.start for c, _ in cuts] == [0] + [c.stop for c, _ in cuts[:-1]] and cuts[-1][0].stop == 6
        for cut, total in cuts:
            assert total == sum(counts[cut]) <= capacity
            if cut.stop < 6:      # greedy: the next row did not fit
                assert total + counts[cut.stop] > capacity
    with pytest.raises(ValueError):      # (the reference checks the launch's first row only where the rows begin)
        meta.launches(0)
    # rows laid out by columns (no offsets): capacity // columns rows a launch
    plain = harness.Windows(meta.tables, meta.rows, meta.starts, None, meta.firsts, 8)
    assert plain.launches(None) == [(slice(0, 6), None)]
    assert plain.launches(20) == [(slice(0, 2), None), (slice(2, 4), None), (slice(4, 6), None)]
    with pytest.raises(ValueError):
        plain.launches(7)


def test_a_steps_rows_split_by_the_pools_window_and_packed_rows_take_their_tiles_width():
    import crit_amd.paged_kv_attention as pk
    pool = _pool(window=16)
    batch = harness.StepBatch.build([(0, 4, 1), (3, 0, 300), (1, 0, 16), (4, 100, 17), (2, 16, 1)])
    assert harness.split(pool, batch) == ([0, 2, 4], [1, 3])
    meta = harness.windows_of(pool, [batch.row(r) for r in (0, 2, 4)], "cpu")
    for heads in (2, 8, 16):
        group = heads // pool.kv_heads
        rows = pk.tile_for(meta.columns, group, (9, 4), False)[0]
        assert harness.launch_columns(pk, heads, pool, meta) == min(64, max(16, rows // group))
    plain = harness.Windows(meta.tables, meta.rows, meta.starts, None, meta.firsts, 4)
    assert harness.launch_columns(pk, 8, pool, plain) == 4
