"""The pool's device-side bookkeeping on the GPU against the CPU oracle, bit for bit: slots of positions through bound
page tables, the move of an accepted draft-tree path's rows, copies of whole pages; and a decode step (slots -> append
-> attention) captured once and replayed as the sequences grow. Mirrors the reference's
inference/attention-state/tests/test_rounds.py:45-60, 190-215, 275-291. Calls go through the kernels module, which
reaches the HIP kernels through the C ABI."""
import pytest
import torch

from oracle import pool as oracle_pool
from tests.support import STORE, bits, kernels

pytestmark = pytest.mark.gpu
dev = "cuda"


def _round_pool(page, table_pages, lengths, round_slots, seed=0):
    g = torch.Generator().manual_seed(seed)
    pages = round_slots * table_pages
    order = torch.randperm(pages, generator=g).tolist()
    tables = torch.full((round_slots, table_pages), pages, dtype=torch.int32)
    capacity = torch.zeros(round_slots, dtype=torch.int64)
    for s, n in lengths:
        held = -(-n // page)
        tables[s, :held] = torch.tensor([order.pop() for _ in range(held)], dtype=torch.int32)
        capacity[s] = n
    return tables, capacity, pages


def test_slots_are_the_closed_form_inside_capacity_and_the_dump_page_outside():
    pk = kernels()
    page = 16
    tables, capacity, dump = _round_pool(page, 40, [(0, 600), (1, 17), (3, 640), (5, 1)], 6)
    wide = torch.full((6, 48), -5, dtype=torch.int32, device=dev)      # the tables as a view of wider rows
    wide[:, :40] = tables.to(dev)
    tables_dev = wide[:, :40]
    g = torch.Generator().manual_seed(3)
    n = 70001      # more than one workgroup's, not a multiple of anything
    slot = torch.randint(0, 6, (n,), generator=g)
    where = torch.randint(-3, 700, (n,), generator=g)
    where[:4] = torch.tensor([0, 599, 600, -1])
    slot[:4] = 0
    want = oracle_pool.slots_at(tables, capacity, slot, where, page, dump)
    got = pk.slots_at(tables_dev, capacity.to(dev), slot.to(dev), where.to(dev), page, dump)
    assert torch.equal(got.cpu(), want)
    # any shape, and an output given (test_rounds.py:283-289)
    out = torch.full((10, 7), -7, dtype=torch.int64, device=dev)
    pk.slots_at(tables_dev, capacity.to(dev), slot[:70].view(10, 7).to(dev), where[:70].view(10, 7).to(dev), page, dump,
                out=out)
    assert torch.equal(out.cpu(), want[:70].view(10, 7))
    # a round's reserve: each token's row's slot first (pages.py:652-653)
    slots_t = torch.tensor([3, 0, 5, 2])
    rows_t = torch.randint(0, 4, (300,), generator=g)
    positions = torch.randint(0, 660, (300,), generator=g)
    want = oracle_pool.reserve_round(tables, capacity, slots_t, rows_t, positions, page, dump)
    got = pk.slots_at(tables_dev, capacity.to(dev), slots_t.to(dev), positions.to(dev), page, dump, rows=rows_t.to(dev))
    assert torch.equal(got.cpu(), want)
    # round slots that do not exist read as slots without capacity
    got = pk.slots_at(tables_dev, capacity.to(dev), torch.tensor([6, -1, 0], device=dev),
                      torch.tensor([0, 0, 0], device=dev), page, dump)
    assert got.tolist() == [dump * page, dump * page, int(tables[0, 0]) * page]
    assert pk.slots_at(tables_dev, capacity.to(dev), slot[:0].to(dev), where[:0].to(dev), page, dump).numel() == 0


def _stores(kind, layers, slots, hkv, d, seed, one_allocation=False):
    g = torch.Generator().manual_seed(seed)
    if kind in ("bf16", "fp16"):
        make = lambda: torch.randn(layers, slots, hkv, d, generator=g).to(STORE[kind])
    else:
        make = lambda: torch.randint(0, 256, (layers, slots, hkv, d), generator=g, dtype=torch.uint8).view(
            torch.int8 if kind == "int8" else torch.float8_e4m3fn)
    found = [make(), make()]
    if kind in ("fp8:row", "int8"):
        found += [torch.rand(layers, slots, hkv, generator=g), torch.rand(layers, slots, hkv, generator=g)]
    return found


def _on_device(stores, interleaved):
    """The stores on the GPU; interleaved: keys and values as two views of one allocation, a layer's keys followed by its
    values (a layer stride that is not the layer's size)."""
    if not interleaved:
        return [s.to(dev) for s in stores]
    k, v = stores[0], stores[1]
    both = torch.stack([bits(k), bits(v)], dim=1).to(dev).contiguous()      # [layers][2][slots][hkv][d]
    return [both[:, 0].view(k.dtype), both[:, 1].view(v.dtype)] + [s.to(dev) for s in stores[2:]]


def _same(got, want, what=""):
    for i, (a, b) in enumerate(zip(got, want)):
        assert torch.equal(bits(a).cpu(), bits(b)), f"{what} store {i}"


@pytest.mark.parametrize("kind,hkv,d", [("bf16", 2, 16), ("bf16", 8, 128), ("fp8:row", 8, 128), ("int8", 2, 64), ("fp8", 3, 20)])
@pytest.mark.parametrize("interleaved", [False, True])
def test_compact_moves_accepted_paths_as_index_copy_of_index_select_does(kind, hkv, d, interleaved):
    pk = kernels()
    page, layers, rows = 16, 3, 5
    tables, capacity, dump = _round_pool(page, 12, [(0, 80), (1, 190), (2, 100), (3, 64), (4, 33)], 6, seed=4)
    slots = (dump + 1) * page
    stores = _stores(kind, layers, slots, hkv, d, 5)
    start = torch.tensor([30, 100, 7, 50, 20, 0])
    emitted = torch.tensor([3, 6, 0, 9, 4, 0])
    # row 0: the reference's own case (test_rounds.py:208); row 1: a deeper path; row 2 held; row 3: no tree, a
    # permutation whose targets are later sources; row 4: moved already
    path = torch.full((rows, 12), -1, dtype=torch.int64)
    path[0, :3] = torch.tensor([0, 2, 5])
    path[1, :6] = torch.tensor([0, 3, 4, 7, 10, 11])
    path[2, :4] = torch.tensor([0, 1, 2, 3])
    path[3, :9] = torch.tensor([0, 2, 1, 4, 3, 8, 7, 6, 5])
    path[4, :4] = torch.tensor([0, 2, 4, 6])
    moved = torch.tensor([0, 0, 0, 0, 1, 0])
    for dtype in (torch.int64, torch.int32):
        want = [s.clone() for s in stores]
        want_moved = moved.clone()
        oracle_pool.compact(want, slots, tables, capacity, start, emitted, path, want_moved, page, dump)
        got = _on_device(stores, interleaved)
        got_moved = moved.to(dev)
        pk.compact(got, slots, tables.to(dev), capacity.to(dev), start.to(dev), emitted.to(dev), path.to(dtype).to(dev),
                   got_moved, page, dump)
        _same(got, want, f"path {dtype}")
        assert got_moved.tolist() == want_moved.tolist() == [1, 1, 1, 1, 1, 0]
        assert not torch.equal(bits(want[0]), bits(stores[0]))
        # a second commit of the round finds the paths moved (test_rounds.py:211)
        pk.compact(got, slots, tables.to(dev), capacity.to(dev), start.to(dev), emitted.to(dev), path.to(dtype).to(dev),
                   got_moved, page, dump)
        _same(got, want, "second commit")


def test_compact_of_the_widest_path_and_of_sources_past_capacity():
    pk = kernels()
    page, layers = 16, 2
    tables, capacity, dump = _round_pool(page, 40, [(0, 600), (1, 300)], 2, seed=6)
    slots = (dump + 1) * page
    stores = _stores("fp8:row", layers, slots, 8, 128, 7)
    g = torch.Generator().manual_seed(8)
    # 256 columns: a random increasing path (a tree's) in row 0; in row 1 every second accepted node lies past the
    # slot's capacity, whose source is then the dump page's first slot
    path = torch.full((2, 256), -1, dtype=torch.int64)
    path[0] = torch.cat([torch.zeros(1, dtype=torch.int64), torch.sort(torch.randperm(330, generator=g)[:255] + 1).values])
    path[1, :40] = torch.arange(40) * 2
    path[1, 1:40:2] += 400
    start, emitted, moved = torch.tensor([200, 100]), torch.tensor([256, 40]), torch.zeros(2, dtype=torch.int64)
    want = [s.clone() for s in stores]
    oracle_pool.compact(want, slots, tables, capacity, start, emitted, path, moved.clone(), page, dump)
    got = [s.to(dev) for s in stores]
    pk.compact(got, slots, tables.to(dev), capacity.to(dev), start.to(dev), emitted.to(dev), path.to(dev), moved.to(dev),
               page, dump)
    _same(got, want)
    with pytest.raises(ValueError):
        pk.compact(got, slots, tables.to(dev), capacity.to(dev), start.to(dev), emitted.to(dev),
                   torch.zeros(2, 257, dtype=torch.int64, device=dev), moved.to(dev), page, dump)
    with pytest.raises(ValueError):      # more rows than round slots
        pk.compact(got, slots, tables.to(dev), capacity.to(dev), start.to(dev), emitted.to(dev),
                   torch.zeros(3, 4, dtype=torch.int64, device=dev), moved.to(dev), page, dump)
    with pytest.raises(ValueError):      # rows of 6 bytes
        pk.compact([torch.zeros(layers, slots, 3, dtype=torch.bfloat16, device=dev)], slots, tables.to(dev), capacity.to(dev),
                   start.to(dev), emitted.to(dev), path.to(dev), moved.to(dev), page, dump)


def test_compact_reads_the_dump_page_as_it_was_and_leaves_it_so():
    # Rows whose windows run past their slots' capacity: their targets there are the dump page's first slot, and so is
    # the source of an accepted node past the capacity. index_copy_(index_select()) reads every source first, so such
    # a node's target gets the dump page's row as it was before the move, whatever other rows send there meanwhile;
    # what the dump page holds afterwards is one of the rows sent to it in the reference (undefined which) and the
    # row it held here. Every other slot: equal to the reference's.
    pk = kernels()
    page, layers, rows = 16, 4, 9
    lengths = [(s, 40 + 3 * s) for s in range(rows)]
    tables, capacity, dump = _round_pool(page, 12, lengths, rows, seed=11)
    slots = (dump + 1) * page
    stores = _stores("fp8:row", layers, slots, 3, 16, 12)
    start = capacity - 4                      # a window of 12 columns: 8 of them past the capacity
    emitted = torch.full((rows,), 12)
    path = torch.arange(12).repeat(rows, 1)
    path[:, 1] = 9                            # column 1 (inside) takes node 9 (past the capacity: the dump page's row)
    path[:, 2] = 3
    path[:, 3] = 2
    moved = torch.zeros(rows, dtype=torch.int64)
    want = [s.clone() for s in stores]
    oracle_pool.compact(want, slots, tables, capacity, start, emitted, path, moved.clone(), page, dump)
    for _ in range(5):      # (which workgroup runs first differs from launch to launch)
        got = [s.to(dev) for s in stores]
        pk.compact(got, slots, tables.to(dev), capacity.to(dev), start.to(dev), emitted.to(dev), path.to(dev), moved.to(dev), page, dump)
        for i, (a, b, before) in enumerate(zip(got, want, stores)):
            a, b, before = (bits(x).cpu().reshape(layers, slots, -1) for x in (a, b, before))
            assert torch.equal(a[:, :dump * page], b[:, :dump * page]), f"store {i}"
            assert torch.equal(a[:, dump * page:], before[:, dump * page:]), f"store {i}: the dump page"
            r = int(oracle_pool.slots_at(tables, capacity, torch.tensor([0]), start[:1] + 1, page, dump)[0])
            assert torch.equal(a[:, r], before[:, dump * page]), "the dump page's row as it was"


@pytest.mark.parametrize("kind,hkv,d,page", [("bf16", 8, 128, 16), ("fp8:row", 8, 128, 16), ("int8", 2, 64, 4), ("fp16", 1, 6, 2)])
@pytest.mark.parametrize("interleaved", [False, True])
def test_pages_are_copied_whole_in_every_layer_and_store(kind, hkv, d, page, interleaved):
    pk = kernels()
    pages, layers = 40, 3
    stores = _stores(kind, layers, pages * page, hkv, d, 9)
    source = torch.tensor([3, -1, 7, 39, 12, 3, 40, 2])      # (40: the first id past the pages)
    target = torch.tensor([0, 5, 9, 1, -1, 38, 4, 41])
    want = [s.clone() for s in stores]
    oracle_pool.copy_pages(want, pages * page, source[:6], target[:6], page)      # (the last two pairs are skipped)
    got = _on_device(stores, interleaved)
    pk.copy_pages(got, pages * page, source.to(dev), target.to(dev), page)
    _same(got, want)
    assert not torch.equal(bits(want[0]), bits(stores[0]))
    pk.copy_pages(got, pages * page, source[:0].to(dev), target[:0].to(dev), page)
    _same(got, want, "no pages")


def test_a_decode_step_from_positions_on_the_device_replays_from_one_graph():
    # The hot loop without the host (pages.py:646-660 and the step's kernels): slots of each row's next position from the
    # bound tables, the token's keys and values appended there, attention over the row up to it, for two layers, captured
    # once; every replay after the lengths moved on the device equals the same step launched eagerly, bit for bit, and
    # the oracle over the pool as the eager launches left it.
    from oracle import attend as oracle_attend
    pk = kernels()
    page, layers, hq, hkv, d, B = 16, 2, 8, 2, 128, 3
    tables, capacity, dump = _round_pool(page, 32, [(0, 500), (1, 500), (2, 500)], 4, seed=10)
    tables, capacity = tables.contiguous().to(dev), capacity.to(dev)
    g = torch.Generator().manual_seed(11)

    def fresh_pool():
        g2 = torch.Generator().manual_seed(12)
        k = (torch.randn(layers, dump + 1, page, hkv, d, generator=g2) * 0.5).bfloat16().to(dev)
        v = (torch.randn(layers, dump + 1, page, hkv, d, generator=g2) * 0.5).bfloat16().to(dev)
        return k, v
    pools = {"graph": fresh_pool(), "eager": fresh_pool()}
    lengths = torch.tensor([40, 333, 7], dtype=torch.int64, device=dev)
    slot_ids = torch.arange(B, dtype=torch.int64, device=dev)
    rows = torch.arange(B, dtype=torch.int32, device=dev)
    starts = torch.arange(B, dtype=torch.int32, device=dev)
    keys = torch.randn(layers, B, hkv, d, generator=g).bfloat16().to(dev)
    values = torch.randn(layers, B, hkv, d, generator=g).bfloat16().to(dev)
    q = torch.randn(layers, B, hq, d, generator=g).bfloat16().to(dev)
    parts = pk.partitions(torch.device(dev), hkv, "bf16")
    workspace = torch.empty(pk.workspace_floats(B, hq, parts, d), dtype=torch.float32, device=dev)

    def step(which, slots, out):
        k, v = pools[which]
        pk.slots_at(tables, capacity, slot_ids, lengths, page, dump, out=slots)
        for layer in range(layers):
            pk.write(keys[layer], values[layer], slots, k[layer], v[layer], "bf16")
            pk.attend(q[layer], k[layer], v[layer], "bf16", tables, rows, starts, lengths, 1, page, out=out[layer],
                      workspace=workspace)
    slots_g, out_g = torch.empty(B, dtype=torch.int64, device=dev), torch.empty(layers, B, hq, d, dtype=torch.bfloat16, device=dev)
    slots_e, out_e = torch.empty_like(slots_g), torch.empty_like(out_g)
    step("graph", slots_g, out_g)      # (the first launches on a device look addresses up: outside the capture)
    torch.cuda.synchronize()
    pools["graph"] = fresh_pool()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step("graph", slots_g, out_g)
    pools["graph"][0].copy_(pools["eager"][0]), pools["graph"][1].copy_(pools["eager"][1])
    for n in range(6):
        graph.replay()
        torch.cuda.synchronize()
        step("eager", slots_e, out_e)
        torch.cuda.synchronize()
        assert torch.equal(slots_g, slots_e), n
        assert torch.equal(out_g, out_e), n
        assert torch.equal(pools["graph"][0], pools["eager"][0]) and torch.equal(pools["graph"][1], pools["eager"][1]), n
        at = lengths.tolist()
        want_slots = [int(tables[s, p // page]) * page + p % page for s, p in enumerate(at)]
        assert slots_g.tolist() == want_slots
        k_cpu, v_cpu = pools["eager"][0][1].cpu(), pools["eager"][1][1].cpu()
        for s in range(B):
            want, _ = oracle_attend.window_reference(q[1, s:s + 1].float().cpu(), k_cpu, v_cpu, "bf16", tables[s].cpu(), at[s], 1,
                                                     page, d ** -0.5)
            torch.testing.assert_close(out_g[1, s:s + 1].double().cpu(), want, atol=2e-2, rtol=2e-2)
        lengths += torch.tensor([1, 16, 3], device=dev)      # the sequences grow on the device


def test_a_rounds_lengths_start_and_commit_on_the_device():
    # KVPool.start_round / commit_round's lengths (pages.py:623-644) against the oracle on random rounds, and the
    # reference's known answers (tests/test_rounds.py:66-72, 113-133).
    pk = kernels()
    g = torch.Generator().manual_seed(21)
    slots, rows = 700, 613
    lengths = torch.randint(0, 5000, (slots,), generator=g)
    start, moved = torch.full((slots,), -1), torch.ones(slots, dtype=torch.int64)
    d_lengths, d_start, d_moved = lengths.to(dev), start.to(dev), moved.to(dev)
    for _ in range(3):
        emitted = torch.randint(0, 3, (rows,), generator=g)
        frontier = torch.randint(0, 6000, (rows,), generator=g)
        oracle_pool.start_round(lengths, start, moved, rows)
        pk.start_round(d_lengths, d_start, d_moved, rows)
        assert torch.equal(d_start.cpu(), start) and torch.equal(d_moved.cpu(), moved)
        moved[:rows] = 1
        d_moved[:rows] = 1
        oracle_pool.commit_round(lengths, start, emitted, frontier)
        pk.commit_round(d_lengths, d_start, emitted.to(dev), frontier.to(dev))
        assert torch.equal(d_lengths.cpu(), lengths)
    lengths, start = torch.tensor([20, 30, 7], device=dev), torch.tensor([-1, -1, -1], device=dev)
    pk.start_round(lengths, start, None, 2)
    pk.commit_round(lengths, start, torch.tensor([3, 0], device=dev), torch.tensor([23, 30], device=dev))
    pk.commit_round(lengths, start, torch.tensor([2, 0], device=dev), torch.tensor([22, 30], device=dev))
    assert lengths.tolist() == [22, 30, 7] and start.tolist() == [20, 30, -1]
    lengths[1] = 27
    pk.start_round(lengths, start, None, 2)
    pk.commit_round(lengths, start, torch.tensor([2, 0], device=dev), torch.tensor([24, 31], device=dev))
    assert lengths.tolist() == [24, 27, 7]
    pk.start_round(lengths, start, None, 0)      # no rows: nothing launched
    with pytest.raises(ValueError):
        pk.commit_round(lengths, start, torch.zeros(4, dtype=torch.int64, device=dev), torch.zeros(4, dtype=torch.int64, device=dev))


def _bound(page, table_pages, held, round_slots, seed):
    """Round tables of sequences bound with all the pages they hold, and the same tables as the host's lists."""
    tables, capacity, dump = _round_pool(page, table_pages, held, round_slots, seed)
    lists = {s: tables[s, :-(-n // page)].tolist() for s, n in held}
    return tables, capacity, dump, lists


@pytest.mark.parametrize("rows_n,window", [(1, 1), (7, 4), (300, 16), (1000, 3)])
def test_a_steps_buffers_built_on_the_device_are_the_ones_the_host_builds(rows_n, window):
    # StepBatch.build + reserve()'s slots + _step_buffers (device.py:600-616, pages.py:337-397) for bound sequences.
    pk = kernels()
    page, table_pages, round_slots = 16, 24, rows_n + 3
    g = torch.Generator().manual_seed(rows_n)
    held = [(s, int(torch.randint(40, table_pages * page + 1, (1,), generator=g))) for s in range(round_slots) if s % 5 != 4]
    tables, capacity, dump, lists = _bound(page, table_pages, held, round_slots, seed=rows_n + 1)
    bound = torch.tensor([s for s, _ in held])
    slot = bound[torch.randperm(len(bound), generator=g)[:rows_n]]
    rows_n = slot.numel()
    counts = torch.randint(1, 2 * window + 1, (rows_n,), generator=g)
    counts[::3] = 1
    lengths = torch.zeros(round_slots, dtype=torch.int64)
    for s, n in held:
        lengths[s] = int(torch.randint(0, n - 2 * window + 1, (1,), generator=g))      # every token inside the capacity
    rows = [(int(s), int(lengths[s]), int(c)) for s, c in zip(slot, counts)]
    starts, positions, row_of = oracle_pool.step_batch(rows)
    slots, d_starts, d_counts, d_firsts, d_offsets, d_tables = oracle_pool.step_buffers(lists, rows, page, dump, window, table_pages)
    n, k = len(d_starts), len(slots)
    step_rows, step_tokens = rows_n + 5, k + 9
    buffers = pk.StepBuffers(step_rows, step_tokens, table_pages, dump, dev)
    for t in (buffers.d_slots, buffers.positions_t, buffers.rows_t, buffers.starts_t, buffers.d_starts, buffers.d_counts,
              buffers.d_firsts, buffers.d_offsets, buffers.d_tables):
        t.fill_(-77)
    found = pk.step_buffers(buffers, tables.to(dev), capacity.to(dev), lengths.to(dev), slot.to(dev), page, window,
                            counts=counts.to(dev))
    assert found is buffers and buffers.totals.tolist() == [k, n, sum(d_counts), 0]
    assert buffers.d_slots[:k].tolist() == slots and buffers.positions_t[:k].tolist() == positions
    assert buffers.rows_t[:k].tolist() == row_of and buffers.starts_t[:rows_n + 1].tolist() == starts
    assert buffers.d_slots[k:].eq(-77).all() and buffers.positions_t[k:].eq(-77).all()
    assert buffers.d_starts[:n].tolist() == d_starts and buffers.d_counts[:n].tolist() == d_counts
    assert buffers.d_firsts[:n].tolist() == d_firsts and buffers.d_offsets[:n].tolist() == d_offsets
    assert buffers.d_tables[:n].tolist() == d_tables and buffers.d_rows.tolist() == list(range(step_rows))
    # entries past the window rows are empty: no tokens, every page the dump page
    assert buffers.d_counts[n:].eq(0).all() and buffers.d_tables[n:].eq(dump).all() and buffers.d_starts[n:].eq(0).all()
    assert buffers.d_offsets[n:].eq(sum(d_counts)).all()
    # one count for every row, first positions given, buffers that are too small
    firsts = torch.tensor([r[1] for r in rows])
    pk.step_buffers(buffers, tables.to(dev), capacity.to(dev), None, slot.to(dev), page, window, count=window, firsts=firsts.to(dev))
    same = [(s, f, window) for s, f, _ in rows]
    slots2, d_starts2, _, d_firsts2, d_offsets2, _ = oracle_pool.step_buffers(lists, same, page, dump, window, table_pages)
    if len(slots2) <= step_tokens:
        assert buffers.totals.tolist() == [len(slots2), rows_n, len(slots2), 0]
        assert buffers.d_slots[:len(slots2)].tolist() == slots2 and buffers.d_starts[:rows_n].tolist() == d_starts2
        assert buffers.d_firsts[:rows_n].tolist() == d_firsts2 and buffers.d_offsets[:rows_n].tolist() == d_offsets2
    small = pk.StepBuffers(max(1, n - 1), max(1, n - 1, k // 2), table_pages, dump, dev) if rows_n > 1 else None
    if small is not None and rows_n <= small.step_rows:
        pk.step_buffers(small, tables.to(dev), capacity.to(dev), lengths.to(dev), slot.to(dev), page, window, counts=counts.to(dev))
        assert small.totals.tolist() == [k, n, sum(d_counts), 1]
        assert small.d_slots.tolist() == slots[:small.step_tokens]


def test_a_step_row_of_an_unbound_slot_lands_on_the_dump_page():
    pk = kernels()
    page, table_pages = 16, 4
    tables, capacity, dump, _ = _bound(page, table_pages, [(0, 64), (2, 20)], 3, seed=5)
    buffers = pk.StepBuffers(4, 16, table_pages, dump, dev)
    lengths = torch.tensor([10, 3, 19], device=dev)
    slot = torch.tensor([2, 1, 7, 0], device=dev)      # slot 1 holds nothing, slot 7 does not exist
    pk.step_buffers(buffers, tables.to(dev), capacity.to(dev), lengths, slot, page, 2, count=2)
    t = tables.tolist()
    assert buffers.d_slots[:8].tolist() == [t[2][1] * 16 + 3, dump * 16, dump * 16, dump * 16, dump * 16, dump * 16,
                                            t[0][0] * 16 + 10, t[0][0] * 16 + 11]      # (position 20 of slot 2: past its capacity)
    assert buffers.d_firsts.tolist() == [19, 3, 0, 10] and buffers.d_tables[2].tolist() == [dump] * 4
    assert buffers.d_tables[1].tolist() == t[1] and buffers.totals.tolist() == [8, 4, 8, 0]
    with pytest.raises(ValueError):
        pk.step_buffers(buffers, tables.to(dev), capacity.to(dev), lengths, torch.zeros(5, dtype=torch.int64, device=dev), page, 2)
    with pytest.raises(ValueError):
        pk.step_buffers(buffers, tables.to(dev), capacity.to(dev), None, slot, page, 2)


def test_a_whole_step_buffers_append_attention_commit_replays_from_one_graph():
    # A decode step with nothing built on the host: the step's buffers from the bound tables and the lengths on the
    # device, the tokens' keys and values appended at the buffers' slots, attention over the buffers' window entries (two
    # of the six entries stay empty), the lengths committed; captured once. Every replay equals the same step built the
    # reference's way on the host (oracle lists -> tensors) and launched eagerly, bit for bit.
    pk = kernels()
    page, layers, hq, hkv, d, B, width = 16, 2, 8, 2, 128, 4, 2
    table_pages = 32
    tables, capacity, dump, lists = _bound(page, table_pages, [(0, 500), (1, 500), (2, 500), (3, 500)], 5, seed=30)
    tables_d, capacity_d = tables.contiguous().to(dev), capacity.to(dev)
    g = torch.Generator().manual_seed(31)

    def fresh_pool():
        g2 = torch.Generator().manual_seed(32)
        k = (torch.randn(layers, dump + 1, page, hkv, d, generator=g2) * 0.5).bfloat16().to(dev)
        v = (torch.randn(layers, dump + 1, page, hkv, d, generator=g2) * 0.5).bfloat16().to(dev)
        return k, v
    pools = {"graph": fresh_pool(), "eager": fresh_pool()}
    lengths = torch.tensor([40, 333, 7, 90, 0], dtype=torch.int64, device=dev)
    host_lengths = lengths.tolist()
    slot = torch.tensor([3, 0, 2, 1], dtype=torch.int64, device=dev)
    counts = torch.tensor([1, 2, 2, 1], dtype=torch.int64, device=dev)
    T = int(counts.sum())
    step_rows, step_tokens = 6, 8
    buffers = pk.StepBuffers(step_rows, step_tokens, table_pages, dump, dev)
    start, emitted, frontier = torch.zeros(5, dtype=torch.int64, device=dev), torch.ones(B, dtype=torch.int64, device=dev), \
        torch.zeros(step_rows, dtype=torch.int64, device=dev)
    keys = torch.randn(layers, step_tokens, hkv, d, generator=g).bfloat16().to(dev)
    values = torch.randn(layers, step_tokens, hkv, d, generator=g).bfloat16().to(dev)
    q = torch.randn(layers, step_tokens, hq, d, generator=g).bfloat16().to(dev)
    parts = pk.partitions(torch.device(dev), hkv, "bf16")
    workspace = torch.empty(pk.workspace_floats(step_tokens, hq, parts, d), dtype=torch.float32, device=dev)
    out_g = torch.zeros(layers, step_tokens, hq, d, dtype=torch.bfloat16, device=dev)
    out_e = torch.zeros_like(out_g)

    def device_step():
        k, v = pools["graph"]
        pk.step_buffers(buffers, tables_d, capacity_d, lengths, slot, page, width, counts=counts)
        # (tokens past the step's are appended nowhere: their slots are set below zero once, outside the capture)
        for layer in range(layers):
            pk.write(keys[layer], values[layer], buffers.d_slots, k[layer], v[layer], "bf16")
            pk.attend(q[layer], k[layer], v[layer], "bf16", buffers.d_tables, buffers.d_rows, buffers.d_starts, buffers.d_firsts,
                      width, page, counts=buffers.d_counts, offsets=buffers.d_offsets, tokens=step_tokens, out=out_g[layer],
                      workspace=workspace)
        torch.add(buffers.d_firsts, buffers.d_counts, out=frontier)
        pk.commit_round(lengths, start, emitted, frontier[:B])      # (round slot r is row r: see below)

    def host_step(at):
        k, v = pools["eager"]
        rows = [(int(s), at[int(s)], int(c)) for s, c in zip(slot.tolist(), counts.tolist())]
        slots, d_starts, d_counts, d_firsts, d_offsets, d_tables = oracle_pool.step_buffers(lists, rows, page, dump, width, table_pages)
        i32 = dict(dtype=torch.int32, device=dev)
        slots_t = torch.tensor(slots + [-1] * (step_tokens - T), device=dev)
        for layer in range(layers):
            pk.write(keys[layer], values[layer], slots_t, k[layer], v[layer], "bf16")
            pk.attend(q[layer], k[layer], v[layer], "bf16", torch.tensor(d_tables, **i32), torch.arange(B, **i32),
                      torch.tensor(d_starts, **i32), torch.tensor(d_firsts, device=dev), width, page,
                      counts=torch.tensor(d_counts, **i32), offsets=torch.tensor(d_offsets, **i32), tokens=step_tokens,
                      out=out_e[layer], workspace=workspace)
        return slots
    # The commit writes round row r's length: with the rows in round-slot order the frontier of row r is slot r's. Here the
    # rows are a permutation of the slots, so the lengths are committed through the same permutation on the host side of
    # the comparison: round_lengths[r] = frontier[r] for r < B.
    buffers.d_slots.fill_(-1)
    device_step()      # (the first launches on a device look addresses up: outside the capture)
    torch.cuda.synchronize()
    pools["graph"] = fresh_pool()
    lengths.copy_(torch.tensor(host_lengths))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        device_step()
    pools["graph"][0].copy_(pools["eager"][0]), pools["graph"][1].copy_(pools["eager"][1])
    lengths.copy_(torch.tensor(host_lengths))
    for n in range(5):
        at = lengths.tolist()
        graph.replay()
        torch.cuda.synchronize()
        slots = host_step(at)
        torch.cuda.synchronize()
        assert buffers.d_slots[:T].tolist() == slots and buffers.totals.tolist() == [T, B, T, 0], n
        assert torch.equal(out_g[:, :T], out_e[:, :T]), n
        assert torch.equal(pools["graph"][0], pools["eager"][0]) and torch.equal(pools["graph"][1], pools["eager"][1]), n
        want = [at[int(s)] + int(c) for s, c in zip(slot.tolist(), counts.tolist())]      # row r's frontier
        assert lengths[:B].tolist() == want, n
        # (the next step reads the lengths by slot: any values below the capacity do, the comparison builds from the same)


def test_the_transactional_state_is_a_sequences_length_on_the_device():
    # KVState (inference/attention-state/code/implementation.py:5-50; oracle.state) beside the device pool: staged rows are
    # appended past the sequence's valid length, a commit of n moves the length by n (the rest is dropped: the next rows
    # overwrite it), a rollback leaves it; attend() over the committed rows, or with the pending ones, is one decode row.
    from oracle.state import KVState
    pk = kernels()
    page, width, hd = 16, 4, 16
    tables, capacity, dump, _ = _bound(page, width, [(0, 64)], 1, seed=40)
    tables_d, capacity_d = tables.to(dev), capacity.to(dev)
    k = torch.zeros(dump + 1, page, 1, hd, dtype=torch.bfloat16, device=dev)
    v = torch.zeros_like(k)
    lengths, start = torch.zeros(1, dtype=torch.int64, device=dev), torch.zeros(1, dtype=torch.int64, device=dev)
    state = KVState(64, hd, hd)
    g = torch.Generator().manual_seed(41)
    slot0 = torch.zeros(1, dtype=torch.int64, device=dev)
    pending = 0

    def stage(n):
        nonlocal pending
        keys, values = torch.randn(n, 1, hd, generator=g).bfloat16(), torch.randn(n, 1, hd, generator=g).bfloat16()
        for key, value in zip(keys[:, 0].float().tolist(), values[:, 0].float().tolist()):
            state.stage(key, value)
        at = int(lengths[0]) + pending + torch.arange(n, device=dev)
        slots = pk.slots_at(tables_d, capacity_d, slot0.expand(n).contiguous(), at, page, dump)
        pk.write(keys.to(dev), values.to(dev), slots, k, v, "bf16")
        pending += n

    def commit(n):
        nonlocal pending
        state.commit(n)
        pk.start_round(lengths, start, None, 1)
        frontier = lengths + n
        pk.commit_round(lengths, start, torch.tensor([n], device=dev), frontier)
        pending = 0

    def check(include_pending):
        q = torch.randn(1, 1, hd, generator=g).bfloat16()
        want = state.attend(q[0, 0].float().tolist(), include_pending=include_pending)
        rows = int(lengths[0]) + (pending if include_pending else 0)
        got = pk.attend(q.to(dev), k, v, "bf16", tables_d, torch.zeros(1, dtype=torch.int32, device=dev),
                        torch.zeros(1, dtype=torch.int32, device=dev), torch.tensor([rows - 1], device=dev), 1, page)
        torch.testing.assert_close(got[0, 0].double().cpu(), torch.tensor(want, dtype=torch.float64), atol=2e-2, rtol=2e-2)
    stage(5)
    check(True)
    commit(3)                      # two speculative rows rejected
    assert int(lengths[0]) == len(state.committed) == 3
    check(False)
    stage(4)
    check(True)
    check(False)                   # the committed prefix alone, the staged rows lying past it
    state.rollback()
    pending = 0                    # (nothing to do on the device: the length did not move)
    check(False)
    stage(20)
    commit(20)
    assert int(lengths[0]) == len(state.committed) == 23
    check(False)
    commit(0)                      # a held row: the length stays
    assert int(lengths[0]) == 23
