"""The pool's device-side bookkeeping of crit's paged KV pool, restated on torch-CPU. Test infrastructure only: nothing
that ships may import this.

Follows inference/attention-state/code/pages.py: _slots_at (655-660), _reserve_round (646-653), _compact (662-684),
_copy (861-869), start_round / commit_round (623-644) and reserve's loop with _step_buffers (337-397), and
core/python/crit_plugins/device.py: StepBatch.build (600-616). Pinned (tests/test_oracle.py) by the slot closed form looped in Python, by the reference's known answers
(tests/test_rounds.py:45-60, 190-215, 275-291: positions past a slot's capacity land on the dump page; the accepted path
[0, 2, 5] of a window at 30 leaves rows [30, 32, 35] at 30..32; a second commit moves nothing) and by a row-at-a-time
model of the move in which a target that is a later source must still deliver its old row; the round's lengths by
tests/test_rounds.py:66-72, 113-133 (20 -> 23; a held row and a truncation's second commit -> (22, 30); a keep between
rounds -> (24, 27)); the step's buffers by a step worked out by hand, by cumulative sums and by slots_at() over the
same positions.
"""
import torch


def slots_at(round_tables, round_capacity, slot, positions, page, dump):
    """KV slots of `positions` of the sequences in round slots `slot` (both int64, one shape), the dump page's first
    slot where a position lies outside its slot's capacity (pages.py:655-660)."""
    table_pages = round_tables.shape[1]
    capacity = round_capacity.index_select(0, slot.reshape(-1)).view(slot.shape)
    entry = round_tables[slot, (positions // page).clamp(0, table_pages - 1)]
    inside = (positions >= 0) & (positions < capacity)
    return torch.where(inside, entry.long() * page + positions % page, torch.full_like(positions, dump * page))


def reserve_round(round_tables, round_capacity, slots_t, rows_t, positions_t, page, dump):
    """A round's slots: each token's row's round slot, then slots_at (pages.py:652-653)."""
    return slots_at(round_tables, round_capacity, slots_t.index_select(0, rows_t), positions_t, page, dump)


def compact(stores, slots, round_tables, round_capacity, start, emitted, path, moved, page, dump):
    """The accepted tree path's rows (node path[r][j] at start[r] + path[r][j]) to positions start[r] + j, 0 < j <
    emitted[r], in every layer of every store, once a round (pages.py:662-684). stores: tensors [layers][...] whose layer
    holds `slots` rows; changed in place, and moved[:rows] set to 1."""
    rows, width = path.shape
    columns = torch.arange(width)
    first = start[:rows]
    keep = (columns[None, :] < emitted[:rows, None]) & (columns[None, :] > 0) & (path >= 0) & (moved[:rows, None] == 0)
    slot = torch.arange(rows)[:, None].expand(rows, width).reshape(-1)
    nowhere = torch.full_like(path.long(), -1)
    source = slots_at(round_tables, round_capacity, slot, torch.where(keep, first[:, None] + path.long(), nowhere).reshape(-1), page, dump)
    target = slots_at(round_tables, round_capacity, slot, torch.where(keep, first[:, None] + columns[None, :], nowhere).reshape(-1), page, dump)
    for store in stores:
        if store is None:
            continue
        flat = store.view(torch.uint8) if store.dtype == torch.float8_e4m3fn else store
        flat = flat.view(flat.shape[0], slots, -1)
        flat.index_copy_(1, target, flat.index_select(1, source))
    moved[:rows] = 1


def copy_pages(stores, slots, source, target, page):
    """Each page source[i] copied to page target[i] in every layer of every store, one after the other as the host loop
    over KVPool._copy does (pages.py:861-869); a pair with a negative id skipped."""
    for a, b in zip(source.tolist(), target.tolist()):
        if a < 0 or b < 0:
            continue
        for store in stores:
            if store is None:
                continue
            flat = store.view(torch.uint8) if store.dtype == torch.float8_e4m3fn else store
            flat = flat.view(flat.shape[0], slots // page, -1)
            flat[:, b].copy_(flat[:, a].clone())


def start_round(round_lengths, start, moved, rows):
    """A round begins (pages.py:623-628): start = the lengths as found, no path moved."""
    start[:rows] = round_lengths[:rows]
    moved[:rows] = 0


def commit_round(round_lengths, start, emitted, frontier):
    """The length update that ends commit_round (pages.py:644): the frontier where a row emitted, else what the round
    found."""
    rows = emitted.numel()
    round_lengths[:rows] = torch.where(emitted > 0, frontier[:rows], start[:rows])


def step_batch(rows):
    """StepBatch.build (device.py:600-616) for rows of (sequence, first position, count): starts (rows + 1), every
    token's position, every token's row."""
    starts, positions, row_of = [0], [], []
    for r, (_, first, count) in enumerate(rows):
        starts.append(starts[-1] + count)
        positions += range(first, first + count)
        row_of += [r] * count
    return starts, positions, row_of


def step_buffers(tables, rows, page, dump, window, table_pages):
    """A step's slots and window entries as reserve() and _step_buffers make them on the host (pages.py:337-349,
    359-397), for a pool without a sliding ring: tables maps a sequence to its page ids (all the pages it holds), rows
    are (sequence, first position, count). Returns (slots, d_starts, d_counts, d_firsts, d_offsets, d_tables) as lists:
    a window row is one of up to `window` tokens; its table is the sequence's, the dump page's id past it."""
    starts, _, _ = step_batch(rows)
    slots, found = [], []
    for sequence, first, count in rows:
        table = tables[sequence]
        slots += [table[q // page] * page + q % page for q in range(first, first + count)]
    offset = 0
    for r, (sequence, first, count) in enumerate(rows):
        if count > window:
            continue
        table = list(tables[sequence])
        found.append((starts[r], count, first, offset, table + [dump] * (table_pages - len(table))))
        offset += count
    return (slots, [f[0] for f in found], [f[1] for f in found], [f[2] for f in found], [f[3] for f in found],
            [f[4] for f in found])
