"""The caller's side of the kernels module, restated for the tests: how crit's attention plugin turns a step's rows into
launches. Test infrastructure only: nothing that ships imports this.

Restates, in plain Python over host lists:
  - StepBatch.build / row (core/python/crit_plugins/device.py:586-633): rows of (sequence, first position, count) packed
    into tokens; row(r) = (sequence, first token, count, first position);
  - Windows and its launches() (inference/attention-state/code/device_attention.py:123-152);
  - _windows_of (device_attention.py:1082-1105): each window row's page table cut at the pages its positions reach,
    padded with the dump page to a width in multiples of TABLE_WIDTH = 16; partial rows packed by the rows' tokens
    (offsets); the launch width the widest row's next power of two;
  - _launch_columns (device_attention.py:847-863): packed rows take max(columns, tile rows // group), at most 64;
  - the split of a step (device_attention.py:416-440): rows of up to pool.window tokens are window rows of one attend()
    launch (or several, by the partials' capacity), the others prompt rows, one prefill() launch each over the
    sequence's own table (_prefill_rows, device_attention.py:901-916).
What they state in closed form is pinned by tests/test_harness.py.
"""
import math

import torch

TABLE_WIDTH = 16      # device_attention.py:1077-1079


class StepBatch:
    """device.py:586-633, the host lists and the device tensors."""

    def __init__(self, sequences, starts, positions, device=None):
        self.sequences, self.starts, self.positions, self.device = sequences, starts, positions, device
        self.starts_t = self.positions_t = self.rows_t = None

    @classmethod
    def build(cls, rows, device=None):
        sequences, starts, positions, row_of = [], [0], [], []
        for r, (sequence, first, count) in enumerate(rows):
            if count < 1 or first < 0:
                raise ValueError("a row is one or more tokens at non-negative positions")
            sequences.append(sequence)
            starts.append(starts[-1] + count)
            positions += range(first, first + count)
            row_of += [r] * count
        batch = cls(sequences, starts, positions, device)
        batch.starts_t = torch.tensor(starts, dtype=torch.int32, device=device)
        batch.positions_t = torch.tensor(positions, dtype=torch.int64, device=device)
        batch.rows_t = torch.tensor(row_of, dtype=torch.int64, device=device)
        return batch

    @property
    def rows(self):
        return len(self.sequences)

    @property
    def tokens(self):
        return self.starts[-1]

    def row(self, r):
        first = self.starts[r]
        return self.sequences[r], first, self.starts[r + 1] - first, self.positions[first]


class Windows:
    """device_attention.py:123-152."""

    def __init__(self, tables, rows, starts, counts, firsts, columns, offsets=None, bounds=None, total=None):
        self.tables, self.rows, self.starts, self.counts, self.firsts = tables, rows, starts, counts, firsts
        self.columns, self.offsets, self.bounds, self.total = int(columns), offsets, bounds, total

    def launches(self, capacity):
        count = int(self.starts.shape[0])
        if self.offsets is None:
            step = count if capacity is None else capacity // self.columns
            if step < 1:
                raise ValueError(f"a row of {self.columns} tokens needs more partials than the workspace holds")
            return [(slice(a, min(count, a + step)), None) for a in range(0, count, step)]
        found, first, used = [], 0, 0
        for r, bound in enumerate(self.bounds):
            if capacity is not None and min(used + bound, self.total) > capacity:
                if r == first:
                    raise ValueError(f"a row of {bound} tokens needs more partials than the workspace holds")
                found.append((slice(first, r), min(used, self.total)))
                first, used = r, 0
            used += bound
        found.append((slice(first, count), min(used, self.total)))
        return found


class PoolView:
    """What the plugin reads of a KVPool (inference/attention-state/code/pages.py): its geometry, each sequence's page ids
    (table()), the dump page, the window, one layer's pages (layer_pages() -> keys, values[, key scales, value scales])
    and each sequence's table on the device (device_tables)."""

    def __init__(self, kind, page, dump, window, tables, pages, multipliers=(1.0, 1.0), device="cpu"):
        self.dtype, self.page, self.dump, self.window = kind, int(page), int(dump), int(window)
        self._tables, self._pages, self.multipliers, self.device = tables, pages, multipliers, device
        self.kv_heads, self.head_dim, self.value_dim = pages[0].shape[-2], pages[0].shape[-1], pages[1].shape[-1]
        self.device_tables = {}

    def table(self, sequence):
        return self._tables[sequence]

    def layer_pages(self, layer=0):
        return self._pages

    def device_table(self, sequence):
        if sequence not in self.device_tables:
            self.device_tables[sequence] = torch.tensor(self._tables[sequence], dtype=torch.int32, device=self.device)
        return self.device_tables[sequence]


def windows_of(pool, rows, device):
    """device_attention.py:1082-1105 for rows of (sequence, first token, count, first position)."""
    tables = [pool.table(sequence)[:math.ceil((position + count) / pool.page)] for sequence, _, count, position in rows]
    width = -(-max(len(t) for t in tables) // TABLE_WIDTH) * TABLE_WIDTH
    grid = torch.full((len(rows), width), pool.dump, dtype=torch.int32)
    for i, t in enumerate(tables):
        grid[i, :len(t)] = torch.tensor(t, dtype=torch.int32)
    counts = [count for _, _, count, _ in rows]
    offsets = [sum(counts[:i]) for i in range(len(rows))]
    meta = torch.tensor([[first, count, position, offset] for (_, first, count, position), offset in zip(rows, offsets)],
                        dtype=torch.int64)
    grid, meta = grid.to(device), meta.to(device)
    widest = max(counts)
    return Windows(grid, torch.arange(len(rows), dtype=torch.int32, device=device), meta[:, 0].to(torch.int32),
                   meta[:, 1].to(torch.int32), meta[:, 2].contiguous(), 1 << (widest - 1).bit_length(),
                   offsets=meta[:, 3].to(torch.int32), bounds=counts, total=sum(counts))


def launch_columns(pk, heads, pool, meta, fused=False, capability=(9, 4)):
    """device_attention.py:847-863."""
    if meta.offsets is None:
        return meta.columns
    group = heads // pool.kv_heads
    rows = pk.tile_for(meta.columns, group, capability, fused)[0]
    return min(pk.MAX_COLUMNS, max(meta.columns, rows // group))


def split(pool, batch):
    """device_attention.py:428-440: (window rows, prompt rows) of a step."""
    short = [r for r in range(batch.rows) if batch.row(r)[2] <= pool.window]
    rest = [r for r in range(batch.rows) if batch.row(r)[2] > pool.window]
    return short, rest


def forward(pk, q, pool, batch, scale=None, lse=False, partial_rows=None, **features):
    """A step's attention as DeviceAttention._forward launches it over a paged pool with crit's kernels (reader split,
    prompt reader prefill): the window rows through attend() with their tables, packed partials and launch width, the
    prompt rows through prefill() one row a launch. partial_rows: the partial rows the workspace holds (None: any).
    Returns out [tokens][heads][value_dim] (and lse [tokens][heads])."""
    tokens, heads = q.shape[0], q.shape[1]
    out = q.new_empty(tokens, heads, pool.value_dim)
    found = q.new_empty(tokens, heads, dtype=torch.float32) if lse else None
    pages = pool.layer_pages()
    scaled = len(pages) == 4
    common = dict(key_scales=pages[2] if scaled else None, value_scales=pages[3] if scaled else None,
                  multipliers=pool.multipliers, scale=scale)
    short, rest = split(pool, batch)
    launched = {"attend": 0, "prefill": 0}
    if short:
        meta = windows_of(pool, [batch.row(r) for r in short], q.device)
        columns = launch_columns(pk, heads, pool, meta)
        for cut, total in meta.launches(partial_rows):
            part = (lambda t: t[cut]) if not cut.start else (lambda t: t[cut].clone())
            pk.attend(q, pages[0], pages[1], pool.dtype, meta.tables, part(meta.rows), part(meta.starts), part(meta.firsts),
                      columns, pool.page, counts=part(meta.counts), offsets=part(meta.offsets), tokens=total, out=out,
                      lse=found, **common, **features)
            launched["attend"] += 1
    for r in rest:
        sequence, first, count, position = batch.row(r)
        span = slice(first, first + count)
        pk.prefill(q[span], pages[0], pages[1], pool.dtype, pool.device_table(sequence), position, pool.page, out=out[span],
                   lse=found[span] if found is not None else None, **common)
        launched["prefill"] += 1
    forward.launched = launched
    return (out, found) if lse else out
