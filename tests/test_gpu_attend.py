"""Paged decode / verify-window attention on the GPU against the CPU oracle (float64 attention over the stored values),
and the bit-for-bit invariances the reference demands of its split-KV reader. Mirrors the reference's
kernels/techniques/attention/paged-kv-attention/tests/test_paged_kv_attention.py:132-188, 275-297, 401-456, 501-512,
tests/test_nonfinite.py, tests/test_sinks.py and tests/test_sliding.py. Tolerances: the reference's own (8e-3 abs +
2e-2 rel, lse 1e-3), tighter than the 2e-2 (bf16) / 5e-2 (fp8) the task allows."""
import math

import pytest
import torch

from tests.support import KINDS, Cache, kernels, rand_q

pytestmark = pytest.mark.gpu
dev = "cuda"
ATOL, RTOL = 8e-3, 2e-2


def _close(got, want, what=None):
    torch.testing.assert_close(got.double().cpu(), want, atol=ATOL, rtol=RTOL, msg=None if what is None else str(what))


def _close_lse(got, want, what=None):
    torch.testing.assert_close(got.double().cpu(), want, atol=1e-3, rtol=1e-4, msg=None if what is None else str(what))


# The reference's own shapes (test_paged_kv_attention.py:129, keys and values of different widths among them), the
# benchmark's, one and three KV heads (a wavefront of the 128-wide kernel then serves one head, not two), and the
# narrowest heads.
SHAPES = [(8, 2, 128, 128), (32, 8, 128, 128), (40, 8, 128, 128), (24, 4, 256, 256), (12, 2, 64, 128), (12, 2, 64, 64),
          (56, 8, 128, 128), (6, 1, 128, 128), (12, 3, 128, 128), (8, 2, 128, 64), (4, 2, 16, 32), (6, 1, 32, 16),
          (5, 1, 256, 64)]


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("hq,hkv,d,dv", SHAPES)
@pytest.mark.parametrize("page", [16, 48])
def test_windows_match_float64_attention(kind, hq, hkv, d, dv, page):
    cache = Cache(kind, hkv, d, dv, page, [130, 64, 1, 517])
    cols = 5
    rows, starts, firsts, counts = [0, 1, 2, 3], [0, 5, 10, 15], [125, 59, 0, 400], [5, 5, 1, 3]
    q = rand_q(20, hq, d, 3)
    lse = torch.full((20, hq), 7.0, device=dev)
    out = cache.attend(q, rows, starts, firsts, cols, lse=lse,
                       counts=torch.tensor(counts, dtype=torch.int32, device=dev))
    for s, start, first, count in zip(rows, starts, firsts, counts):
        want, want_lse = cache.want(q[start:start + count], s, first, count)
        _close(out[start:start + count], want, (s, first))
        _close_lse(lse[start:start + count], want_lse, (s, first))
    assert bool((lse[11:15] == 7.0).all()) and bool((lse[18:] == 7.0).all())      # only the rows' tokens are written


def test_the_cpu_reference_configuration():
    # batch 4, 8 query heads, 2 KV heads, head_dim 128, page 16, contexts {64, 200, 333, 512}, a seeded permutation of
    # 128 physical pages, scale 1/sqrt(128); one new token appended per sequence, then attended.
    pk = kernels()
    g = torch.Generator().manual_seed(0)
    lengths = [64, 200, 333, 512]
    hq, hkv, d, page, n_pages = 8, 2, 128, 16, 128
    perm = torch.randperm(n_pages, generator=g)
    widths = [-(-(n + 1) // page) for n in lengths]
    tables = torch.full((4, 48), n_pages, dtype=torch.int32)          # unused entries: the dump page
    at = 0
    for s, w in enumerate(widths):
        tables[s, :w] = perm[at:at + w].to(torch.int32)
        at += w
    for kind, tol in (("bf16", 2e-2), ("fp8", 5e-2)):
        store = torch.bfloat16 if kind == "bf16" else torch.float8_e4m3fn
        k = torch.zeros(n_pages + 1, page, hkv, d, dtype=store, device=dev)
        v = torch.zeros_like(k)
        mult = (1.0, 1.0) if kind == "bf16" else (4.5 / 448, 4.5 / 448)
        raw = []
        from oracle import append as oa
        for s, n in enumerate(lengths):
            keys, values = torch.randn(n + 1, hkv, d, generator=g), torch.randn(n + 1, hkv, d, generator=g)
            raw.append((keys, values))
            slots = oa.slots(tables[s], torch.arange(n), page)
            pk.write(keys[:n].to(dev), values[:n].to(dev), slots.to(dev), k, v, kind, multipliers=mult)
        # the step: one new token per sequence
        new_slots = torch.stack([oa.slots(tables[s], torch.tensor([n]), page)[0] for s, n in enumerate(lengths)])
        pk.write(torch.stack([r[0][-1] for r in raw]).to(dev), torch.stack([r[1][-1] for r in raw]).to(dev),
                 new_slots.to(dev), k, v, kind, multipliers=mult)
        q = torch.randn(4, hq, d, generator=g)
        out = pk.attend(q.to(dev).bfloat16(), k, v, kind, tables.to(dev), torch.arange(4, dtype=torch.int32, device=dev),
                        torch.arange(4, dtype=torch.int32, device=dev),
                        torch.tensor(lengths, dtype=torch.int64, device=dev), 1, page, multipliers=mult, scale=d ** -0.5)
        from oracle import attend as oatt
        for s, n in enumerate(lengths):
            want, _ = oatt.window_reference(q[s:s + 1], k.cpu(), v.cpu(), kind, tables[s], n, 1, page, d ** -0.5,
                                            multipliers=mult)
            torch.testing.assert_close(out[s:s + 1].double().cpu(), want, atol=tol, rtol=tol)
            # and against the raw (unquantised) FP32 inputs through the reference's CPU path: gather + SDPA in FP32
            exact = torch.nn.functional.scaled_dot_product_attention(
                q[s].view(1, hq, 1, d), raw[s][0].transpose(0, 1).unsqueeze(0), raw[s][1].transpose(0, 1).unsqueeze(0),
                scale=d ** -0.5, enable_gqa=True)[0, :, 0]
            torch.testing.assert_close(out[s].float().cpu(), exact, atol=tol, rtol=tol)


@pytest.mark.parametrize("kind", ["bf16", "fp8", "fp8:row", "int8"])
@pytest.mark.parametrize("hkv,d,dv", [(4, 128, 128), (1, 128, 128), (3, 128, 128), (2, 64, 128)])
def test_rows_and_columns_are_invariant_bit_for_bit(kind, hkv, d, dv):
    pk = kernels()
    cache = Cache(kind, hkv, d, dv, 16, [700, 300, 2100])
    q = rand_q(24, 4 * hkv, d, 5)
    together = cache.attend(q, [0, 1, 2], [0, 8, 16], [690, 290, 2090], 8)
    for s, start, first in zip([0, 1, 2], [0, 8, 16], [690, 290, 2090]):
        alone = cache.attend(q[start:start + 8], [s], [0], [first], 8)
        assert torch.equal(alone, together[start:start + 8])
        for c in range(8):    # each column decoded alone, in a launch of one column
            one = cache.attend(q[start + c:start + c + 1], [s], [0], [first + c], 1)
            assert torch.equal(one[0], together[start + c]), (s, c)
        wide = cache.attend(q[start:start + 8], [s], [0], [first], 16,
                            counts=torch.tensor([8], dtype=torch.int32, device=dev))
        assert torch.equal(wide, together[start:start + 8])
    counts = torch.tensor([3, 1, 4], dtype=torch.int32, device=dev)
    offsets = torch.tensor([0, 3, 4], dtype=torch.int32, device=dev)
    floats = pk.workspace_floats(8, 4 * hkv, pk.partitions(dev, hkv, kind), dv)
    packed = cache.attend(q, [0, 1, 2], [0, 8, 16], [690, 290, 2090], 8, counts=counts, offsets=offsets, tokens=8,
                          workspace=torch.full((floats,), float("nan"), dtype=torch.float32, device=dev))
    for start, count in zip([0, 8, 16], [3, 1, 4]):
        assert torch.equal(packed[start:start + count], together[start:start + count])


@pytest.mark.parametrize("kind", ["bf16", "fp8"])
@pytest.mark.parametrize("hkv,sliding", [(2, 0), (3, 0), (2, 700), (3, 41)])
def test_windows_of_many_tiles_share_a_workgroup_and_keep_each_tokens_bits(hkv, sliding, kind):
    # Pages of 128-wide heads: a window of three tiles or more (12 columns x 4 heads: six tiles of 8 rows with two KV
    # heads a wavefront, three of 16 with one) is read four tiles a workgroup (16-bit pages) or two (FP8 pages); a
    # token's bits stay those of its own one-column launch and of the fused launch, with and without a sliding window,
    # and rows of fewer columns beside it.
    cache = Cache(kind, hkv, 128, 128, 16, [1500, 40, 2100])
    q = rand_q(36, 4 * hkv, 128, 21)
    counts = torch.tensor([12, 5, 12], dtype=torch.int32, device=dev)
    firsts = [1480, 30, 2085]
    lse = torch.empty(36, 4 * hkv, device=dev)
    together = cache.attend(q, [0, 1, 2], [0, 12, 24], firsts, 12, counts=counts, sliding=sliding, lse=lse)
    assert torch.equal(together[:12], cache.attend(q, [0, 1, 2], [0, 12, 24], firsts, 12, counts=counts, sliding=sliding, fused=True)[:12])
    for s, start, first, count in zip([0, 1, 2], [0, 12, 24], firsts, [12, 5, 12]):
        want, want_lse = cache.want(q[start:start + count], s, first, count, sliding=sliding)
        _close(together[start:start + count], want)
        _close_lse(lse[start:start + count], want_lse)
        for c in (0, count // 2, count - 1):
            one = cache.attend(q[start + c:start + c + 1], [s], [0], [first + c], 1, sliding=sliding)
            assert torch.equal(one[0], together[start + c]), (s, c)


def test_a_count_past_the_columns_reads_as_the_columns():
    cache = Cache("bf16", 2, 128, 128, 16, [300, 300])
    q = rand_q(8, 8, 128, 11)
    want = cache.attend(q, [0, 1], [0, 4], [290, 280], 4)
    got = cache.attend(q, [0, 1], [0, 4], [290, 280], 4, counts=torch.tensor([9, 4], dtype=torch.int32, device=dev))
    assert torch.equal(got, want)


@pytest.mark.parametrize("kind", ["bf16", "fp8", "int8"])
@pytest.mark.parametrize("hq,hkv,d,dv", [(32, 8, 128, 128), (24, 4, 256, 256), (6, 1, 128, 128), (12, 3, 128, 128),
                                         (12, 2, 64, 128)])
def test_a_fused_launch_gives_a_column_the_split_launchs_bits(kind, hq, hkv, d, dv):
    for length in (40, 700, 5000):
        cache = Cache(kind, hkv, d, dv, 64, [length], seed=1)
        T = min(130, length)
        pos0 = length - T
        q = rand_q(T, hq, d, 2)
        starts = list(range(0, T, 64))
        counts = torch.tensor([min(64, T - s) for s in starts], dtype=torch.int32, device=dev)
        lse, one_lse = torch.empty(T, hq, device=dev), torch.empty(T, hq, device=dev)
        fused = cache.attend(q, [0] * len(starts), starts, [pos0 + s for s in starts], 64, counts=counts, fused=True,
                             lse=lse)
        alone = cache.attend(q, [0] * T, list(range(T)), [pos0 + i for i in range(T)], 1, lse=one_lse)
        assert torch.equal(fused, alone), (kind, length)
        assert torch.equal(lse, one_lse), (kind, length)
        want, want_lse = cache.want(q[:3], 0, pos0, 3)
        _close(fused[:3], want)
        _close_lse(lse[:3], want_lse)


@pytest.mark.parametrize("kind,hq,hkv,d,dv", [("bf16", 8, 2, 128, 128), ("fp8", 24, 4, 256, 256), ("bf16", 8, 2, 64, 64),
                                              # value rows narrower than a wavefront: the merge's lanes past them
                                              # still take a partition each
                                              ("bf16", 4, 2, 16, 16), ("int8", 6, 2, 32, 32), ("fp8:row", 2, 1, 128, 16),
                                              ("bf16", 3, 3, 32, 64)])
def test_a_row_of_many_partitions_merges_to_the_fused_launchs_bits(kind, hq, hkv, d, dv):
    # Long rows cut into many partitions (the long-context split): the merge takes the maxima and exponentials of a
    # batch of partitions on as many lanes and keeps only the sums in order; the fused launch folds one partition
    # after another. The same bits for 9 partitions (the first count past the one-by-one merge), one batch exactly,
    # a few batches with a ragged last one, a count no row fills; with sinks; and the oracle.
    pk = kernels()
    block = pk.flash_block(d, dv, hq, hkv, 16, kind)
    cache = Cache(kind, hkv, d, dv, 16, [40 * block * 5 + 7], seed=51)
    n = cache.lengths[0]
    q = rand_q(3, hq, d, 52)
    sinks = torch.linspace(-1, 1, hq, device=dev)
    for parts, piece in ((9, block * 23), (32, block * 6), (16, block * 6), (77, block * 2), (500, block)):
        lse, fused_lse = torch.empty(3, hq, device=dev), torch.empty(3, hq, device=dev)
        split = cache.attend(q, [0], [0], [n - 3], 3, partitions=parts, piece=piece, lse=lse)
        fused = cache.attend(q, [0], [0], [n - 3], 3, partitions=parts, piece=piece, lse=fused_lse, fused=True)
        assert torch.equal(split, fused), (parts, piece)
        assert torch.equal(lse, fused_lse), (parts, piece)
        want, want_lse = cache.want(q, 0, n - 3, 3)
        _close(split, want)
        _close_lse(lse, want_lse)
        assert torch.equal(cache.attend(q, [0], [0], [n - 3], 3, partitions=parts, piece=piece, sinks=sinks),
                           cache.attend(q, [0], [0], [n - 3], 3, partitions=parts, piece=piece, sinks=sinks, fused=True))
        # a sliding window that leaves most partitions without a visible position (empty states between live ones)
        window = 5 * block + 3
        slid = cache.attend(q, [0], [0], [n - 3], 3, partitions=parts, piece=piece, sliding=window)
        assert torch.equal(slid, cache.attend(q, [0], [0], [n - 3], 3, partitions=parts, piece=piece, sliding=window, fused=True))
        want, _ = cache.want(q, 0, n - 3, 3, sliding=window)
        _close(slid, want)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 128), (24, 4, 256), (12, 2, 64)])
def test_rows_read_their_fresh_positions_beside_the_pages(kind, hq, hkv, d):
    # attend(fresh=(keys, values, shift, first)): a prompt chunk of 130 tokens at position 300 as window rows of up to
    # 64 columns (DeviceAttention._decode_rows' pieces, device_attention.py:751-783), its own positions from 16-bit
    # rows as the projections gave them (row = position - shift, unscaled), the prefix from the pages: against the
    # oracle, one shift and first for every row and one a row (a row whose first lies past every position reads the
    # pages only); split = fused = each row alone, bit for bit; with a sliding window and sinks.
    position, T = 300, 130
    cache = Cache(kind, hkv, d, d, 16, [position + T], seed=71)
    q = rand_q(T, hq, d, 72)
    q_dtype = torch.float16 if kind == "fp16" else torch.bfloat16
    g = torch.Generator().manual_seed(73)
    fk, fv = torch.randn(T, hkv, d, generator=g).to(q_dtype).to(dev), torch.randn(T, hkv, d, generator=g).to(q_dtype).to(dev)
    starts = [0, 64, 128]
    counts = torch.tensor([64, 64, 2], dtype=torch.int32, device=dev)
    firsts = [position + s for s in starts]
    i64 = lambda x: torch.tensor(x, dtype=torch.int64, device=dev)
    one = (fk, fv, i64([position]), i64([position]))
    lse, fused_lse = torch.empty(T, hq, device=dev), torch.empty(T, hq, device=dev)
    out = cache.attend(q, [0, 0, 0], starts, firsts, 64, counts=counts, fresh=one, lse=lse)
    fused = cache.attend(q, [0, 0, 0], starts, firsts, 64, counts=counts, fresh=one, lse=fused_lse, fused=True)
    assert torch.equal(out, fused) and torch.equal(lse, fused_lse)
    for t in (0, 1, 63, 64, 129):
        want, want_lse = cache.want(q[t:t + 1], 0, position + t, 1, fresh=(fk.cpu(), fv.cpu(), position, position))
        _close(out[t:t + 1], want, f"token {t}")
        _close_lse(lse[t:t + 1], want_lse, f"lse {t}")
    alone = cache.attend(q[64:128], [0], [0], [position + 64], 64, fresh=one)
    assert torch.equal(alone, out[64:128])
    # a shift and a first for each row: the second row's own positions only (its first 64 positions back in the
    # pages), the third row none
    each = (fk, fv, i64([position] * 3), i64([position, position + 64, 1 << 62]))
    mixed = cache.attend(q, [0, 0, 0], starts, firsts, 64, counts=counts, fresh=each)
    assert torch.equal(mixed[:64], out[:64])
    want, _ = cache.want(q[100:101], 0, position + 100, 1, fresh=(fk.cpu(), fv.cpu(), position, position + 64))
    _close(mixed[100:101], want, "second row")
    want, _ = cache.want(q[129:130], 0, position + 129, 1)
    _close(mixed[129:130], want, "third row")
    sinks = torch.linspace(-1, 1, hq, device=dev)
    slid = cache.attend(q, [0, 0, 0], starts, firsts, 64, counts=counts, fresh=one, sliding=90, sinks=sinks, lse=lse)
    assert torch.equal(slid, cache.attend(q, [0, 0, 0], starts, firsts, 64, counts=counts, fresh=one, sliding=90,
                                          sinks=sinks, fused=True))
    plain_lse = torch.empty(T, hq, device=dev)
    plain = cache.attend(q, [0, 0, 0], starts, firsts, 64, counts=counts, fresh=one, sliding=90, lse=plain_lse)
    want, want_lse = cache.want(q[70:71], 0, position + 70, 1, sliding=90, fresh=(fk.cpu(), fv.cpu(), position, position))
    _close(plain[70:71], want, "window")
    _close_lse(plain_lse[70:71], want_lse, "window lse")
    weight = torch.exp(plain_lse) / (torch.exp(plain_lse) + torch.exp(sinks)[None, :])
    torch.testing.assert_close(slid.float(), plain.float() * weight[..., None], atol=8e-3, rtol=2e-2)


def test_fresh_rows_that_do_not_fit_are_refused():
    cache = Cache("bf16", 2, 128, 128, 16, [100])
    q = rand_q(4, 8, 128, 1)
    fk = torch.zeros(4, 2, 128, dtype=torch.bfloat16, device=dev)
    i64 = lambda x: torch.tensor(x, dtype=torch.int64, device=dev)
    with pytest.raises(ValueError):
        cache.attend(q, [0], [0], [96], 4, fresh=(fk[:, :1], fk, i64([96]), i64([96])))
    with pytest.raises(ValueError):
        cache.attend(q, [0], [0], [96], 4, fresh=(fk.float(), fk.float(), i64([96]), i64([96])))
    with pytest.raises(ValueError):
        cache.attend(q, [0], [0], [96], 4, fresh=(fk, fk, i64([96, 96]), i64([96, 96])))
    with pytest.raises(ValueError):
        cache.attend(q, [0], [0], [96], 4, fresh=(fk, fk, i64([96]), i64([96])),
                     blocks=torch.zeros(4, 2, dtype=torch.int32, device=dev), block_size=16)


def test_a_given_workspace_holds_the_partials_and_a_small_one_is_refused():
    pk = kernels()
    cache = Cache("bf16", 2, 128, 128, 16, [300])
    q = rand_q(4, 8, 128, 9)
    floats = pk.workspace_floats(4, 8, 16, 128)
    own = cache.attend(q, [0], [0], [296], 4, partitions=16)
    given = cache.attend(q, [0], [0], [296], 4, partitions=16,
                         workspace=torch.full((floats,), float("nan"), dtype=torch.float32, device=dev))
    assert torch.equal(own, given)
    with pytest.raises(ValueError, match="workspace"):
        cache.attend(q, [0], [0], [296], 4, partitions=16,
                     workspace=torch.empty(floats - 1, dtype=torch.float32, device=dev))


@pytest.mark.parametrize("kind,chunk", [("bf16", 512), ("bf16", 1024), ("fp8", 2048)])
def test_contiguous_splits_match_float64_and_do_not_depend_on_the_table_width(kind, chunk):
    cache = Cache(kind, 8, 128, 128, 16, [5000, 900])
    q = rand_q(2, 40, 128, 21)
    lse = torch.empty(2, 40, device=dev)
    out = cache.attend(q, [0, 1], [0, 1], [4999, 899], 1, flash=True, chunk=chunk, lse=lse)
    for s, first in ((0, 4999), (1, 899)):
        want, want_lse = cache.want(q[s:s + 1], s, first, 1)
        _close(out[s:s + 1], want)
        _close_lse(lse[s:s + 1], want_lse)
    # a wider table (more splits in the grid, none of them holding a position) changes no bit
    wider = torch.cat([cache.tables, torch.zeros(2, 4096, dtype=torch.int32, device=dev)], 1).contiguous()
    narrow, cache.tables = cache.tables, wider
    again = cache.attend(q, [0, 1], [0, 1], [4999, 899], 1, flash=True, chunk=chunk)
    cache.tables = narrow
    assert torch.equal(again, out)


def test_one_graph_replays_at_every_length():
    pk = kernels()
    cache = Cache("fp8:row", 4, 128, 128, 16, [5000, 5000])
    q = rand_q(10, 16, 128, 8).to(torch.bfloat16)
    rows = torch.tensor([0, 1], dtype=torch.int32, device=dev)
    starts = torch.tensor([0, 5], dtype=torch.int32, device=dev)
    firsts = torch.tensor([10, 20], dtype=torch.int64, device=dev)
    out = torch.empty(10, 16, 128, dtype=torch.bfloat16, device=dev)
    workspace = torch.empty(pk.workspace_floats(10, 16, pk.partitions(dev, 4, "fp8:row"), 128), dtype=torch.float32,
                            device=dev)

    def launch(into):
        return pk.attend(q, cache.k, cache.v, "fp8:row", cache.tables, rows, starts, firsts, 5, 16,
                         key_scales=cache.ks, value_scales=cache.vs, out=into, workspace=workspace)
    launch(out)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch(out)
    for a, b in ((10, 20), (4000, 63), (64, 4990), (1, 2)):
        firsts.copy_(torch.tensor([a, b], device=dev))
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        eager = launch(torch.empty_like(out))
        torch.cuda.synchronize()
        assert torch.equal(got, eager), (a, b)


def test_work_follows_the_rows_length_not_the_capacity():
    # Every position past the row's own is poisoned (NaN scales) before the launch: a read of any would show.
    pk = kernels()
    cache = Cache("fp8:row", 4, 128, 128, 64, [20_000])
    q = rand_q(1, 16, 128, 1).to(torch.bfloat16)
    args = lambda firsts: (q, cache.k, cache.v, "fp8:row", cache.tables, torch.zeros(1, dtype=torch.int32, device=dev),
                           torch.zeros(1, dtype=torch.int32, device=dev), firsts, 1, 64)
    kw = dict(key_scales=cache.ks, value_scales=cache.vs)
    for first in (19_000, 4_000):
        firsts = torch.tensor([first], device=dev)
        want = pk.attend(*args(firsts), **kw).clone()
        past = cache.slots(0, torch.arange(first + 1, 20_000, device=dev))
        cache.ks.view(-1, 4)[past] = float("nan")
        cache.vs.view(-1, 4)[past] = float("nan")
        got = pk.attend(*args(firsts), **kw)
        assert bool(torch.isfinite(got).all()), first
        assert torch.equal(got, want), first


def test_a_nan_query_poisons_only_its_own_token_and_head():
    cache = Cache("bf16", 2, 128, 128, 16, [300, 300])
    q = rand_q(4, 8, 128, 4)
    clean = cache.attend(q, [0, 1], [0, 2], [298, 298], 2)
    q[1, 3, 7] = float("nan")
    dirty = cache.attend(q, [0, 1], [0, 2], [298, 298], 2)
    assert bool(torch.isnan(dirty[1, 3]).all())
    mask = torch.ones(4, 8, dtype=torch.bool, device=dev)
    mask[1, 3] = False
    assert torch.equal(dirty[mask], clean[mask])


def test_a_window_of_one_position_returns_that_positions_value():
    cache = Cache("bf16", 2, 128, 128, 16, [40])
    q = rand_q(1, 8, 128, 4)
    one = cache.attend(q, [0], [0], [5], 1, sliding=1)
    stored = cache.v.view(-1, 2, 128)[cache.slots(0, torch.tensor([5]))][0]         # [hkv][dv]
    assert torch.equal(one[0], stored.repeat_interleave(4, 0))
    zero = cache.attend(q, [0], [0], [0], 1)                                       # position 0 sees itself only
    stored = cache.v.view(-1, 2, 128)[cache.slots(0, torch.tensor([0]))][0]
    assert torch.equal(zero[0], stored.repeat_interleave(4, 0))


@pytest.mark.parametrize("kind", ["bf16", "fp8:row"])
@pytest.mark.parametrize("window", [1, 100, 128, 1000])
def test_a_sliding_window_sees_only_its_last_positions(kind, window):
    cache = Cache(kind, 2, 128, 128, 16, [3000])
    q = rand_q(4, 8, 128, 4)
    lse = torch.empty(4, 8, device=dev)
    out = cache.attend(q, [0], [0], [2996], 4, sliding=window, lse=lse)
    want, want_lse = cache.want(q, 0, 2996, 4, sliding=window)
    _close(out, want)
    _close_lse(lse, want_lse)
    for c in range(4):
        one = cache.attend(q[c:c + 1], [0], [0], [2996 + c], 1, sliding=window)
        assert torch.equal(one[0], out[c])


def test_sinks_add_one_valueless_position_to_every_softmax():
    cache = Cache("bf16", 2, 128, 128, 16, [500])
    q = rand_q(2, 8, 128, 4)
    sinks = torch.tensor([0.0, 1.0, -1.0, float("-inf"), 3.0, 0.5, -0.5, 2.0], device=dev)
    lse, plain_lse = torch.empty(2, 8, device=dev), torch.empty(2, 8, device=dev)
    out = cache.attend(q, [0], [0], [498], 2, sinks=sinks, lse=lse)
    plain = cache.attend(q, [0], [0], [498], 2, lse=plain_lse)
    # out = plain * sum / (sum + e^sink); lse = log(e^plain_lse + e^sink)
    weight = torch.exp(plain_lse) / (torch.exp(plain_lse) + torch.exp(sinks)[None, :])
    torch.testing.assert_close(out.float(), plain.float() * weight[..., None], atol=8e-3, rtol=2e-2)
    torch.testing.assert_close(lse, torch.logaddexp(plain_lse, sinks[None, :].expand(2, 8)), atol=1e-3, rtol=1e-4)
    assert torch.equal(out[:, 3], plain[:, 3])
    fused = cache.attend(q, [0], [0], [498], 2, sinks=sinks, fused=True)
    assert torch.equal(fused, out)


def test_outputs_in_fp32_and_fp16_pages():
    cache = Cache("fp16", 2, 128, 128, 16, [333])
    q = rand_q(1, 8, 128, 4)
    out32 = torch.empty(1, 8, 128, dtype=torch.float32, device=dev)
    cache.attend(q, [0], [0], [332], 1, out=out32)
    want, _ = cache.want(q, 0, 332, 1)
    _close(out32, want)
    out16 = cache.attend(q, [0], [0], [332], 1)
    assert out16.dtype == torch.float16
    assert torch.equal(out32.half(), out16)


def test_later_launches_of_a_step_take_absolute_offsets():
    # DeviceAttention hands a later launch cloned slices whose offsets keep their absolute values: the partial rows
    # count from the launch's first row (inference/attention-state/code/device_attention.py:692-699).
    cache = Cache("bf16", 2, 128, 128, 16, [300, 300, 300])
    q = rand_q(3, 8, 128, 4)
    whole = cache.attend(q, [0, 1, 2], [0, 1, 2], [299, 299, 299], 1,
                         counts=torch.ones(3, dtype=torch.int32, device=dev),
                         offsets=torch.tensor([0, 1, 2], dtype=torch.int32, device=dev), tokens=3)
    out = torch.zeros_like(whole)
    pk = kernels()
    floats = pk.workspace_floats(2, 8, pk.partitions(dev, 2, "bf16"), 128)
    cache.attend(q, [1, 2], [1, 2], [299, 299], 1, counts=torch.ones(2, dtype=torch.int32, device=dev),
                 offsets=torch.tensor([1, 2], dtype=torch.int32, device=dev), tokens=2, out=out,
                 workspace=torch.empty(floats, dtype=torch.float32, device=dev))
    assert torch.equal(out[1:], whole[1:]) and not bool(out[0].any())


def test_merge_shards_equals_attention_over_the_whole_sequence():
    # inference/partitioned-attention/tests/test_device.py:44-77
    pk = kernels()
    g = torch.Generator().manual_seed(1)
    keys, values = torch.randn(300, 2, 128, generator=g), torch.randn(300, 2, 128, generator=g)
    q = torch.randn(1, 4, 128, generator=g).to(dev)
    caches = {}
    for name, (a, b) in {"s": (0, 300), "a": (0, 120), "b": (120, 300)}.items():
        c = Cache("bf16", 2, 128, 128, 16, [b - a], seed=7)
        c.write(0, 0, keys[a:b].to(dev), values[a:b].to(dev))
        caches[name] = c

    def step(c, n):
        lse = torch.empty(1, 4, device=dev)
        return c.attend(q, [0], [0], [n - 1], 1, lse=lse), lse
    out, lse = step(caches["s"], 300)
    parts = [step(caches["a"], 120), step(caches["b"], 180)]
    merged, merged_lse = pk.merge_shards([o for o, _ in parts], [x for _, x in parts])
    torch.testing.assert_close(merged, out.float(), atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(merged_lse, lse, atol=2e-3, rtol=1e-4)
    from oracle import attend as oatt
    want, want_lse = oatt.merge([o.cpu() for o, _ in parts], [x.cpu() for _, x in parts])
    torch.testing.assert_close(merged.cpu(), want, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(merged_lse.cpu(), want_lse, atol=1e-5, rtol=1e-5)
    outs = [torch.ones(2, 1, 128, device=dev), torch.zeros(2, 1, 128, device=dev)]
    lses = [torch.tensor([[0.5], [float("-inf")]], device=dev), torch.full((2, 1), float("-inf"), device=dev)]
    o, l = pk.merge_shards(outs, lses)
    assert bool((o[0] == 1).all()) and not bool(o[1].any()) and float(l[1, 0]) == float("-inf")
    assert abs(float(l[0, 0]) - 0.5) < 1e-6


def test_bad_geometry_is_refused():
    cache = Cache("bf16", 2, 128, 128, 16, [100])
    q = rand_q(1, 8, 128, 4)
    with pytest.raises(ValueError):
        cache.attend(q, [0], [0], [99], 65)
    with pytest.raises(ValueError):
        cache.attend(q[:, :7], [0], [0], [99], 1)
    with pytest.raises(ValueError, match="offsets"):
        cache.attend(q, [0], [0], [99], 1, offsets=torch.zeros(1, dtype=torch.int32, device=dev))
    with pytest.raises(ValueError):
        cache.attend(q, [0], [0], [99], 1, derive=(q, 0))      # (not a Derive: derive() makes one)


def test_launches_that_overlap_on_two_streams_do_not_share_counters():
    # The split launch's workgroups pull their units from two counters the module hands the launch, one pair per
    # stream: launches in flight together (two streams here, many each) must not disturb one another, and every one
    # must leave its pair zeroed for the next launch on its stream.
    caches = [Cache("bf16", 4, 128, 128, 16, [3000, 1700, 900], seed=s) for s in (1, 2)]
    qs = [rand_q(3, 16, 128, 20 + s) for s in range(2)]
    want = [c.attend(q, [0, 1, 2], [0, 1, 2], [2999, 1699, 899], 1) for c, q in zip(caches, qs)]
    torch.cuda.synchronize()
    pk = kernels()
    floats = pk.workspace_floats(3, 16, pk.partitions(dev, 4, "bf16"), 128)
    # (each stream its own partials: the module's default workspace is one per device and owner, as the reference's)
    spaces = [torch.empty(floats, dtype=torch.float32, device=dev) for _ in range(2)]
    streams = [torch.cuda.Stream() for _ in range(2)]
    outs = [[], []]
    for rep in range(65):
        for i, stream in enumerate(streams):
            with torch.cuda.stream(stream):
                outs[i].append(caches[i].attend(qs[i], [0, 1, 2], [0, 1, 2], [2999, 1699, 899], 1, workspace=spaces[i]))
    torch.cuda.synchronize()
    for i in range(2):
        for got in outs[i]:
            assert torch.equal(got, want[i])


def test_an_owners_graph_replays_beside_another_owners_eager_launches():
    # Owner A captures a step of 32 launches and replays it on one stream while owner B issues more than 64 eager
    # launches on another: each owner's launch counters and partials are its own (a captured launch bakes its counters'
    # address in, so it must never be an address an eager launch or another graph is handed), and both get the bits
    # of their launches run alone.
    pk = kernels()
    lengths = [3000, 1700, 900, 2500]
    caches = [Cache("bf16", 4, 128, 128, 16, lengths, seed=s) for s in (31, 32)]
    qs = [rand_q(4, 16, 128, 40 + s) for s in range(2)]
    firsts = [n - 1 for n in lengths]
    rows = torch.arange(4, dtype=torch.int32, device=dev)
    firsts_t = torch.tensor(firsts, dtype=torch.int64, device=dev)
    want = [c.attend(q, rows, rows, firsts_t, 1) for c, q in zip(caches, qs)]
    torch.cuda.synchronize()
    layers = 32
    out_a = torch.zeros(layers, 4, 16, 128, dtype=torch.bfloat16, device=dev)

    def step_a():
        for layer in range(layers):
            caches[0].attend(qs[0], rows, rows, firsts_t, 1, out=out_a[layer])
    with pk.owner("a"):
        step_a()      # (the owner's partials and counters are allocated outside the capture)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step_a()
    streams = [torch.cuda.Stream() for _ in range(2)]
    got_b = []
    for rep in range(3):
        out_a.zero_()
        torch.cuda.synchronize()
        with torch.cuda.stream(streams[0]):
            graph.replay()
        with torch.cuda.stream(streams[1]), pk.owner("b"):
            for i in range(70):
                got_b.append(caches[1].attend(qs[1], rows, rows, firsts_t, 1))
        torch.cuda.synchronize()
        for layer in range(layers):
            assert torch.equal(out_a[layer], want[0]), (rep, layer)
    for got in got_b:
        assert torch.equal(got, want[1])
    # the two owners hold different counters, and a capture's are not the eager stream's
    held = {key: h for key, h in pk._holdings.items() if key[1] in ("a", "b")}
    assert len(held) == 2
    pairs = [at for h in held.values() for at in h.pair_of.values()]
    assert len(pairs) == len(set(pairs)) >= 3
    pk.release("a"), pk.release("b")
    assert not [key for key in pk._holdings if key[1] in ("a", "b")]


def test_a_launch_without_counters_deals_its_units_in_turn():
    # The C ABI with launch_state NULL (a host that keeps no counters): units are dealt to the workgroups in turn,
    # the same bits as the pulled launch.
    from crit_amd.paged_kv_attention import _abi
    cache = Cache("fp8", 8, 128, 128, 16, [5000, 300, 1200, 64, 2048, 4097], seed=33)
    q = rand_q(6, 32, 128, 34)
    rows = torch.arange(6, dtype=torch.int32, device=dev)
    firsts = torch.tensor([n - 1 for n in cache.lengths], dtype=torch.int64, device=dev)
    want = cache.attend(q, rows, rows, firsts, 1)
    lib, seen = _abi.load(), []
    real = lib.crit_pkv_attend

    def without_counters(params, stream):
        params.launch_state = None
        seen.append(1)
        return real(params, stream)
    lib.crit_pkv_attend = without_counters
    try:
        got = cache.attend(q, rows, rows, firsts, 1)
    finally:
        lib.crit_pkv_attend = real
    torch.cuda.synchronize()
    assert len(seen) == 1
    assert torch.equal(got, want)


def test_more_units_than_resident_workgroups_and_ragged_rows():
    # 96 rows of very different lengths over 8 KV heads: several thousand units for a few hundred resident
    # workgroups, most of the list's (row, partition) slots empty; every row against its own launch, bit for bit.
    g = torch.Generator().manual_seed(9)
    lengths = [int(x) for x in torch.randint(1, 6000, (96,), generator=g)]
    lengths[5], lengths[50] = 1, 5999
    cache = Cache("fp8", 8, 128, 128, 16, lengths, seed=4)
    q = rand_q(96, 32, 128, 6)
    firsts = [n - 1 for n in lengths]
    together = cache.attend(q, list(range(96)), list(range(96)), firsts, 1)
    for s in (0, 5, 17, 50, 95):
        alone = cache.attend(q[s:s + 1], [s], [0], [firsts[s]], 1)
        assert torch.equal(alone[0], together[s]), s
        want, _ = cache.want(q[s:s + 1].to(torch.bfloat16), s, firsts[s], 1)
        _close(together[s:s + 1], want, s)


@pytest.mark.parametrize("kind,hq,hkv,d,page", [("bf16", 8, 2, 128, 16), ("int8", 8, 2, 128, 16), ("fp8", 32, 8, 128, 16),
                                                 ("bf16", 12, 2, 64, 16), ("fp8:row", 8, 2, 128, 48)])
def test_a_tree_sees_its_ancestors_and_a_chain_is_causal(kind, hq, hkv, d, page):
    # the reference's tree test (tests/test_cuda.py:110-129, tests/test_flash.py:74-92)
    cache = Cache(kind, hkv, d, d, page, [400, 300])
    parents = torch.tensor([-1, 0, 0, 1, 1, 2, 5, 3], dtype=torch.int64, device=dev)
    q = rand_q(8, hq, d, 6)
    out = cache.attend(q, [0], [0], [392], 8, parents=parents)
    want, _ = cache.want(q.to(torch.bfloat16), 0, 392, 8, parents=parents.tolist())
    _close(out, want)
    chain = cache.attend(q, [0], [0], [392], 8, parents=torch.arange(-1, 7, device=dev))
    assert torch.equal(chain, cache.attend(q, [0], [0], [392], 8))
    assert not torch.equal(chain, out)
    assert torch.equal(cache.attend(q, [0], [0], [392], 8, parents=parents.int(), fused=True), out)
    assert torch.equal(cache.attend(q, [0], [0], [392], 8, parents=parents, flash=True, chunk=128),
                       cache.attend(q, [0], [0], [392], 8, parents=parents, flash=True, chunk=128, fused=True))
    # two rows in one launch, the second a shorter tree behind the first row's tokens: each as alone
    both = torch.cat([parents, torch.tensor([-1, 0, 1, 1, 0], dtype=torch.int64, device=dev)])
    q2 = rand_q(13, hq, d, 7)
    together = cache.attend(q2, [0, 1], [0, 8], [392, 295], 8, parents=both,
                            counts=torch.tensor([8, 5], dtype=torch.int32, device=dev))
    alone = cache.attend(q2[8:13], [1], [0], [295], 8, parents=both[8:13].contiguous(),
                         counts=torch.tensor([5], dtype=torch.int32, device=dev))
    assert torch.equal(together[8:13], alone)
    want2, _ = cache.want(q2[8:13].to(torch.bfloat16), 1, 295, 5, parents=both[8:13].tolist())
    _close(together[8:13], want2)
    with pytest.raises(ValueError):
        cache.attend(q, [0], [0], [392], 8, parents=parents.float())


@pytest.mark.parametrize("kind,hq,hkv,d,page", [("bf16", 8, 2, 128, 16), ("int8", 8, 2, 128, 16), ("fp8", 32, 8, 128, 16),
                                                 ("bf16", 12, 2, 64, 16), ("fp8:row", 10, 2, 128, 48), ("fp16", 6, 2, 256, 16)])
@pytest.mark.parametrize("block_size", [4, 16, 80])
def test_block_lists_see_only_their_blocks(kind, hq, hkv, d, page, block_size):
    # the reference's test (tests/test_paged_kv_attention.py:372-397): four tokens of one row, each with its own list
    # of 10 - t blocks out of the sequence's, -1 behind them; a token sees its listed blocks' positions up to its own.
    cache = Cache(kind, hkv, d, d, page, [1000])
    g = torch.Generator().manual_seed(9)
    q = rand_q(4, hq, d, 7)
    nblk = math.ceil(1000 / block_size)
    blocks = torch.full((4, 12), -1, dtype=torch.int32)
    for t in range(4):
        chosen = torch.randperm(nblk, generator=g)[:10 - t].sort().values
        blocks[t, :len(chosen)] = chosen.to(torch.int32)
    lse = torch.empty(4, hq, device=dev)
    out = cache.attend(q, [0], [0], [996], 4, blocks=blocks.to(dev), block_size=block_size, lse=lse, partitions=4)
    q_dtype = torch.float16 if kind == "fp16" else torch.bfloat16
    want, want_lse = cache.want(q.to(q_dtype), 0, 996, 4, blocks=blocks, block_size=block_size)
    _close(out, want)
    _close_lse(lse, want_lse)
    # the lists in another order, and in a wider tensor of lists: the same positions (sums in another order)
    wide = torch.full((4, 40), -1, dtype=torch.int32)
    wide[:, 5:17] = blocks.flip(1)
    again = cache.attend(q, [0], [0], [996], 4, blocks=wide.to(dev)[:, 5:17], block_size=block_size, partitions=4)
    _close(again, want)


def test_block_lists_rows_are_their_own_and_empty_lists_see_nothing():
    cache = Cache("bf16", 4, 128, 128, 16, [3000, 700])
    q = rand_q(3, 16, 128, 8)
    blocks = torch.full((3, 6), -1, dtype=torch.int32)
    blocks[0, :4] = torch.tensor([0, 7, 20, 46])        # row 0: two columns at 2998, 2999; block 46 = positions 2944 .. 3007
    blocks[1, :3] = torch.tensor([46, 3, 11])
    # token 2 (row 1, position 699) lists nothing: zeros and -inf
    lse = torch.empty(3, 16, device=dev)
    both = cache.attend(q, [0, 1], [0, 2], [2998, 699], 2, blocks=blocks.to(dev), block_size=64, lse=lse,
                        counts=torch.tensor([2, 1], dtype=torch.int32, device=dev))
    want, _ = cache.want(q[:2].to(torch.bfloat16), 0, 2998, 2, blocks=blocks[:2], block_size=64)
    _close(both[:2], want)
    assert bool((both[2] == 0).all()) and bool(torch.isinf(lse[2]).all())
    alone = cache.attend(q[:2], [0], [0], [2998], 2, blocks=blocks[:2].to(dev), block_size=64)
    assert torch.equal(alone, both[:2])
    # a block past the token's own position, or past the page table, is masked: listing it changes nothing
    more = blocks.clone()
    more[0, 4], more[0, 5] = 47, 100000
    assert torch.equal(cache.attend(q[:2], [0], [0], [2998], 2, blocks=more[:2].to(dev), block_size=64)[0], alone[0])
    with pytest.raises(ValueError):
        cache.attend(q[:2], [0], [0], [2998], 2, blocks=blocks[:2].to(dev), block_size=64, fused=True)
    with pytest.raises(ValueError):
        cache.attend(q[:2], [0], [0], [2998], 2, blocks=blocks[:2].to(dev), block_size=64, sliding=8)
    with pytest.raises(ValueError):
        cache.attend(q[:2], [0], [0], [2998], 2, blocks=blocks[:2].to(dev))
    with pytest.raises(ValueError):
        cache.attend(q[:2], [0], [0], [2998], 2, blocks=blocks[:2].long().to(dev), block_size=64)


@pytest.mark.parametrize("kind,block_size", [("bf16", 64), ("fp8", 32), ("bf16", 24)])
def test_block_lists_with_a_draft_tree_over_long_lists(kind, block_size):
    # Lists long enough for several pieces and partitions (blocks of 64 and 32 walk their lists in the 128-wide kernel,
    # blocks of 24 in the generic one), a draft tree on top: a column sees its listed blocks' positions below the
    # window and, of the window, its ancestors' and its own where listed.
    cache = Cache(kind, 2, 128, 128, 16, [6000])
    g = torch.Generator().manual_seed(13)
    parents = torch.tensor([-1, 0, 0, 1, 2], dtype=torch.int32, device=dev)
    first = 5990
    q = rand_q(5, 8, 128, 11)
    nblk = math.ceil(6000 / block_size)
    blocks = torch.full((5, 70), -1, dtype=torch.int32)
    for t in range(5):
        chosen = torch.randperm(nblk - 1, generator=g)[:60 - 7 * t]
        blocks[t, :len(chosen)] = chosen.to(torch.int32)
        blocks[t, 65] = nblk - 1                      # the window's own block, behind a gap of -1
    out = cache.attend(q, [0], [0], [first], 5, parents=parents, blocks=blocks.to(dev), block_size=block_size, partitions=3)
    want, _ = cache.want(q.to(torch.bfloat16), 0, first, 5, parents=parents.tolist(), blocks=blocks, block_size=block_size)
    _close(out, want)
    more = cache.attend(q, [0], [0], [first], 5, parents=parents, blocks=blocks.to(dev), block_size=block_size, partitions=16)
    _close(more, want)


@pytest.mark.parametrize("kind", ["bf16", "fp8:row"])
def test_a_round_hands_its_slots_over_as_int64_rows(kind):
    # A captured round's launch (device_attention.py:561-576): the pool's round tables, the batch's round slots as they
    # are (int64, device.py:661, 681), starts int32, the frontier int64, no counts: the same bits as int32 rows, through
    # the 128-wide kernel, the generic one (a head width of 64) and the fused launch.
    for hq, hkv, d in ((8, 2, 128), (4, 2, 64)):
        cache = Cache(kind, hkv, d, d, 16, [700, 90, 300], seed=81)
        cols = 4
        q = rand_q(3 * cols, hq, d, 82)
        slots_t = torch.tensor([2, 0, 1], dtype=torch.int64, device=dev)
        starts_t = (torch.arange(4, dtype=torch.int32, device=dev) * cols)[:3]
        frontier = torch.tensor([290, 640, 70], dtype=torch.int64, device=dev)
        for fused in (False, True):
            got = cache.attend(q, slots_t, starts_t, frontier, cols, fused=fused)
            want = cache.attend(q, slots_t.to(torch.int32), starts_t, frontier, cols, fused=fused)
            assert torch.equal(got, want)
        ref, _ = cache.want(q[cols:2 * cols], 0, 640, cols)
        _close(got[cols:2 * cols], ref)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("sliding,sinks", [(0, False), (40, False), (0, True)])
def test_window_rows_equal_the_references_torch_fallback_over_the_same_tables(kind, sliding, sinks):
    # The reader against the arithmetic the reference tests its own reader with: windows_torch's FP32 online softmax in
    # passes of 1,024 positions over the page tables (device_attention.py:1204-1288; oracle.attend.windows_online), the
    # same Windows metadata into both.
    from oracle import attend as oracle_attend
    hq, hkv, d, page = 8, 2, 128, 16
    cache = Cache(kind, hkv, d, d, page, [1100, 64, 2300])
    rows, starts, counts, firsts = [2, 0, 1], [0, 4, 6], [4, 2, 1], [2290, 1098, 63]
    q = rand_q(7, hq, d, 5)
    q_dtype = torch.float16 if kind == "fp16" else torch.bfloat16
    sink = torch.tensor([0.5, -1.0, float("-inf"), 2.0, 0.0, 1.5, -3.0, 0.25]) if sinks else None
    lse = torch.empty(7, hq, device=dev)
    out = cache.attend(q, rows, starts, firsts, 4, lse=lse, counts=torch.tensor(counts, dtype=torch.int32, device=dev),
                       sliding=sliding, sinks=None if sink is None else sink.to(dev))
    k, v, ks, vs, tables = cache.cpu()
    want, want_lse = oracle_attend.windows_online(q.to(q_dtype).float().cpu(), k, v, kind, tables, rows, starts, counts, firsts, 4,
                                                  page, d ** -0.5, ks, vs, cache.multipliers, extent=2300, sliding=sliding,
                                                  sinks=sink)
    _close(out, want.double(), (kind, sliding, sinks))
    _close_lse(lse, want_lse.double(), (kind, sliding, sinks))
