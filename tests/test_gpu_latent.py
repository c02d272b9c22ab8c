"""Latent attention on the GPU against the float64 oracle (oracle.latent, the reference's latent_attention.py) over the
rows as the cache stores them: decode tokens and verify windows over shuffled pages at the ranks and heads of the models
that use it, sinks and log-sum-exps, BF16, FP16 and E4M3 caches (two scales a position, or one); a token's bits the same
alone, in a verify window, beside other rows, fused or not and in a prompt chunk; one graph replayed at other lengths;
what the module refuses. The cases cover those of the reference's kernels/techniques/attention/latent-attention/tests/
test_latent_attention.py, at its tolerances (8e-3 + 2e-2 |ref|; log-sum-exp 1e-3). Calls go through the module, which
reaches the HIP kernels through the C ABI."""
import pytest
import torch

from oracle import latent as oracle_latent

pytestmark = pytest.mark.gpu
dev = "cuda"


def module():
    import crit_amd.latent_attention as la
    return la


class Cache:
    """A latent cache of several sequences: a position's row is its latent (R values) then its rotary key (P values),
    appended by the module's own write() into pages handed out from a shuffled list, a spare page a sequence. scales: 0
    (a 16-bit cache), 2 (E4M3 codes, the latent and the rotary key each at its own scale) or 1 (E4M3 codes at one
    scale a row, as a KV pool's fp8:row pages of one head hold them)."""

    def __init__(self, rank, rope, page, lengths, seed=0, dtype=torch.bfloat16, scales=0):
        self.la = module()
        self.rank, self.rope, self.page = rank, rope, page
        draw = torch.Generator().manual_seed(seed)
        each = 1 + max((n + page - 1) // page for n in lengths)
        total = each * len(lengths) + 2
        self.tables = torch.randperm(total, generator=draw)[:each * len(lengths)].reshape(len(lengths), each).to(
            device=dev, dtype=torch.int32)
        self.cache = torch.zeros(total, page, rank + rope, dtype=dtype, device=dev)
        self.scales = torch.zeros(total, page, 2, device=dev) if scales else None
        for s, n in enumerate(lengths):
            latent = torch.randn(n, rank, generator=draw).to(dev)
            rotary = torch.randn(n, rope, generator=draw).to(dev) * (3 if scales else 1)      # (two scales that differ)
            self.la.write(latent, rotary, self.slot_of(s, torch.arange(n, device=dev)), self.cache, self.scales)
        if scales == 1:
            self._recode_at_one_scale(total)

    def _recode_at_one_scale(self, total):
        width = self.rank + self.rope
        two = self.scales.reshape(-1, 2)
        by_value = torch.cat([two[:, :1].expand(-1, self.rank), two[:, 1:].expand(-1, self.rope)], dim=1)
        values = self.cache.reshape(-1, width).float() * by_value
        one = (values.abs().amax(dim=-1) / 448.0).clamp(min=1e-30)
        codes = (values / one.unsqueeze(-1)).clamp(-448, 448).to(torch.float8_e4m3fn)
        self.cache, self.scales = codes.reshape(total, self.page, width), one.reshape(total, self.page, 1).contiguous()

    def slot_of(self, s, positions):
        pages = self.tables[s].long()[torch.div(positions, self.page, rounding_mode="floor")]
        return pages * self.page + positions % self.page

    def rows(self, s, n):
        """Positions 0 .. n - 1 of sequence s as the cache stores them: (latent [n][R], rotary key [n][P]), float64."""
        scales = None if self.scales is None else self.scales.cpu()
        return oracle_latent.stored(self.cache.cpu(), scales, self.tables[s].cpu(), n, self.page, self.rank)

    def attend(self, q, rows, starts, firsts, columns, **kw):
        ints = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
        return self.la.attend(q, self.cache, self.tables, ints(rows), ints(starts),
                              torch.tensor(firsts, dtype=torch.int64, device=dev), columns, self.page, rank=self.rank,
                              scales=self.scales, **kw)

    def check(self, q, out, lse, s, start, first, count, scale, sinks=None, lse_tol=1e-3):
        """Tokens start .. start + count - 1 against float64 latent attention of window row (s, first, count)."""
        latent, rotary = self.rows(s, first + count)
        own = first + torch.arange(count)
        seen = torch.arange(first + count).unsqueeze(0) <= own.unsqueeze(1)
        tokens = slice(start, start + count)
        queries = q[tokens].double().cpu()
        want, want_lse = oracle_latent.latent_attention(queries[..., :self.rank], queries[..., self.rank:], latent, rotary, seen,
                                                        scale, None if sinks is None else sinks.cpu())
        torch.testing.assert_close(out[tokens].double().cpu(), want, atol=8e-3, rtol=2e-2)
        if lse is not None:
            torch.testing.assert_close(lse[tokens].double().cpu(), want_lse, atol=lse_tol, rtol=1e-4)


def _q(tokens, heads, width, seed, dtype=torch.bfloat16):
    draw = torch.Generator().manual_seed(seed)
    return torch.randn(tokens, heads, width, generator=draw).mul_(0.5).to(dev, dtype)


@pytest.mark.parametrize("rank,rope,heads,page", [(512, 64, 16, 64), (512, 64, 128, 16), (256, 64, 8, 32), (128, 32, 20, 16),
                                                 (64, 32, 3, 48), (128, 64, 5, 16), (64, 64, 40, 16), (1024, 64, 16, 64),
                                                 (512, 128, 24, 16), (1024, 32, 2, 16), (1024, 128, 4, 32), (1024, 256, 16, 16),
                                                 (512, 32, 16, 64), (512, 256, 3, 16), (256, 32, 6, 16), (256, 128, 8, 32),
                                                 (256, 256, 1, 16), (128, 128, 5, 16), (128, 256, 20, 16), (64, 128, 2, 48),
                                                 (64, 256, 7, 16),
                                                 # ranks and rotary widths below the matrix tiles: the vector kernel
                                                 (16, 16, 3, 16), (32, 16, 16, 48), (16, 256, 5, 16), (32, 64, 8, 64),
                                                 (1024, 16, 2, 16), (512, 16, 16, 32), (64, 16, 7, 16), (32, 32, 4, 16),
                                                 (16, 64, 1, 16), (128, 16, 6, 16), (256, 16, 3, 16), (16, 32, 2, 16),
                                                 (16, 128, 2, 16), (32, 128, 3, 16), (32, 256, 2, 16)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_windows_match_float64_latent_attention(rank, rope, heads, page, dtype):
    cache = Cache(rank, rope, page, [130, 64, 1, 517], dtype=dtype)
    rows, starts, firsts, counts = [0, 1, 2, 3], [0, 5, 10, 15], [125, 59, 0, 400], [5, 5, 1, 3]
    q = _q(20, heads, rank + rope, 3, dtype)
    scale = 192 ** -0.5
    sinks = torch.randn(heads, generator=torch.Generator().manual_seed(9)).to(dev)
    sinks[0] = float("-inf")
    for given in (None, sinks):
        lse = torch.full((20, heads), 7.0, device=dev)
        out = cache.attend(q, rows, starts, firsts, 5, scale=scale, lse=lse,
                           counts=torch.tensor(counts, dtype=torch.int32, device=dev), sinks=given)
        for s, start, first, count in zip(rows, starts, firsts, counts):
            cache.check(q, out, lse, s, start, first, count, scale, given)
        assert bool((lse[11:15] == 7.0).all()) and bool((lse[18:] == 7.0).all())      # only the rows' tokens are written


def test_a_tokens_bits_are_its_own_alone_in_a_window_and_beside_other_rows():
    cache = Cache(512, 64, 64, [700, 300, 2100], seed=2)
    q = _q(24, 16, 576, 5)
    together = cache.attend(q, [0, 1, 2], [0, 8, 16], [690, 290, 2090], 8)
    for r, (start, first) in enumerate(zip([0, 8, 16], [690, 290, 2090])):
        for c in range(8):
            alone = cache.attend(q[start + c:start + c + 1], [r], [0], [first + c], 1)
            assert torch.equal(alone[0], together[start + c]), (r, c)
        window = cache.attend(q[start:start + 8], [r], [0], [first], 8)
        assert torch.equal(window, together[start:start + 8]), r
    # rows launched a few at a time (their partials bounded) and a round's int64 rows: the same bits
    la = cache.la
    limit = la.PARTIAL_BYTES
    try:
        la.PARTIAL_BYTES = 8 * 16 * la.partitions(torch.device(dev), 16, 512, 64, 64) * 514 * 4      # one row's
        sliced = cache.attend(q, [0, 1, 2], [0, 8, 16], [690, 290, 2090], 8, fused=True)
    finally:
        la.PARTIAL_BYTES = limit
    assert torch.equal(sliced, together)
    as_slots = la.attend(q, cache.cache, cache.tables, torch.tensor([0, 1, 2], device=dev), torch.tensor([0, 8, 16], dtype=torch.int32, device=dev),
                         torch.tensor([690, 290, 2090], device=dev), 8, 64, rank=512)
    assert torch.equal(as_slots, together)


@pytest.mark.parametrize("tile_rows", [128, 16])
def test_many_heads_either_kernel_matches_float64_and_a_tokens_bits_follow_the_kernel_alone(tile_rows):
    # 128 heads of DeepSeek's shape: the many-heads kernel (128 query rows a workgroup; the default here) or, asked for,
    # the small tiles. Either way a token's bits are its own: alone, in a verify window, beside other rows (the longest
    # rows go first inside the launch), in launches of a few rows at a time; and the lengths straddle pieces, tiles of 32
    # positions and pages.
    cache = Cache(512, 64, 16, [1500, 33, 2100, 600], seed=31)
    la = cache.la
    assert la.tile_rows(128, 512, 64, 16) == 128 and la.tile_rows(128, 512, 64, 16, asked=16) == 16
    assert la.tile_rows(64, 512, 64, 16) == 16 and la.tile_rows(128, 512, 64, 24) == 16 and la.tile_rows(128, 512, 64, 16, 1) == 128
    assert la.tile_rows(64, 512, 64, 16, asked=128) == 128
    q = _q(16, 128, 576, 32)
    rows, starts, firsts = [0, 1, 2, 3], [0, 4, 8, 12], [1496, 29, 2096, 511]
    sinks = torch.randn(128, generator=torch.Generator().manual_seed(33)).to(dev)
    lse = torch.empty(16, 128, device=dev)
    together = cache.attend(q, rows, starts, firsts, 4, lse=lse, sinks=sinks, tile_rows=tile_rows)
    for s_, start, first in zip(rows, starts, firsts):
        cache.check(q, together, lse, s_, start, first, 4, 576 ** -0.5, sinks)
        window = cache.attend(q[start:start + 4], [s_], [0], [first], 4, sinks=sinks, tile_rows=tile_rows)
        assert torch.equal(window, together[start:start + 4]), s_
        for c in (0, 3):
            alone = cache.attend(q[start + c:start + c + 1], [s_], [0], [first + c], 1, sinks=sinks, tile_rows=tile_rows)
            assert torch.equal(alone[0], together[start + c]), (s_, c)
    limit = la.PARTIAL_BYTES
    try:
        la.PARTIAL_BYTES = 4 * 128 * la.partitions(torch.device(dev), 128, 512, 64, 16, 0, tile_rows) * 514 * 4      # one row's
        sliced = cache.attend(q, rows, starts, firsts, 4, sinks=sinks, tile_rows=tile_rows)
    finally:
        la.PARTIAL_BYTES = limit
    assert torch.equal(sliced, together)
    other = cache.attend(q, rows, starts, firsts, 4, sinks=sinks, tile_rows=144 - tile_rows)
    torch.testing.assert_close(other.float(), together.float(), atol=8e-3, rtol=2e-2)      # the same attention, other sums
    with pytest.raises(ValueError):
        cache.attend(q, rows, starts, firsts, 4, tile_rows=64)
    odd = Cache(512, 64, 24, [40], seed=34)
    with pytest.raises(ValueError):      # pages of no multiple of 16 positions: not the many-heads kernel's
        odd.attend(_q(1, 128, 576, 35), [0], [0], [39], 1, tile_rows=128)
    assert torch.equal(odd.attend(_q(1, 128, 576, 35), [0], [0], [39], 1), odd.attend(_q(1, 128, 576, 35), [0], [0], [39], 1, tile_rows=16))


@pytest.mark.parametrize("heads", [16, 128])
def test_a_nan_query_reaches_its_own_rows_output_only(heads):
    cache = Cache(512, 64, 64, [700, 300], seed=4)
    q = _q(2, heads, 576, 6)
    clean = cache.attend(q, [0, 1], [0, 1], [650, 250], 1)
    q[0, 3, 5] = float("nan")
    lse = torch.empty(2, heads, device=dev)
    out = cache.attend(q, [0, 1], [0, 1], [650, 250], 1, lse=lse)
    assert bool(torch.isnan(out[0, 3]).all()) and bool(torch.isnan(lse[0, 3]))
    keep = torch.ones(heads, dtype=torch.bool, device=dev)
    keep[3] = False
    assert torch.equal(out[0][keep], clean[0][keep]) and torch.equal(out[1], clean[1])


def test_one_graph_replays_at_every_length():
    cache = Cache(512, 64, 64, [4000], seed=3)
    la = cache.la
    q = _q(1, 16, 576, 7)
    first = torch.tensor([10], dtype=torch.int64, device=dev)
    args = (cache.cache, cache.tables, torch.zeros(1, dtype=torch.int32, device=dev), torch.zeros(1, dtype=torch.int32, device=dev),
            first, 1, 64)
    out = torch.empty(1, 16, 512, dtype=torch.bfloat16, device=dev)
    la.attend(q, *args, rank=512, out=out)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        la.attend(q, *args, rank=512, out=out)
    for at in (0, 63, 64, 1000, 3999):
        first.fill_(at)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, cache.attend(q, [0], [0], [at], 1)), at


def test_what_it_cannot_read_is_refused():
    cache = Cache(512, 64, 64, [10])
    la = cache.la
    q = _q(1, 16, 576, 1)
    some = lambda: (torch.zeros(1, dtype=t, device=dev) for t in (torch.int32, torch.int32, torch.int64))
    with pytest.raises(ValueError, match="BF16 or FP16 in the cache's dtype"):
        cache.attend(q.float(), [0], [0], [5], 1)
    with pytest.raises(ValueError, match="powers of two"):
        la.attend(q, cache.cache, cache.tables, *some(), 1, 64, rank=500)
    with pytest.raises(ValueError, match="columns a row"):
        cache.attend(q, [0], [0], [5], 65)
    with pytest.raises(ValueError, match="sinks: one FP32 logit a head"):
        cache.attend(q, [0], [0], [5], 1, sinks=torch.zeros(3, device=dev))
    codes = torch.zeros(4, 64, 576, dtype=torch.float8_e4m3fn, device=dev)
    with pytest.raises(ValueError, match="E4M3 cache takes its scales"):
        la.attend(q, codes, cache.tables, *some(), 1, 64, rank=512)
    with pytest.raises(ValueError, match="multiple of 32"):
        cache.attend(q, [0], [0], [5], 1, piece=48)


@pytest.mark.parametrize("rank,rope", [(512, 64), (64, 32), (128, 32), (256, 128), (1024, 256), (64, 256), (16, 16), (32, 64),
                                       (512, 16), (16, 256)])
@pytest.mark.parametrize("scales", [2, 1])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_an_e4m3_cache_matches_float64_over_its_stored_values_and_keeps_a_tokens_bits(scales, dtype, rank, rope):
    cache = Cache(rank, rope, 64, [130, 517], seed=6, dtype=torch.float8_e4m3fn, scales=scales)
    q = _q(8, 16, rank + rope, 8, dtype)
    lse = torch.empty(8, 16, device=dev)
    scale = 192 ** -0.5
    out = cache.attend(q, [0, 1], [0, 4], [126, 513], 4, scale=scale, lse=lse)
    for s, start, first in ((0, 0, 126), (1, 4, 513)):
        cache.check(q, out, lse, s, start, first, 4, scale)
        for c in range(4):
            alone = cache.attend(q[start + c:start + c + 1], [s], [0], [first + c], 1, scale=scale)
            assert torch.equal(alone[0], out[start + c]), (s, c)


@pytest.mark.parametrize("rank,rope", [(16, 16), (32, 64), (1024, 16)])
@pytest.mark.parametrize("coded", [0, 2])
def test_shapes_below_the_matrix_tiles_keep_a_tokens_bits_and_deal_their_pieces_round(rank, rope, coded):
    kind = dict(dtype=torch.float8_e4m3fn, scales=coded) if coded else {}
    cache = Cache(rank, rope, 16, [3000, 70], seed=21, **kind)
    q = _q(8, 6, rank + rope, 22)
    lse = torch.empty(8, 6, device=dev)
    scale = 0.11
    together = cache.attend(q, [0, 1], [0, 4], [2990, 60], 4, scale=scale, lse=lse)
    for s, start, first in ((0, 0, 2990), (1, 4, 60)):
        cache.check(q, together, lse, s, start, first, 4, scale)
        for c in range(4):
            alone = cache.attend(q[start + c:start + c + 1], [s], [0], [first + c], 1, scale=scale)
            assert torch.equal(alone[0], together[start + c]), (s, c)
    # few partitions: partition b reads pieces b, b + partitions, ...; a piece that is no multiple of a step of 64
    for parts, piece in ((1, 512), (3, 96), (5, 32)):
        out = cache.attend(q, [0, 1], [0, 4], [2990, 60], 4, scale=scale, lse=lse, partitions=parts, piece=piece)
        for s, start, first in ((0, 0, 2990), (1, 4, 60)):
            cache.check(q, out, lse, s, start, first, 4, scale)


@pytest.mark.parametrize("scales", [2, 1])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_an_e4m3_cache_under_the_many_heads_kernel_matches_float64_and_keeps_a_tokens_bits(scales, dtype):
    # 128 heads over codes: the many-heads kernel converts each tile in LDS, one step ahead; rows that end inside a tile,
    # a page and a piece, one tile long and many pieces long; a packed prompt chunk of few heads on the same kernel.
    cache = Cache(512, 64, 16, [1500, 33, 2100, 600], seed=41, dtype=torch.float8_e4m3fn, scales=scales)
    la = cache.la
    assert la.tile_rows(128, 512, 64, 16, 1) == 128
    q = _q(16, 128, 576, 42, dtype)
    rows, starts, firsts = [0, 1, 2, 3], [0, 4, 8, 12], [1496, 29, 2096, 511]
    sinks = torch.randn(128, generator=torch.Generator().manual_seed(43)).to(dev)
    lse = torch.empty(16, 128, device=dev)
    scale = 192 ** -0.5
    together = cache.attend(q, rows, starts, firsts, 4, scale=scale, lse=lse, sinks=sinks)
    for s_, start, first in zip(rows, starts, firsts):
        cache.check(q, together, lse, s_, start, first, 4, scale, sinks)
        for c in (0, 3):
            alone = cache.attend(q[start + c:start + c + 1], [s_], [0], [first + c], 1, scale=scale, sinks=sinks)
            assert torch.equal(alone[0], together[start + c]), (s_, c)
    small = cache.attend(q, rows, starts, firsts, 4, scale=scale, sinks=sinks, tile_rows=16)
    torch.testing.assert_close(small.float(), together.float(), atol=8e-3, rtol=2e-2)      # the same attention, other sums
    few = _q(40, 16, 576, 44, dtype)
    lse = torch.empty(40, 16, device=dev)
    packed = la.prefill(few, cache.cache, cache.tables[2], 2060, 16, rank=512, scale=scale, scales=cache.scales, lse=lse, packed=True)
    cache.check(few, packed, lse, 2, 0, 2060, 40, scale)


@pytest.mark.parametrize("rank,rope,heads,page", [(512, 64, 16, 64), (512, 64, 128, 16), (128, 32, 20, 16), (32, 16, 4, 16)])
def test_prompt_chunks_match_float64_and_are_their_positions_decoded(rank, rope, heads, page):
    cache = Cache(rank, rope, page, [900], seed=11)
    la = cache.la
    sinks = torch.randn(heads, generator=torch.Generator().manual_seed(12)).to(dev)
    scale = 192 ** -0.5
    for position, T in ((0, 70), (400, 133), (899 - 37, 38)):
        q = _q(T, heads, rank + rope, position + 1)
        for given in (None, sinks):
            lse = torch.empty(T, heads, device=dev)
            out = la.prefill(q, cache.cache, cache.tables[0], position, page, rank=rank, scale=scale, lse=lse, sinks=given)
            cache.check(q, out, lse, 0, 0, position, T, scale, given, lse_tol=2e-3)
        for t in (0, T // 2, T - 1):
            alone = cache.attend(q[t:t + 1], [0], [0], [position + t], 1, scale=scale, sinks=sinks)
            assert torch.equal(alone[0], out[t]), (position, t)


@pytest.mark.parametrize("heads", [16, 24, 64])
def test_packed_prompt_chunks_of_few_heads_match_float64_and_a_tokens_bits_do_not_follow_the_chunk(heads):
    # packed=True: the many-heads kernel reads the chunk, a tile of 128 query rows being 128 / heads tokens (with 24
    # heads a token straddles two tiles). Against the exact result at the module's tolerance; a token's bits are those of
    # the same position read alone by the same kernel (tile_rows=128), whatever the chunk's length; against the small
    # tiles' decode bits they are another rounding of the same sums, inside the same tolerance.
    cache = Cache(512, 64, 16, [1200], seed=41)
    la = cache.la
    sinks = torch.randn(heads, generator=torch.Generator().manual_seed(42)).to(dev)
    for position, T in ((0, 70), (500, 133), (1199 - 300, 301)):
        q = _q(T, heads, 576, position + 3)
        lse = torch.empty(T, heads, device=dev)
        out = la.prefill(q, cache.cache, cache.tables[0], position, 16, rank=512, lse=lse, sinks=sinks, packed=True)
        cache.check(q, out, lse, 0, 0, position, T, 576 ** -0.5, sinks, lse_tol=2e-3)
        for t in (0, T // 2, T - 1):
            alone = cache.attend(q[t:t + 1], [0], [0], [position + t], 1, sinks=sinks, tile_rows=128)
            assert torch.equal(alone[0], out[t]), (position, t)
        assert torch.equal(la.prefill(q[:T // 2], cache.cache, cache.tables[0], position, 16, rank=512, sinks=sinks, packed=True), out[:T // 2])
        decoded = la.prefill(q, cache.cache, cache.tables[0], position, 16, rank=512, sinks=sinks)
        torch.testing.assert_close(out.float(), decoded.float(), atol=8e-3, rtol=2e-2)


def test_a_prompt_tokens_bits_do_not_follow_its_chunks_length_and_a_graph_replays_at_device_positions():
    cache = Cache(512, 64, 64, [3000], seed=13)
    la = cache.la
    q = _q(200, 16, 576, 14)
    full = la.prefill(q, cache.cache, cache.tables[0], 2000, 64, rank=512)
    for T in (1, 37, 64, 129):
        assert torch.equal(la.prefill(q[:T], cache.cache, cache.tables[0], 2000, 64, rank=512), full[:T]), T
    position = torch.tensor([0], dtype=torch.int64, device=dev)
    out = torch.empty(200, 16, 512, dtype=torch.bfloat16, device=dev)
    la.prefill(q, cache.cache, cache.tables[0], position, 64, rank=512, out=out)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        la.prefill(q, cache.cache, cache.tables[0], position, 64, rank=512, out=out)
    for at in (0, 700, 2799):
        position.fill_(at)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, la.prefill(q, cache.cache, cache.tables[0], at, 64, rank=512)), at


def test_the_partitions_are_a_knob_the_caller_or_the_tuning_sets():
    # Fewer partitions: the same attention (other sums), fewer partials; the engine's tuned PARTS and PIECE (what crit's
    # kernel build writes beside the module) are what a call without arguments takes, decode and prompt alike.
    cache = Cache(512, 64, 64, [3000, 900], seed=6)
    la = cache.la
    q = _q(16, 128, 576, 8)
    scale = 192 ** -0.5
    default = cache.attend(q, [0, 1], [0, 8], [2990, 890], 8, scale=scale)
    for parts in (1, 4, 16):
        lse = torch.empty(16, 128, device=dev)
        out = cache.attend(q, [0, 1], [0, 8], [2990, 890], 8, scale=scale, lse=lse, partitions=parts)
        for s, start, first in ((0, 0, 2990), (1, 8, 890)):
            cache.check(q, out, lse, s, start, first, 8, scale)

    class Tuning:      # the generated accessor's shape (kernels/crit_kernels/build.py:255-313)
        @staticmethod
        def knobs(structure, key, rows):
            assert structure == "window" and key == {"R": 512, "P": 64, "H": 128, "PAGE": 64, "KIND": 0}
            return {"PARTS": 4, "PIECE": 512}

    four = cache.attend(q, [0, 1], [0, 8], [2990, 890], 8, scale=scale, partitions=4, piece=512)
    la._crit_tuning = Tuning
    try:
        assert la.partitions(torch.device(dev), 128, 512, 64, 64) == 4
        tuned = cache.attend(q, [0, 1], [0, 8], [2990, 890], 8, scale=scale)
        chunk = la.prefill(q[:8], cache.cache, cache.tables[0], 2990, 64, rank=512, scale=scale)
    finally:
        la._crit_tuning = None
    assert torch.equal(tuned, four) and torch.equal(chunk, four[:8])
    assert torch.equal(cache.attend(q, [0, 1], [0, 8], [2990, 890], 8, scale=scale), default)
    for bad in (0, 65):
        with pytest.raises(ValueError):
            cache.attend(q, [0, 1], [0, 8], [2990, 890], 8, partitions=bad)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_write_keeps_every_bit_of_rows_of_the_caches_own_type(dtype):
    # every 16-bit pattern once (NaNs with their payloads and signs, subnormals, both zeros) as latents and rotary keys
    la = module()
    patterns = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
    latent, rope_k = patterns[:49152].reshape(384, 128), patterns[49152:].reshape(512, 32)[:384]
    slots = torch.randperm(400, generator=torch.Generator().manual_seed(5))[:384]
    cache = torch.zeros(25, 16, 160, dtype=dtype, device=dev)
    la.write(latent.to(dev), rope_k.to(dev), slots.to(dev), cache)
    rows = cache.cpu().view(torch.int16).reshape(400, 160)[slots]
    assert torch.equal(rows[:, :128], latent.view(torch.int16)) and torch.equal(rows[:, 128:], rope_k.view(torch.int16))


@pytest.mark.parametrize("source", [torch.float32, torch.bfloat16, torch.float16])
def test_write_stores_the_bytes_and_scales_of_the_reference_rule(source):
    # oracle.latent.write is the reference's torch rule (latent_attention/__init__.py:74-97); the module's write is one
    # HIP launch and must leave the same bytes: rows of zeros (the 1e-30 floor), NaN and infinite inputs, values that
    # saturate, an untouched row, and a skipped slot.
    la = module()
    g = torch.Generator().manual_seed(21)
    n, R, P, page, pages = 37, 128, 32, 16, 6
    latent = torch.randn(n, R, generator=g) * 3
    rope_k = torch.randn(n, P, generator=g) * 40
    latent[3] = 0
    rope_k[4] = 0
    latent[5, 7] = float("nan")
    rope_k[6, 1] = float("inf")
    latent[8, 0] = -0.0
    latent, rope_k = latent.to(source), rope_k.to(source)
    slots = torch.randperm(pages * page, generator=g)[:n]
    for dtype in (torch.bfloat16, torch.float16, torch.float8_e4m3fn):
        coded = dtype == torch.float8_e4m3fn
        want = torch.zeros(pages, page, R + P, dtype=dtype)
        want_scales = torch.zeros(pages, page, 2) if coded else None
        oracle_latent.write(latent, rope_k, slots, want, want_scales)
        got = torch.zeros(pages, page, R + P, dtype=dtype, device=dev)
        got_scales = torch.zeros(pages, page, 2, device=dev) if coded else None
        dropped = slots.clone().to(dev)
        la.write(latent.to(dev), rope_k.to(dev), dropped, got, got_scales)
        raw = torch.uint8 if coded else torch.int16

        def same(a, b):      # bit for bit; a 16-bit NaN that went through a cast only as a NaN (its payload differs
            if coded or source == dtype:      # between torch's own casts); rows of the cache's own type: every bit
                return torch.equal(a.view(raw), b.view(raw))
            nan = torch.isnan(b.float())
            return torch.equal(torch.isnan(a.float()), nan) and torch.equal(a.view(raw)[~nan], b.view(raw)[~nan])
        assert same(got.cpu(), want), dtype
        if coded:
            found, nan = got_scales.cpu(), torch.isnan(want_scales)      # (a NaN row's scale is a NaN, whatever its payload)
            assert torch.equal(torch.isnan(found), nan) and torch.equal(found.view(torch.int32)[~nan], want_scales.view(torch.int32)[~nan])
        # a token whose slot is negative is skipped; strided inputs are read where they lie
        got.zero_()
        dropped[0] = -1
        wide = torch.zeros(n, R + 8, dtype=source, device=dev)
        wide[:, :R] = latent.to(dev)
        la.write(wide[:, :R], rope_k.to(dev), dropped, got, got_scales)
        kept = want.clone().view(-1, R + P)
        kept[slots[0]] = 0
        assert same(got.cpu(), kept.view(pages, page, R + P)), dtype


def test_two_owners_launch_on_two_streams_without_sharing_partials_and_an_outgrown_buffer_outlives_its_graph():
    import crit_amd.paged_kv_attention as pk
    cache = Cache(512, 64, 64, [3000, 900, 2000], seed=31)
    la = cache.la
    q = _q(3, 16, 576, 32)
    rows = torch.tensor([0, 1, 2], dtype=torch.int32, device=dev)
    starts = torch.tensor([0, 1, 2], dtype=torch.int32, device=dev)
    firsts = torch.tensor([2990, 890, 1990], dtype=torch.int64, device=dev)
    args = (cache.cache, cache.tables, rows, starts, firsts, 1, 64)
    serial = la.attend(q, *args, rank=512)
    torch.cuda.synchronize()
    one, two = torch.cuda.Stream(), torch.cuda.Stream()
    out_a = torch.empty_like(serial)
    out_b = [torch.empty_like(serial) for _ in range(6)]
    try:
        with pk.owner("a"), torch.cuda.stream(one):
            la.attend(q, *args, rank=512, out=out_a)      # (the owner's partials exist before the capture)
            one.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=one):
                la.attend(q, *args, rank=512, out=out_a)
        held = pk._holdings[(torch.cuda.current_device(), "a")].latent
        for i in range(6):      # owner a's graph replays on one stream while owner b launches on another
            out_a.zero_()
            with torch.cuda.stream(one):
                graph.replay()
            with pk.owner("b"), torch.cuda.stream(two):
                la.attend(q, *args, rank=512, out=out_b[i])
        torch.cuda.synchronize()
        assert torch.equal(out_a, serial)
        assert all(torch.equal(o, serial) for o in out_b)
        assert pk._holdings[(torch.cuda.current_device(), "b")].latent.data_ptr() != held.data_ptr()
        # owner a outgrows its buffer with a larger eager launch: the graph still replays into the old one, which is
        # kept, so memory allocated afterwards is not what the replay writes
        wide_q = _q(24, 128, 576, 33)
        with pk.owner("a"):
            cache.attend(wide_q, [0, 1, 2], [0, 8, 16], [2990, 890, 1990], 8)
            grown = pk._holdings[(torch.cuda.current_device(), "a")].latent
        assert grown.data_ptr() != held.data_ptr() and grown.numel() > held.numel()
        fresh = [torch.full((held.numel(),), 5.0, device=dev) for _ in range(4)]
        out_a.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_a, serial)
        assert all(bool((t == 5.0).all()) for t in fresh)
        del graph
    finally:
        pk.release("a")
        pk.release("b")


@pytest.mark.parametrize("coded", [0, 2, 1])
def test_many_heads_units_longer_than_the_lanes_hold_tiles_for_and_rows_beyond_the_ranked_launches(coded):
    # A unit of more than 64 tiles of 32 positions refills the lanes' table of tiles on the way (one partition over
    # 9,000 positions is 282 tiles); a launch of more than 64 batch rows keeps the caller's order instead of ranking the
    # rows by length, and one of fewer than 16 deals (row, partition) pairs, not whole rows, to the XCDs. 16-bit rows,
    # and E4M3 rows with two scales a position or one.
    kind = dict(dtype=torch.float8_e4m3fn, scales=coded) if coded else {}
    long = Cache(512, 64, 64, [9000], seed=51, **kind)
    q = _q(1, 128, 576, 52)
    lse = torch.empty(1, 128, device=dev)
    for parts, piece in ((1, 512), (3, 512), (5, 96)):
        out = long.attend(q, [0], [0], [8999], 1, lse=lse, partitions=parts, piece=piece)
        long.check(q, out, lse, 0, 0, 8999, 1, 576 ** -0.5)
    lengths = [40 + 37 * (i % 9) for i in range(70)]
    many = Cache(512, 64, 16, lengths, seed=53, **kind)
    q = _q(70, 128, 576, 54)
    rows, starts, firsts = list(range(70)), list(range(70)), [n - 1 for n in lengths]
    together = many.attend(q, rows, starts, firsts, 1)
    for s_ in (0, 8, 33, 69):
        many.check(q, together, None, s_, s_, firsts[s_], 1, 576 ** -0.5)
        assert torch.equal(many.attend(q[s_:s_ + 1], [s_], [0], [firsts[s_]], 1)[0], together[s_])
    assert torch.equal(many.attend(q[:20], rows[:20], starts[:20], firsts[:20], 1), together[:20])
