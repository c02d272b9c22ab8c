"""Keys derived from the value rows on read (attend's and prefill's derive=): a pool of value pages only, each row read as
its value and, normed and rotated, as its key. Against float64 attention whose keys are derived in float64 on the host
(oracle.attend.derived_keys) from the rows as the pages store them: every page kind, every head width, GQA, a rotation
over part of the head (any even width) and no norm weight, positions at page boundaries, a long row, a sliding window, sinks, trees; a
column's bits the same alone, in any window, fused or split; a prompt chunk's tokens the same positions decoded; what the
reference refuses is refused. Mirrors the reference's tests/test_derived_keys.py at its tolerances (8e-3 + 2e-2 |ref|,
log-sum-exp 1e-3)."""
import itertools

import pytest
import torch

from oracle import attend as oracle_attend
from tests.support import KINDS, STORE, kernels, rand_q

pytestmark = pytest.mark.gpu
dev = "cuda"
EPS = 1e-6


class ValuePool:
    """One layer of a pool that keeps value rows only: `lengths[s]` positions of sequence s written through the module's
    own append into pages handed out from a shuffled list (one spare page a sequence, so windows may end on a page's
    last slot). The rows' magnitudes vary by position and head: the norm takes them to one, so a derived key is not its
    row."""

    def __init__(self, kind, hkv, d, page, lengths, seed=0, multiplier=0.03):
        self.pk = kernels()
        self.kind, self.hkv, self.d, self.page = kind, hkv, d, page
        self.multipliers = (1.0, multiplier if kind == "fp8" else 1.0)
        draw = torch.Generator().manual_seed(seed)
        each = 1 + max((n + page - 1) // page for n in lengths)
        total = each * len(lengths) + 3
        shuffled = torch.randperm(total, generator=draw)[:each * len(lengths)]
        self.tables = shuffled.reshape(len(lengths), each).to(device=dev, dtype=torch.int32)
        self.v = torch.zeros(total, page, hkv, d, dtype=STORE[kind], device=dev)
        self.vs = torch.zeros(total, page, hkv, dtype=torch.float32, device=dev) if kind in ("fp8:row", "int8") else None
        for s, n in enumerate(lengths):
            loud = 0.5 + 3.0 * torch.rand(n, hkv, 1, generator=draw)
            rows = torch.randn(n, hkv, d, generator=draw) * loud
            self.pk.write(None, rows.to(dev), self.slot_of(s, torch.arange(n, device=dev)), None, self.v, kind, None, self.vs,
                          multipliers=self.multipliers)

    @property
    def q_dtype(self):
        return torch.float16 if self.kind == "fp16" else torch.bfloat16

    def slot_of(self, s, positions):
        pages = self.tables[s].long()[torch.div(positions, self.page, rounding_mode="floor")]
        return pages * self.page + positions % self.page

    def stored(self, s, n):
        """Positions 0 .. n - 1 of sequence s as the pages hold them (codes times their scale or multiplier): float64
        [n][hkv][d] on the CPU."""
        at = self.slot_of(s, torch.arange(n, device=dev))
        rows = self.v.reshape(-1, self.hkv, self.d)[at].double() * self.multipliers[1]
        if self.vs is not None:
            rows = rows * self.vs.reshape(-1, self.hkv)[at].double().unsqueeze(-1)
        return rows.cpu()

    def attend(self, q, rows, starts, firsts, columns, derive, **kw):
        ints = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
        return self.pk.attend(q.to(self.q_dtype), None, self.v, self.kind, self.tables, ints(rows), ints(starts),
                              torch.tensor(firsts, dtype=torch.int64, device=dev), columns, self.page, value_scales=self.vs,
                              multipliers=self.multipliers, derive=derive, **kw)

    def check(self, q, out, lse, derive, s, start, first, count, sliding=0, sinks=None, seen_of=None):
        """Tokens start .. start + count - 1 of out (and lse) against float64 attention of window row (s, first, count)
        over keys derived in float64 from the stored rows."""
        values = self.stored(s, first + count)
        weight = None if derive[0] is None else derive[0].cpu()
        keys = oracle_attend.derived_keys(values, weight, derive[1], derive[2].cpu(), derive[3])
        queries = q.to(self.q_dtype).double().cpu()
        positions = torch.arange(first + count)
        for c in range(count):
            own = first + c
            seen = seen_of(c, positions) if seen_of is not None else positions <= own
            if sliding:
                seen = seen & (positions > own - sliding)
            want, want_lse = oracle_attend.reference(queries[start + c], keys, values, seen, self.d ** -0.5)
            if sinks is not None:      # a sink logit a head joins the softmax's denominator
                with_sink = torch.logaddexp(want_lse, sinks.double().cpu())
                want, want_lse = want * torch.exp(want_lse - with_sink).unsqueeze(-1), with_sink
            torch.testing.assert_close(out[start + c].double().cpu(), want, atol=8e-3, rtol=2e-2)
            if lse is not None:
                torch.testing.assert_close(lse[start + c].double().cpu(), want_lse, atol=1e-3, rtol=1e-4)


def derive_for(pk, d, rotary_dim, weighted=True, seed=5, packed=True):
    """A layer's derive=: inverse frequencies of base 10,000 over the rotary width, a norm weight around 1 (or none);
    packed by pk.derive() or left a plain tuple."""
    exponents = torch.arange(0, rotary_dim, 2, dtype=torch.float64) / rotary_dim
    freqs = torch.pow(torch.tensor(10000.0, dtype=torch.float64), -exponents).float().to(dev)
    weight = None
    if weighted:
        weight = (1.0 + 0.3 * torch.randn(d, generator=torch.Generator().manual_seed(seed))).to(dev)
    given = (weight, EPS, freqs, rotary_dim)
    return pk.derive(*given) if packed else given


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("hq,hkv,d,rot,weighted", [(8, 2, 128, 128, True), (12, 2, 64, 64, True), (8, 4, 128, 64, False),
                                                   (16, 2, 64, 32, True), (3, 1, 128, 16, True),
                                                   # rotary widths whose halves are not whole lanes of 8 elements
                                                   # (12, 1, 25 and 50 apart), and the other head widths
                                                   (8, 2, 128, 24, True), (4, 2, 64, 2, False), (8, 2, 64, 50, True),
                                                   (4, 2, 32, 32, True), (4, 1, 16, 10, False), (6, 2, 256, 100, True),
                                                   (4, 4, 256, 256, False)])
@pytest.mark.parametrize("fused", [False, True])
def test_windows_with_derived_keys_match_float64_attention(kind, hq, hkv, d, rot, weighted, fused):
    # four window rows in one launch: windows that start and end at page boundaries (15 / 16, 31 / 32), a sequence of a
    # single position, a window deep in a longer sequence
    windows = [(0, 127, 5), (1, 31, 5), (2, 0, 1), (3, 400, 3)]      # (sequence, first position, columns)
    cache = ValuePool(kind, hkv, d, 16, [140, 64, 1, 517])
    derive = derive_for(cache.pk, d, rot, weighted)
    starts = [5 * i for i in range(len(windows))]
    q = rand_q(5 * len(windows), hq, d, 3)
    lse = torch.empty(q.shape[0], hq, device=dev)
    out = cache.attend(q, [w[0] for w in windows], starts, [w[1] for w in windows], 5, derive, lse=lse, fused=fused,
                       counts=torch.tensor([w[2] for w in windows], dtype=torch.int32, device=dev))
    for (s, first, count), start in zip(windows, starts):
        cache.check(q, out, lse, derive, s, start, first, count)


@pytest.mark.parametrize("kind", ["bf16", "fp8:row", "int8", "fp8"])
def test_a_long_row_and_a_sliding_windows_edges_with_sinks(kind):
    hq, hkv, d, n = 8, 2, 128, 4096
    cache = ValuePool(kind, hkv, d, 64, [n + 4], seed=2)
    derive = derive_for(cache.pk, d, 128, packed=False)      # (a plain tuple is packed at the call)
    q = rand_q(4, hq, d, 7)
    sinks = torch.tensor([0.5, -1.0, float("-inf"), 2.0, 0.0, 1.5, -3.0, 0.25], device=dev)
    lse = torch.empty(4, hq, device=dev)
    out = cache.attend(q, [0], [0], [n], 4, derive, lse=lse, sinks=sinks)
    cache.check(q, out, lse, derive, 0, 0, n, 4, sinks=sinks)
    out = cache.attend(q, [0], [0], [n], 4, derive, lse=lse, sliding=130)
    cache.check(q, out, lse, derive, 0, 0, n, 4, sliding=130)


@pytest.mark.parametrize("kind", ["bf16", "fp8:row"])
def test_a_columns_bits_are_its_own_alone_in_any_window_fused_or_split(kind):
    hq, hkv, d = 8, 2, 128
    cache = ValuePool(kind, hkv, d, 16, [300, 90], seed=3)
    derive = derive_for(cache.pk, d, 64)
    q = rand_q(8, hq, d, 9)
    out = cache.attend(q, [0, 1], [0, 4], [290, 80], 4, derive)
    fused = cache.attend(q, [0, 1], [0, 4], [290, 80], 4, derive, fused=True)
    assert torch.equal(out, fused)
    for start, s, first in ((2, 0, 292), (4, 1, 80), (7, 1, 83)):
        alone = cache.attend(q[start:start + 1], [s], [0], [first], 1, derive)
        assert torch.equal(alone[0], out[start])
    wider = cache.attend(q, [1, 0], [4, 0], [80, 290], 8, derive, counts=torch.tensor([4, 4], dtype=torch.int32, device=dev))
    assert torch.equal(wider, out)


def test_a_tree_with_derived_keys_sees_its_ancestors():
    hq, hkv, d = 4, 1, 64
    cache = ValuePool("bf16", hkv, d, 16, [70], seed=4)
    derive = derive_for(cache.pk, d, 64)
    q = rand_q(5, hq, d, 11)
    parents = torch.tensor([-1, 0, 0, 1, 2], dtype=torch.int32, device=dev)
    lse = torch.empty(5, hq, device=dev)
    out = cache.attend(q, [0], [0], [65], 5, derive, lse=lse, parents=parents)
    paths = {0: {0}, 1: {0, 1}, 2: {0, 2}, 3: {0, 1, 3}, 4: {0, 2, 4}}
    cache.check(q, out, lse, derive, 0, 0, 65, 5,
                seen_of=lambda c, n: (n < 65) | torch.tensor([int(x) - 65 in paths[c] for x in n]))


@pytest.mark.parametrize("kind,d,rot", [("bf16", 128, 128), ("fp8", 64, 64), ("int8", 32, 6), ("fp8:row", 256, 200)])
def test_a_prompt_chunk_with_derived_keys_is_its_positions_decoded(kind, d, rot):
    pk = kernels()
    hq, hkv, T, prefix = 8, 2, 150, 37
    cache = ValuePool(kind, hkv, d, 16, [prefix + T], seed=6)
    derive = derive_for(pk, d, rot)
    q = rand_q(T, hq, d, 13).to(cache.q_dtype)
    lse = torch.empty(T, hq, device=dev)
    out = pk.prefill(q, None, cache.v, kind, cache.tables[0], prefix, 16, value_scales=cache.vs, multipliers=cache.multipliers,
                     lse=lse, derive=derive)
    for t in (0, 63, 64, 149):
        cache.check(q, out, lse, derive, 0, t, prefix + t, 1)
        one = cache.attend(q[t:t + 1], [0], [0], [prefix + t], 1, derive)
        assert torch.equal(one[0], out[t])
    on_device = pk.prefill(q, None, cache.v, kind, cache.tables[0], torch.tensor([prefix], device=dev), 16,
                           value_scales=cache.vs, multipliers=cache.multipliers, derive=derive)
    assert torch.equal(on_device, out)


def _check_with_fresh(cache, q, out, lse, derive, fv, at, split, tokens, window=0):
    """Tokens of a chunk at position `at` whose positions from at + split on are the fresh value rows fv[split:]: float64
    attention over the stored rows then the fresh ones, every key derived from its row."""
    weight, eps, freqs, rot = derive[:4]
    values = torch.cat([cache.stored(0, at + split), fv[split:].double().cpu()])
    keys = oracle_attend.derived_keys(values, None if weight is None else weight.cpu(), eps, freqs.cpu(), rot)
    qd = q.double().cpu()
    n = torch.arange(at + fv.shape[0])
    for t in tokens:
        seen = n <= at + t
        if window:
            seen = seen & (n > at + t - window)
        want, want_lse = oracle_attend.reference(qd[t], keys, values, seen, cache.d ** -0.5)
        torch.testing.assert_close(out[t].double().cpu(), want, atol=8e-3, rtol=2e-2, msg=f"{at} {split} {window} {t}")
        torch.testing.assert_close(lse[t].double().cpu(), want_lse, atol=1e-3, rtol=1e-4, msg=f"lse {at} {split} {window} {t}")


@pytest.mark.parametrize("kind", KINDS)
def test_a_fused_chunk_derives_its_fresh_rows_keys(kind):
    # A chunk of 100 tokens read as two window rows (64 + 36 columns) of one fused launch; its own positions come as
    # fresh value rows with no keys: a fresh position's key is derived from its fresh row as a stored position's is from
    # its stored row. The chunk's position and the first fresh position are device tensors (no host value in the launch).
    tokens, cut = 100, 64
    cache = ValuePool(kind, 2, 128, 16, [700], multiplier=0.04)
    pk = cache.pk
    derive = derive_for(pk, 128, 128)
    q = rand_q(tokens, 8, 128, 22).to(cache.q_dtype)
    fv = torch.randn(tokens, 2, 128, generator=torch.Generator().manual_seed(21)).to(dev).to(cache.q_dtype)
    shift = torch.zeros(1, dtype=torch.int64, device=dev)
    fresh_from = torch.zeros(1, dtype=torch.int64, device=dev)
    window = dict(counts=torch.tensor([cut, tokens - cut], dtype=torch.int32, device=dev), value_scales=cache.vs,
                  multipliers=cache.multipliers, fused=True, derive=derive)
    same_table = torch.zeros(2, dtype=torch.int32, device=dev)
    first_tokens = torch.tensor([0, cut], dtype=torch.int32, device=dev)

    def read(at, fresh, lse=None):
        firsts = torch.tensor([at, at + cut], dtype=torch.int64, device=dev)
        return pk.attend(q, None, cache.v, kind, cache.tables, same_table, first_tokens, firsts, 64, 16, lse=lse, fresh=fresh, **window)

    for at, split in itertools.product((0, 200, 600), (0, 37, 100)):
        shift.fill_(at)
        fresh_from.fill_(at + split)
        lse = torch.empty(tokens, 8, device=dev)
        out = read(at, (None, fv, shift, fresh_from), lse)
        _check_with_fresh(cache, q, out, lse, derive, fv, at, split, (0, 41, 99))
    with pytest.raises(ValueError, match="fresh keys None"):
        read(0, (fv, fv, shift, fresh_from))


@pytest.mark.parametrize("kind", KINDS)
def test_a_prompt_chunk_derives_its_fresh_rows_keys_with_a_sliding_window(kind):
    cache = ValuePool(kind, 2, 128, 16, [700])
    pk = cache.pk
    derive = derive_for(pk, 128, 64)
    g = torch.Generator().manual_seed(21)
    q = rand_q(100, 8, 128, 22).to(cache.q_dtype)
    fv = torch.randn(100, 2, 128, generator=g).to(dev).to(cache.q_dtype)
    for at, split, window in ((0, 0, 0), (200, 37, 0), (600, 100, 0), (200, 37, 50)):
        lse = torch.empty(100, 8, device=dev)
        out = pk.prefill(q, None, cache.v, kind, cache.tables[0], at, 16, value_scales=cache.vs, multipliers=cache.multipliers,
                         lse=lse, fresh=(None, fv, at + split), derive=derive, sliding=window)
        _check_with_fresh(cache, q, out, lse, derive, fv, at, split, (0, 41, 99), window)


def test_what_derived_keys_do_not_take_is_refused():
    pk = kernels()
    cache = ValuePool("bf16", 2, 128, 16, [40])
    derive = derive_for(pk, 128, 128)
    q = rand_q(1, 8, 128, 1)
    with pytest.raises(ValueError, match="flash structures"):
        cache.attend(q, [0], [0], [39], 1, derive, flash=True)
    with pytest.raises(ValueError, match="block lists"):
        cache.attend(q, [0], [0], [39], 1, derive, blocks=torch.zeros(1, 1, dtype=torch.int32, device=dev), block_size=16)
    with pytest.raises(ValueError, match="key_pages None"):
        pk.attend(q.bfloat16(), cache.v, cache.v, "bf16", cache.tables, torch.zeros(1, dtype=torch.int32, device=dev),
                  torch.zeros(1, dtype=torch.int32, device=dev), torch.tensor([39], device=dev), 1, 16, derive=derive)
    with pytest.raises(ValueError, match="int8_qk"):
        pk.prefill(q.bfloat16(), None, cache.v, "bf16", cache.tables[0], 39, 16, derive=derive, int8_qk=True)
    freqs = derive.freqs
    for bad, match in (((None, EPS, freqs, 130), "rotary_dim"), ((None, EPS, freqs[:3], 128), "freqs"),
                       ((torch.ones(64, device=dev), EPS, freqs, 128), "weight"), ((None, -1.0, freqs, 128), "eps")):
        with pytest.raises(ValueError, match=match):
            cache.attend(q, [0], [0], [39], 1, bad)
    with pytest.raises(ValueError, match="rotary_dim"):      # (any even width is taken; an odd one is not a width)
        cache.attend(q, [0], [0], [39], 1, (None, EPS, freqs[:4], 9))
    # a plain tuple needs packing, which a capture cannot do; a Derive made by derive() holds its table
    assert derive.table.numel() == 64 + 128
