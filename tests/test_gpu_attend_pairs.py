"""Decode and verify windows over 64-wide heads, which the bandwidth kernel reads in pairs of adjacent KV heads as
128-wide ones (an even number of KV heads, pages of a power of two from 16 positions up): every page kind against float64
attention over the stored values at GQA groups of 1, 2, 4 and 6 and at head counts whose pairs fill a wavefront's tile
(two pairs) or do not (one pair, three pairs); an FP8 pool's multipliers a KV head and the row scales of the row-scaled
kinds follow each query row's own head; a token's bits alone, in a window, fused and split; a chain of parents is the
causal window; sliding windows and sinks; a long row of many partitions; graphs. An odd number of KV heads, or pages the
kernel does not walk, stay on the generic kernel and are checked beside them."""
import pytest
import torch

from tests.support import KINDS, Cache, rand_q

pytestmark = pytest.mark.gpu
dev = "cuda"
ATOL, RTOL = 8e-3, 2e-2

# (query heads, KV heads): one pair, two pairs (one wavefront's tile), three pairs, four pairs; groups of 6, 4, 2, 1, 4
HEADS = [(12, 2), (16, 4), (12, 6), (8, 8), (32, 8)]


def close(got, want, what):
    torch.testing.assert_close(got.double().cpu(), want, atol=ATOL, rtol=RTOL, msg=str(what))


def close_lse(got, want, what):
    torch.testing.assert_close(got.double().cpu(), want, atol=1e-3, rtol=1e-4, msg=str(what))


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("hq,hkv", HEADS)
@pytest.mark.parametrize("fused", [False, True])
def test_pairs_of_narrow_heads_match_float64_attention(kind, hq, hkv, fused):
    # the heads' magnitudes differ (a head's scores must not feel its pair's keys), windows end at page boundaries
    cache = Cache(kind, hkv, 64, 64, 16, [130, 64, 1, 517], seed=hq + hkv)
    loud = torch.linspace(0.3, 3.0, hkv, device=dev)[None, :, None]
    for s, n in enumerate(cache.lengths):
        g = torch.Generator().manual_seed(100 + s)
        keys, values = torch.randn(n, hkv, 64, generator=g).to(dev) * loud, torch.randn(n, hkv, 64, generator=g).to(dev) * loud.flip(1)
        cache.write(s, 0, keys, values)
    windows = [(0, 125, 5), (1, 59, 5), (2, 0, 1), (3, 400, 3)]
    starts = [5 * i for i in range(4)]
    q = rand_q(20, hq, 64, 3)
    lse = torch.full((20, hq), 7.0, device=dev)
    out = cache.attend(q, [w[0] for w in windows], starts, [w[1] for w in windows], 5, lse=lse, fused=fused,
                       counts=torch.tensor([w[2] for w in windows], dtype=torch.int32, device=dev))
    for (s, first, count), start in zip(windows, starts):
        want, want_lse = cache.want(q[start:start + count], s, first, count)
        close(out[start:start + count], want, (s, first))
        close_lse(lse[start:start + count], want_lse, (s, first))
    assert bool((lse[11:15] == 7.0).all()) and bool((lse[18:] == 7.0).all())      # only the rows' tokens are written


def test_an_fp8_pools_multipliers_follow_each_query_rows_own_head():
    hq, hkv = 16, 4
    per_head = torch.tensor([[0.010, 0.035, 0.020, 0.050], [0.040, 0.015, 0.030, 0.012]])      # keys', then values'
    cache = Cache("fp8", hkv, 64, 64, 16, [300, 77], multipliers=per_head)
    q = rand_q(6, hq, 64, 5)
    lse = torch.empty(6, hq, device=dev)
    for fused in (False, True):
        out = cache.attend(q, [0, 1], [0, 3], [290, 70], 3, lse=lse, fused=fused)
        for s, start, first in ((0, 0, 290), (1, 3, 70)):
            want, want_lse = cache.want(q[start:start + 3], s, first, 3)
            close(out[start:start + 3], want, (fused, s))
            close_lse(lse[start:start + 3], want_lse, (fused, s))


@pytest.mark.parametrize("kind", ["bf16", "fp8", "fp8:row", "int8"])
@pytest.mark.parametrize("hq,hkv", [(12, 2), (32, 8), (12, 6)])
def test_a_tokens_bits_are_its_own_alone_in_a_window_fused_or_split(kind, hq, hkv):
    cache = Cache(kind, hkv, 64, 64, 16, [700, 300, 2100], seed=2)
    q = rand_q(24, hq, 64, 5)
    rows, starts, firsts = [0, 1, 2], [0, 8, 16], [690, 290, 2090]
    together = cache.attend(q, rows, starts, firsts, 8)
    assert torch.equal(cache.attend(q, rows, starts, firsts, 8, fused=True), together)
    for r, start, first in zip(rows, starts, firsts):
        for c in (0, 3, 7):
            alone = cache.attend(q[start + c:start + c + 1], [r], [0], [first + c], 1)
            assert torch.equal(alone[0], together[start + c]), (r, c)
        assert torch.equal(cache.attend(q[start:start + 8], [r], [0], [first], 8), together[start:start + 8]), r
    # a window twice as wide with the same live columns, the rows in another order
    wider = cache.attend(q, rows[::-1], starts[::-1], firsts[::-1], 16, counts=torch.full((3,), 8, dtype=torch.int32, device=dev))
    assert torch.equal(wider, together)


@pytest.mark.parametrize("kind", ["bf16", "int8"])
def test_a_chain_of_parents_is_the_causal_window_and_a_tree_sees_its_ancestors(kind):
    hq, hkv = 16, 4
    cache = Cache(kind, hkv, 64, 64, 16, [80], seed=4)
    q = rand_q(5, hq, 64, 11)
    plain = cache.attend(q, [0], [0], [70], 5)
    chain = torch.tensor([-1, 0, 1, 2, 3], dtype=torch.int32, device=dev)
    assert torch.equal(cache.attend(q, [0], [0], [70], 5, parents=chain), plain)
    tree = torch.tensor([-1, 0, 0, 1, 2], dtype=torch.int32, device=dev)
    lse = torch.empty(5, hq, device=dev)
    out = cache.attend(q, [0], [0], [70], 5, parents=tree, lse=lse)
    want, want_lse = cache.want(q, 0, 70, 5, parents=tree.cpu())
    close(out, want, "tree")
    close_lse(lse, want_lse, "tree")


@pytest.mark.parametrize("kind", ["bf16", "fp8:row"])
def test_sliding_windows_and_sinks(kind):
    hq, hkv = 12, 6
    cache = Cache(kind, hkv, 64, 64, 32, [1500], seed=6)
    q = rand_q(4, hq, 64, 7)
    lse = torch.empty(4, hq, device=dev)
    for window in (1, 100, 1000):
        out = cache.attend(q, [0], [0], [1400], 4, sliding=window, lse=lse)
        want, want_lse = cache.want(q, 0, 1400, 4, sliding=window)
        close(out, want, window)
        close_lse(lse, want_lse, window)
    assert torch.equal(cache.attend(q, [0], [0], [1400], 4, sliding=5000), cache.attend(q, [0], [0], [1400], 4))
    sinks = torch.linspace(-2.0, 2.0, hq, device=dev)
    plain = cache.attend(q, [0], [0], [1400], 4, lse=lse)
    weight = torch.exp(lse) / (torch.exp(lse) + torch.exp(sinks)[None, :])
    with_sinks = cache.attend(q, [0], [0], [1400], 4, sinks=sinks)
    torch.testing.assert_close(with_sinks.float(), plain.float() * weight[..., None], atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("kind", ["bf16", "fp8"])
def test_a_long_row_of_many_partitions_merges_to_the_fused_launchs_bits(kind):
    hq, hkv, n = 32, 8, 40000
    cache = Cache(kind, hkv, 64, 64, 16, [n + 2], seed=8, scale=0.5)
    q = rand_q(2, hq, 64, 9)
    lse = torch.empty(2, hq, device=dev)
    split = cache.attend(q, [0], [0], [n], 2, lse=lse)
    assert torch.equal(cache.attend(q, [0], [0], [n], 2, fused=True), split)
    want, want_lse = cache.want(q, 0, n, 2)
    close(split, want, "long row")
    close_lse(lse, want_lse, "long row")


def test_one_graph_replays_at_every_length():
    hq, hkv = 16, 4
    cache = Cache("bf16", hkv, 64, 64, 16, [3000], seed=10)
    q = rand_q(1, hq, 64, 12).bfloat16()
    first = torch.tensor([10], dtype=torch.int64, device=dev)
    zero = torch.zeros(1, dtype=torch.int32, device=dev)
    out = torch.empty(1, hq, 64, dtype=torch.bfloat16, device=dev)
    read = lambda: cache.pk.attend(q, cache.k, cache.v, "bf16", cache.tables, zero, zero, first, 1, 16, out=out)
    read()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        read()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            read()
    for at in (0, 15, 16, 1000, 2999):
        first.fill_(at)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, cache.attend(q, [0], [0], [at], 1)), at


@pytest.mark.parametrize("kind", ["bf16", "fp8:row"])
@pytest.mark.parametrize("hq,hkv,page", [(12, 3, 16), (12, 2, 48), (5, 1, 16)])
def test_what_does_not_pair_stays_on_the_generic_kernel(kind, hq, hkv, page):
    # an odd number of KV heads, pages that are no power of two: the same answers from the other kernel
    cache = Cache(kind, hkv, 64, 64, page, [333, 90], seed=3)
    q = rand_q(6, hq, 64, 13)
    out = cache.attend(q, [0, 1], [0, 3], [320, 80], 3)
    assert torch.equal(cache.attend(q, [0, 1], [0, 3], [320, 80], 3, fused=True), out)
    for s, start, first in ((0, 0, 320), (1, 3, 80)):
        close(out[start:start + 3], cache.want(q[start:start + 3], s, first, 3)[0], (s, first))
