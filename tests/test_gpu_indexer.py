"""crit_amd.sparse_indexer on the GPU against the float64 oracle (oracle.indexer), written from the operation's
definition (inference/attention-state/code/sparse_index.py of the reference):

    score[t][s] = sum over heads of weight[t][h] * scale * max(0, q[t][h] . key[s])   for s < ends[t], else -inf
    picks[t]    = the positions of the k largest scores below ends[t], ascending, then -1; ties to the lower position,
                  a NaN below every number

Scores over 16-bit and E4M3 keys at the head counts and widths the module takes, causal ends; picks with ties, fewer
valid keys than k, empty rows, NaN and -inf, rows of every length class the select kernels are built for; a token's bits
the same alone and beside other tokens; select in groups the same as one call; keys read in place; captured calls; what
the module refuses. The cases cover those of the reference's tests/test_sparse_indexer.py, at its bounds."""
import itertools

import numpy as np
import pytest
import torch

from crit_amd import sparse_indexer as si
from oracle import indexer as ref

pytestmark = pytest.mark.gpu
dev = torch.device("cuda")
NAN, NINF = float("nan"), float("-inf")


def compressed(rows, e4m3):
    """Key rows [n][D] (16-bit, on the device) as the index keeps them: as they are, or E4M3 codes with one FP32 scale a
    key (amax / 448, at least 1e-30). Returns (keys, scales or None, the FP32 values the keys stand for)."""
    if not e4m3:
        return rows, None, rows.float()
    scales = (rows.float().abs().amax(dim=1) / 448.0).clamp_min(1e-30)
    codes = (rows.float() / scales[:, None]).to(torch.float8_e4m3fn)
    return codes, scales, codes.float() * scales[:, None]


class Call:
    """The operands of one scores / select call: `tokens` query tokens of `heads` heads over `n` keys of `width`."""

    def __init__(self, tokens, heads, width, n, seed=0, e4m3=False, dtype=torch.bfloat16):
        g = torch.Generator().manual_seed(7919 * seed + 13)
        rows = torch.empty(n, width).normal_(0.0, 0.5, generator=g).to(dev).to(dtype)
        self.q = torch.empty(tokens, heads, width).normal_(0.0, 0.5, generator=g).to(dev).to(dtype)
        self.w = (torch.empty(tokens, heads).normal_(generator=g) / heads ** 0.5).to(dev)
        ends = (torch.rand(tokens, generator=g) * (n + 1)).long().clamp_(max=n)      # causal ends anywhere in 0 .. n
        ends[0] = n                                                                    # (one token sees every key)
        self.ends = ends.to(torch.int32).to(dev)
        self.keys, self.scales, self.values = compressed(rows, e4m3)
        self.scale = width ** -0.5

    def scores(self, tokens=slice(None), **kw):
        return si.scores(self.q[tokens], self.keys, self.w[tokens], self.ends[tokens], key_scales=self.scales, **kw)

    def exact(self, absolute=False):
        """The oracle's scores in float64 [tokens][n]; absolute: of the operands' magnitudes (an error bound's base)."""
        f = (lambda x: x.abs()) if absolute else (lambda x: x)
        return ref.sparse_scores(f(self.q).double().cpu().numpy(), f(self.values).double().cpu().numpy(),
                                 f(self.w).double().cpu().numpy(), self.ends.cpu().numpy(), self.scale)


def exact_picks(scores, ends, k):
    return torch.from_numpy(ref.sparse_index(scores.double().cpu().numpy(), ends.cpu().numpy(), k))


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device=dev)


def same_bits(a, b):
    return torch.equal(a.view(torch.int32), b.view(torch.int32))


SHAPES = [(64, 128), (32, 64), (16, 256), (8, 128), (128, 256), (1, 64)]


@pytest.mark.parametrize("heads,width,e4m3,dtype", [(h, d, e, t) for (h, d), e, t in
                                                    itertools.product(SHAPES, (False, True), (torch.bfloat16, torch.float16))])
def test_scores_match_the_oracle(heads, width, e4m3, dtype):
    call = Call(37, heads, width, 1000, seed=heads + width, e4m3=e4m3, dtype=dtype)
    got = call.scores().cpu().numpy()
    want = call.exact()
    # FP32 sums of exact 16-bit products: within 1e-4 of the sum of the terms' magnitudes (the reference's bound)
    slack = call.exact(absolute=True) * 1e-4 + 1e-6
    seen = np.isfinite(want)
    assert np.array_equal(seen, np.isfinite(got)), "the causal ends"
    assert (got[~seen] == -np.inf).all()
    assert (np.abs(got.astype(np.float64)[seen] - want[seen]) <= slack[seen]).all()


@pytest.mark.parametrize("heads,width,e4m3,n", [(64, 128, False, 700), (8, 64, True, 900), (128, 256, False, 900), (1, 64, False, 333)])
def test_a_tokens_scores_are_its_own(heads, width, e4m3, n):
    call = Call(33, heads, width, n, seed=3 + heads, e4m3=e4m3)
    together = call.scores()
    assert same_bits(call.scores(), together), "a second launch"
    for t in (0, 1, 16, 32):
        assert same_bits(call.scores(slice(t, t + 1))[0], together[t]), t
    # the block of keys a workgroup takes follows the launch's size: forty times the tokens, the same bits
    many = si.scores(call.q.repeat(40, 1, 1), call.keys, call.w.repeat(40, 1), call.ends.repeat(40), key_scales=call.scales)
    assert same_bits(many[33 * 7:33 * 8], together)


def test_scores_into_a_wider_out_and_strided_queries():
    call = Call(6, 16, 128, 250, seed=21)
    want = call.scores()
    wide = torch.full((8, 300), 7.0, device=dev)
    call.scores(out=wide)
    assert torch.equal(wide[:6, :250], want) and bool((wide[:, 250:] == 7.0).all()) and bool((wide[6:] == 7.0).all())
    big = torch.zeros(6, 16, 256, dtype=call.q.dtype, device=dev)
    big[:, :, :128] = call.q
    assert torch.equal(si.scores(big[:, :, :128], call.keys, call.w, call.ends), want)


def tied_rows(rows, n, seed, nans=False):
    """Score rows for the select: normal draws with a third of the columns set to one value (ties across the k-th),
    optionally NaNs and -inf sprinkled in."""
    g = torch.Generator().manual_seed(seed)
    s = torch.empty(rows, n).normal_(generator=g)
    s[:, torch.randperm(n, generator=g)[:n // 3]] = 0.0
    if nans:
        s[:, torch.randperm(n, generator=g)[:max(1, n // 50)]] = NAN
        s[:, torch.randperm(n, generator=g)[:max(1, n // 40)]] = NINF
    return s


@pytest.mark.parametrize("n,k", [(5000, 512), (700, 64), (300, 512), (1, 1), (4097, 2048)])
def test_topk_picks_the_oracles_positions(n, k):
    s = tied_rows(9, n, seed=n + k)
    s[2] = 1.0      # a row of nothing but ties
    s = s.to(dev)
    # ends: everything, one short, fewer than k, none, k exactly, one
    ends = i32([n, n - 1, n, k // 2, 0, max(1, n - 300), k, n, 1]).clamp(0, n)
    assert torch.equal(si.topk(s, ends, k).long().cpu(), exact_picks(s, ends, k))


@pytest.mark.parametrize("row,k,picks", [
    ([1.0, NAN, NINF, 2.0, NAN], 4, [0, 1, 2, 3]),      # 2, 1, -inf, then the first NaN
    ([1.0, NAN, NINF, 2.0, NAN], 3, [0, 2, 3]),
    ([0.0, -0.0, 0.0, -0.0, -1.0], 2, [0, 1]),          # the zeros tie whatever their sign
    ([NAN, NAN, NAN, NAN, NAN], 2, [0, 1]),
    ([NINF, 3.0, NINF, 3.0, 3.0], 2, [1, 3]),
])
def test_a_nan_ranks_below_every_number(row, k, picks):
    s = torch.tensor([row], device=dev)
    assert si.topk(s, i32([len(row)]), k).tolist() == [picks]


# (rows of 9,000, 13,000, 20,000 and 30,000: each of the element counts a thread of the kernel that holds a row is built
# for; 128 rows or more of up to 64,512: a workgroup holds such a row whole)
@pytest.mark.parametrize("n,k,t", [(200000, 512, 1), (60000, 4096, 2), (8192, 512, 3), (5, 512, 1), (33000, 16, 4),
                                   (4096, 1, 2), (9000, 2048, 2), (13000, 64, 2), (20000, 2048, 2), (30000, 300, 2),
                                   (50000, 2048, 2), (36000, 2048, 130), (50000, 2048, 130), (57000, 100, 128),
                                   (64512, 2048, 129), (64513, 700, 128)])
def test_long_rows_with_ties_nans_and_rows_cut_short(n, k, t):
    s = tied_rows(t, n, seed=n * 7 + k, nans=True)
    s[-1, : n // 2] = 2.5   # more ties at the threshold than k
    s = s.to(dev)
    for cut in (0, 1, 3, n // 2, n):
        ends = torch.full((t,), n, dtype=torch.int32, device=dev)
        ends[0] = max(0, n - cut)
        assert torch.equal(si.topk(s, ends, k).long().cpu(), exact_picks(s, ends, k)), (n, k, t, cut)


def test_scores_that_are_not_16_byte_aligned_are_picked_the_same():
    # a row that starts 4 bytes into a buffer, rows an odd stride apart: the select falls back to 4-byte loads
    n, k = 9001, 300
    base = tied_rows(3, n + 5, seed=77, nans=True).to(dev)
    odd = base[:, 1:n + 1]
    ends = i32([n, n - 7, 40])
    assert odd.data_ptr() % 16 != 0
    assert torch.equal(si.topk(odd, ends, k).long().cpu(), exact_picks(odd.contiguous(), ends, k))


def test_rows_of_a_batch_pick_what_they_pick_alone():
    n, k, rows = 20000, 2048, 200
    s = tied_rows(rows, n, seed=n)
    s[1, 100:] = 0.5
    s = s.to(dev)
    ends = torch.full((rows,), n, dtype=torch.int32, device=dev)
    ends[2], ends[3] = n - 777, k + 5
    together = si.topk(s, ends, k)
    for t in range(4):
        assert torch.equal(si.topk(s[t:t + 1].contiguous(), ends[t:t + 1], k)[0], together[t]), t
    assert torch.equal(together[:4].long().cpu(), exact_picks(s[:4], ends[:4], k))


def picks_within_the_products_error(got, exact, exact_scores, slack=1e-3):
    """Where the kernel's picks differ from the exact ones, every pick it took instead scores within `slack` of the
    exact k-th score (the kernel ranks FP32 sums, the oracle float64 ones)."""
    for t in range(len(exact)):
        mine, theirs = set(got[t].tolist()) - {-1}, set(exact[t].tolist()) - {-1}
        if mine != theirs:
            kth = exact_scores[t][list(theirs)].min()
            assert float(exact_scores[t][list(mine - theirs)].min()) >= float(kth) - slack, t


def test_select_in_groups_is_one_call_and_matches_the_oracle():
    call = Call(50, 64, 128, 3000, seed=9, e4m3=True)
    args = (call.q, call.keys, call.w, call.ends, 256)
    at_once = si.select(*args, key_scales=call.scales, workspace_bytes=1 << 30)
    in_groups = si.select(*args, key_scales=call.scales, workspace=torch.empty(7 * 3000, device=dev))      # 7 tokens a launch
    assert torch.equal(at_once, in_groups)
    assert torch.equal(si.topk(call.scores(), call.ends, 256), at_once)
    want = call.exact()
    picks_within_the_products_error(at_once, ref.sparse_index(want, call.ends.cpu().numpy(), 256), want)


def key_store(rows, width, seed, e4m3):
    g = torch.Generator().manual_seed(seed)
    return compressed(torch.empty(rows, width).normal_(0.0, 0.5, generator=g).to(dev).to(torch.bfloat16), e4m3)[:2]


@pytest.mark.parametrize("e4m3,kind", [(False, torch.int32), (False, torch.int64), (True, torch.int32), (True, torch.int64)])
def test_keys_read_in_place_score_as_their_gathered_copy(e4m3, kind):
    groups, each, n = 3, 4, 700
    call = Call(groups * each, 64, 128, n, seed=11)
    store, scales = key_store(5000, 128, 5, e4m3)
    g = torch.Generator().manual_seed(55)
    slots = torch.stack([torch.randperm(5000, generator=g)[:n] for _ in range(groups)]).to(dev).to(kind)
    in_place = si.scores(call.q, store, call.w, call.ends, key_scales=scales, slots=slots)
    for r in range(groups):
        span, at = slice(r * each, (r + 1) * each), slots[r].long()
        gathered = si.scores(call.q[span], store[at], call.w[span], call.ends[span], key_scales=None if scales is None else scales[at])
        assert torch.equal(in_place[span], gathered), r
    first = slice(0, each)
    one_list = si.scores(call.q[first], store, call.w[first], call.ends[first], key_scales=scales, slots=slots[0])      # [n]: one sequence
    assert torch.equal(one_list, in_place[first])
    picked = si.select(call.q[first], store, call.w[first], call.ends[first], 16, key_scales=scales, slots=slots[0])
    assert torch.equal(picked, si.topk(in_place[first], call.ends[first], 16))
    with pytest.raises(ValueError):      # 5 tokens are not 3 groups
        si.scores(call.q[:5], store, call.w[:5], call.ends[:5], key_scales=scales, slots=slots)
    with pytest.raises(ValueError):      # slots are integers
        si.scores(call.q, store, call.w, call.ends, key_scales=scales, slots=slots.float())


def test_graphs_capture_a_select():
    call = Call(4, 64, 128, 2048, seed=4)
    out = torch.empty(4, 512, dtype=torch.int32, device=dev)
    room = torch.empty(4 * 2048, device=dev)
    select = lambda: si.select(call.q, call.keys, call.w, call.ends, 512, out=out, workspace=room)
    select()
    want = out.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        select()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            select()
    for _ in range(3):
        out.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)


def test_it_refuses_what_it_does_not_take():
    call = Call(2, 64, 128, 10)
    q, keys, w, ends = call.q, call.keys, call.w, call.ends
    refused = [
        lambda: si.scores(q.float(), keys, w, ends),                           # FP32 queries
        lambda: si.scores(q, keys.half(), w, ends),                            # keys of another 16-bit type than the queries
        lambda: si.scores(q, keys.to(torch.float8_e4m3fn), w, ends),           # E4M3 keys without their scales
        lambda: si.scores(q, keys, w, ends.long()),                            # int64 ends
        lambda: si.scores(q[:, :48], keys, w[:, :48], ends),                   # heads not a power of two
        lambda: si.topk(torch.zeros(2, 10, device=dev), ends, 0),              # k of nothing
        lambda: si.scores(q.cpu(), keys.cpu(), w.cpu(), ends.cpu()),           # there is no CPU path
    ]
    for call_it in refused:
        with pytest.raises(ValueError):
            call_it()


def test_one_list_for_many_tokens_takes_the_shared_kernel_whatever_their_count():
    # One slot list [n] for every token (a prompt chunk of one sequence): 19 or 21 tokens fill no whole workgroups of 4
    # or 8, and share their keys through LDS all the same; every token scores as it does alone.
    n = 900
    g = torch.Generator().manual_seed(15)
    store = (torch.randn(4000, 128, generator=g) * 0.5).to(dev).to(torch.bfloat16)
    slots = torch.randperm(4000, generator=g)[:n].to(dev)
    for tokens in (19, 21):
        call = Call(tokens, 64, 128, n, seed=16 + tokens)
        q, w, ends = call.q, call.w, call.ends
        got = si.scores(q, store, w, ends, slots=slots)
        assert torch.equal(got, si.scores(q, store[slots], w, ends))
        for t in (0, 7, tokens - 1):
            assert torch.equal(got[t], si.scores(q[t:t + 1], store, w[t:t + 1], ends[t:t + 1], slots=slots)[0]), t


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("each", [16, 12])
def test_a_rounds_rows_share_their_keys_in_place(fp8, each):
    # Many tokens in groups (a round's rows, each a sequence with its own slots): groups of 16 fill the workgroups that
    # share keys through LDS, groups of 12 do not and go a token a workgroup; either way the gathered keys' bits.
    rows, n = 4, 900
    call = Call(rows * each, 64, 128, n, seed=13)
    q, w, ends = call.q, call.w, call.ends
    g = torch.Generator().manual_seed(6)
    store = (torch.randn(4000, 128, generator=g) * 0.5).to(dev).to(torch.bfloat16)
    scales = None
    if fp8:
        scales = (store.float().abs().amax(1) / 448.0).clamp_min(1e-30)
        store = (store.float() / scales[:, None]).to(torch.float8_e4m3fn)
    slots = torch.stack([torch.randperm(4000, generator=g)[:n] for _ in range(rows)]).to(dev)
    got = si.scores(q, store, w, ends, key_scales=scales, slots=slots)
    for r in range(rows):
        span = slice(r * each, (r + 1) * each)
        want = si.scores(q[span], store[slots[r]], w[span], ends[span], key_scales=None if scales is None else scales[slots[r]])
        assert torch.equal(got[span].view(torch.int32), want.view(torch.int32)), r
        alone = si.scores(q[span][:1], store, w[span][:1], ends[span][:1], key_scales=scales, slots=slots[r].to(torch.int32))
        assert torch.equal(alone[0].view(torch.int32), got[span][0].view(torch.int32)), r


def test_calls_past_a_launchs_tokens_go_in_runs(monkeypatch):
    monkeypatch.setattr(si, "_LAUNCH_TOKENS", 40)
    call = Call(100, 8, 64, 300, seed=17)
    q, keys, w, ends = call.q, call.keys, call.w, call.ends
    runs = si.scores(q, keys, w, ends)
    g = torch.Generator().manual_seed(7)
    slots = torch.stack([torch.randperm(300, generator=g)[:200] for _ in range(5)]).to(dev)      # 5 groups of 20
    ends2 = ends.clamp(max=200)
    grouped = si.scores(q, keys, w, ends2, slots=slots)
    wide = si.scores(q, keys, w, ends2, slots=slots[:2].repeat_interleave(1, 0)[:2])            # 2 groups of 50: past 40 each
    monkeypatch.setattr(si, "_LAUNCH_TOKENS", 65535)
    assert torch.equal(runs, si.scores(q, keys, w, ends))
    assert torch.equal(grouped, si.scores(q, keys, w, ends2, slots=slots))
    assert torch.equal(wide, si.scores(q, keys, w, ends2, slots=slots[:2]))


@pytest.mark.parametrize("kind,fp8_keys", [("bf16", False), ("fp8", True)])
def test_a_sparse_decode_step_reads_the_blocks_the_index_selects(kind, fp8_keys):
    # What the reference's sparse reader does with the two modules (inference/attention-state/code/sparse_index.py, then
    # paged_kv_attention.attend(blocks=)): four decode tokens of one sequence of 4,000 positions, one index key per
    # block of 64 positions; each token scores the blocks it may see, its 8 best become its block list, and the
    # attention reads those blocks only. The picks against the oracle's, the attention against float64 attention over
    # the listed blocks.
    from tests.support import Cache, rand_q
    block, n_pos, k = 64, 4000, 8
    n_blocks = -(-n_pos // block)
    cache = Cache(kind, 2, 128, 128, 16, [n_pos])
    index = Call(4, 16, 64, n_blocks, seed=21, e4m3=fp8_keys)
    q, keys, scales, w = index.q, index.keys, index.scales, index.w
    firsts = n_pos - 4
    ends = torch.tensor([(firsts + t) // block + 1 for t in range(4)], dtype=torch.int32, device=dev)   # the blocks a token may see
    picked = si.select(q, keys, w, ends, k, key_scales=scales)
    assert picked.dtype == torch.int32 and picked.shape == (4, k)
    index.ends = ends
    want_scores = index.exact()
    exact = ref.sparse_index(want_scores, ends.cpu().numpy(), k)
    for t in range(4):
        a, b = set(picked[t].tolist()), set(exact[t].tolist())
        if a != b:      # a pick that differs scores within the products' error of the k-th
            assert float(want_scores[t][list(a - b)].min()) >= float(want_scores[t][list(b)].min()) - 1e-3, t
    qa = rand_q(4, 8, 128, 5)
    lse = torch.empty(4, 8, device=dev)
    zero = torch.zeros(1, dtype=torch.int32, device=dev)
    at = torch.tensor([firsts], dtype=torch.int64, device=dev)
    out = cache.attend(qa, zero, zero, at, 4, blocks=picked, block_size=block, lse=lse, partitions=4)
    want, want_lse = cache.want(qa.to(torch.bfloat16), 0, firsts, 4, blocks=picked.cpu(), block_size=block)
    torch.testing.assert_close(out.double().cpu(), want, atol=8e-3, rtol=2e-2)
    torch.testing.assert_close(lse.double().cpu(), want_lse, atol=1e-3, rtol=1e-4)
    # the same step as one captured graph: no host work between the index and the attention
    graph = torch.cuda.CUDAGraph()
    again, picked_again = torch.empty_like(out), torch.empty_like(picked)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        si.select(q, keys, w, ends, k, key_scales=scales, out=picked_again)
        cache.attend(qa, zero, zero, at, 4, blocks=picked_again, block_size=block, partitions=4, out=again)
        torch.cuda.synchronize()
        picked_again.fill_(-1), again.zero_()
        with torch.cuda.graph(graph, stream=stream):
            si.select(q, keys, w, ends, k, key_scales=scales, out=picked_again)
            cache.attend(qa, zero, zero, at, 4, blocks=picked_again, block_size=block, partitions=4, out=again)
    for _ in range(2):
        picked_again.fill_(-1), again.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(picked_again, picked) and torch.equal(again, out)


@pytest.mark.parametrize("fp8", [False, True])
def test_a_decode_steps_sequences_score_their_own_keys_in_place(fp8):
    # 64 sequences of one token, each over its own 50,000 keys where a store holds them (pages of 64 rows at random
    # places): blocks of thousands of keys a workgroup, the launch whose wavefronts keep three tiles of key rows in
    # flight. A sequence's scores are bit for bit those of the sequence alone over a gathered copy of its keys.
    groups, n, page = 64, 50000, 64
    call = Call(groups, 64, 128, 8, seed=31)
    q, w = call.q, call.w
    g = torch.Generator(device=dev).manual_seed(6)
    rows = groups * (n // page + 1) * page
    store = (torch.randn(rows, 128, device=dev, generator=g) * 0.5).to(torch.bfloat16)
    scales = None
    if fp8:
        scales = (store.float().abs().amax(1) / 448.0).clamp_min(1e-30)
        store = (store.float() / scales[:, None]).to(torch.float8_e4m3fn)
    pages = torch.randperm(rows // page, device=dev, generator=g).view(groups, -1)
    slots = (pages[:, :, None] * page + torch.arange(page, device=dev)[None, None, :]).reshape(groups, -1)[:, :n]
    slots = slots.to(torch.int32).contiguous()
    ends = torch.randint(n - 5000, n + 1, (groups,), generator=torch.Generator().manual_seed(2)).to(torch.int32).to(dev)
    ends[0], ends[1], ends[2], ends[3] = n, 0, 17, 4160
    got = si.scores(q, store, w, ends, key_scales=scales, slots=slots)
    assert bool((got[1] == float("-inf")).all())
    for s in (0, 2, 3, 4, 33, 63):
        keys = store[slots[s].long()]
        alone = si.scores(q[s:s + 1], keys, w[s:s + 1], ends[s:s + 1], key_scales=None if scales is None else scales[slots[s].long()])
        assert torch.equal(got[s], alone[0]), s
        seen = int(ends[s])
        assert bool(torch.isfinite(got[s, :seen]).all()) and bool((got[s, seen:] == float("-inf")).all())
    picked = si.topk(got, ends, 64)
    assert torch.equal(picked[0], exact_picks(got[:1], ends[:1], 64)[0].to(dev))
